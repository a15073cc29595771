"""TEST INFRASTRUCTURE -- CPU oracle for the CSR SpMV / SpMM path (see oracle.py)."""
