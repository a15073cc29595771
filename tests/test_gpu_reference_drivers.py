"""The reference's OWN GPU test programs (test/dcu/level2/mv_csr_?_dcu_test.cpp, mv_coo_?, mv_ell_?
for ? in s, d, c, z; spmv_{csr,coo,ell}_s; test/dcu/level3/mm_csr_?_dcu_test.cpp,
mm_csr_s_dcu_row_test.cpp; and the CPU programs test/arm/mv_?_csr_arm_test.c, mm_?_csr_arm_test.c), compiled unchanged
against this repository's headers and library by `make -C oracle ref_drivers` (into oracle/_ref/,
where the reference tree is present) and run here on a coordinate file: they read the file, take
the COO -> CSR / ELL route, call alphasparse_dcu_?_csrmv / _csrmm / _coomv / _ellmv and compare with
rocSPARSE through check_s / check_d, printing "correct,<ratio>".  Skipped where the programs were
not built."""
import os
import subprocess

import numpy as np
import pytest
import scipy.io
import scipy.sparse as sp

from helpers import announce

pytestmark = pytest.mark.gpu
HERE = os.path.dirname(os.path.abspath(__file__))
BIN = os.path.join(os.path.dirname(HERE), "oracle", "_ref")

PROGRAMS = {
    "mv_csr_s_dcu_test": [[], ["--transA=T"]],
    "mv_csr_d_dcu_test": [[], ["--transA=T"]],
    "mv_coo_s_dcu_test": [[]],
    "mv_coo_d_dcu_test": [[]],
    "mv_ell_s_dcu_test": [[]],
    "mv_ell_d_dcu_test": [[]],
    "spmv_csr_s_dcu_test": [[]],
    "spmv_coo_s_dcu_test": [[]],
    "spmv_ell_s_dcu_test": [[]],
    "mm_csr_s_dcu_test": [["--columns=8", "--layout=C"], ["--columns=70", "--layout=C"]],
    "mm_csr_d_dcu_test": [["--columns=8", "--layout=C"]],
    "mm_csr_s_dcu_row_test": [["--columns=64"]],
    # complex element types (the coordinate reader gives every entry equal real and imaginary parts);
    # mv_csr_c / mv_csr_z pass rocSPARSE a half-initialised beta and are left out
    "mv_coo_c_dcu_test": [[]],
    "mv_coo_z_dcu_test": [[]],
    "mv_ell_c_dcu_test": [[]],
    "mv_ell_z_dcu_test": [[]],
    "mm_csr_c_dcu_test": [["--columns=8", "--layout=C"]],
    "mm_csr_z_dcu_test": [["--columns=8", "--layout=C"]],
    # the CPU test programs (test/arm/*.c): alphasparse_?_mv / _mm against the _plain variants through
    # check_?_l2 / _l3; both run on the GPU here, through different kernels
    "mv_s_csr_arm_test": [[], ["--transA=T"]],
    "mv_d_csr_arm_test": [[], ["--transA=T"]],
    "mv_c_csr_arm_test": [[], ["--transA=T"], ["--transA=H"]],
    "mv_z_csr_arm_test": [[], ["--transA=T"], ["--transA=H"]],
    "mm_s_csr_arm_test": [["--columns=8"], ["--columns=8", "--layout=C"], ["--columns=8", "--transA=T"]],
    "mm_d_csr_arm_test": [["--columns=8"], ["--columns=8", "--layout=C", "--transA=T"]],
    "mm_c_csr_arm_test": [["--columns=8"], ["--columns=8", "--layout=C", "--transA=H"]],
    "mm_z_csr_arm_test": [["--columns=8"], ["--columns=8", "--transA=H"]],
}


@pytest.fixture(scope="module")
def matrix_file(tmp_path_factory):
    d = tmp_path_factory.mktemp("mtx")
    rng = np.random.default_rng(12)
    m, n = 3000, 2500
    lens = np.minimum(1 + rng.zipf(1.7, m), 400)       # skewed rows, none empty
    rows = np.repeat(np.arange(m), lens)
    cols = np.concatenate([rng.choice(n, k, replace=False) for k in lens])
    vals = rng.uniform(-1, 1, rows.size)
    path = str(d / "skewed.mtx")
    scipy.io.mmwrite(path, sp.coo_matrix((vals, (rows, cols)), shape=(m, n)), precision=9)
    return path


@pytest.mark.parametrize("program", sorted(PROGRAMS))
def test_reference_program_passes_its_own_check(gpu, matrix_file, program):
    exe = os.path.join(BIN, program)
    if not os.path.exists(exe):
        pytest.skip("%s was not built (make -C oracle ref_drivers needs the reference tree, hipcc and rocSPARSE)" % program)
    for extra in PROGRAMS[program]:
        cmd = [exe, "--data-file=" + matrix_file, "--check"] + extra
        announce("reference program", " ".join(cmd))
        r = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=120)
        out = r.stdout
        assert r.returncode == 0, out[-2000:]
        assert "correct," in out and "error," not in out, out[-2000:]
