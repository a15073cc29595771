"""Hand-shaped CSR matrices for tests (no GPU, no library needed)."""
import numpy as np

from alsparse_amd import workloads as wl


def csr_from_lengths(lengths, cols, dtype, seed=7, base=0):
    """CSR with the given row lengths, sorted distinct random columns, values in [-1, 1)."""
    rng = np.random.default_rng(seed)
    lengths = np.minimum(np.asarray(lengths, dtype=np.int64), cols)
    row_ptr = np.zeros(len(lengths) + 1, dtype=np.int64)
    np.cumsum(lengths, out=row_ptr[1:])
    col = np.empty(int(row_ptr[-1]), dtype=np.int32)
    for r, n in enumerate(lengths):
        if n:
            if n * 4 < cols:
                c = np.unique(rng.integers(0, cols, size=int(n * 1.3) + 8))
                while c.size < n:
                    c = np.unique(np.concatenate([c, rng.integers(0, cols, size=int(n))]))
                c = np.sort(rng.choice(c, size=int(n), replace=False))
            else:
                c = np.sort(rng.choice(cols, size=int(n), replace=False))
            col[row_ptr[r]:row_ptr[r + 1]] = c
    vals = rng.uniform(-1, 1, size=col.size).astype(dtype)
    return wl.Csr(len(lengths), cols, (row_ptr + base).astype(np.int32), col + np.int32(base), vals, base,
                  "lengths(m=%d,nnz=%d)" % (len(lengths), col.size))


# complex-valued variants of the seeded workloads
real_dtype, complex_vector, complexify = wl.real_dtype, wl.complex_vector, wl.complexify
