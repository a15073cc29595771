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


def real_dtype(dtype):
    """float32 for complex64, float64 for complex128, the dtype itself for real types."""
    return np.empty(0, dtype=dtype).real.dtype


def complex_vector(n, dtype, stream):
    """Seeded complex vector: real parts from generator stream `stream`, imaginary from stream + 100."""
    rd = real_dtype(dtype)
    return (wl.uniform(n, rd, stream) + 1j * wl.uniform(n, rd, stream + 100)).astype(dtype)


def complexify(a, dtype, stream=200):
    """The structure of a real workload with seeded complex values of the given complex dtype."""
    return wl.Csr(a.rows, a.cols, a.row_ptr, a.col_ind, complex_vector(a.nnz, dtype, stream), a.base,
                  a.name + ":" + np.dtype(dtype).name)
