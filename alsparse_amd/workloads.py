"""Seeded synthetic CSR workloads (bindings of ``libasamd_workloads.so``).

The five benchmark shapes, each also available scaled down for tests:

* ``random_points``   config 1: ``draws`` random (row, col) points, duplicates merged
* ``laplace2d``       config 2: 5-point Laplacian on an nx x ny grid
* ``uniform_rows``    configs 3 and 5: exactly k sorted distinct random columns per row
* ``powerlaw_rmat``   config 4: Zipf(2) row lengths, R-MAT columns

Values and vectors come from the same counter-based generator
(streams 2 = matrix values, 3 = x, 4 = y / C, 5 = B).
"""
import ctypes
import os
from ctypes import c_double, c_int32, c_int64, c_uint64, c_void_p

import numpy as np

from .build import WORKLOADS_PATH

SEED = 20250101
_lib = None


def _load():
    global _lib
    if _lib is None:
        if not os.path.exists(WORKLOADS_PATH):
            raise RuntimeError("%s is missing: run __graft_entry__.build()" % WORKLOADS_PATH)
        lib = ctypes.CDLL(WORKLOADS_PATH)
        lib.wl_draw.restype = c_uint64
        lib.wl_draw.argtypes = [c_uint64, c_uint64, c_uint64]
        for n in ("wl_fill_uniform_f32", "wl_fill_uniform_f64"):
            getattr(lib, n).restype = None
            getattr(lib, n).argtypes = [c_void_p, c_int64, c_uint64, c_uint64, c_double, c_double]
        lib.wl_uniform_rows.restype = c_int64
        lib.wl_uniform_rows.argtypes = [c_int32, c_int32, c_int32, c_uint64, c_int32, c_void_p, c_void_p]
        lib.wl_laplace2d.restype = c_int64
        lib.wl_laplace2d.argtypes = [c_int32, c_int32, c_int32, c_void_p, c_void_p, c_void_p, c_void_p]
        lib.wl_powerlaw_rmat.restype = c_int64
        lib.wl_powerlaw_rmat.argtypes = [c_int32, c_int32, c_uint64, c_int32, c_void_p, c_void_p]
        lib.wl_random_points.restype = c_int64
        lib.wl_random_points.argtypes = [c_int32, c_int32, c_int64, c_uint64, c_int32, c_void_p, c_void_p]
        lib.wl_checksum.restype = c_uint64
        lib.wl_checksum.argtypes = [c_void_p, c_int64]
        _lib = lib
    return _lib


def _p(a):
    return None if a is None else a.ctypes.data_as(c_void_p)


def uniform(n, dtype, stream, seed=SEED, lo=-1.0, hi=1.0):
    """n values uniform in [lo, hi) from the given stream."""
    out = np.empty(int(n), dtype=dtype)
    fn = _load().wl_fill_uniform_f32 if out.dtype == np.float32 else _load().wl_fill_uniform_f64
    fn(_p(out), out.size, seed, stream, lo, hi)
    return out


class Csr:
    """Host CSR triple plus its shape; ``base`` is the index base of row_ptr / col_ind."""

    def __init__(self, rows, cols, row_ptr, col_ind, values, base=0, name=""):
        self.rows, self.cols, self.base, self.name = int(rows), int(cols), int(base), name
        self.row_ptr, self.col_ind, self.values = row_ptr, col_ind, values
        self.nnz = int(row_ptr[-1]) - self.base

    @property
    def dtype(self):
        return self.values.dtype


def real_dtype(dtype):
    """float32 for complex64, float64 for complex128, the dtype itself for real types."""
    return np.empty(0, dtype=dtype).real.dtype


def complex_vector(n, dtype, stream, seed=SEED):
    """Seeded complex vector: real parts from generator stream `stream`, imaginary parts from stream + 100."""
    rd = real_dtype(dtype)
    out = np.empty(int(n), dtype=dtype)
    out.real = uniform(n, rd, stream, seed)
    out.imag = uniform(n, rd, stream + 100, seed)
    return out


def complexify(a, dtype, stream=200):
    """The structure of a real workload with seeded complex values of the given complex dtype."""
    return Csr(a.rows, a.cols, a.row_ptr, a.col_ind, complex_vector(a.nnz, dtype, stream), a.base,
               a.name + ":" + np.dtype(dtype).name)


def uniform_rows(rows, cols, k, dtype=np.float32, seed=SEED, base=0, lo=-1.0, hi=1.0):
    lib = _load()
    k = min(k, cols)
    row_ptr = np.empty(rows + 1, dtype=np.int32)
    col_ind = np.empty(rows * k, dtype=np.int32)
    lib.wl_uniform_rows(rows, cols, k, seed, base, _p(row_ptr), _p(col_ind))
    vals = uniform(rows * k, dtype, 2, seed, lo, hi)
    return Csr(rows, cols, row_ptr, col_ind, vals, base, "uniform_rows(%d,%d,%d)" % (rows, cols, k))


def bimodal_rows(rows, cols, k_short, k_long, every, dtype=np.float32, seed=SEED, base=0):
    """Rows of two lengths: every `every`-th row has k_long entries, the others k_short, columns uniform random
    (sorted, distinct) in both.  Not a benchmark configuration: the workload that the row-length bins are for."""
    if rows % every:
        raise ValueError("rows must be a multiple of `every`")
    periods = rows // every
    short = uniform_rows(periods * (every - 1), cols, k_short, dtype, seed, base)
    long_ = uniform_rows(periods, cols, k_long, dtype, seed + 1, base)
    ks, kl = min(k_short, cols), min(k_long, cols)
    per = (every - 1) * ks + kl
    col = np.empty((periods, per), dtype=np.int32)
    col[:, :(every - 1) * ks] = short.col_ind.reshape(periods, (every - 1) * ks)
    col[:, (every - 1) * ks:] = long_.col_ind.reshape(periods, kl)
    lengths = np.full(rows, ks, dtype=np.int64)
    lengths[every - 1::every] = kl
    row_ptr = np.zeros(rows + 1, dtype=np.int64)
    np.cumsum(lengths, out=row_ptr[1:])
    vals = uniform(periods * per, dtype, 2, seed)
    return Csr(rows, cols, (row_ptr + base).astype(np.int32), col.reshape(-1), vals, base,
               "bimodal_rows(%d,%d,%d,%d,%d)" % (rows, cols, k_short, k_long, every))


def stencil3d(nx, ny, nz, dtype=np.float64, seed=SEED, base=0):
    """The 27-point stencil on an nx x ny x nz grid (x fastest): every grid point is coupled to itself and to its
    neighbours within one step in each direction, 8 to 27 entries per row, columns ascending, random values.
    Not a benchmark configuration: the structure of a trilinear finite-element matrix, rows of similar lengths
    whose x entries neighbouring rows share."""
    rows = nx * ny * nz
    idx = np.arange(rows, dtype=np.int64)
    ix, iy, iz = idx % nx, (idx // nx) % ny, idx // (nx * ny)
    offsets = [(dz, dy, dx) for dz in (-1, 0, 1) for dy in (-1, 0, 1) for dx in (-1, 0, 1)]  # ascending columns
    masks = [((ix + dx >= 0) & (ix + dx < nx) & (iy + dy >= 0) & (iy + dy < ny) & (iz + dz >= 0) & (iz + dz < nz))
             for dz, dy, dx in offsets]
    lengths = np.zeros(rows, dtype=np.int64)
    for mk in masks:
        lengths += mk
    row_ptr = np.zeros(rows + 1, dtype=np.int64)
    np.cumsum(lengths, out=row_ptr[1:])
    nnz = int(row_ptr[-1])
    if nnz >= 2 ** 31:
        raise ValueError("more than 2^31 - 1 entries")
    col_ind = np.empty(nnz, dtype=np.int32)
    pos = row_ptr[:-1].copy()
    for (dz, dy, dx), mk in zip(offsets, masks):
        col_ind[pos[mk]] = (idx[mk] + (dz * ny + dy) * nx + dx + base).astype(np.int32)
        pos += mk
    vals = uniform(nnz, dtype, 2, seed)
    return Csr(rows, rows, (row_ptr + base).astype(np.int32), col_ind, vals, base, "stencil3d(%d,%d,%d)" % (nx, ny, nz))


def laplace2d(nx, ny, dtype=np.float64, base=0):
    lib = _load()
    rows = nx * ny
    nnz = lib.wl_laplace2d(nx, ny, base, None, None, None, None)
    row_ptr = np.empty(rows + 1, dtype=np.int32)
    col_ind = np.empty(nnz, dtype=np.int32)
    vals = np.empty(nnz, dtype=dtype)
    if vals.dtype == np.float64:
        lib.wl_laplace2d(nx, ny, base, _p(row_ptr), _p(col_ind), _p(vals), None)
    else:
        lib.wl_laplace2d(nx, ny, base, _p(row_ptr), _p(col_ind), None, _p(vals))
    return Csr(rows, rows, row_ptr, col_ind, vals, base, "laplace2d(%d,%d)" % (nx, ny))


def powerlaw_rmat(levels, max_len=200000, dtype=np.float32, seed=SEED, base=0):
    lib = _load()
    rows = 1 << levels
    row_ptr = np.empty(rows + 1, dtype=np.int32)
    nnz = lib.wl_powerlaw_rmat(levels, max_len, seed, base, _p(row_ptr), None)
    col_ind = np.empty(nnz, dtype=np.int32)
    lib.wl_powerlaw_rmat(levels, max_len, seed, base, _p(row_ptr), _p(col_ind))
    vals = uniform(nnz, dtype, 2, seed, 0.0, 1.0)
    return Csr(rows, rows, row_ptr, col_ind, vals, base, "powerlaw_rmat(2^%d)" % levels)


def random_points(rows, cols, draws, dtype=np.float32, seed=SEED, base=0):
    lib = _load()
    nnz = lib.wl_random_points(rows, cols, draws, seed, base, None, None)
    row_ptr = np.empty(rows + 1, dtype=np.int32)
    col_ind = np.empty(nnz, dtype=np.int32)
    lib.wl_random_points(rows, cols, draws, seed, base, _p(row_ptr), _p(col_ind))
    vals = uniform(nnz, dtype, 2, seed)
    return Csr(rows, cols, row_ptr, col_ind, vals, base, "random_points(%d,%d,%d)" % (rows, cols, draws))


def checksum(a):
    a = np.ascontiguousarray(a)
    return int(_load().wl_checksum(_p(a), a.nbytes))


# ---- the five benchmark configurations (scale < 1 shrinks them for tests) ------
def config(idx, scale_log2=0):
    """Returns (csr, x, y0, alpha, beta, extra).  ``scale_log2`` = s shrinks the
    row count by 2^s (s = 0 is the full benchmark shape)."""
    s = scale_log2
    if idx == 1:
        a = random_points(1000, 1000, 5000, np.float32)
        return a, uniform(a.cols, np.float32, 3), np.zeros(a.rows, np.float32), 1.0, 0.0, {}
    if idx == 2:
        n = 2048 >> (s // 2)
        a = laplace2d(n, n, np.float64)
        return a, uniform(a.cols, np.float64, 3), np.zeros(a.rows, np.float64), 1.0, 0.0, {}
    if idx == 3:
        rows = (1 << 24) >> s
        a = uniform_rows(rows, rows, 16, np.float32)
        return a, uniform(a.cols, np.float32, 3), uniform(a.rows, np.float32, 4), 1.0, 0.5, {}
    if idx == 4:
        a = powerlaw_rmat(23 - s, 200000, np.float32)
        return a, uniform(a.cols, np.float32, 3), np.zeros(a.rows, np.float32), 1.0, 0.0, {}
    if idx == 5:
        rows = (1 << 20) >> s
        a = uniform_rows(rows, rows, 32, np.float32)
        n = 64
        B = uniform(a.cols * n, np.float32, 5).reshape(a.cols, n)
        C = uniform(a.rows * n, np.float32, 4).reshape(a.rows, n)
        return a, B, C, 1.5, 0.5, {"n": n}
    raise ValueError("config index 1..5")


def spmv_bytes(rows, cols, nnz, itemsize, beta):
    """Algorithmic (compulsory) traffic of y = alpha*A*x + beta*y."""
    return nnz * (itemsize + 4) + (rows + 1) * 4 + cols * itemsize + rows * itemsize * (2 if beta != 0 else 1)


def spmm_bytes(rows, k, n, nnz, itemsize, beta):
    """Algorithmic (compulsory) traffic of C = alpha*A*B + beta*C."""
    return nnz * (itemsize + 4) + (rows + 1) * 4 + k * n * itemsize + rows * n * itemsize * (2 if beta != 0 else 1)
