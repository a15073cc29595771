"""Seeded random structures through the kernels that read 16-bit column numbers or hold x in LDS: matrices of few
columns (x in one LDS fill), of several fills (column slices over a copy of the entries), and bands (the staged row
blocks with 16-bit column distances); row lengths uniform, geometric, constant, or short with a few long rows; both
index bases, both real types, arrays off their 16-byte alignment.  Every result is compared with the CPU oracle
(the reference's one kernel for every shape: src/kernel/dcu/level2/mv/csrmv/dcu_gemv_vector.h:14-57)."""
import numpy as np
import pytest

from alsparse_amd import workloads as wl
from helpers import DeviceCsr, announce, check_spmv, run_plan_csrmv
from helpers_shapes import csr_from_lengths

pytestmark = pytest.mark.gpu


def _draw(seed):
    rng = np.random.default_rng(7000 + seed)
    dtype = (np.float32, np.float64)[seed % 2]
    kind = ("one_fill", "slices", "band")[seed % 3]
    fill = 163840 // np.dtype(dtype).itemsize
    m = int(rng.integers(1, 6000))
    cols = (int(rng.integers(2, fill)) if kind == "one_fill" else
            int(rng.integers(fill + 1, 9 * fill)) if kind == "slices" else m + int(rng.integers(0, 50)))
    law = int(rng.integers(0, 4))
    if law == 0:
        lengths = rng.integers(0, 60, size=m)
    elif law == 1:
        lengths = rng.geometric(1.0 / 20.0, size=m) - 1
    elif law == 2:
        lengths = np.full(m, int(rng.integers(1, 40)))
    else:
        lengths = rng.integers(0, 8, size=m)
        lengths[rng.integers(0, m, size=max(1, m // 50))] = rng.integers(100, 3000)
    base = int(rng.integers(0, 2))
    lengths = np.minimum(lengths, cols)
    if kind != "band":
        return kind, csr_from_lengths(list(lengths), cols, dtype, seed=seed + 1, base=base), int(rng.integers(0, 4))
    lengths = np.minimum(lengths, min(120, cols))  # (the staged kernel takes rows of up to 128 8-byte entries)
    row_ptr = np.zeros(m + 1, dtype=np.int64)
    np.cumsum(lengths, out=row_ptr[1:])
    col = np.empty(int(row_ptr[-1]), dtype=np.int64)
    for r in range(m):  # columns within 2 000 of the diagonal, on both sides
        lo, hi = max(0, r - 2000), min(cols, r + 2000)
        col[row_ptr[r]:row_ptr[r + 1]] = np.sort(rng.choice(np.arange(lo, hi), size=int(lengths[r]), replace=False))
    a = wl.Csr(m, cols, (row_ptr + base).astype(np.int32), (col + base).astype(np.int32),
               wl.uniform(int(row_ptr[-1]), dtype, 7, seed), base, "band")
    return kind, a, 0


@pytest.mark.parametrize("seed", range(24))
def test_random_structure(gpu, seed):
    kind, a, shift = _draw(seed)
    if a.nnz < 4:
        pytest.skip("drew a matrix of fewer than four entries")
    algo = "stream" if kind == "band" else "xlds"
    x, y0 = wl.uniform(a.cols, a.dtype, 3, seed), wl.uniform(a.rows, a.dtype, 4, seed)
    da = DeviceCsr(a, shift=shift)
    try:
        for alpha, beta in ((1.0, 0.0), (-1.5, 0.75)):
            announce("random structure", seed, kind, a.dtype.name, a.rows, a.cols, "base", a.base, alpha, beta)
            y = run_plan_csrmv(da, algo, alpha, x, beta, y0)
            if y is None:
                pytest.skip("this structure cannot run " + algo)
            check_spmv(a, alpha, x, beta, y0, y, "seed %d %s" % (seed, (alpha, beta)))
    finally:
        da.free()
