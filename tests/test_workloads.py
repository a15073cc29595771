"""The seeded workload generators: structural invariants of every benchmark shape and
64-bit checksums of their arrays (tests/golden/workload_checksums.json), so that the
GPU box and this container multiply the same matrices."""
import json
import os

import numpy as np
import pytest

from alsparse_amd import workloads as wl
from golden_cases import checksum_cases

SUMS = json.load(open(os.path.join(os.path.dirname(__file__), "golden", "workload_checksums.json")))


def test_generated_arrays_match_committed_checksums():
    cases = checksum_cases()
    assert sorted(cases) == sorted(SUMS)
    for key, arrays in cases.items():
        for name, v in arrays.items():
            got = int(v) if np.isscalar(v) else "%016x" % wl.checksum(v)
            assert got == SUMS[key][name], (key, name)


def _check_csr(a, sorted_rows=True):
    rp = a.row_ptr.astype(np.int64) - a.base
    assert rp[0] == 0 and rp[-1] == a.nnz and np.all(np.diff(rp) >= 0)
    ci = a.col_ind.astype(np.int64) - a.base
    assert ci.size == a.nnz and (ci >= 0).all() and (ci < a.cols).all()
    if sorted_rows and a.nnz:
        d = np.diff(ci)
        row_start = np.zeros(a.nnz, bool)
        row_start[rp[1:-1][rp[1:-1] < a.nnz]] = True
        assert np.all((d > 0) | row_start[1:]), "columns must be strictly increasing inside a row"


def test_config1_random_points():
    a, x, y0, alpha, beta, _ = wl.config(1)
    assert (a.rows, a.cols) == (1000, 1000) and 4900 < a.nnz <= 5000 and a.dtype == np.float32
    _check_csr(a)
    assert (alpha, beta) == (1.0, 0.0) and np.all(y0 == 0) and np.abs(x).max() <= 1 and np.abs(a.values).max() <= 1


def test_config2_laplacian_counts_and_values():
    a = wl.laplace2d(2048, 2048, np.float64)
    assert a.rows == 4194304 and a.nnz == 20963328
    _check_csr(a)
    lens = np.diff(a.row_ptr)
    assert lens.min() == 3 and lens.max() == 5 and (lens == 3).sum() == 4
    diag = a.col_ind == np.repeat(np.arange(a.rows, dtype=np.int32), lens)
    assert np.all(a.values[diag] == 4.0) and np.all(a.values[~diag] == -1.0) and diag.sum() == a.rows
    # symmetric structure with neighbours at +-1 and +-nx
    off = a.col_ind.astype(np.int64) - np.repeat(np.arange(a.rows), lens)
    assert set(np.unique(off).tolist()) == {-2048, -1, 0, 1, 2048}
    small = wl.laplace2d(5, 3, np.float32, base=1)
    _check_csr(small)
    assert small.nnz == 5 * 15 - 2 * 5 - 2 * 3


@pytest.mark.parametrize("rows,cols,k", [(4096, 1 << 24, 16), (2048, 1 << 20, 32), (100, 20, 16), (50, 8, 16)])
def test_uniform_rows_exact_count_sorted_distinct(rows, cols, k):
    a = wl.uniform_rows(rows, cols, k, np.float32)
    kk = min(k, cols)
    assert a.nnz == rows * kk and np.all(np.diff(a.row_ptr) == kk)
    _check_csr(a)
    assert np.abs(a.values).max() <= 1
    # rows are generated independently: a prefix of a larger matrix is the same matrix
    b = wl.uniform_rows(rows // 2, cols, k, np.float32)
    assert np.array_equal(b.col_ind, a.col_ind[: b.nnz]) and np.array_equal(b.values, a.values[: b.nnz])


def test_config4_powerlaw_rmat_statistics():
    a = wl.powerlaw_rmat(18, 200000, np.float32)
    _check_csr(a)
    lens = np.diff(a.row_ptr)
    assert lens.min() >= 1 and lens.max() <= 200000
    # P(L >= k) = 1/k before de-duplication: about half the rows have one entry, a quarter at most... and a heavy tail
    assert 0.47 < (lens == 1).mean() < 0.53
    assert 0.72 < (lens <= 3).mean() < 0.80
    assert lens.max() > 5000
    assert (a.values >= 0).all() and (a.values < 1).all()
    # R-MAT skew: column bits are 0 with probability ~0.75-0.79, so the low half of the columns holds most entries
    assert (a.col_ind < a.cols // 2).mean() > 0.7
    # one-based variant is the same matrix shifted
    b = wl.powerlaw_rmat(12, 500, np.float32, base=1)
    c = wl.powerlaw_rmat(12, 500, np.float32, base=0)
    assert np.array_equal(b.row_ptr - 1, c.row_ptr) and np.array_equal(b.col_ind - 1, c.col_ind)


def test_vectors_are_counter_based():
    x = wl.uniform(1000, np.float32, 3)
    assert np.array_equal(wl.uniform(500, np.float32, 3), x[:500])
    assert not np.array_equal(wl.uniform(1000, np.float32, 4), x)
    assert -1 <= x.min() and x.max() < 1 and abs(x.mean()) < 0.1
    assert wl.spmv_bytes(16777216, 16777216, 268435456, 4, 0.5) == 2415919108
    assert wl.spmv_bytes(4194304, 4194304, 20963328, 8, 0.0) == 335446020
    assert wl.spmm_bytes(1048576, 1048576, 64, 33554432, 4, 0.5) == 1077936132
