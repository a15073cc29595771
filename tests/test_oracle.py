"""Pins the CPU oracle (test infrastructure) before anything is compared with it.

The reference stores no golden vectors for this path (its tests are differential
runs on time-seeded random matrices), so the oracle is pinned by
  * brute-force dense products in fp64 on tiny matrices (empty rows, 1-entry rows, a full row),
  * scipy.sparse as an independent library routine,
  * closed forms (identity, diagonal, Laplacian times ones, alpha = 0, beta = 1),
  * invariants (linearity in alpha, row permutation, additive splitting),
  * bit-for-bit agreement with the reference's own sources compiled into oracle/_ref
    (skipped where that library is absent) and with the committed fixtures it produced.
A dropped term, a wrong sign, a transposed operand or a shifted index fails at least one."""
import os
from ctypes import Structure, byref, c_bool, c_double, c_float, c_int32, c_void_p

import numpy as np
import pytest
import scipy.sparse as sp

from alsparse_amd import workloads as wl
from oracle import oracle as orc
from helpers_shapes import csr_from_lengths

DT = [np.float32, np.float64]
EPS = {np.dtype(np.float32): 2.0 ** -24, np.dtype(np.float64): 2.0 ** -53}


def dense(a):
    D = np.zeros((a.rows, a.cols), dtype=np.float64)
    rp, ci = a.row_ptr - a.base, a.col_ind - a.base
    for r in range(a.rows):
        for k in range(rp[r], rp[r + 1]):
            D[r, ci[k]] += float(a.values[k])
    return D


def gamma_bound(a, alpha, x, beta, y0, slack=4):
    """|error| <= slack * (len + 2) * eps * (|alpha| sum|a x| + |beta y0|), per row."""
    rp = a.row_ptr - a.base
    absA = sp.csr_matrix((np.abs(a.values.astype(np.float64)), a.col_ind - a.base, rp), shape=(a.rows, a.cols))
    mag = abs(alpha) * (absA @ np.abs(x.astype(np.float64))) + np.abs(beta * y0.astype(np.float64))
    return slack * (np.diff(rp) + 2) * EPS[a.dtype] * mag


@pytest.mark.parametrize("dtype", DT)
def test_spmv_plain_against_brute_force_dense(dtype):
    lengths = [0, 1, 12, 3, 0, 0, 5, 1, 12, 2, 7, 0]          # empty rows, single entries, full rows (cols = 12)
    for base in (0, 1):
        a = csr_from_lengths(lengths, 12, dtype, seed=11, base=base)
        rng = np.random.default_rng(5)
        x = rng.uniform(-1, 1, a.cols).astype(dtype)
        y0 = rng.uniform(-1, 1, a.rows).astype(dtype)
        for alpha, beta in ((1.0, 0.0), (2.0, 3.0), (-0.5, 1.0), (0.0, 0.75)):
            want = alpha * (dense(a) @ x.astype(np.float64)) + beta * y0.astype(np.float64)
            for got in (orc.csrmv_plain(a, alpha, x, beta, y0), orc.csrmv_omp(a, alpha, x, beta, y0, threads=3),
                        orc.csrmv_omp(a, alpha, x, beta, y0, threads=5, fast=False)):
                assert np.all(np.abs(got - want) <= gamma_bound(a, alpha, x, beta, y0) + 1e-300)
            assert np.allclose(orc.csrmv_f64acc(a, alpha, x, beta, y0), want, rtol=1e-13, atol=1e-13)


@pytest.mark.parametrize("dtype", DT)
def test_spmv_against_scipy_on_every_workload_shape(dtype):
    shapes = [wl.random_points(300, 200, 1500, dtype), wl.laplace2d(31, 17, dtype), wl.uniform_rows(500, 700, 16, dtype),
              wl.powerlaw_rmat(10, 400, dtype), wl.uniform_rows(64, 64, 64, dtype)]
    for a in shapes:
        x = wl.uniform(a.cols, dtype, 3)
        y0 = wl.uniform(a.rows, dtype, 4)
        A = sp.csr_matrix((a.values.astype(np.float64), a.col_ind, a.row_ptr), shape=(a.rows, a.cols))
        want = 1.5 * (A @ x.astype(np.float64)) - 0.25 * y0.astype(np.float64)
        for got in (orc.csrmv_plain(a, 1.5, x, -0.25, y0), orc.csrmv_omp(a, 1.5, x, -0.25, y0, threads=4)):
            assert np.all(np.abs(got - want) <= gamma_bound(a, 1.5, x, -0.25, y0) + 1e-300), a.name


@pytest.mark.parametrize("dtype", DT)
def test_spmv_closed_forms(dtype):
    n = 257
    ident = wl.Csr(n, n, np.arange(n + 1, dtype=np.int32), np.arange(n, dtype=np.int32), np.ones(n, dtype), 0)
    x = wl.uniform(n, dtype, 3)
    y0 = wl.uniform(n, dtype, 4)
    # identity: y = alpha*x + beta*y exactly as two rounded products and a sum
    got = orc.csrmv_plain(ident, 2.0, x, 3.0, y0)
    assert np.array_equal(got, (y0 * dtype(3.0)) + dtype(2.0) * x)
    # diagonal
    d = wl.uniform(n, dtype, 2)
    diag = wl.Csr(n, n, ident.row_ptr, ident.col_ind, d, 0)
    assert np.array_equal(orc.csrmv_plain(diag, 1.0, x, 0.0, y0), d * x)
    # alpha = 0 leaves beta*y; beta = 1, alpha = 0 leaves y untouched
    a = wl.powerlaw_rmat(9, 100, dtype)
    xx, yy = wl.uniform(a.cols, dtype, 3), wl.uniform(a.rows, dtype, 4)
    assert np.array_equal(orc.csrmv_plain(a, 0.0, xx, 0.5, yy), yy * dtype(0.5))
    assert np.array_equal(orc.csrmv_plain(a, 0.0, xx, 1.0, yy), yy)
    # 5-point Laplacian times ones: 4 - (#neighbours), exact in any precision
    nx, ny = 23, 9
    lap = wl.laplace2d(nx, ny, dtype)
    got = orc.csrmv_plain(lap, 1.0, np.ones(lap.cols, dtype), 0.0, np.zeros(lap.rows, dtype)).reshape(ny, nx)
    want = np.zeros((ny, nx))
    want[0, :] += 1
    want[-1, :] += 1
    want[:, 0] += 1
    want[:, -1] += 1
    assert np.array_equal(got, want)


@pytest.mark.parametrize("dtype", DT)
def test_spmv_invariants(dtype):
    a = wl.powerlaw_rmat(10, 300, dtype)
    x, y0 = wl.uniform(a.cols, dtype, 3), wl.uniform(a.rows, dtype, 4)
    base = orc.csrmv_plain(a, 1.0, x, 0.0, y0)
    # power-of-two scaling commutes with rounding: A(4x) = 4 Ax and alpha = 4 likewise
    assert np.array_equal(orc.csrmv_plain(a, 1.0, (4 * x).astype(dtype), 0.0, y0), 4 * base)
    assert np.array_equal(orc.csrmv_plain(a, 4.0, x, 0.0, y0), 4 * base)
    # row permutation equivariance (bit-exact: each row is computed independently)
    perm = np.random.default_rng(1).permutation(a.rows)
    lens = np.diff(a.row_ptr)[perm]
    rp = np.zeros(a.rows + 1, np.int32)
    np.cumsum(lens, out=rp[1:])
    ci = np.concatenate([a.col_ind[a.row_ptr[r]:a.row_ptr[r + 1]] for r in perm]) if a.nnz else a.col_ind
    va = np.concatenate([a.values[a.row_ptr[r]:a.row_ptr[r + 1]] for r in perm])
    ap = wl.Csr(a.rows, a.cols, rp, ci.astype(np.int32), va, 0)
    assert np.array_equal(orc.csrmv_plain(ap, 1.0, x, 0.0, y0), base[perm])
    # additive splitting A = A1 + A2 (even / odd columns)
    for keep in (0, 1):
        pass
    m1 = (a.col_ind % 2) == 0
    parts = []
    for mask in (m1, ~m1):
        rows = np.repeat(np.arange(a.rows), np.diff(a.row_ptr))[mask]
        rp2 = np.zeros(a.rows + 1, np.int32)
        np.add.at(rp2, rows + 1, 1)
        np.cumsum(rp2, out=rp2)
        parts.append(wl.Csr(a.rows, a.cols, rp2, a.col_ind[mask], a.values[mask], 0))
    s = orc.csrmv_f64acc(parts[0], 1.0, x, 0.0, y0) + orc.csrmv_f64acc(parts[1], 1.0, x, 0.0, y0)
    assert np.allclose(s, orc.csrmv_f64acc(a, 1.0, x, 0.0, y0), rtol=1e-12, atol=1e-12)


@pytest.mark.parametrize("dtype", DT)
def test_spmm_plain_against_dense_and_scipy(dtype):
    a = csr_from_lengths([0, 3, 9, 1, 0, 4, 9, 2], 9, dtype, seed=3)
    rng = np.random.default_rng(8)
    n = 5
    B = rng.uniform(-1, 1, (a.cols, n)).astype(dtype)
    C0 = rng.uniform(-1, 1, (a.rows, n)).astype(dtype)
    for alpha, beta in ((1.5, 0.5), (1.0, 0.0), (0.0, 2.0)):
        want = alpha * (dense(a) @ B.astype(np.float64)) + beta * C0.astype(np.float64)
        tol = 64 * EPS[np.dtype(dtype)] * (abs(alpha) * (np.abs(dense(a)) @ np.abs(B.astype(np.float64))) + abs(beta) * np.abs(C0)) + 1e-300
        row = orc.csrmm_plain(a, alpha, B, beta, C0, layout="row")
        rowp = orc.csrmm_plain(a, alpha, B, beta, C0, layout="row", omp=True)
        col = orc.csrmm_plain(a, alpha, np.asfortranarray(B), beta, np.asfortranarray(C0), layout="col")
        assert row.flags.c_contiguous and col.flags.f_contiguous
        for got in (row, rowp, col):
            assert np.all(np.abs(got - want) <= tol)
        assert np.array_equal(row, rowp)          # same per-row arithmetic, rows independent
    a = wl.uniform_rows(200, 150, 8, dtype)
    B = wl.uniform(a.cols * 7, dtype, 5).reshape(a.cols, 7)
    C0 = wl.uniform(a.rows * 7, dtype, 4).reshape(a.rows, 7)
    A = sp.csr_matrix((a.values.astype(np.float64), a.col_ind, a.row_ptr), shape=(a.rows, a.cols))
    want = 1.5 * (A @ B.astype(np.float64)) + 0.5 * C0
    assert np.allclose(orc.csrmm_plain(a, 1.5, B, 0.5, C0), want, rtol=0, atol=200 * EPS[np.dtype(dtype)] * 8)
    # one dense column == SpMV, bit for bit (same loop order)
    x = np.ascontiguousarray(B[:, 0])
    y = orc.csrmv_plain(a, 1.0, x, 0.0, np.zeros(a.rows, dtype))
    c = orc.csrmm_plain(a, 1.0, x.reshape(-1, 1), 0.0, np.zeros((a.rows, 1), dtype))
    assert np.array_equal(c[:, 0], y)


def test_partition_rows_by_nnz_matches_definition():
    """partition[i] = lower_bound(rows_end[0 .. rows-1), i * (nnz / T)); partition[T] = rows
    (src/util/partition.c:79-92)."""
    rng = np.random.default_rng(0)
    for rows, T in ((1, 1), (17, 4), (1000, 16), (50, 64)):
        lens = rng.integers(0, 9, rows)
        lens[rng.integers(0, rows)] += 200
        re = np.cumsum(lens).astype(np.int32)
        got = orc.partition_rows_by_nnz(re, T)
        ave = int(re[-1]) // T
        want = [0] + [int(np.searchsorted(re[:rows - 1], ave * i, side="left")) for i in range(1, T)] + [rows]
        assert got.tolist() == want
        assert all(got[i] <= got[i + 1] for i in range(T))


def test_csr2coo_and_csr2ell_definitions():
    for base in (0, 1):
        a = csr_from_lengths([0, 3, 0, 0, 5, 1, 0, 2, 0], 7, np.float32, seed=2, base=base)
        rp0 = a.row_ptr - base
        # closed form: coo_row[k] = (upper_bound(row_ptr, k) - 1) + base
        want = np.searchsorted(rp0, np.arange(a.nnz), side="right") - 1 + base
        assert np.array_equal(orc.csr2coo(a), want)
        w = orc.csr2ell_width(a)
        assert w == 5
        for ell_base in (0, 1):
            ev, ec = orc.csr2ell(a, ell_base=ell_base)
            assert ev.shape == (w * a.rows,)
            # brute force, column-major [slot*m + row], padding (0, ell_base)
            for r in range(a.rows):
                for s in range(w):
                    k = rp0[r] + s
                    if k < rp0[r + 1]:
                        assert ev[s * a.rows + r] == a.values[k] and ec[s * a.rows + r] == a.col_ind[k] - base + ell_base
                    else:
                        assert ev[s * a.rows + r] == 0 and ec[s * a.rows + r] == ell_base
            # round trip ELL -> CSR drops the padding
            E = ev.reshape(w, a.rows).T
            keep = np.arange(w)[None, :] < np.diff(rp0)[:, None]
            assert np.array_equal(E[keep], a.values)
    big = wl.Csr(1 << 23, 4, np.zeros((1 << 23) + 1, np.int32), np.zeros(0, np.int32), np.zeros(0, np.float32), 0)
    with pytest.raises(OverflowError):
        orc.csr2ell(big, width=256)             # 2^31 entries: the reference aborts here


@pytest.mark.parametrize("dtype", DT)
def test_coomv_and_ellmv_against_brute_force_and_csr(dtype):
    """COO and ELL products: fp64 brute force straight from the format's arrays (so a
    row-major / column-major mix-up or a shifted slot fails), any entry order for COO,
    out-of-range ELL slots skipped, and bit-equality with the CSR oracle on integer data
    (where every partial sum is exact, so the order and fma contraction cannot matter)."""
    rng = np.random.default_rng(11)
    for a in (csr_from_lengths([0, 3, 0, 0, 5, 1, 0, 2, 0, 70], 90, dtype, seed=2), wl.laplace2d(9, 7, dtype),
              wl.powerlaw_rmat(7, 300, dtype)):
        x, y0 = wl.uniform(a.cols, dtype, 3), wl.uniform(a.rows, dtype, 4)
        rows = orc.csr2coo(a)
        alpha, beta = 2.0, 3.0
        want = beta * y0.astype(np.float64)
        for k in range(a.nnz):
            want[rows[k]] += alpha * float(a.values[k]) * float(x[a.col_ind[k]])
        bound = gamma_bound(a, alpha, x, beta, y0)
        assert np.all(np.abs(orc.coomv_plain(a, rows, alpha, x, beta, y0) - want) <= bound)
        # any storage order gives the same product
        perm = rng.permutation(a.nnz)
        shuffled = wl.Csr(a.rows, a.cols, a.row_ptr, a.col_ind[perm], a.values[perm], 0)
        assert np.all(np.abs(orc.coomv_plain(shuffled, rows[perm], alpha, x, beta, y0) - want) <= bound)
        # ELL: brute force from the column-major arrays themselves
        w = orc.csr2ell_width(a)
        ev, ec = orc.csr2ell(a)
        ec = ec.copy()
        want = beta * y0.astype(np.float64)
        for r in range(a.rows):
            for s_ in range(w):
                want[r] += alpha * float(ev[s_ * a.rows + r]) * float(x[ec[s_ * a.rows + r]])
        assert np.all(np.abs(orc.ellmv(a.rows, a.cols, ev, ec, w, alpha, x, beta, y0) - want) <= bound)
        # a slot whose index is >= n is skipped (dcu_gemv_x_ell.cpp:33), whatever its value
        pad = np.flatnonzero(ev == 0)
        if pad.size:
            ev2, ec2 = ev.copy(), ec.copy()
            ev2[pad[0]], ec2[pad[0]] = 1e6, a.cols
            assert np.array_equal(orc.ellmv(a.rows, a.cols, ev2, ec2, w, alpha, x, beta, y0),
                                  orc.ellmv(a.rows, a.cols, ev, ec, w, alpha, x, beta, y0))
        # integer data: exact in every order
        ai = wl.Csr(a.rows, a.cols, a.row_ptr, a.col_ind, rng.integers(-4, 5, a.nnz).astype(dtype), 0)
        xi, yi = rng.integers(-4, 5, a.cols).astype(dtype), rng.integers(-4, 5, a.rows).astype(dtype)
        ref = orc.csrmv_plain(ai, 2.0, xi, 3.0, yi)
        assert np.array_equal(orc.coomv_plain(ai, rows, 2.0, xi, 3.0, yi), ref)
        evi, eci = orc.csr2ell(ai)
        assert np.array_equal(orc.ellmv(a.rows, a.cols, evi, eci, w, 2.0, xi, 3.0, yi), ref)
        # beta = 0 still multiplies: y0 = 0 stays 0 on empty rows
        assert orc.coomv_plain(a, rows, 1.0, x, 0.0, y0)[0] == 0 or np.diff(a.row_ptr)[0] > 0


@pytest.mark.parametrize("dtype", DT)
def test_transposed_spmv_against_dense_scipy_and_the_untransposed_oracle(dtype):
    """y = alpha A^T x + beta y: dense fp64 brute force on rectangular matrices (a swapped
    m / n or a forgotten transpose cannot pass), scipy, and the plain oracle applied to an
    explicitly transposed matrix (same sums in another order: within the rounding bound;
    bit-equal on integer data)."""
    rng = np.random.default_rng(13)
    for a in (csr_from_lengths([0, 3, 0, 0, 5, 1, 0, 2, 0, 70], 90, dtype, seed=2), wl.laplace2d(9, 7, dtype),
              wl.powerlaw_rmat(7, 300, dtype), wl.uniform_rows(50, 400, 8, dtype, base=1)):
        x, y0 = wl.uniform(a.rows, dtype, 3), wl.uniform(a.cols, dtype, 4)
        at = orc.transpose(a)
        assert (at.rows, at.cols, at.nnz) == (a.cols, a.rows, a.nnz)
        D = dense(a)
        assert np.array_equal(dense(at), D.T)
        for alpha, beta in ((1.0, 0.0), (2.0, 3.0), (-0.5, 1.0)):
            got = orc.csrmv_trans_plain(a, alpha, x, beta, y0)
            want = alpha * (D.T @ x.astype(np.float64)) + beta * y0.astype(np.float64)
            bound = gamma_bound(at, alpha, x, beta, y0)
            assert np.all(np.abs(got - want) <= bound)
            sp_want = alpha * (sp.csr_matrix(D).T @ x.astype(np.float64)) + beta * y0.astype(np.float64)
            assert np.all(np.abs(got - sp_want) <= bound)
            assert np.all(np.abs(got - orc.csrmv_plain(at, alpha, x, beta, y0)) <= 2 * bound)
        ai = wl.Csr(a.rows, a.cols, a.row_ptr, a.col_ind, rng.integers(-4, 5, a.nnz).astype(dtype), a.base)
        xi, yi = rng.integers(-4, 5, a.rows).astype(dtype), rng.integers(-4, 5, a.cols).astype(dtype)
        assert np.array_equal(orc.csrmv_trans_plain(ai, 2.0, xi, 3.0, yi), orc.csrmv_plain(orc.transpose(ai), 2.0, xi, 3.0, yi))


def test_error_metric_detects_planted_errors():
    a = wl.uniform_rows(400, 300, 16, np.float32)
    x, y0 = wl.uniform(a.cols, np.float32, 3), wl.uniform(a.rows, np.float32, 4)
    ref = orc.csrmv_plain(a, 1.0, x, 0.5, y0)
    assert orc.csrmv_err(a, 1.0, x, 0.5, y0, ref, ref).full == 0
    bad = ref.copy()
    bad[123] += 1e-2
    e = orc.csrmv_err(a, 1.0, x, 0.5, y0, bad, ref)
    assert e.row == 123 and e.full > 1e-4 and e.strict >= e.full
    bad = ref.copy()
    bad[7] = np.nan
    assert orc.csrmv_err(a, 1.0, x, 0.5, y0, bad, ref).full == np.inf
    empty = csr_from_lengths([0, 2, 0], 5, np.float32)
    xe, ye = np.ones(5, np.float32), np.ones(3, np.float32)
    r = orc.csrmv_plain(empty, 1.0, xe, 0.5, ye)
    wrong = r.copy()
    wrong[2] += 1e-7
    assert orc.csrmv_err(empty, 1.0, xe, 0.5, ye, wrong, r).zero_den_mismatch == 1


# ---- the reference's own kernels, compiled from its sources ---------------------
needs_ref = pytest.mark.skipif(not orc.ref_available(), reason="oracle/_ref not built (reference tree absent)")


def _ref_mv(name, a, alpha, x, beta, y0, threads=None):
    T = c_float if a.dtype == np.float32 else c_double
    fn, mat = orc.ref_call(name, a, threads=threads)
    fn.argtypes = [T, c_void_p, c_void_p, T, c_void_p]
    y = y0.copy()
    assert fn(T(alpha), byref(mat.s), x.ctypes.data_as(c_void_p), T(beta), y.ctypes.data_as(c_void_p)) == 0
    return y


def _ref_mm(name, a, alpha, B, ldb, beta, C0, ldc, n):
    T = c_float if a.dtype == np.float32 else c_double
    fn, mat = orc.ref_call(name, a)
    fn.argtypes = [T, c_void_p, c_void_p, c_int32, c_int32, T, c_void_p, c_int32]
    C = C0.copy(order="K")
    assert fn(T(alpha), byref(mat.s), B.ctypes.data_as(c_void_p), n, ldb, T(beta), C.ctypes.data_as(c_void_p), ldc) == 0
    return C


class _RefCoo(Structure):  # spmat_coo_?_t, include/alphasparse/spmat.h:73-86 of the reference
    _fields_ = [("values", c_void_p), ("row_indx", c_void_p), ("col_indx", c_void_p), ("rows", c_int32),
                ("cols", c_int32), ("nnz", c_int32), ("ordered", c_bool), ("d_rows_indx", c_void_p),
                ("d_cols_indx", c_void_p), ("d_values", c_void_p)]


@needs_ref
@pytest.mark.parametrize("dtype", DT)
def test_coomv_oracle_is_bit_identical_to_reference_kernel(dtype):
    T = c_float if dtype == np.float32 else c_double
    fn = getattr(orc.ref_lib(), "gemv_%s_coo_plain" % ("s" if dtype == np.float32 else "d"))
    fn.argtypes, fn.restype = [T, c_void_p, c_void_p, T, c_void_p], c_int32
    rng = np.random.default_rng(5)
    for a in (wl.random_points(1000, 1000, 5000, dtype), wl.powerlaw_rmat(12, 3000, dtype),
              csr_from_lengths([0, 1, 0, 70, 3, 0], 100, dtype)):
        x, y0 = wl.uniform(a.cols, dtype, 3), wl.uniform(a.rows, dtype, 4)
        rows, cols, vals = orc.csr2coo(a), a.col_ind.copy(), a.values.copy()
        for shuffle in (False, True):
            if shuffle:
                perm = rng.permutation(a.nnz)
                rows, cols, vals = rows[perm].copy(), cols[perm].copy(), vals[perm].copy()
            coo = _RefCoo(vals.ctypes.data, rows.ctypes.data, cols.ctypes.data, a.rows, a.cols, a.nnz, False, None, None, None)
            for alpha, beta in ((1.0, 0.0), (2.0, 3.0)):
                y = y0.copy()
                assert fn(T(alpha), byref(coo), x.ctypes.data_as(c_void_p), T(beta), y.ctypes.data_as(c_void_p)) == 0
                mine = orc.coomv_plain(wl.Csr(a.rows, a.cols, a.row_ptr, cols, vals, 0), rows, alpha, x, beta, y0)
                assert np.array_equal(mine, y), (a.name, shuffle, alpha, beta)


@needs_ref
@pytest.mark.parametrize("dtype", DT)
def test_oracle_is_bit_identical_to_reference_kernels(dtype):
    shapes = [wl.random_points(1000, 1000, 5000, dtype), wl.laplace2d(40, 25, dtype), wl.uniform_rows(3000, 2000, 16, dtype),
              wl.powerlaw_rmat(12, 3000, dtype), csr_from_lengths([0, 1, 0, 70, 3, 0], 100, dtype)]
    for a in shapes:
        x, y0 = wl.uniform(a.cols, dtype, 3), wl.uniform(a.rows, dtype, 4)
        for alpha, beta in ((1.0, 0.0), (2.0, 3.0), (1.0, 0.5)):
            assert np.array_equal(orc.csrmv_plain(a, alpha, x, beta, y0), _ref_mv("gemv_{t}_csr_plain", a, alpha, x, beta, y0)), a.name
            xt, yt = wl.uniform(a.rows, dtype, 3), wl.uniform(a.cols, dtype, 4)
            assert np.array_equal(orc.csrmv_trans_plain(a, alpha, xt, beta, yt),
                                  _ref_mv("gemv_{t}_csr_trans_plain", a, alpha, xt, beta, yt)), a.name
            for th in (1, 3, 8):
                assert np.array_equal(orc.csrmv_omp(a, alpha, x, beta, y0, threads=th, fast=False),
                                      _ref_mv("gemv_{t}_csr", a, alpha, x, beta, y0, threads=th)), (a.name, th)
        n = 6
        B = wl.uniform(a.cols * n, dtype, 5).reshape(a.cols, n)
        C0 = wl.uniform(a.rows * n, dtype, 4).reshape(a.rows, n)
        assert np.array_equal(orc.csrmm_plain(a, 1.5, B, 0.5, C0), _ref_mm("gemm_{t}_csr_row_plain", a, 1.5, B, n, 0.5, C0, n, n))
        assert np.array_equal(orc.csrmm_plain(a, 1.5, B, 0.5, C0, omp=True), _ref_mm("gemm_{t}_csr_row", a, 1.5, B, n, 0.5, C0, n, n))
        Bf, Cf = np.asfortranarray(B), np.asfortranarray(C0)
        assert np.array_equal(orc.csrmm_plain(a, 1.5, Bf, 0.5, Cf, layout="col"),
                              _ref_mm("gemm_{t}_csr_col_plain", a, 1.5, Bf, a.cols, 0.5, Cf, a.rows, n))
