"""Pins the complex-valued CPU oracle (oracle/complex_oracle.c), without any GPU:
brute force and numpy / scipy products in higher precision, closed forms, reductions to the
real oracle, conjugation identities, planted-error detection by the metric and, where it was
built, bit-for-bit agreement with the reference's own kernels compiled with -DCOMPLEX."""
from ctypes import byref, c_int32, c_void_p

import numpy as np
import pytest
import scipy.sparse as sp

from alsparse_amd import workloads as wl
from helpers_shapes import complex_vector, complexify, csr_from_lengths, real_dtype
from oracle import oracle as orc

CX = [np.complex64, np.complex128]
IDS = ["c64", "c128"]
EPS = {np.dtype(np.complex64): 2.0 ** -24, np.dtype(np.complex128): 2.0 ** -53}
SCALARS = [(1.0, 0.0), (1.25 - 0.5j, 0.5 + 0.75j), (-2j, 1.0), (0.0, 0.5 - 0.25j)]


def shapes(dtype):
    rd = real_dtype(dtype)
    return [complexify(a, dtype) for a in (
        wl.random_points(300, 260, 1500, rd), wl.laplace2d(17, 13, rd), wl.uniform_rows(400, 350, 16, rd),
        wl.powerlaw_rmat(10, 700, rd), csr_from_lengths([0, 1, 0, 70, 3, 0, 0, 129], 200, rd),
        wl.uniform_rows(120, 90, 5, rd, base=1))]


def scipy_csr(a):
    return sp.csr_matrix((a.values.astype(np.complex128), a.col_ind.astype(np.int64) - a.base,
                          a.row_ptr.astype(np.int64) - a.base), shape=(a.rows, a.cols))


def bound(a, alpha, x, beta, y0, terms):
    """gamma-style bound on |oracle - exact| per output element: every product and sum of the
    three-multiplication form loses a few ulps of (|re|+|im|)^2 <= 2|a|^2."""
    A = abs(scipy_csr(a))
    return 16 * (terms + 4) * EPS[a.dtype] * (abs(alpha) * (A @ np.abs(x)) + abs(beta) * np.abs(y0)) + 1e-300


@pytest.mark.parametrize("dtype", CX, ids=IDS)
def test_complex_spmv_against_brute_force_and_scipy(dtype):
    for a in shapes(dtype):
        x, y0 = complex_vector(a.cols, dtype, 3), complex_vector(a.rows, dtype, 4)
        dense = scipy_csr(a).toarray()
        maxlen = int(np.diff(a.row_ptr).max())
        for alpha, beta in SCALARS:
            y = orc.csrmv_plain(a, alpha, x, beta, y0)
            brute = np.array([alpha * sum(dense[r, c] * complex(x[c]) for c in np.nonzero(dense[r])[0]) + beta * complex(y0[r])
                              for r in range(a.rows)]) if a.rows <= 200 else None
            exact = alpha * (scipy_csr(a) @ x.astype(np.complex128)) + beta * y0.astype(np.complex128)
            lim = bound(a, alpha, x, beta, y0, maxlen)
            assert np.all(np.abs(y - exact) <= lim), (a.name, alpha, beta)
            if brute is not None:
                assert np.all(np.abs(y - brute) <= lim), (a.name, alpha, beta)
            err = orc.csrmv_err(a, alpha, x, beta, y0, y, exact.astype(dtype))
            assert err.full <= 64 * EPS[a.dtype] * (maxlen + 4)   # (empty rows: beta*y0 rounds differently in numpy)


@pytest.mark.parametrize("dtype", CX, ids=IDS)
def test_complex_spmv_closed_forms(dtype):
    rd = real_dtype(dtype)
    n = 50
    ident = wl.Csr(n, n, np.arange(n + 1, dtype=np.int32), np.arange(n, dtype=np.int32), np.ones(n, dtype=dtype), 0, "I")
    x, y0 = complex_vector(n, dtype, 3), complex_vector(n, dtype, 4)

    def mul(p, q):  # the four-multiplication product, every operation rounded in the real type
        p, q = np.asarray(p, dtype=dtype), np.asarray(q, dtype=dtype)
        return ((p.real * q.real - p.imag * q.imag) + 1j * (p.imag * q.real + p.real * q.imag)).astype(dtype)
    # alpha = 0 leaves beta*y0, rounded as one four-multiplication product
    for beta in (0.5 - 0.25j, 1.0, 0.0, 3j):
        assert np.array_equal(orc.csrmv_plain(ident, 0.0, x, beta, y0), mul(np.full(n, beta), y0))
    # beta = 0 on the identity returns alpha*x; the three-multiplication madde forms the real part as
    # (xr - xi) + xi, so this holds to a few ulps of |xr| + |xi| and not exactly, in the reference too
    ulps = 8 * EPS[np.dtype(dtype)] * (np.abs(x.real) + np.abs(x.imag))
    assert np.all(np.abs(orc.csrmv_plain(ident, 1.0, x, 0.0, y0) - x) <= ulps)
    assert np.all(np.abs(orc.csrmv_plain(ident, 1j, x, 0.0, y0) - x * 1j) <= ulps)
    # a diagonal of i: y = i * x (A = i*I)
    diag_i = wl.Csr(n, n, ident.row_ptr, ident.col_ind, np.full(n, 1j, dtype=dtype), 0, "iI")
    assert np.all(np.abs(orc.csrmv_plain(diag_i, 1.0, x, 0.0, y0) - x * 1j) <= ulps)
    # real data in complex storage: the complex oracle reproduces the real oracle bit for bit
    ar = wl.powerlaw_rmat(10, 500, rd)
    ac = wl.Csr(ar.rows, ar.cols, ar.row_ptr, ar.col_ind, ar.values.astype(dtype), 0, "real-in-complex")
    xr, yr = wl.uniform(ar.cols, rd, 3), wl.uniform(ar.rows, rd, 4)
    yc = orc.csrmv_plain(ac, 2.0, xr.astype(dtype), 3.0, yr.astype(dtype))
    assert np.array_equal(yc.real, orc.csrmv_plain(ar, 2.0, xr, 3.0, yr)) and not yc.imag.any()
    # A real, x purely imaginary: y = i * (A x_r), again bit for bit against the real oracle
    yi = orc.csrmv_plain(ac, 1.0, (1j * xr).astype(dtype), 0.0, np.zeros(ar.rows, dtype=dtype))
    assert np.array_equal(yi.imag, orc.csrmv_plain(ar, 1.0, xr, 0.0, np.zeros(ar.rows, dtype=rd))) and not yi.real.any()
    # the Laplacian times the all-(1+i) vector: 4 - #neighbours in both parts, exactly
    lap = wl.laplace2d(9, 7, rd)
    lc = wl.Csr(lap.rows, lap.cols, lap.row_ptr, lap.col_ind, lap.values.astype(dtype), 0, "lap")
    yl = orc.csrmv_plain(lc, 1.0, np.full(lap.cols, 1 + 1j, dtype=dtype), 0.0, np.zeros(lap.rows, dtype=dtype))
    expect = orc.csrmv_plain(lap, 1.0, np.ones(lap.cols, dtype=rd), 0.0, np.zeros(lap.rows, dtype=rd))
    assert np.array_equal(yl.real, expect) and np.array_equal(yl.imag, expect) and set(expect) <= {0.0, 1.0, 2.0}


@pytest.mark.parametrize("dtype", CX, ids=IDS)
def test_complex_transposed_and_conjugate_transposed_spmv(dtype):
    for a in shapes(dtype):
        x, y0 = complex_vector(a.rows, dtype, 5), complex_vector(a.cols, dtype, 6)
        A = scipy_csr(a)
        maxcol = int(np.bincount(a.col_ind.astype(np.int64) - a.base, minlength=a.cols).max())
        for alpha, beta in SCALARS:
            for conj in (False, True):
                y = orc.csrmv_trans_plain(a, alpha, x, beta, y0, conj=conj)
                op = A.conj().T if conj else A.T
                exact = alpha * (op @ x.astype(np.complex128)) + beta * y0.astype(np.complex128)
                at = orc.transpose(a, conj=conj)
                assert np.all(np.abs(y - exact) <= bound(at, alpha, x, beta, y0, maxcol)), (a.name, alpha, beta, conj)
                # the same operator as an explicit CSR matrix through the untransposed kernel
                y2 = orc.csrmv_plain(at, alpha, x, beta, y0)
                assert np.all(np.abs(y - y2) <= 2 * bound(at, alpha, x, beta, y0, maxcol))
        # A^H x is the transposed product with conjugated values, operation for operation
        conj_a = wl.Csr(a.rows, a.cols, a.row_ptr, a.col_ind, np.conj(a.values), a.base, "conj")
        assert np.array_equal(orc.csrmv_trans_plain(a, 1.25 - 0.5j, x, 0.5j, y0, conj=True),
                              orc.csrmv_trans_plain(conj_a, 1.25 - 0.5j, x, 0.5j, y0, conj=False))
    # a matrix with a non-zero imaginary part must tell A^T from A^H
    a = shapes(dtype)[0]
    x, y0 = complex_vector(a.rows, dtype, 5), complex_vector(a.cols, dtype, 6)
    assert not np.allclose(orc.csrmv_trans_plain(a, 1.0, x, 0.0, y0), orc.csrmv_trans_plain(a, 1.0, x, 0.0, y0, conj=True))


@pytest.mark.parametrize("dtype", CX, ids=IDS)
def test_complex_spmm_coomv_ellmv_csr2ell(dtype):
    rng = np.random.default_rng(3)
    for a in shapes(dtype):
        A = scipy_csr(a)
        maxlen = int(np.diff(a.row_ptr).max())
        n = 5
        B = complex_vector(a.cols * n, dtype, 7).reshape(a.cols, n)
        C0 = complex_vector(a.rows * n, dtype, 8).reshape(a.rows, n)
        for alpha, beta in SCALARS[:3]:
            exact = alpha * (A @ B.astype(np.complex128)) + beta * C0.astype(np.complex128)
            lim = 16 * (maxlen + 4) * EPS[a.dtype] * (abs(alpha) * (abs(A) @ np.abs(B)) + abs(beta) * np.abs(C0)) + 1e-300
            Cr = orc.csrmm_plain(a, alpha, B, beta, C0)
            Cc = orc.csrmm_plain(a, alpha, np.asfortranarray(B), beta, np.asfortranarray(C0), layout="col")
            assert np.all(np.abs(Cr - exact) <= lim) and np.all(np.abs(Cc - exact) <= lim), (a.name, alpha, beta)
            assert orc.csrmm_err(a, alpha, B, beta, C0, Cr, exact.astype(dtype)).full <= 64 * EPS[a.dtype] * (maxlen + 4)
            # one dense column of the row-major product is the SpMV, operation for operation
            y = orc.csrmm_plain(a, alpha, B[:, :1].copy(), beta, C0[:, :1].copy())[:, 0]
            x, y0 = B[:, 0].copy(), C0[:, 0].copy()
            assert np.all(np.abs(y - orc.csrmv_plain(a, alpha, x, beta, y0)) <= 2 * bound(a, alpha, x, beta, y0, maxlen))
        x, y0 = complex_vector(a.cols, dtype, 3), complex_vector(a.rows, dtype, 4)
        rows = orc.csr2coo(a) - a.base
        exact = (1.25 - 0.5j) * (A @ x.astype(np.complex128)) + 0.5j * y0.astype(np.complex128)
        lim = bound(a, 1.25 - 0.5j, x, 0.5j, y0, maxlen)
        assert np.all(np.abs(orc.coomv_plain(a, rows, 1.25 - 0.5j, x, 0.5j, y0) - exact) <= lim)
        perm = rng.permutation(a.nnz)   # any storage order gives the same sums up to rounding
        shuffled = wl.Csr(a.rows, a.cols, a.row_ptr, a.col_ind[perm].copy(), a.values[perm].copy(), a.base, "shuffled")
        assert np.all(np.abs(orc.coomv_plain(shuffled, rows[perm].copy(), 1.25 - 0.5j, x, 0.5j, y0) - exact) <= lim)
        # csr2ell: values moved bit for bit, padding (0, index ell_base); ELL SpMV equals the CSR one
        w = orc.csr2ell_width(a)
        ev, ec = orc.csr2ell(a, w)
        assert ev.dtype == a.dtype
        lens = np.diff(a.row_ptr)
        for r in range(0, a.rows, max(1, a.rows // 25)):
            b = int(a.row_ptr[r] - a.base)
            for s in range(w):
                if s < lens[r]:
                    assert ev[s * a.rows + r] == a.values[b + s] and ec[s * a.rows + r] == a.col_ind[b + s] - a.base
                else:
                    assert ev[s * a.rows + r] == 0 and ec[s * a.rows + r] == 0
        assert np.all(np.abs(orc.ellmv(a.rows, a.cols, ev, ec, w, 1.25 - 0.5j, x, 0.5j, y0) - exact) <= lim)


def test_complex_error_metric_detects_planted_errors():
    a = shapes(np.complex64)[2]
    x, y0 = complex_vector(a.cols, np.complex64, 3), complex_vector(a.rows, np.complex64, 4)
    ref = orc.csrmv_plain(a, 1.5, x, 0.5, y0)
    assert orc.csrmv_err(a, 1.5, x, 0.5, y0, ref, ref).full == 0
    wrong = ref.copy()
    wrong[7] += 1e-2j          # an error in the imaginary part only
    e = orc.csrmv_err(a, 1.5, x, 0.5, y0, wrong, ref)
    assert e.full > 1e-4 and e.row == 7
    # a conjugated (wrong-sign) result is far outside the tolerance
    assert orc.csrmv_err(a, 1.5, x, 0.5, y0, np.conj(ref), ref).full > 1e-2
    empty = complexify(csr_from_lengths([0, 2, 0], 5, np.float32), np.complex64)
    xe, ye = complex_vector(5, np.complex64, 3), complex_vector(3, np.complex64, 4)
    r = orc.csrmv_plain(empty, 1.0, xe, 0.5j, ye)
    bad = r.copy()
    bad[2] += 1e-7j
    assert orc.csrmv_err(empty, 1.0, xe, 0.5j, ye, bad, r).zero_den_mismatch == 1
    assert orc.csrmv_err(empty, 1.0, xe, 0.5j, ye, r, r).zero_den_mismatch == 0


# ---- the reference's own kernels, compiled from its sources with -DCOMPLEX -------------------
def _have_ref():
    if not orc.ref_available():
        return False
    return hasattr(orc.ref_lib(), "gemv_c_csr_conj_plain")


needs_ref = pytest.mark.skipif(not _have_ref(), reason="oracle/_ref not built with the complex kernels")


@needs_ref
@pytest.mark.parametrize("dtype", CX, ids=IDS)
def test_complex_oracle_is_bit_identical_to_reference_kernels(dtype):
    T, t = orc._ct(dtype), orc._pre(dtype)
    L = orc.ref_lib()

    def mv(name, a, alpha, x, beta, y0):
        fn = getattr(L, name % t)
        fn.restype, fn.argtypes = c_int32, [T, c_void_p, c_void_p, T, c_void_p]
        mat = orc.RefCsr(a)
        y = y0.copy()
        assert fn(T(alpha), byref(mat.s), x.ctypes.data_as(c_void_p), T(beta), y.ctypes.data_as(c_void_p)) == 0
        return y

    def mm(name, a, alpha, B, ldb, beta, C0, ldc, n):
        fn = getattr(L, name % t)
        fn.restype, fn.argtypes = c_int32, [T, c_void_p, c_void_p, c_int32, c_int32, T, c_void_p, c_int32]
        mat = orc.RefCsr(a)
        C = C0.copy(order="K")
        assert fn(T(alpha), byref(mat.s), B.ctypes.data_as(c_void_p), n, ldb, T(beta), C.ctypes.data_as(c_void_p), ldc) == 0
        return C

    for a in shapes(dtype):
        x, y0 = complex_vector(a.cols, dtype, 3), complex_vector(a.rows, dtype, 4)
        xt, yt = complex_vector(a.rows, dtype, 5), complex_vector(a.cols, dtype, 6)
        for alpha, beta in SCALARS:
            assert np.array_equal(orc.csrmv_plain(a, alpha, x, beta, y0), mv("gemv_%s_csr_plain", a, alpha, x, beta, y0)), a.name
            assert np.array_equal(orc.csrmv_trans_plain(a, alpha, xt, beta, yt),
                                  mv("gemv_%s_csr_trans_plain", a, alpha, xt, beta, yt)), a.name
            assert np.array_equal(orc.csrmv_trans_plain(a, alpha, xt, beta, yt, conj=True),
                                  mv("gemv_%s_csr_conj_plain", a, alpha, xt, beta, yt)), a.name
        n = 6
        B = complex_vector(a.cols * n, dtype, 7).reshape(a.cols, n)
        C0 = complex_vector(a.rows * n, dtype, 8).reshape(a.rows, n)
        assert np.array_equal(orc.csrmm_plain(a, 1.5 - 0.5j, B, 0.5j, C0),
                              mm("gemm_%s_csr_row_plain", a, 1.5 - 0.5j, B, n, 0.5j, C0, n, n))
        Bf, Cf = np.asfortranarray(B), np.asfortranarray(C0)
        assert np.array_equal(orc.csrmm_plain(a, 1.5 - 0.5j, Bf, 0.5j, Cf, layout="col"),
                              mm("gemm_%s_csr_col_plain", a, 1.5 - 0.5j, Bf, a.cols, 0.5j, Cf, a.rows, n))
        # COO kernel: spmat_coo_?_t, include/alphasparse/spmat.h:120-158 of the reference
        from test_oracle import _RefCoo
        rows, cols, vals = orc.csr2coo(a) - a.base, (a.col_ind - a.base).astype(np.int32), a.values.copy()
        coo = _RefCoo(vals.ctypes.data, rows.ctypes.data, cols.ctypes.data, a.rows, a.cols, a.nnz, False, None, None, None)
        fn = getattr(L, "gemv_%s_coo_plain" % t)
        fn.restype, fn.argtypes = c_int32, [T, c_void_p, c_void_p, T, c_void_p]
        y = y0.copy()
        assert fn(T(1.5 - 0.5j), byref(coo), x.ctypes.data_as(c_void_p), T(0.5j), y.ctypes.data_as(c_void_p)) == 0
        assert np.array_equal(orc.coomv_plain(a, rows, 1.5 - 0.5j, x, 0.5j, y0), y), a.name
