"""alphasparse_?_mv / _mm and their _plain variants on host arrays, all four value types, every
operation the reference's tables hold (A, A^T, and A^H for complex types), both dense layouts:
results against the CPU oracle on the same inputs, and the two variants against each other, which is
the comparison the reference's own CPU test programs make (test/arm/mv_s_csr_arm_test.c)."""
from ctypes import byref

import numpy as np
import pytest

from alsparse_amd import capi, workloads as wl
from oracle import oracle as orc
from helpers import announce
from helpers_shapes import complex_vector, complexify, csr_from_lengths, real_dtype

pytestmark = pytest.mark.gpu
DT = [np.float32, np.float64, np.complex64, np.complex128]
IDS = ["f32", "f64", "c64", "c128"]
TOL = {np.dtype(np.float32): 1e-4, np.dtype(np.float64): 1e-12, np.dtype(np.complex64): 1e-4,
       np.dtype(np.complex128): 1e-12}
N, T_, H_ = 0, 1, 2


def vec(n, dtype, stream):
    return complex_vector(n, dtype, stream) if orc.is_complex(dtype) else wl.uniform(n, dtype, stream)


def matrices(dtype):
    rd = real_dtype(dtype)
    out = [wl.powerlaw_rmat(12, 900, rd), wl.uniform_rows(5000, 3000, 9, rd), csr_from_lengths([0, 3, 0, 700, 1, 0], 800, rd),
           wl.uniform_rows(700, 900, 5, rd, base=1)]
    return [complexify(a, dtype) for a in out] if orc.is_complex(dtype) else out


def make_handle(lib, a):
    h = capi.alphasparse_matrix_t()
    rp = np.ascontiguousarray(a.row_ptr)
    st = getattr(lib, "alphasparse_%s_create_csr" % capi.prefix(a.dtype))(
        byref(h), a.base, a.rows, a.cols, capi.ptr(rp[:-1].copy()), capi.ptr(rp[1:].copy()), capi.ptr(a.col_ind),
        capi.ptr(a.values))
    assert st == 0, st
    return h


def ops_of(dtype):
    return (N, T_, H_) if orc.is_complex(dtype) else (N, T_)


def scalars(dtype):
    return (1.25 - 0.5j, 0.5 + 0.75j) if orc.is_complex(dtype) else (1.25, 0.5)


@pytest.mark.parametrize("dtype", DT, ids=IDS)
def test_host_mv_and_mv_plain(gpu, dtype):
    lib = capi.load()
    p, T = capi.prefix(dtype), capi.scalar_type(dtype)
    alpha, beta = scalars(dtype)
    descr = capi.alpha_matrix_descr(0, 0, 0)
    for a in matrices(dtype):
        h = make_handle(lib, a)
        try:
            for op in ops_of(dtype):
                xlen, ylen = (a.cols, a.rows) if op == N else (a.rows, a.cols)
                x, y0 = vec(xlen, dtype, 3), vec(ylen, dtype, 4)
                if op == N:
                    metric, ref = a, orc.csrmv_plain(a, alpha, x, beta, y0)
                else:
                    metric, ref = orc.transpose(a, conj=op == H_), orc.csrmv_trans_plain(a, alpha, x, beta, y0, conj=op == H_)
                got = {}
                for name in ("mv", "mv_plain"):
                    y = y0.copy()
                    announce("host", name, np.dtype(dtype).name, a.name, op)
                    assert getattr(lib, "alphasparse_%s_%s" % (p, name))(op, T(alpha), h, descr, capi.ptr(x), T(beta), capi.ptr(y)) == 0
                    err = orc.csrmv_err(metric, alpha, x, beta, y0, y, ref)
                    assert err.zero_den_mismatch == 0 and err.full <= TOL[np.dtype(dtype)], (name, a.name, op, err)
                    got[name] = y
                # the reference's own drivers compare the two entry points with each other
                err = orc.csrmv_err(metric, alpha, x, beta, y0, got["mv"], got["mv_plain"])
                assert err.full <= TOL[np.dtype(dtype)]
                if op == N and not orc.is_complex(dtype):
                    # one lane, storage order, fused multiply-adds: only the contraction separates the
                    # plain GPU kernel from the CPU oracle, a few ulps of the row's magnitude
                    assert orc.csrmv_err(a, alpha, x, beta, y0, got["mv_plain"], ref).full <= 64 * np.finfo(dtype).eps
        finally:
            assert lib.alphasparse_destroy(h) == 0


@pytest.mark.parametrize("layout", ["row", "col"])
@pytest.mark.parametrize("dtype", DT, ids=IDS)
def test_host_mm_and_mm_plain_every_operation(gpu, dtype, layout):
    lib = capi.load()
    p, T = capi.prefix(dtype), capi.scalar_type(dtype)
    alpha, beta = scalars(dtype)
    descr = capi.alpha_matrix_descr(0, 0, 0)
    lay = capi.ALPHA_SPARSE_LAYOUT_ROW_MAJOR if layout == "row" else capi.ALPHA_SPARSE_LAYOUT_COLUMN_MAJOR
    for a in matrices(dtype)[:3]:
        h = make_handle(lib, a)
        try:
            for op in ops_of(dtype):
                eff = a if op == N else orc.transpose(a, conj=op == H_)   # op(A) as an explicit matrix
                for n in (1, 7, 40):
                    B = vec(eff.cols * n, dtype, 5).reshape(eff.cols, n)
                    C0 = vec(eff.rows * n, dtype, 6).reshape(eff.rows, n)
                    ref = orc.csrmm_plain(eff, alpha, B, beta, C0)
                    for name in ("mm", "mm_plain"):
                        if layout == "row":
                            X, Y = np.ascontiguousarray(B), C0.copy()
                            ldx, ldy = n, n
                        else:
                            X, Y = np.asfortranarray(B), np.asfortranarray(C0).copy(order="F")
                            ldx, ldy = eff.cols, eff.rows
                        announce("host", name, np.dtype(dtype).name, a.name, op, layout, n)
                        st = getattr(lib, "alphasparse_%s_%s" % (p, name))(op, T(alpha), h, descr, lay, capi.ptr(X), n, ldx, T(beta),
                                                                          capi.ptr(Y), ldy)
                        assert st == 0, (name, st)
                        err = orc.csrmm_err(eff, alpha, B, beta, C0, np.asarray(Y), ref)
                        assert err.zero_den_mismatch == 0 and err.full <= TOL[np.dtype(dtype)], (name, a.name, op, n, err)
        finally:
            assert lib.alphasparse_destroy(h) == 0


def test_plain_entry_points_share_the_validation(gpu):
    lib = capi.load()
    a = wl.uniform_rows(50, 40, 3, np.float32)
    h = make_handle(lib, a)
    descr = capi.alpha_matrix_descr(0, 0, 0)
    x, y = wl.uniform(50, np.float32, 3), wl.uniform(50, np.float32, 4)
    try:
        S = capi
        for name in ("alphasparse_s_mv", "alphasparse_s_mv_plain"):
            f = getattr(lib, name)
            assert f(0, 1.0, h, descr, None, 0.0, capi.ptr(y)) == S.ALPHA_SPARSE_STATUS_NOT_INITIALIZED
            assert f(2, 1.0, h, descr, capi.ptr(x), 0.0, capi.ptr(y)) == S.ALPHA_SPARSE_STATUS_INVALID_VALUE   # real + conjugate
            assert f(0, 1.0, h, capi.alpha_matrix_descr(1, 0, 0), capi.ptr(x), 0.0, capi.ptr(y)) == S.ALPHA_SPARSE_STATUS_NOT_SUPPORTED
        assert lib.alphasparse_d_mv_plain(0, 1.0, h, descr, capi.ptr(x), 0.0, capi.ptr(y)) == S.ALPHA_SPARSE_STATUS_INVALID_VALUE
        for name in ("alphasparse_s_mm", "alphasparse_s_mm_plain"):
            f = getattr(lib, name)
            assert f(0, 1.0, h, descr, 5, capi.ptr(x), 1, 1, 0.0, capi.ptr(y), 1) == S.ALPHA_SPARSE_STATUS_INVALID_VALUE      # layout
            assert f(0, 1.0, h, descr, 0, capi.ptr(x), 0, 1, 0.0, capi.ptr(y), 1) == S.ALPHA_SPARSE_STATUS_INVALID_VALUE      # columns
            assert f(0, 1.0, h, descr, 0, capi.ptr(x), 2, 1, 0.0, capi.ptr(y), 2) == S.ALPHA_SPARSE_STATUS_INVALID_VALUE      # ldx < columns
    finally:
        assert lib.alphasparse_destroy(h) == 0
