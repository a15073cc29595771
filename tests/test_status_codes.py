"""Argument validation of the C API: every status code and its precedence as in
the reference (alphasparse_dcu_x_csrmv.cpp:52-97, alphasparse_dcu_x_csrmm.cpp:72-110,
alphasparse_dcu_x_csrmv_analysis.cpp:280-333, alphasparse_x_mv.c:1670-1691).
Validation precedes any HIP call, so all of this runs without a GPU: the handle
is a dummy block of memory that a correct implementation never dereferences on
these paths, device pointers are dummy non-NULL addresses."""
import ctypes
from ctypes import byref, c_double, c_float, c_int32, c_void_p

import numpy as np
import pytest

from alsparse_amd import capi

S = capi
DUMMY = ctypes.create_string_buffer(4096)
H = ctypes.cast(DUMMY, c_void_p)      # non-NULL "handle"
P = c_void_p(0x1000)                  # non-NULL "device pointer"
NULL = c_void_p(None)


@pytest.fixture(scope="module")
def lib():
    return capi.load()


def descr(base=0, mtype=0):
    return capi.make_descr(base=base, mtype=mtype)


@pytest.mark.parametrize("p,T", [("s", c_float), ("d", c_double)])
def test_csrmv_status_precedence(lib, p, T):
    f = getattr(lib, "alphasparse_dcu_%s_csrmv" % p)
    a, b, d = T(1), T(0), descr()

    def call(h=H, trans=0, m=4, n=4, nnz=8, alpha=byref(a), de=byref(d), val=P, rp=P, ci=P, x=P, beta=byref(b), y=P):
        return f(h, trans, m, n, nnz, alpha, de, val, rp, ci, None, x, beta, y)

    assert call(h=NULL) == S.ALPHA_SPARSE_STATUS_INVALID_HANDLE
    assert call(h=NULL, de=None) == S.ALPHA_SPARSE_STATUS_INVALID_HANDLE          # handle first
    assert call(de=None) == S.ALPHA_SPARSE_STATUS_INVALID_POINTER
    bad = descr(base=7)
    assert call(de=byref(bad)) == S.ALPHA_SPARSE_STATUS_INVALID_VALUE
    assert call(de=byref(bad), m=-1) == S.ALPHA_SPARSE_STATUS_INVALID_VALUE
    for kw in ({"m": -1}, {"n": -1}, {"nnz": -1}):
        assert call(**kw) == S.ALPHA_SPARSE_STATUS_INVALID_VALUE
    # quick return beats the pointer checks and leaves y alone
    for kw in ({"m": 0}, {"n": 0}, {"nnz": 0}):
        assert call(alpha=None, val=NULL, y=NULL, **kw) == S.ALPHA_SPARSE_STATUS_SUCCESS
    assert call(alpha=None) == S.ALPHA_SPARSE_STATUS_INVALID_POINTER
    assert call(beta=None) == S.ALPHA_SPARSE_STATUS_INVALID_POINTER
    for kw in ({"val": NULL}, {"rp": NULL}, {"ci": NULL}, {"x": NULL}, {"y": NULL}):
        assert call(**kw) == S.ALPHA_SPARSE_STATUS_INVALID_POINTER
    sym = descr(mtype=S.ALPHA_SPARSE_MATRIX_TYPE_SYMMETRIC)
    assert call(de=byref(sym)) == S.ALPHA_SPARSE_STATUS_NOT_SUPPORTED
    assert call(de=byref(sym), val=NULL) == S.ALPHA_SPARSE_STATUS_INVALID_POINTER  # pointers before type
    # the transposed product is supported (and needs a GPU); the conjugate of a real matrix is not
    assert call(trans=S.ALPHA_SPARSE_OPERATION_CONJUGATE_TRANSPOSE) == S.ALPHA_SPARSE_STATUS_NOT_SUPPORTED


@pytest.mark.parametrize("p", ["s", "d"])
def test_csrmv_analysis_status_precedence(lib, p):
    f = getattr(lib, "alphasparse_dcu_%s_csrmv_analysis" % p)
    d = descr()
    info = (capi._alphasparse_dcu_mat_info * 1)()

    def call(h=H, m=4, n=4, nnz=8, de=byref(d), val=P, rp=P, ci=P, inf=info):
        return f(h, 0, m, n, nnz, de, val, rp, ci, inf)

    assert call(h=NULL) == S.ALPHA_SPARSE_STATUS_INVALID_HANDLE
    assert call(de=None) == S.ALPHA_SPARSE_STATUS_INVALID_POINTER
    assert call(inf=None) == S.ALPHA_SPARSE_STATUS_INVALID_POINTER
    bad = descr(base=3)
    assert call(de=byref(bad)) == S.ALPHA_SPARSE_STATUS_INVALID_VALUE
    sym = descr(mtype=1)
    assert call(de=byref(sym)) == S.ALPHA_SPARSE_STATUS_NOT_SUPPORTED
    assert call(de=byref(sym), m=-1) == S.ALPHA_SPARSE_STATUS_NOT_SUPPORTED       # type before sizes here
    assert call(m=-1) == S.ALPHA_SPARSE_STATUS_INVALID_VALUE
    assert call(nnz=0, rp=NULL) == S.ALPHA_SPARSE_STATUS_SUCCESS
    for kw in ({"val": NULL}, {"rp": NULL}, {"ci": NULL}):
        assert call(**kw) == S.ALPHA_SPARSE_STATUS_INVALID_POINTER
    assert lib.alphasparse_dcu_csrmv_clear(NULL, info) == S.ALPHA_SPARSE_STATUS_INVALID_HANDLE
    assert lib.alphasparse_dcu_csrmv_clear(H, None) == S.ALPHA_SPARSE_STATUS_INVALID_POINTER
    assert lib.alphasparse_dcu_csrmv_clear(H, info) == S.ALPHA_SPARSE_STATUS_SUCCESS  # nothing recorded: no-op


@pytest.mark.parametrize("p,T", [("s", c_float), ("d", c_double)])
def test_csrmm_status_precedence(lib, p, T):
    f = getattr(lib, "alphasparse_dcu_%s_csrmm" % p)
    a, b, d = T(1), T(0), descr()

    def call(h=H, ta=0, tb=0, layout=0, m=4, n=4, k=4, nnz=8, alpha=byref(a), de=byref(d), val=P, rp=P, ci=P,
             B=P, ldb=4, beta=byref(b), C=P, ldc=4):
        return f(h, ta, tb, layout, m, n, k, nnz, alpha, de, val, rp, ci, B, ldb, beta, C, ldc)

    assert call(h=NULL) == S.ALPHA_SPARSE_STATUS_INVALID_HANDLE
    assert call(de=None) == S.ALPHA_SPARSE_STATUS_INVALID_POINTER
    bad = descr(base=2)
    assert call(de=byref(bad)) == S.ALPHA_SPARSE_STATUS_INVALID_VALUE
    for kw in ({"m": -1}, {"n": -1}, {"k": 0}, {"k": -1}, {"nnz": -1}, {"ldb": -1}, {"ldc": -1}):
        assert call(**kw) == S.ALPHA_SPARSE_STATUS_INVALID_VALUE
    for kw in ({"m": 0}, {"n": 0}, {"nnz": 0}, {"ldb": 0}, {"ldc": 0}):
        assert call(alpha=None, B=NULL, **kw) == S.ALPHA_SPARSE_STATUS_SUCCESS
    assert call(alpha=None) == S.ALPHA_SPARSE_STATUS_INVALID_POINTER
    assert call(beta=None) == S.ALPHA_SPARSE_STATUS_INVALID_POINTER
    for kw in ({"val": NULL}, {"rp": NULL}, {"ci": NULL}, {"B": NULL}, {"C": NULL}):
        assert call(**kw) == S.ALPHA_SPARSE_STATUS_INVALID_POINTER
    sym = descr(mtype=1)
    for layout in (0, 1):
        assert call(layout=layout, de=byref(sym)) == S.ALPHA_SPARSE_STATUS_NOT_SUPPORTED
        assert call(layout=layout, ta=1) == S.ALPHA_SPARSE_STATUS_NOT_SUPPORTED
        assert call(layout=layout, tb=2) == S.ALPHA_SPARSE_STATUS_NOT_SUPPORTED
    assert call(layout=0, tb=1) == S.ALPHA_SPARSE_STATUS_NOT_SUPPORTED   # row-major with op(B) = B^T


@pytest.mark.parametrize("p,T", [("s", c_float), ("d", c_double)])
def test_coomv_and_ellmv_status_precedence(lib, p, T):
    """alphasparse_dcu_x_coomv.cpp:50-95 and alphasparse_dcu_x_ellmv.cpp:48-93."""
    a, b, d = T(1), T(0), descr()
    coomv, ellmv = getattr(lib, "alphasparse_dcu_%s_coomv" % p), getattr(lib, "alphasparse_dcu_%s_ellmv" % p)

    def coo(h=H, trans=0, m=4, n=4, nnz=8, alpha=byref(a), de=byref(d), val=P, ri=P, ci=P, x=P, beta=byref(b), y=P):
        return coomv(h, trans, m, n, nnz, alpha, de, val, ri, ci, x, beta, y)

    def ell(h=H, trans=0, m=4, n=4, alpha=byref(a), de=byref(d), val=P, ci=P, width=2, x=P, beta=byref(b), y=P):
        return ellmv(h, trans, m, n, alpha, de, val, ci, width, x, beta, y)

    bad, sym = descr(base=7), descr(mtype=S.ALPHA_SPARSE_MATRIX_TYPE_SYMMETRIC)
    for call, sizes, zero, ptrs in ((coo, ("m", "n", "nnz"), ("m", "n", "nnz"), ("val", "ri", "ci", "x", "y")),
                                    (ell, ("m", "n"), ("m", "n", "width"), ("val", "ci", "x", "y"))):
        assert call(h=NULL, de=None) == S.ALPHA_SPARSE_STATUS_INVALID_HANDLE
        assert call(de=None) == S.ALPHA_SPARSE_STATUS_INVALID_POINTER
        assert call(de=byref(bad), m=-1) == S.ALPHA_SPARSE_STATUS_INVALID_VALUE
        for k in sizes:
            assert call(**{k: -1}) == S.ALPHA_SPARSE_STATUS_INVALID_VALUE
        for k in zero:  # quick return beats the pointer checks
            assert call(alpha=None, val=NULL, y=NULL, **{k: 0}) == S.ALPHA_SPARSE_STATUS_SUCCESS
        assert call(alpha=None) == S.ALPHA_SPARSE_STATUS_INVALID_POINTER
        assert call(beta=None) == S.ALPHA_SPARSE_STATUS_INVALID_POINTER
        for k in ptrs:
            assert call(**{k: NULL}) == S.ALPHA_SPARSE_STATUS_INVALID_POINTER
        assert call(de=byref(sym)) == S.ALPHA_SPARSE_STATUS_NOT_SUPPORTED
        assert call(de=byref(sym), val=NULL) == S.ALPHA_SPARSE_STATUS_INVALID_POINTER
        assert call(trans=S.ALPHA_SPARSE_OPERATION_TRANSPOSE) == S.ALPHA_SPARSE_STATUS_NOT_SUPPORTED
    assert ell(width=-3) == S.ALPHA_SPARSE_STATUS_INVALID_VALUE


def test_generic_spmv_status_codes(lib):
    """src/core/op_dcu/generic/alphasparse_dcu_spmv.cpp:30-76: check order, size query."""
    from ctypes import c_size_t
    SM, DV = capi.alphasparse_dcu_spmat_descr, capi.alphasparse_dcu_dnvec_descr
    d = descr()
    a, b = c_float(1), c_float(0)

    def mat(**kw):
        m = SM(True, True, 4, 4, 8, P, P, None, P, S.ALPHA_SPARSE_DCU_INDEXTYPE_I32, S.ALPHA_SPARSE_DCU_INDEXTYPE_I32,
               S.ALPHA_SPARSE_DATATYPE_FLOAT, 0, S.ALPHA_SPARSE_FORMAT_CSR, ctypes.pointer(d), None)
        for k, v in kw.items():
            setattr(m, k, v)
        return m

    x, y = DV(True, 4, P, S.ALPHA_SPARSE_DATATYPE_FLOAT), DV(True, 4, P, S.ALPHA_SPARSE_DATATYPE_FLOAT)
    size = c_size_t(0)
    buf = P

    def call(h=H, m=None, xx=x, yy=y, al=byref(a), be=byref(b), ct=S.ALPHA_SPARSE_DATATYPE_FLOAT, alg=0, bs=byref(size), tb=None):
        m = mat() if m is None else m
        return lib.alphasparse_dcu_spmv(h, 0, al, byref(m) if m is not False else None, byref(xx) if xx is not None else None, be,
                                        byref(yy) if yy is not None else None, ct, alg, bs, tb)

    assert call(h=NULL) == S.ALPHA_SPARSE_STATUS_INVALID_HANDLE
    for kw in ({"m": False}, {"xx": None}, {"yy": None}, {"al": None}, {"be": None}):
        assert call(**kw) == S.ALPHA_SPARSE_STATUS_INVALID_POINTER
    assert call(m=mat(init=False)) == S.ALPHA_SPARSE_STATUS_INVALID_VALUE
    assert call(xx=DV(False, 4, P, 0)) == S.ALPHA_SPARSE_STATUS_INVALID_VALUE
    assert call(ct=S.ALPHA_SPARSE_DATATYPE_DOUBLE) == S.ALPHA_SPARSE_STATUS_NOT_SUPPORTED       # mixed precision
    assert call(m=mat(row_type=S.ALPHA_SPARSE_DCU_INDEXTYPE_I64)) == S.ALPHA_SPARSE_STATUS_NOT_SUPPORTED
    assert call(m=mat(col_type=S.ALPHA_SPARSE_DCU_INDEXTYPE_U16)) == S.ALPHA_SPARSE_STATUS_NOT_SUPPORTED
    # size query on an already analysed matrix: no device work, 4 bytes
    assert call() == S.ALPHA_SPARSE_STATUS_SUCCESS and size.value == 4
    # complex data reaches the typed entry points' validation; unknown data types and formats other
    # than COO / CSR / ELL are refused
    cx = S.ALPHA_SPARSE_DATATYPE_FLOAT_COMPLEX
    assert call(m=mat(data_type=cx, val_data=None), xx=DV(True, 4, P, cx), yy=DV(True, 4, P, cx), ct=cx,
                tb=buf) == S.ALPHA_SPARSE_STATUS_INVALID_POINTER
    assert call(m=mat(data_type=cx, rows=0), xx=DV(True, 4, P, cx), yy=DV(True, 4, P, cx), ct=cx,
                tb=buf) == S.ALPHA_SPARSE_STATUS_SUCCESS
    assert call(m=mat(data_type=7), xx=DV(True, 4, P, 7), yy=DV(True, 4, P, 7), ct=7, tb=buf) == S.ALPHA_SPARSE_STATUS_NOT_SUPPORTED
    assert call(m=mat(format=S.ALPHA_SPARSE_FORMAT_COO_AOS), tb=buf) == S.ALPHA_SPARSE_STATUS_NOT_SUPPORTED
    assert call(m=mat(format=S.ALPHA_SPARSE_FORMAT_BSR), tb=buf) == S.ALPHA_SPARSE_STATUS_NOT_SUPPORTED
    # the typed entry points' own validation shows through
    assert call(m=mat(val_data=None), tb=buf) == S.ALPHA_SPARSE_STATUS_INVALID_POINTER
    assert call(m=mat(rows=0), tb=buf) == S.ALPHA_SPARSE_STATUS_SUCCESS
    assert call(m=mat(rows=1 << 40), tb=buf) == S.ALPHA_SPARSE_STATUS_INVALID_VALUE


def test_conversion_status_codes(lib):
    d = descr()
    w = c_int32(-5)
    assert lib.alphasparse_dcu_csr2coo(NULL, P, 8, 4, P, 0) == S.ALPHA_SPARSE_STATUS_INVALID_HANDLE
    assert lib.alphasparse_dcu_csr2coo(H, P, 8, 4, P, 5) == S.ALPHA_SPARSE_STATUS_INVALID_VALUE
    assert lib.alphasparse_dcu_csr2coo(H, P, -1, 4, P, 0) == S.ALPHA_SPARSE_STATUS_INVALID_VALUE
    assert lib.alphasparse_dcu_csr2coo(H, NULL, 0, 4, NULL, 0) == S.ALPHA_SPARSE_STATUS_SUCCESS
    assert lib.alphasparse_dcu_csr2coo(H, NULL, 8, 4, P, 0) == S.ALPHA_SPARSE_STATUS_INVALID_POINTER
    assert lib.alphasparse_dcu_csr2ell_width(NULL, 4, byref(d), P, byref(d), byref(w)) == S.ALPHA_SPARSE_STATUS_INVALID_HANDLE
    assert lib.alphasparse_dcu_csr2ell_width(H, 4, None, P, byref(d), byref(w)) == S.ALPHA_SPARSE_STATUS_INVALID_POINTER
    assert lib.alphasparse_dcu_csr2ell_width(H, -1, byref(d), P, byref(d), byref(w)) == S.ALPHA_SPARSE_STATUS_INVALID_VALUE
    assert lib.alphasparse_dcu_csr2ell_width(H, 4, byref(d), P, byref(d), None) == S.ALPHA_SPARSE_STATUS_INVALID_POINTER
    assert lib.alphasparse_dcu_csr2ell_width(H, 0, byref(d), NULL, byref(d), byref(w)) == S.ALPHA_SPARSE_STATUS_SUCCESS
    assert w.value == 0
    for name in ("alphasparse_dcu_scsr2ell", "alphasparse_dcu_dcsr2ell"):
        f = getattr(lib, name)
        assert f(NULL, 4, byref(d), P, P, P, byref(d), 2, P, P) == S.ALPHA_SPARSE_STATUS_INVALID_HANDLE
        assert f(H, 4, byref(d), P, P, P, None, 2, P, P) == S.ALPHA_SPARSE_STATUS_INVALID_POINTER
        assert f(H, 4, byref(d), P, P, P, byref(d), -2, P, P) == S.ALPHA_SPARSE_STATUS_INVALID_VALUE
        # width * m >= 2^31: the host converter aborts (convert_ell_x_coo.c:53-56), here an error status
        assert f(H, 1 << 23, byref(d), P, P, P, byref(d), 256, P, P) == S.ALPHA_SPARSE_STATUS_INVALID_VALUE
        assert f(H, 8388608, byref(d), P, P, P, byref(d), 200000, P, P) == S.ALPHA_SPARSE_STATUS_INVALID_VALUE
        assert f(H, 4, byref(d), NULL, NULL, NULL, byref(d), 0, NULL, NULL) == S.ALPHA_SPARSE_STATUS_SUCCESS
        assert f(H, 4, byref(d), NULL, P, P, byref(d), 2, P, P) == S.ALPHA_SPARSE_STATUS_INVALID_POINTER


def test_descr_and_info_lifecycle(lib):
    d = capi.alpha_dcu_matrix_descr_t()
    assert lib.alphasparse_dcu_create_mat_descr(None) == S.ALPHA_SPARSE_STATUS_INVALID_POINTER
    assert lib.alphasparse_dcu_create_mat_descr(byref(d)) == 0
    # defaults of src/util_cpp/handle.cpp:259-262
    assert (d.contents.type, d.contents.mode, d.contents.diag, d.contents.base) == (0, 0, 0, 0)
    assert lib.alphasparse_dcu_destroy_mat_descr(d) == 0
    info = capi.alphasparse_dcu_mat_info_t()
    assert lib.alphasparse_dcu_create_mat_info(None) == S.ALPHA_SPARSE_STATUS_INVALID_POINTER
    assert lib.alphasparse_dcu_create_mat_info(byref(info)) == 0
    assert not info.contents.csrmv_info and info.contents.boost_enable == 0
    assert lib.alphasparse_dcu_destroy_mat_info(info) == 0
    assert lib.alphasparse_dcu_destroy_mat_info(None) == 0
    ci = ctypes.POINTER(capi._alphasparse_dcu_csrmv_info)()
    assert lib.alphasparse_dcu_create_csrmv_info(byref(ci), True) == 0
    assert ci.contents.algo_tuning and ci.contents.algo == 0 and ci.contents.size == 0 and not ci.contents.row_blocks
    assert lib.alphasparse_dcu_destroy_csrmv_info(ci) == 0
    assert lib.alphasparse_dcu_destroy_csrmv_info(None) == 0
    # hip status mapping, src/util_cpp/handle.cpp:21-53
    m = lib.get_alphasparse_dcu_status_for_hip_status
    assert m(0) == 0 and m(2) == S.ALPHA_SPARSE_STATUS_ALLOC_FAILED and m(1) == S.ALPHA_SPARSE_STATUS_INTERNAL_ERROR
    assert m(17) == S.ALPHA_SPARSE_STATUS_INVALID_POINTER and m(101) == S.ALPHA_SPARSE_STATUS_INVALID_HANDLE
    assert m(400) == S.ALPHA_SPARSE_STATUS_INVALID_HANDLE and m(999) == S.ALPHA_SPARSE_STATUS_INTERNAL_ERROR


@pytest.mark.parametrize("p,dt,T", [("s", np.float32, c_float), ("d", np.float64, c_double)])
def test_create_export_destroy_and_host_api_validation(lib, p, dt, T):
    rp = np.array([1, 3, 3, 6], dtype=np.int32)       # one-based, an empty row
    ci = np.array([1, 4, 2, 3, 4], dtype=np.int32)
    v = np.array([1, 2, 3, 4, 5], dtype=dt)
    A = capi.alphasparse_matrix_t()
    create = getattr(lib, "alphasparse_%s_create_csr" % p)
    rs, re = np.ascontiguousarray(rp[:-1]), np.ascontiguousarray(rp[1:])
    assert create(None, 1, 3, 4, capi.ptr(rs), capi.ptr(re), capi.ptr(ci), capi.ptr(v)) == S.ALPHA_SPARSE_STATUS_INVALID_POINTER
    assert create(byref(A), 1, 0, 4, capi.ptr(rs), capi.ptr(re), capi.ptr(ci), capi.ptr(v)) == S.ALPHA_SPARSE_STATUS_INVALID_VALUE
    assert create(byref(A), 1, 3, 4, capi.ptr(rs), capi.ptr(re), capi.ptr(ci), capi.ptr(v)) == 0
    assert A.contents.format == S.ALPHA_SPARSE_FORMAT_CSR
    assert A.contents.datatype == (0 if p == "s" else 1)
    assert not A.contents.dcu_info and not A.contents.inspector          # zero-initialised, unlike the reference
    mat = ctypes.cast(A.contents.mat, ctypes.POINTER(capi.spmat_csr_s_t if p == "s" else capi.spmat_csr_d_t)).contents
    assert (mat.rows, mat.cols) == (3, 4) and not mat.d_values and not mat.d_row_ptr
    # deep copy, shifted to base zero; rows_end aliases rows_start + 1
    assert [mat.rows_start[i] for i in range(4)] == [0, 2, 2, 5]
    assert ctypes.addressof(mat.rows_end.contents) == ctypes.addressof(mat.rows_start.contents) + 4
    assert [mat.col_indx[i] for i in range(5)] == [0, 3, 1, 2, 3]
    v[0] = 99                                                              # caller keeps ownership of its arrays
    assert mat.values[0] == 1
    base, rows, cols = ctypes.c_int(-1), c_int32(), c_int32()
    prs, pre, pci, pv = c_void_p(), c_void_p(), c_void_p(), c_void_p()
    export = getattr(lib, "alphasparse_%s_export_csr" % p)
    assert export(A, byref(base), byref(rows), byref(cols), byref(prs), byref(pre), byref(pci), byref(pv)) == 0
    assert base.value == 0 and (rows.value, cols.value) == (3, 4)         # always reports base zero
    assert prs.value == ctypes.addressof(mat.rows_start.contents) and pre.value == prs.value + 4
    other = getattr(lib, "alphasparse_%s_export_csr" % ("d" if p == "s" else "s"))
    assert other(A, byref(base), byref(rows), byref(cols), byref(prs), byref(pre), byref(pci), byref(pv)) == S.ALPHA_SPARSE_STATUS_INVALID_VALUE

    # host-pointer entry points: validation order of alphasparse_x_mv.c:1670-1679 (all before any device work)
    mv = getattr(lib, "alphasparse_%s_mv" % p)
    mm = getattr(lib, "alphasparse_%s_mm" % p)
    x = np.ones(4, dtype=dt)
    y = np.ones(3, dtype=dt)
    gen = capi.alpha_matrix_descr(0, 0, 0)
    assert mv(0, T(1), None, gen, capi.ptr(x), T(0), capi.ptr(y)) == S.ALPHA_SPARSE_STATUS_NOT_INITIALIZED
    assert mv(0, T(1), A, gen, None, T(0), capi.ptr(y)) == S.ALPHA_SPARSE_STATUS_NOT_INITIALIZED
    assert mv(0, T(1), A, gen, capi.ptr(x), T(0), None) == S.ALPHA_SPARSE_STATUS_NOT_INITIALIZED
    assert mv(2, T(1), A, gen, capi.ptr(x), T(0), capi.ptr(y)) == S.ALPHA_SPARSE_STATUS_INVALID_VALUE     # real + conj
    assert mv(0, T(1), A, capi.alpha_matrix_descr(1, 0, 0), capi.ptr(x), T(0), capi.ptr(y)) == S.ALPHA_SPARSE_STATUS_NOT_SUPPORTED
    wrong = getattr(lib, "alphasparse_%s_mv" % ("d" if p == "s" else "s"))
    WT = c_double if p == "s" else c_float
    assert wrong(0, WT(1), A, gen, capi.ptr(x), WT(0), capi.ptr(y)) == S.ALPHA_SPARSE_STATUS_INVALID_VALUE
    assert mm(0, T(1), None, gen, 0, capi.ptr(x), 1, 1, T(0), capi.ptr(y), 1) == S.ALPHA_SPARSE_STATUS_NOT_INITIALIZED
    assert mm(2, T(1), A, gen, 0, capi.ptr(x), 1, 1, T(0), capi.ptr(y), 1) == S.ALPHA_SPARSE_STATUS_INVALID_VALUE
    assert mm(0, T(1), A, gen, 0, capi.ptr(x), 0, 1, T(0), capi.ptr(y), 1) == S.ALPHA_SPARSE_STATUS_INVALID_VALUE
    # device entry with a handle that has no mirror yet: mv_dcu forwards NULL device arrays -> INVALID_POINTER
    mvd = getattr(lib, "alphasparse_%s_mv_dcu" % p)
    a_, b_, dd = T(1), T(0), descr()
    assert mvd(H, 0, byref(a_), None, byref(dd), P, byref(b_), P) == S.ALPHA_SPARSE_STATUS_NOT_INITIALIZED
    assert mvd(H, 0, byref(a_), A, byref(dd), P, byref(b_), P) == S.ALPHA_SPARSE_STATUS_INVALID_POINTER
    assert mvd(NULL, 0, byref(a_), A, byref(dd), P, byref(b_), P) == S.ALPHA_SPARSE_STATUS_INVALID_HANDLE
    h2d = getattr(lib, "host2device_%s_csr" % p)
    assert h2d(None) == S.ALPHA_SPARSE_STATUS_INVALID_POINTER
    assert getattr(lib, "host2device_%s_csr" % ("d" if p == "s" else "s"))(A) == S.ALPHA_SPARSE_STATUS_INVALID_VALUE
    assert lib.alphasparse_destroy(A) == 0
    assert lib.alphasparse_destroy(None) == 0
