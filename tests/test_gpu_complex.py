"""Complex element types (ALPHA_Complex8 / ALPHA_Complex16) on the GPU through the C API:
csrmv for A, A^T and A^H with and without analysis, every kernel family a complex plan can run,
csrmm in the three layouts, coomv / ellmv / csr2ell, matrix handles (CSR, COO, ELL), the
host-pointer entry points and the descriptor API, each against the complex CPU oracle.
Tolerance: per output element |dy| <= 1e-4 (complex64) / 1e-12 (complex128) of
|alpha| sum|a||x| (+ |beta y0|), moduli of complex numbers; outputs without a non-zero product
must equal the oracle's beta*y0 exactly; csr2ell bit for bit."""
from ctypes import byref, c_int, c_int32, c_size_t, c_void_p

import numpy as np
import pytest

from alsparse_amd import capi, hiprt, workloads as wl
from oracle import oracle as orc
from helpers import ALGOS, DeviceCsr, announce, check_beta_rows
from helpers_shapes import complex_vector, complexify, csr_from_lengths, real_dtype
from test_gpu_formats_mv import dev, run_coomv, run_ellmv

pytestmark = pytest.mark.gpu
CX = [np.complex64, np.complex128]
IDS = ["c64", "c128"]
TOL = {np.dtype(np.complex64): 1e-4, np.dtype(np.complex128): 1e-12}
N, T_, H_ = (capi.ALPHA_SPARSE_OPERATION_NON_TRANSPOSE, capi.ALPHA_SPARSE_OPERATION_TRANSPOSE,
             capi.ALPHA_SPARSE_OPERATION_CONJUGATE_TRANSPOSE)
OPS = {"N": N, "T": T_, "H": H_}
SCALARS = [(1.0, 0.0), (1.25 - 0.5j, 0.5 + 0.75j), (-2j, 1.0)]

SHAPES = {
    "uniform16": lambda rd: wl.uniform_rows(40000, 30000, 16, rd),
    "powerlaw": lambda rd: wl.powerlaw_rmat(14, 20000, rd),
    "laplace": lambda rd: wl.laplace2d(211, 177, rd),
    "long_and_empty": lambda rd: csr_from_lengths([0] * 300 + [9000] + [0] * 200 + [2, 4097, 4095, 0, 0, 1, 63, 64, 65],
                                                  20000, rd),
    "base_one": lambda rd: wl.uniform_rows(3000, 2500, 7, rd, base=1),
    # 2^20 entries or more and few columns: x in LDS; without analysis the transposed operations add up in LDS
    "tall": lambda rd: wl.uniform_rows(70000, 8000, 16, rd, base=1),
    "tiny": lambda rd: csr_from_lengths([2, 0, 1], 5, rd),
    # rows of similar lengths: the staged row-block kernel with several lanes per row
    "stencil27": lambda rd: wl.stencil3d(14, 11, 9, rd),
    "regular_40_60": lambda rd: csr_from_lengths(list(40 + (np.arange(1200) * 7) % 21), 3000, rd, base=1),
}


def make(shape, dtype):
    return complexify(SHAPES[shape](real_dtype(dtype)), dtype)


def oracle_mv(a, op, alpha, x, beta, y0):
    if op == N:
        return a, orc.csrmv_plain(a, alpha, x, beta, y0)
    conj = op == H_
    return orc.transpose(a, conj=conj), orc.csrmv_trans_plain(a, alpha, x, beta, y0, conj=conj)


def check(metric_matrix, alpha, x, beta, y0, y, ref, what):
    err = orc.csrmv_err(metric_matrix, alpha, x, beta, y0, y, ref)
    tol = TOL[metric_matrix.dtype]
    assert err.zero_den_mismatch == 0, "%s: %d outputs without products differ" % (what, err.zero_den_mismatch)
    assert err.full <= tol, "%s: error %.3e at %d exceeds %g" % (what, err.full, err.row, tol)
    if beta == 0:
        assert err.strict <= tol, "%s: strict error %.3e exceeds %g" % (what, err.strict, tol)
    else:
        check_beta_rows(metric_matrix, alpha, x, beta, y0, y, ref, tol, what)


def run_csrmv(h, da, op, alpha, x, beta, y0, info=None):
    a = da.a
    lib = capi.load()
    T = capi.scalar_type(a.dtype)
    descr = capi.make_descr(base=a.base)
    dx, dy = dev(x), dev(y0)
    al, be = T(alpha), T(beta)
    st = getattr(lib, "alphasparse_dcu_%s_csrmv" % capi.prefix(a.dtype))(
        h.h, op, a.rows, a.cols, a.nnz, byref(al), byref(descr), da.val.c_ptr(), da.row_ptr.c_ptr(), da.col.c_ptr(),
        info, dx.c_ptr(), byref(be), dy.c_ptr())
    assert st == 0, "csrmv status %d" % st
    hiprt.synchronize()
    y = dy.to_numpy()
    dx.free()
    dy.free()
    return y


@pytest.mark.parametrize("op", list(OPS), ids=list(OPS))
@pytest.mark.parametrize("shape", list(SHAPES))
@pytest.mark.parametrize("dtype", CX, ids=IDS)
def test_complex_csrmv_with_and_without_analysis(gpu, dtype, shape, op):
    lib = capi.load()
    a = make(shape, dtype)
    opv = OPS[op]
    xlen, ylen = (a.cols, a.rows) if opv == N else (a.rows, a.cols)
    x, y0 = complex_vector(xlen, dtype, 3), complex_vector(ylen, dtype, 4)
    da = DeviceCsr(a)
    info = capi.alphasparse_dcu_mat_info_t()
    assert lib.alphasparse_dcu_create_mat_info(byref(info)) == 0
    descr = capi.make_descr(base=a.base)
    try:
        for alpha, beta in SCALARS:
            m, ref = oracle_mv(a, opv, alpha, x, beta, y0)
            announce("complex csrmv, no analysis", np.dtype(dtype).name, shape, op, alpha, beta)
            check(m, alpha, x, beta, y0, run_csrmv(gpu, da, opv, alpha, x, beta, y0), ref, "%s %s lazy" % (shape, op))
        announce("complex csrmv analysis", np.dtype(dtype).name, shape, op)
        assert getattr(lib, "alphasparse_dcu_%s_csrmv_analysis" % capi.prefix(dtype))(
            gpu.h, opv, a.rows, a.cols, a.nnz, byref(descr), da.val.c_ptr(), da.row_ptr.c_ptr(), da.col.c_ptr(), info) == 0
        st = lib.asamd_analysis_stats(info).contents
        assert st.algo != capi.ASAMD_SPMV_ROWCONST
        assert st.transpose_built == {N: 0, T_: 1, H_: 2}[opv]
        first = None
        for alpha, beta in SCALARS:
            m, ref = oracle_mv(a, opv, alpha, x, beta, y0)
            announce("complex csrmv, analysed", np.dtype(dtype).name, shape, op, alpha, beta)
            y = run_csrmv(gpu, da, opv, alpha, x, beta, y0, info)
            check(m, alpha, x, beta, y0, y, ref, "%s %s analysed" % (shape, op))
            first = y if first is None else first
        # analysed multiplies use no atomics: bit-reproducible
        assert np.array_equal(first, run_csrmv(gpu, da, opv, *SCALARS[0][:1], x, SCALARS[0][1], y0, info))
    finally:
        lib.alphasparse_dcu_destroy_mat_info(info)
        da.free()


@pytest.mark.parametrize("algo", ["vector", "merge", "scalar", "stream", "ell", "rowconst", "tiled", "hot", "binned", "xlds"])
@pytest.mark.parametrize("dtype", CX, ids=IDS)
def test_complex_kernel_families(gpu, dtype, algo):
    """The thin kernel ABI with a forced family; the constant-row-length family (128-bit quads of
    reals) is refused for complex plans."""
    lib = capi.load()
    T, p = capi.scalar_type(dtype), capi.prefix(dtype)
    ran = 0
    for shape in ("uniform16", "powerlaw", "laplace", "long_and_empty", "base_one", "tiny", "stencil27", "regular_40_60"):
        a = make(shape, dtype)
        x, y0 = complex_vector(a.cols, dtype, 3), complex_vector(a.rows, dtype, 4)
        da = DeviceCsr(a)
        plan = c_void_p()
        announce("complex plan", np.dtype(dtype).name, shape, algo)
        assert lib.asamd_csr_plan_create_dtype(None, a.rows, a.cols, a.nnz, da.row_ptr.c_ptr(), da.col.c_ptr(),
                                               da.val.c_ptr(), a.base, capi.dtype_tag(dtype), 2, byref(plan)) == 0
        try:
            if lib.asamd_csr_plan_set_algo(plan, ALGOS[algo]) != 0:
                assert algo in ("rowconst", "stream", "ell", "hot", "xlds"), (algo, shape)
                continue
            assert algo != "rowconst"
            ws = capi.Workspace(lib, plan)
            for alpha, beta in SCALARS:
                dx, dy = dev(x), dev(y0)
                announce("complex family", np.dtype(dtype).name, shape, algo, alpha, beta)
                assert capi.plan_csrmv(lib, None, plan, 0, T(alpha), da.val.c_ptr(), da.row_ptr.c_ptr(), da.col.c_ptr(),
                                       dx.c_ptr(), T(beta), dy.c_ptr(), ws) == 0
                hiprt.synchronize()
                check(a, alpha, x, beta, y0, dy.to_numpy(), orc.csrmv_plain(a, alpha, x, beta, y0), "%s %s" % (shape, algo))
                dx.free()
                dy.free()
            ran += 1
        finally:
            lib.asamd_csr_plan_destroy(plan)
            da.free()
    # refused for complex plans: the constant-row-length family; for 16-byte values: the hot-column family
    refused = algo == "rowconst" or (algo == "hot" and np.dtype(dtype).itemsize == 16)
    assert ran >= (0 if refused else 2), "family %s ran on %d shapes" % (algo, ran)


@pytest.mark.parametrize("layout", ["row", "col", "col_transB"])
@pytest.mark.parametrize("dtype", CX, ids=IDS)
def test_complex_csrmm(gpu, dtype, layout):
    lib = capi.load()
    T, p = capi.scalar_type(dtype), capi.prefix(dtype)
    for shape in ("uniform16", "powerlaw", "base_one", "tiny"):
        a = make(shape, dtype)
        da = DeviceCsr(a)
        descr = capi.make_descr(base=a.base)
        try:
            for n in (1, 3, 16, 17, 32, 64, 130, 300):
                if a.rows * n > 6_000_000:
                    continue
                B = complex_vector(a.cols * n, dtype, 5).reshape(a.cols, n)
                C0 = complex_vector(a.rows * n, dtype, 6).reshape(a.rows, n)
                for alpha, beta in SCALARS[:2]:
                    al, be = T(alpha), T(beta)
                    if layout == "row":
                        ref = orc.csrmm_plain(a, alpha, B, beta, C0)
                        dB, dC = dev(B), dev(C0)
                        args = (0, 0, capi.ALPHA_SPARSE_LAYOUT_ROW_MAJOR, n, n)
                    elif layout == "col":
                        ref = orc.csrmm_plain(a, alpha, np.asfortranarray(B), beta, np.asfortranarray(C0), layout="col")
                        dB, dC = dev(B.T.copy()), dev(C0.T.copy())      # column-major k x n, ldb = k
                        args = (0, 0, capi.ALPHA_SPARSE_LAYOUT_COLUMN_MAJOR, a.cols, a.rows)
                    else:
                        ref = orc.csrmm_plain(a, alpha, np.asfortranarray(B), beta, np.asfortranarray(C0), layout="col")
                        dB, dC = dev(B.copy()), dev(C0.T.copy())        # B stored n x k column-major == k x n row-major
                        args = (0, 1, capi.ALPHA_SPARSE_LAYOUT_COLUMN_MAJOR, n, a.rows)
                    announce("complex csrmm", np.dtype(dtype).name, shape, layout, n, alpha, beta)
                    st = getattr(lib, "alphasparse_dcu_%s_csrmm" % p)(
                        gpu.h, args[0], args[1], args[2], a.rows, n, a.cols, a.nnz, byref(al), byref(descr), da.val.c_ptr(),
                        da.row_ptr.c_ptr(), da.col.c_ptr(), dB.c_ptr(), args[3], byref(be), dC.c_ptr(), args[4])
                    assert st == 0, st
                    hiprt.synchronize()
                    got = dC.to_numpy().reshape(a.rows, n) if layout == "row" else dC.to_numpy().reshape(n, a.rows).T
                    err = orc.csrmm_err(a, alpha, B, beta, C0, got, np.asarray(ref))
                    assert err.zero_den_mismatch == 0 and err.full <= TOL[np.dtype(dtype)], (shape, layout, n, err)
                    dB.free()
                    dC.free()
        finally:
            da.free()


@pytest.mark.parametrize("shape", ["uniform16", "powerlaw", "laplace", "long_and_empty", "base_one", "tiny"])
@pytest.mark.parametrize("dtype", CX, ids=IDS)
def test_complex_coomv_ellmv_csr2ell(gpu, dtype, shape):
    lib = capi.load()
    p = capi.prefix(dtype)
    a = make(shape, dtype)
    x, y0 = complex_vector(a.cols, dtype, 3), complex_vector(a.rows, dtype, 4)
    rows = orc.csr2coo(a)
    rng = np.random.default_rng(2)
    for alpha, beta in SCALARS:
        ref = orc.csrmv_plain(a, alpha, x, beta, y0)
        announce("complex coomv", np.dtype(dtype).name, shape, alpha, beta)
        check(a, alpha, x, beta, y0, run_coomv(gpu, a.rows, a.cols, a.values, rows, a.col_ind, a.base, alpha, x, beta, y0),
              ref, "coomv %s" % shape)
    perm = rng.permutation(a.nnz)
    announce("complex coomv shuffled", np.dtype(dtype).name, shape)
    check(a, 1.25 - 0.5j, x, 0.5j, y0,
          run_coomv(gpu, a.rows, a.cols, a.values[perm].copy(), rows[perm].copy(), a.col_ind[perm].copy(), a.base,
                    1.25 - 0.5j, x, 0.5j, y0), orc.csrmv_plain(a, 1.25 - 0.5j, x, 0.5j, y0), "coomv shuffled %s" % shape)
    w = orc.csr2ell_width(a)
    if w * a.rows > 8_000_000:
        return
    da = DeviceCsr(a)
    try:
        for ell_base in (0, 1):
            ev, ec = orc.csr2ell(a, w, ell_base=ell_base)
            dev_v, dev_c = hiprt.DeviceArray(max(w * a.rows, 1), dtype), hiprt.DeviceArray(max(w * a.rows, 1), np.int32)
            d_csr, d_ell = capi.make_descr(base=a.base), capi.make_descr(base=ell_base)
            announce("complex csr2ell", np.dtype(dtype).name, shape, ell_base)
            assert getattr(lib, "alphasparse_dcu_%scsr2ell" % p)(
                gpu.h, a.rows, byref(d_csr), da.val.c_ptr(), da.row_ptr.c_ptr(), da.col.c_ptr(), byref(d_ell), w,
                dev_v.c_ptr(), dev_c.c_ptr()) == 0
            hiprt.synchronize()
            gv, gc = dev_v.to_numpy()[:w * a.rows], dev_c.to_numpy()[:w * a.rows]
            assert np.array_equal(gv.view(np.uint8), ev.view(np.uint8)) and np.array_equal(gc, ec)
            for alpha, beta in SCALARS[:2]:
                announce("complex ellmv", np.dtype(dtype).name, shape, ell_base, alpha, beta)
                y = run_ellmv(gpu, a.rows, a.cols, ev, ec, w, ell_base, alpha, x, beta, y0)
                check(a, alpha, x, beta, y0, y, orc.csrmv_plain(a, alpha, x, beta, y0), "ellmv %s" % shape)
                if ell_base == 0:   # same fused chain, same order as the oracle's restatement of the device kernel
                    assert np.array_equal(y, orc.ellmv(a.rows, a.cols, ev, ec, w, alpha, x, beta, y0))
            dev_v.free()
            dev_c.free()
    finally:
        da.free()


@pytest.mark.parametrize("dtype", CX, ids=IDS)
def test_complex_matrix_handles_and_host_entry_points(gpu, dtype):
    """create_coo -> convert_csr / convert_ell -> host2device -> mv_dcu; export; host-pointer mv / mm."""
    lib = capi.load()
    p, T = capi.prefix(dtype), capi.scalar_type(dtype)
    a = make("powerlaw", dtype) if dtype == np.complex64 else complexify(wl.powerlaw_rmat(12, 150, np.float64), dtype)
    x, y0 = complex_vector(a.cols, dtype, 3), complex_vector(a.rows, dtype, 4)
    xt, yt0 = complex_vector(a.rows, dtype, 5), complex_vector(a.cols, dtype, 6)
    perm = np.random.default_rng(1).permutation(a.nnz)
    rows, cols, vals = orc.csr2coo(a)[perm].copy(), a.col_ind[perm].copy(), a.values[perm].copy()
    coo, csr, ell = capi.alphasparse_matrix_t(), capi.alphasparse_matrix_t(), capi.alphasparse_matrix_t()
    assert getattr(lib, "alphasparse_%s_create_coo" % p)(byref(coo), 0, a.rows, a.cols, a.nnz, capi.ptr(rows), capi.ptr(cols),
                                                        capi.ptr(vals)) == 0
    assert lib.alphasparse_convert_csr(coo, 0, byref(csr)) == 0
    al, be = T(1.25 - 0.5j), T(0.5 + 0.75j)
    alpha, beta = 1.25 - 0.5j, 0.5 + 0.75j
    descr = capi.make_descr()
    hdescr = capi.alpha_matrix_descr(0, 0, 0)
    mv_dcu = getattr(lib, "alphasparse_%s_mv_dcu" % p)
    try:
        # the CSR handle holds exactly the source matrix (entries sorted by row, column)
        ib, r_, c_, rs, re_, ci, vv = c_int(), c_int32(), c_int32(), c_void_p(), c_void_p(), c_void_p(), c_void_p()
        assert getattr(lib, "alphasparse_%s_export_csr" % p)(csr, byref(ib), byref(r_), byref(c_), byref(rs), byref(re_),
                                                            byref(ci), byref(vv)) == 0
        assert (r_.value, c_.value, ib.value) == (a.rows, a.cols, 0)
        import ctypes
        got_rp = np.ctypeslib.as_array(ctypes.cast(rs, ctypes.POINTER(c_int32)), (a.rows + 1,))
        got_ci = np.ctypeslib.as_array(ctypes.cast(ci, ctypes.POINTER(c_int32)), (a.nnz,))
        got_v = np.frombuffer((ctypes.c_char * (a.nnz * a.values.itemsize)).from_address(vv.value), dtype=dtype)
        assert np.array_equal(got_rp, a.row_ptr - a.base) and np.array_equal(got_ci, a.col_ind - a.base)
        assert np.array_equal(got_v.view(np.uint8), a.values.view(np.uint8))
        assert getattr(lib, "host2device_%s_csr" % p)(csr) == 0
        for op, xx, yy in ((N, x, y0), (T_, xt, yt0), (H_, xt, yt0), (H_, xt, yt0)):
            m, ref = oracle_mv(a, op, alpha, xx, beta, yy)
            dx, dy = dev(xx), dev(yy)
            announce("complex mv_dcu on a csr handle", np.dtype(dtype).name, op)
            assert mv_dcu(gpu.h, op, byref(al), csr, byref(descr), dx.c_ptr(), byref(be), dy.c_ptr()) == 0
            hiprt.synchronize()
            check(m, alpha, xx, beta, yy, dy.to_numpy(), ref, "mv_dcu op %d" % op)
            dx.free()
            dy.free()
            # host pointers
            yh = yy.copy()
            announce("complex host mv", np.dtype(dtype).name, op)
            assert getattr(lib, "alphasparse_%s_mv" % p)(op, al, csr, hdescr, capi.ptr(xx), be, capi.ptr(yh)) == 0
            check(m, alpha, xx, beta, yy, yh, ref, "host mv op %d" % op)
        n = 9
        B = complex_vector(a.cols * n, dtype, 7).reshape(a.cols, n)
        C0 = complex_vector(a.rows * n, dtype, 8).reshape(a.rows, n)
        C = C0.copy()
        announce("complex host mm", np.dtype(dtype).name)
        assert getattr(lib, "alphasparse_%s_mm" % p)(0, al, csr, hdescr, capi.ALPHA_SPARSE_LAYOUT_ROW_MAJOR, capi.ptr(B), n, n, be,
                                                    capi.ptr(C), n) == 0
        err = orc.csrmm_err(a, alpha, B, beta, C0, C, orc.csrmm_plain(a, alpha, B, beta, C0))
        assert err.zero_den_mismatch == 0 and err.full <= TOL[np.dtype(dtype)], err
        # COO and ELL handles
        assert lib.alphasparse_convert_ell(coo, 0, byref(ell)) == 0
        ref = orc.csrmv_plain(a, alpha, x, beta, y0)
        dx = dev(x)
        for name, h, upload in (("coo", coo, "host2device_%s_coo" % p), ("ell", ell, "host2device_%s_ell" % p)):
            dy = dev(y0)
            announce("complex mv_dcu on a %s handle" % name, np.dtype(dtype).name)
            assert getattr(lib, upload)(h) == 0
            assert mv_dcu(gpu.h, 0, byref(al), h, byref(descr), dx.c_ptr(), byref(be), dy.c_ptr()) == 0
            hiprt.synchronize()
            check(a, alpha, x, beta, y0, dy.to_numpy(), ref, "mv_dcu %s" % name)
            dy.free()
        dx.free()
        # datatype mismatches are refused
        other = "z" if p == "c" else "c"
        assert getattr(lib, "host2device_%s_csr" % other)(csr) == capi.ALPHA_SPARSE_STATUS_INVALID_VALUE
        assert getattr(lib, "alphasparse_%s_mv" % other)(0, capi.scalar_type(np.complex128 if p == "c" else np.complex64)(1),
                                                        csr, hdescr, capi.ptr(x), capi.scalar_type(
                                                            np.complex128 if p == "c" else np.complex64)(0),
                                                        capi.ptr(y0.copy())) == capi.ALPHA_SPARSE_STATUS_INVALID_VALUE
    finally:
        for h in (coo, csr, ell):
            if h:
                assert lib.alphasparse_destroy(h) == 0


@pytest.mark.parametrize("fmt", ["csr", "coo", "ell"])
@pytest.mark.parametrize("dtype", CX, ids=IDS)
def test_complex_generic_spmv(gpu, dtype, fmt):
    lib = capi.load()
    T = capi.scalar_type(dtype)
    dt = capi.dtype_tag(dtype)
    a = make("laplace", dtype)
    x, y0 = complex_vector(a.cols, dtype, 3), complex_vector(a.rows, dtype, 4)
    alpha, beta = 1.25 - 0.5j, 0.5 + 0.75j
    al, be = T(alpha), T(beta)
    descr = capi.make_descr(base=a.base)
    info = capi.alphasparse_dcu_mat_info_t()
    assert lib.alphasparse_dcu_create_mat_info(byref(info)) == 0
    I32 = capi.ALPHA_SPARSE_DCU_INDEXTYPE_I32
    bufs = []
    try:
        if fmt == "csr":
            da = DeviceCsr(a)
            bufs += [da.val, da.row_ptr, da.col]
            mat = capi.alphasparse_dcu_spmat_descr(True, False, a.rows, a.cols, a.nnz, da.row_ptr.c_ptr(), da.col.c_ptr(), None,
                                                   da.val.c_ptr(), I32, I32, dt, a.base, capi.ALPHA_SPARSE_FORMAT_CSR,
                                                   ctypes_pointer(descr), info)
        elif fmt == "coo":
            rows = dev(orc.csr2coo(a))
            cols, vals = dev(a.col_ind), dev(a.values)
            bufs += [rows, cols, vals]
            mat = capi.alphasparse_dcu_spmat_descr(True, False, a.rows, a.cols, a.nnz, rows.c_ptr(), cols.c_ptr(), None,
                                                   vals.c_ptr(), I32, I32, dt, a.base, capi.ALPHA_SPARSE_FORMAT_COO,
                                                   ctypes_pointer(descr), info)
        else:
            w = orc.csr2ell_width(a)
            ev, ec = orc.csr2ell(a, w, ell_base=a.base)
            dv, dc = dev(ev), dev(ec)
            bufs += [dv, dc]
            mat = capi.alphasparse_dcu_spmat_descr(True, False, a.rows, a.cols, w, None, dc.c_ptr(), None, dv.c_ptr(), I32, I32,
                                                   dt, a.base, capi.ALPHA_SPARSE_FORMAT_ELL, ctypes_pointer(descr), info)
        dx, dy = dev(x), dev(y0)
        bufs += [dx, dy]
        xd = capi.alphasparse_dcu_dnvec_descr(True, a.cols, dx.c_ptr(), dt)
        yd = capi.alphasparse_dcu_dnvec_descr(True, a.rows, dy.c_ptr(), dt)
        size = c_size_t(0)
        announce("complex generic spmv", np.dtype(dtype).name, fmt)
        assert lib.alphasparse_dcu_spmv(gpu.h, 0, byref(al), byref(mat), byref(xd), byref(be), byref(yd), dt, 0, byref(size),
                                        None) == 0
        assert size.value == 4 and mat.analysed == (fmt == "csr")
        tmp = hiprt.DeviceArray(16, np.uint8)
        bufs.append(tmp)
        assert lib.alphasparse_dcu_spmv(gpu.h, 0, byref(al), byref(mat), byref(xd), byref(be), byref(yd), dt, 0, byref(size),
                                        tmp.c_ptr()) == 0
        hiprt.synchronize()
        check(a, alpha, x, beta, y0, dy.to_numpy(), orc.csrmv_plain(a, alpha, x, beta, y0), "generic %s" % fmt)
    finally:
        lib.alphasparse_dcu_destroy_mat_info(info)
        for b in bufs:
            b.free()


def ctypes_pointer(obj):
    import ctypes
    return ctypes.pointer(obj)


@pytest.mark.parametrize("dtype", CX, ids=IDS)
def test_misaligned_complex_arrays_are_refused_not_faulted(gpu, dtype):
    """Complex device arrays must be aligned to the element size; anything else is rejected on the
    host before a kernel could touch it."""
    lib = capi.load()
    T = capi.scalar_type(dtype)
    a = make("tiny", dtype)
    da = DeviceCsr(a)
    x, y0 = complex_vector(a.cols + 1, dtype, 3), complex_vector(a.rows + 1, dtype, 4)
    dx, dy = dev(x), dev(y0)
    half = np.dtype(dtype).itemsize // 2
    al, be = T(1), T(0)
    descr = capi.make_descr()
    try:
        announce("misaligned complex x", np.dtype(dtype).name)
        st = getattr(lib, "alphasparse_dcu_%s_csrmv" % capi.prefix(dtype))(
            gpu.h, 0, a.rows, a.cols, a.nnz, byref(al), byref(descr), da.val.c_ptr(), da.row_ptr.c_ptr(), da.col.c_ptr(), None,
            c_void_p(dx.ptr + half), byref(be), dy.c_ptr())
        assert st == capi.ALPHA_SPARSE_STATUS_INVALID_VALUE
        hiprt.synchronize()
        assert np.array_equal(dy.to_numpy(), y0)
    finally:
        da.free()
        dx.free()
        dy.free()
