"""Values changed IN PLACE after an analysis.

The reference's analysis keeps structure only (src/util_cpp/alphasparse_dcu_x_csrmv_analysis.cpp:382-388), so a
caller may rewrite csr_val between multiplies.  Here an analysis may keep re-ordered copies of the values (tiled,
ELL, transposed); the rule is: analyse again after changing values.  A repeated analysis of unchanged structure
arrays only gathers the values again (no sort), a changed structure at the same addresses is noticed through a
fingerprint of the structure arrays, ALSPARSE_AMD_ANALYSIS=structure keeps every analysis free of value copies,
and the host-pointer entry points notice rewritten host values by themselves."""
import os
import time
from ctypes import byref, c_void_p

import numpy as np
import pytest

from alsparse_amd import capi, hiprt, workloads as wl
from oracle import oracle as orc
from helpers import ALGOS, TOL, DeviceCsr, announce, check_spmv, run_csrmv

pytestmark = pytest.mark.gpu


def _new_values(a, seed):
    rng = np.random.default_rng(seed)
    return rng.uniform(-1, 1, size=a.nnz).astype(a.dtype)


def _with_values(a, vals):
    return wl.Csr(a.rows, a.cols, a.row_ptr, a.col_ind, vals, a.base, a.name)


@pytest.mark.parametrize("dtype", [np.float32, np.float64], ids=["f32", "f64"])
@pytest.mark.parametrize("algo", ["tiled", "ell", "merge"])
def test_plan_refresh_values_brings_every_copy_up_to_date(gpu, algo, dtype):
    lib = capi.load()
    a = wl.uniform_rows(6000, 9000, 16, dtype) if algo != "merge" else wl.powerlaw_rmat(13, 3000, dtype)
    x, y0 = wl.uniform(a.cols, a.dtype, 3), wl.uniform(a.rows, a.dtype, 4)
    xt = wl.uniform(a.rows, a.dtype, 5)
    da = DeviceCsr(a)
    T = capi.scalar_type(a.dtype)
    p = capi.prefix(a.dtype)
    plan = c_void_p()
    try:
        announce("refresh", algo, np.dtype(dtype).name)
        assert lib.asamd_csr_plan_create(None, a.rows, a.cols, a.nnz, da.row_ptr.c_ptr(), da.col.c_ptr(), da.val.c_ptr(),
                                         a.base, a.dtype.itemsize, 2, byref(plan)) == 0
        assert lib.asamd_csr_plan_set_algo(plan, ALGOS[algo]) == 0
        assert lib.asamd_csr_plan_build_transpose(None, plan, da.row_ptr.c_ptr(), da.col.c_ptr(), da.val.c_ptr()) == 0

        def multiply(trans):
            dx = hiprt.DeviceArray.from_numpy(xt if trans else x)
            dy = hiprt.DeviceArray.from_numpy(wl.uniform(a.cols, a.dtype, 6) if trans else y0)
            ws = capi.Workspace(lib, plan)
            assert capi.plan_csrmv(lib, None, plan, 1 if trans else 0, T(1.5), da.val.c_ptr(), da.row_ptr.c_ptr(),
                                   da.col.c_ptr(), dx.c_ptr(), T(0.0), dy.c_ptr(), ws) == 0
            hiprt.synchronize()
            out = dy.to_numpy()
            dx.free()
            dy.free()
            return out

        check_spmv(a, 1.5, x, 0.0, y0, multiply(False), "before the change")
        for round_ in range(2):
            b = _with_values(a, _new_values(a, 100 + round_))
            da.val.copy_from(b.values)  # in place: same device address
            assert lib.asamd_csr_plan_refresh_values(None, plan, da.row_ptr.c_ptr(), da.col.c_ptr(), da.val.c_ptr()) == 0
            check_spmv(b, 1.5, x, 0.0, y0, multiply(False), "%s after refresh %d" % (algo, round_))
            yt = multiply(True)
            ref = orc.csrmv_trans_plain(b, 1.5, xt, 0.0, np.zeros(a.cols, a.dtype))
            den = 1.5 * orc.csrmv_trans_plain(_with_values(a, np.abs(b.values)), 1.0, np.abs(xt), 0.0,
                                              np.zeros(a.cols, a.dtype)).astype(np.float64)
            diff = np.abs(yt.astype(np.float64) - ref.astype(np.float64))
            assert np.all(diff[den == 0] == 0)
            assert np.max(diff[den > 0] / den[den > 0]) <= TOL[np.dtype(dtype)], "transposed copy after refresh"
    finally:
        lib.asamd_csr_plan_destroy(plan)
        da.free()


def test_reanalysis_after_values_changed_in_place(gpu):
    """Large enough for the analysis to pick the tiled copy (2 M x 2 M, 16 per row): analyse, multiply, rewrite
    csr_val in place, analyse again (values only: several times faster than the first analysis), multiply."""
    lib = capi.load()
    a = wl.uniform_rows(1 << 21, 1 << 21, 16, np.float32)
    x, y0 = wl.uniform(a.cols, a.dtype, 3), wl.uniform(a.rows, a.dtype, 4)
    da = DeviceCsr(a)
    info = capi.alphasparse_dcu_mat_info_t()
    assert lib.alphasparse_dcu_create_mat_info(byref(info)) == 0
    descr = capi.make_descr(base=a.base)

    def analyse():
        hiprt.synchronize()
        t0 = time.perf_counter()
        assert lib.alphasparse_dcu_s_csrmv_analysis(gpu.h, 0, a.rows, a.cols, a.nnz, byref(descr), da.val.c_ptr(),
                                                    da.row_ptr.c_ptr(), da.col.c_ptr(), info) == 0
        hiprt.synchronize()
        return (time.perf_counter() - t0) * 1e3

    try:
        announce("re-analysis", a.name)
        first_ms = analyse()
        st = lib.asamd_analysis_stats(info).contents
        assert st.tiled_built == 1 and st.algo == capi.ASAMD_SPMV_TILED
        check_spmv(a, 1.5, x, 0.5, y0, run_csrmv(gpu, da, 1.5, x, 0.5, y0, info), "first analysis")
        b = _with_values(a, _new_values(a, 7))
        da.val.copy_from(b.values)
        again_ms = analyse()
        st = lib.asamd_analysis_stats(info).contents
        assert st.tiled_built == 1 and st.algo == capi.ASAMD_SPMV_TILED
        check_spmv(b, 1.5, x, 0.5, y0, run_csrmv(gpu, da, 1.5, x, 0.5, y0, info), "after re-analysis")
        print("analysis %.2f ms, repeated on changed values %.2f ms" % (first_ms, again_ms))
        assert again_ms < 0.5 * first_ms, (first_ms, again_ms)
        # a different structure at the same addresses (same sizes): noticed, laid out afresh
        c = wl.uniform_rows(1 << 21, 1 << 21, 16, np.float32, seed=wl.SEED + 1)
        assert c.nnz == a.nnz and not np.array_equal(c.col_ind, a.col_ind)
        da.col.copy_from(c.col_ind)
        da.val.copy_from(c.values)
        analyse()
        check_spmv(c, 1.5, x, 0.5, y0, run_csrmv(gpu, da, 1.5, x, 0.5, y0, info), "new structure, same addresses")
    finally:
        lib.alphasparse_dcu_destroy_mat_info(info)
        da.free()


def test_structure_only_analysis_reads_values_live(gpu):
    lib = capi.load()
    a = wl.laplace2d(300, 200, np.float64)  # an analysis would keep an ELL copy of this one
    x, y0 = wl.uniform(a.cols, a.dtype, 3), wl.uniform(a.rows, a.dtype, 4)
    da = DeviceCsr(a)
    info = capi.alphasparse_dcu_mat_info_t()
    assert lib.alphasparse_dcu_create_mat_info(byref(info)) == 0
    descr = capi.make_descr(base=a.base)
    os.environ["ALSPARSE_AMD_ANALYSIS"] = "structure"
    try:
        announce("structure-only analysis", a.name)
        assert lib.alphasparse_dcu_d_csrmv_analysis(gpu.h, 0, a.rows, a.cols, a.nnz, byref(descr), da.val.c_ptr(),
                                                    da.row_ptr.c_ptr(), da.col.c_ptr(), info) == 0
        st = lib.asamd_analysis_stats(info).contents
        assert st.ell_built == 0 and st.tiled_built == 0 and st.transpose_built == 0
        check_spmv(a, 2.0, x, 0.0, y0, run_csrmv(gpu, da, 2.0, x, 0.0, y0, info), "structure-only")
        b = _with_values(a, _new_values(a, 3))
        da.val.copy_from(b.values)  # no second analysis
        check_spmv(b, 2.0, x, 0.0, y0, run_csrmv(gpu, da, 2.0, x, 0.0, y0, info), "values changed, no re-analysis")
    finally:
        del os.environ["ALSPARSE_AMD_ANALYSIS"]
        lib.alphasparse_dcu_destroy_mat_info(info)
        da.free()


def test_host_pointer_mv_sees_values_rewritten_through_export_csr(gpu):
    """alphasparse_d_mv reads host arrays in the reference, so values written through the pointers of
    alphasparse_d_export_csr count from the next call on; here the device mirror follows."""
    from ctypes import POINTER, c_double, c_int, c_int32
    lib = capi.load()
    a = wl.laplace2d(120, 90, np.float64)
    x, y0 = wl.uniform(a.cols, a.dtype, 3), wl.uniform(a.rows, a.dtype, 4)
    A = capi.alphasparse_matrix_t()
    rs, re = np.ascontiguousarray(a.row_ptr[:-1]), np.ascontiguousarray(a.row_ptr[1:])
    assert lib.alphasparse_d_create_csr(byref(A), a.base, a.rows, a.cols, capi.ptr(rs), capi.ptr(re), capi.ptr(a.col_ind),
                                        capi.ptr(a.values)) == 0
    descr = capi.alpha_matrix_descr(0, 0, 0)
    try:
        announce("host mv after export_csr edit")
        y = y0.copy()
        assert lib.alphasparse_d_mv(0, c_double(1.5), A, descr, capi.ptr(x), c_double(0.5), capi.ptr(y)) == 0
        check_spmv(a, 1.5, x, 0.5, y0, y, "host mv")
        base, rows, cols = c_int(), c_int32(), c_int32()
        prs, pre, pci, pv = c_void_p(), c_void_p(), c_void_p(), c_void_p()
        assert lib.alphasparse_d_export_csr(A, byref(base), byref(rows), byref(cols), byref(prs), byref(pre), byref(pci),
                                            byref(pv)) == 0
        import ctypes
        host_vals = np.ctypeslib.as_array(ctypes.cast(pv, POINTER(c_double)), shape=(a.nnz,))
        b = _with_values(a, _new_values(a, 11))
        host_vals[:] = b.values  # the library's own host copy, rewritten in place
        for op, ref_fn in ((0, None), (1, orc.csrmv_trans_plain)):
            y = y0.copy() if op == 0 else wl.uniform(a.cols, a.dtype, 6)
            xin = x if op == 0 else wl.uniform(a.rows, a.dtype, 5)
            yin = y.copy()
            assert lib.alphasparse_d_mv(op, c_double(1.5), A, descr, capi.ptr(xin), c_double(0.5), capi.ptr(y)) == 0
            if op == 0:
                check_spmv(b, 1.5, x, 0.5, y0, y, "host mv after edit")
            else:
                ref = ref_fn(b, 1.5, xin, 0.5, yin)
                assert np.max(np.abs(y - ref)) <= 1e-11 * max(1.0, np.max(np.abs(ref)))
    finally:
        lib.alphasparse_destroy(A)
