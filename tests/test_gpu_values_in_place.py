"""csr_val rewritten IN PLACE after an analysis, multiplied again WITHOUT a second analysis.

In the reference the analysis keeps structure only (src/util_cpp/alphasparse_dcu_x_csrmv_analysis.cpp:382-388)
and every multiply reads csr_val (src/kernel/dcu/level2/mv/csrmv/dcu_gemv_vector.h:43-46), so
analysis -> rewrite csr_val -> csrmv(info) is a legal sequence there.  Here an analysis may keep re-ordered
copies of the values (tiled, ELL, A^T, A^H); a guard kernel in front of every multiply that uses such a copy
fingerprints csr_val on the device and the copy is gathered again when the fingerprint moved.  These tests
run that sequence under DEFAULT settings (no environment variable) and compare with the oracle on the
new values; they also run one analysis from two handles on two streams at once, which the reference's
stateless kernels allow (dcu_gemv_vector.h:14-57)."""
import ctypes
import os
import threading
from ctypes import byref, c_void_p

import numpy as np
import pytest

from alsparse_amd import capi, hiprt, workloads as wl
from oracle import oracle as orc
from helpers import ALGOS, DeviceCsr, announce, check_beta_rows
from helpers_shapes import complex_vector, complexify, real_dtype

pytestmark = pytest.mark.gpu
TOL = {np.dtype(np.float32): 1e-4, np.dtype(np.float64): 1e-12, np.dtype(np.complex64): 1e-4,
       np.dtype(np.complex128): 1e-12}
DT = [np.float32, np.float64, np.complex64]
IDS = ["f32", "f64", "c64"]


def _matrix(base, dtype):
    return complexify(base(real_dtype(dtype)), dtype) if np.iscomplexobj(np.zeros(1, dtype)) else base(dtype)


def _vector(n, dtype, seed):
    return complex_vector(n, dtype, seed) if np.iscomplexobj(np.zeros(1, dtype)) else wl.uniform(n, dtype, seed)


def _new_values(a, seed):
    rng = np.random.default_rng(seed)
    v = rng.uniform(-1, 1, size=a.nnz)
    if np.iscomplexobj(a.values):
        v = v + 1j * rng.uniform(-1, 1, size=a.nnz)
    return v.astype(a.dtype)


def _with_values(a, vals):
    return wl.Csr(a.rows, a.cols, a.row_ptr, a.col_ind, vals, a.base, a.name)


def _check(a, op, alpha, x, beta, y0, y, what):
    """per-output criterion against the oracle for op(A)"""
    if op == 0:
        m, ref = a, orc.csrmv_plain(a, alpha, x, beta, y0)
    else:
        m, ref = orc.transpose(a, conj=op == 2), orc.csrmv_trans_plain(a, alpha, x, beta, y0, conj=op == 2)
    err = orc.csrmv_err(m, alpha, x, beta, y0, y, ref)
    assert err.zero_den_mismatch == 0, "%s: %d outputs without products differ" % (what, err.zero_den_mismatch)
    assert err.full <= TOL[a.dtype], "%s: error %.3e at %d exceeds %g" % (what, err.full, err.row, TOL[a.dtype])
    if beta == 0:
        assert err.strict <= TOL[a.dtype], "%s: strict error %.3e" % (what, err.strict)
    else:
        check_beta_rows(m, alpha, x, beta, y0, y, ref, TOL[a.dtype], what)


@pytest.mark.parametrize("dtype", DT, ids=IDS)
@pytest.mark.parametrize("copy", ["tiled", "ell", "transposed", "conj_transposed"])
def test_plan_multiplies_with_the_values_of_the_moment(gpu, copy, dtype):
    """Every kind of value copy, laid out whatever the size (trusted == 2), then csr_val overwritten at the
    same address twice; each multiply -- no refresh, no second analysis -- must see the values of the moment."""
    if copy == "conj_transposed" and not np.iscomplexobj(np.zeros(1, dtype)):
        pytest.skip("a real matrix has no conjugate transpose in the reference's tables")
    lib = capi.load()
    a = _matrix(lambda rd: wl.uniform_rows(7000, 9000, 12, rd), dtype)
    op = {"tiled": 0, "ell": 0, "transposed": 1, "conj_transposed": 2}[copy]
    x = _vector(a.rows if op else a.cols, dtype, 3)
    y0 = _vector(a.cols if op else a.rows, dtype, 4)
    da = DeviceCsr(a)
    T = capi.scalar_type(a.dtype)
    plan = c_void_p()
    alpha, beta = 1.5, 0.5
    try:
        announce("values in place", copy, np.dtype(dtype).name)
        assert lib.asamd_csr_plan_create_dtype(None, a.rows, a.cols, a.nnz, da.row_ptr.c_ptr(), da.col.c_ptr(),
                                               da.val.c_ptr(), a.base, capi.dtype_tag(dtype), 2, byref(plan)) == 0
        st = lib.asamd_csr_plan_stats(plan).contents
        assert st.value_check == 1, "the default is the sampled check"
        if op == 0:
            assert lib.asamd_csr_plan_set_algo(plan, ALGOS[copy]) == 0
        elif op == 1:
            assert lib.asamd_csr_plan_build_transpose(None, plan, da.row_ptr.c_ptr(), da.col.c_ptr(), da.val.c_ptr()) == 0
        else:
            assert lib.asamd_csr_plan_build_conj_transpose(None, plan, da.row_ptr.c_ptr(), da.col.c_ptr(),
                                                           da.val.c_ptr()) == 0
        ws = capi.Workspace(lib, plan)

        def multiply():
            dx, dy = hiprt.DeviceArray.from_numpy(x), hiprt.DeviceArray.from_numpy(y0)
            assert capi.plan_csrmv(lib, None, plan, op, T(alpha), da.val.c_ptr(), da.row_ptr.c_ptr(), da.col.c_ptr(),
                                   dx.c_ptr(), T(beta), dy.c_ptr(), ws) == 0
            hiprt.synchronize()
            out = dy.to_numpy()
            dx.free()
            dy.free()
            return out

        _check(a, op, alpha, x, beta, y0, multiply(), "values of the analysis")
        first = multiply()
        assert np.array_equal(first, multiply()), "unchanged values: the same bits every time"
        for round_ in range(2):
            b = _with_values(a, _new_values(a, 40 + round_))
            da.val.copy_from(b.values)  # in place: same device address, no analysis, no refresh call
            _check(b, op, alpha, x, beta, y0, multiply(), "%s after in-place change %d" % (copy, round_))
        # back to the first values: the product is the first one again, bit for bit
        da.val.copy_from(a.values)
        assert np.array_equal(first, multiply())
    finally:
        lib.asamd_csr_plan_destroy(plan)
        da.free()


@pytest.mark.parametrize("dtype", DT, ids=IDS)
def test_analysis_then_new_values_then_csrmv_through_the_public_api(gpu, dtype):
    """alphasparse_dcu_?_csrmv_analysis -> overwrite csr_val -> alphasparse_dcu_?_csrmv(info), on a matrix large
    enough for the analysis to keep the tiled copy by itself (x beyond an XCD's L2, scattered columns)."""
    lib = capi.load()
    rows = 1 << 21
    a = _matrix(lambda rd: wl.uniform_rows(rows, rows, 16, rd), dtype)
    x, y0 = _vector(a.cols, dtype, 3), _vector(a.rows, dtype, 4)
    da = DeviceCsr(a)
    p, T = capi.prefix(dtype), capi.scalar_type(dtype)
    info = capi.alphasparse_dcu_mat_info_t()
    assert lib.alphasparse_dcu_create_mat_info(byref(info)) == 0
    descr = capi.make_descr(base=a.base)
    dx = hiprt.DeviceArray.from_numpy(x)

    def multiply(alpha, beta):
        dy = hiprt.DeviceArray.from_numpy(y0)
        al, be = T(alpha), T(beta)
        assert getattr(lib, "alphasparse_dcu_%s_csrmv" % p)(gpu.h, 0, a.rows, a.cols, a.nnz, byref(al), byref(descr),
                                                            da.val.c_ptr(), da.row_ptr.c_ptr(), da.col.c_ptr(), info,
                                                            dx.c_ptr(), byref(be), dy.c_ptr()) == 0
        hiprt.synchronize()
        out = dy.to_numpy()
        dy.free()
        return out

    try:
        announce("public API, values in place", a.name, np.dtype(dtype).name)
        assert getattr(lib, "alphasparse_dcu_%s_csrmv_analysis" % p)(gpu.h, 0, a.rows, a.cols, a.nnz, byref(descr),
                                                                     da.val.c_ptr(), da.row_ptr.c_ptr(),
                                                                     da.col.c_ptr(), info) == 0
        st = lib.asamd_analysis_stats(info).contents
        assert st.tiled_built == 1 and st.algo == capi.ASAMD_SPMV_TILED, "this shape is the tiled copy's"
        _check(a, 0, 1.5, x, 0.5, y0, multiply(1.5, 0.5), "after the analysis")
        b = _with_values(a, _new_values(a, 7))
        da.val.copy_from(b.values)
        _check(b, 0, 1.5, x, 0.5, y0, multiply(1.5, 0.5), "values rewritten, no second analysis")
        # a contiguous stretch of at least two sampling runs is always noticed, wherever it lies
        run = int(lib.asamd_value_guard_run(a.nnz * a.dtype.itemsize)) // a.dtype.itemsize
        vals = b.values.copy()
        lo = a.nnz // 3 + 5
        vals[lo:lo + 2 * run] *= -2
        c = _with_values(a, vals)
        da.val.copy_from(c.values)
        _check(c, 0, -1.0, x, 0.0, y0, multiply(-1.0, 0.0), "a stretch of two runs rewritten")
    finally:
        lib.alphasparse_dcu_destroy_mat_info(info)
        da.free()
        dx.free()


def test_full_value_check_notices_a_single_entry(gpu):
    """ALSPARSE_AMD_VALUE_CHECK=full fingerprints every byte: one changed entry anywhere is seen.  (Read when an
    analysis is made.)"""
    lib = capi.load()
    a = wl.uniform_rows(1 << 21, 1 << 21, 16, np.float32)  # 128 MiB of values: the default would sample
    assert a.nnz * 4 > 32 << 20
    x, y0 = wl.uniform(a.cols, a.dtype, 3), wl.uniform(a.rows, a.dtype, 4)
    da = DeviceCsr(a)
    plan = c_void_p()
    os.environ["ALSPARSE_AMD_VALUE_CHECK"] = "full"
    try:
        announce("full value check")
        assert lib.asamd_csr_plan_create(None, a.rows, a.cols, a.nnz, da.row_ptr.c_ptr(), da.col.c_ptr(), da.val.c_ptr(),
                                         a.base, 4, 1, byref(plan)) == 0
        st = lib.asamd_csr_plan_stats(plan).contents
        assert st.value_check == 2 and st.algo == capi.ASAMD_SPMV_TILED
        ws = capi.Workspace(lib, plan)
        dx = hiprt.DeviceArray.from_numpy(x)
        for k in (12345677, a.nnz - 1, 0):
            vals = a.values.copy()
            vals[k] = np.float32(1000.0)
            b = _with_values(a, vals)
            da.val.copy_from(vals)
            dy = hiprt.DeviceArray.from_numpy(y0)
            assert capi.plan_csrmv(lib, None, plan, 0, ctypes.c_float(1.0), da.val.c_ptr(), da.row_ptr.c_ptr(),
                                   da.col.c_ptr(), dx.c_ptr(), ctypes.c_float(0.0), dy.c_ptr(), ws) == 0
            hiprt.synchronize()
            _check(b, 0, 1.0, x, 0.0, y0, dy.to_numpy(), "entry %d poked" % k)
            dy.free()
        dx.free()
    finally:
        del os.environ["ALSPARSE_AMD_VALUE_CHECK"]
        lib.asamd_csr_plan_destroy(plan)
        da.free()


def test_small_workspace_still_multiplies_correctly(gpu):
    """A caller of the plan API who passes no workspace (or too small a one) gets the right product from kernels
    that need none -- and never a copy that could not be checked."""
    lib = capi.load()
    a = wl.powerlaw_rmat(14, 9000, np.float32)
    x, y0 = wl.uniform(a.cols, a.dtype, 3), wl.uniform(a.rows, a.dtype, 4)
    da = DeviceCsr(a)
    plan = c_void_p()
    try:
        announce("no workspace")
        assert lib.asamd_csr_plan_create(None, a.rows, a.cols, a.nnz, da.row_ptr.c_ptr(), da.col.c_ptr(), da.val.c_ptr(),
                                         a.base, 4, 2, byref(plan)) == 0
        dx = hiprt.DeviceArray.from_numpy(x)
        tiny = hiprt.DeviceArray((1024,), np.uint8)
        for algo in ("merge", "tiled", "binned", "hot", "vector"):
            if lib.asamd_csr_plan_set_algo(plan, ALGOS[algo]) != 0:
                continue
            for ws_ptr, ws_bytes in ((None, 0), (tiny.c_ptr(), 1024)):
                dy = hiprt.DeviceArray.from_numpy(y0)
                al, be = ctypes.c_float(2.0), ctypes.c_float(0.5)
                assert lib.asamd_csr_plan_csrmv(None, plan, 0, ctypes.cast(byref(al), c_void_p), da.val.c_ptr(),
                                                da.row_ptr.c_ptr(), da.col.c_ptr(), dx.c_ptr(),
                                                ctypes.cast(byref(be), c_void_p), dy.c_ptr(), ws_ptr, ws_bytes) == 0
                hiprt.synchronize()
                _check(a, 0, 2.0, x, 0.5, y0, dy.to_numpy(), "%s without workspace" % algo)
                dy.free()
        dx.free()
        tiny.free()
    finally:
        lib.asamd_csr_plan_destroy(plan)
        da.free()


@pytest.mark.parametrize("shape", ["powerlaw", "tiled", "slices"])
def test_one_analysis_from_two_handles_at_once(gpu, shape):
    """Two handles, each with a stream of its own, multiply with ONE info concurrently: every scratch word of a
    multiply lives in its handle's buffer, so each result equals the serial one bit for bit."""
    lib, hip = capi.load(), hiprt.lib()
    if shape == "powerlaw":
        a = wl.powerlaw_rmat(20, 1 << 20, np.float32)        # merge-path: carries and head sums per call
    elif shape == "slices":
        a = wl.uniform_rows(1 << 18, 1 << 17, 64, np.float32)  # x in LDS slice by slice: the slices' sums per call
    else:
        a = wl.uniform_rows(1 << 21, 1 << 21, 16, np.float32)  # tiled: the product array per call
    da = DeviceCsr(a)
    info = capi.alphasparse_dcu_mat_info_t()
    assert lib.alphasparse_dcu_create_mat_info(byref(info)) == 0
    descr = capi.make_descr(base=a.base)
    handles = [capi.Handle(), capi.Handle()]
    streams = [c_void_p(), c_void_p()]
    xs = [wl.uniform(a.cols, a.dtype, 10 + i) for i in range(2)]
    y0s = [wl.uniform(a.rows, a.dtype, 20 + i) for i in range(2)]
    dxs = [hiprt.DeviceArray.from_numpy(v) for v in xs]
    dys = [hiprt.DeviceArray.from_numpy(v) for v in y0s]
    scal = [(ctypes.c_float(1.25), ctypes.c_float(0.5)), (ctypes.c_float(-0.75), ctypes.c_float(0.0))]
    try:
        announce("two handles, one analysis", shape)
        for i in range(2):
            hiprt.check(hip.hipStreamCreate(byref(streams[i])), "hipStreamCreate")
            assert lib.asamd_handle_set_stream(handles[i].h, streams[i]) == 0
        assert lib.alphasparse_dcu_s_csrmv_analysis(handles[0].h, 0, a.rows, a.cols, a.nnz, byref(descr), da.val.c_ptr(),
                                                    da.row_ptr.c_ptr(), da.col.c_ptr(), info) == 0
        st = lib.asamd_analysis_stats(info).contents
        want = {"powerlaw": capi.ASAMD_SPMV_MERGE, "slices": capi.ASAMD_SPMV_XLDS, "tiled": capi.ASAMD_SPMV_TILED}[shape]
        assert st.algo == want and (shape != "slices" or st.xlds_slices >= 2), (st.algo, st.xlds_slices)

        def multiply(i, reps):
            for _ in range(reps):
                s = lib.alphasparse_dcu_s_csrmv(handles[i].h, 0, a.rows, a.cols, a.nnz, byref(scal[i][0]), byref(descr),
                                                da.val.c_ptr(), da.row_ptr.c_ptr(), da.col.c_ptr(), info,
                                                dxs[i].c_ptr(), byref(scal[i][1]), dys[i].c_ptr())
                assert s == 0, s

        # serial results first (beta applied once: y is restored before every run)
        serial = []
        for i in range(2):
            dys[i].copy_from(y0s[i])
            multiply(i, 1)
            hiprt.synchronize()
            serial.append(dys[i].to_numpy())
            _check(a, 0, scal[i][0].value, xs[i], scal[i][1].value, y0s[i], serial[i], "serial, handle %d" % i)
        # the second handle's first call grew its buffer; from here on nothing allocates or waits
        for rep in range(3):
            for i in range(2):
                dys[i].copy_from(y0s[i])
            hiprt.synchronize()
            # beta == 0.5 on handle 0: a single multiply per run; handle 1 (beta == 0) repeats to overlap longer
            threads = [threading.Thread(target=multiply, args=(0, 1)), threading.Thread(target=multiply, args=(1, 6))]
            for t in threads:
                t.start()
            for t in threads:
                t.join()
            hiprt.synchronize()
            for i in range(2):
                assert np.array_equal(dys[i].to_numpy().view(np.uint32), serial[i].view(np.uint32)), (
                    "handle %d, concurrent run %d differs from the serial result" % (i, rep))
    finally:
        lib.alphasparse_dcu_destroy_mat_info(info)
        for i in range(2):
            handles[i].close()
            if streams[i]:
                hip.hipStreamDestroy(streams[i])
        for d in dxs + dys:
            d.free()
        da.free()


def test_host_pointer_mv_notices_one_changed_value_and_a_changed_structure(gpu):
    """alphasparse_d_mv reads the caller's host arrays on every call in the reference, so a single value poked
    through alphasparse_d_export_csr's pointers counts from the next call on, and so does an edited column."""
    from ctypes import POINTER, c_double, c_int, c_int32
    lib = capi.load()
    a = wl.uniform_rows(3000, 2500, 9, np.float64)
    x, y0 = wl.uniform(a.cols, a.dtype, 3), wl.uniform(a.rows, a.dtype, 4)
    A = capi.alphasparse_matrix_t()
    rs, re = np.ascontiguousarray(a.row_ptr[:-1]), np.ascontiguousarray(a.row_ptr[1:])
    assert lib.alphasparse_d_create_csr(byref(A), a.base, a.rows, a.cols, capi.ptr(rs), capi.ptr(re), capi.ptr(a.col_ind),
                                        capi.ptr(a.values)) == 0
    descr = capi.alpha_matrix_descr(0, 0, 0)
    try:
        announce("host mv, one value / one column edited")
        y = y0.copy()
        assert lib.alphasparse_d_mv(0, c_double(1.5), A, descr, capi.ptr(x), c_double(0.5), capi.ptr(y)) == 0
        _check(a, 0, 1.5, x, 0.5, y0, y, "host mv")
        base, rows, cols = c_int(), c_int32(), c_int32()
        prs, pre, pci, pv = c_void_p(), c_void_p(), c_void_p(), c_void_p()
        assert lib.alphasparse_d_export_csr(A, byref(base), byref(rows), byref(cols), byref(prs), byref(pre), byref(pci),
                                            byref(pv)) == 0
        host_vals = np.ctypeslib.as_array(ctypes.cast(pv, POINTER(c_double)), shape=(a.nnz,))
        host_cols = np.ctypeslib.as_array(ctypes.cast(pci, POINTER(c_int32)), shape=(a.nnz,))
        vals, col = a.values.copy(), a.col_ind.copy()
        for k in (1, a.nnz // 2 + 3, a.nnz - 1):  # positions chosen without regard to any sampling
            vals[k] = vals[k] * 3.0 + 7.0
            host_vals[k] = vals[k]
            b = wl.Csr(a.rows, a.cols, a.row_ptr, col, vals, a.base, a.name)
            y = y0.copy()
            assert lib.alphasparse_d_mv(0, c_double(1.5), A, descr, capi.ptr(x), c_double(0.5), capi.ptr(y)) == 0
            _check(b, 0, 1.5, x, 0.5, y0, y, "value %d poked" % k)
        # one column index moved to a column the row does not use yet (the row stays sorted or not: the
        # kernels do not care)
        r = a.rows // 2
        k = int(a.row_ptr[r]) - a.base
        used = set(col[k:int(a.row_ptr[r + 1]) - a.base].tolist())
        new_col = next(c for c in range(a.base, a.cols + a.base) if c not in used)
        col[k] = new_col
        host_cols[k] = new_col
        b = wl.Csr(a.rows, a.cols, a.row_ptr, col, vals, a.base, a.name)
        y = y0.copy()
        assert lib.alphasparse_d_mv(0, c_double(1.5), A, descr, capi.ptr(x), c_double(0.5), capi.ptr(y)) == 0
        _check(b, 0, 1.5, x, 0.5, y0, y, "column index edited")
    finally:
        lib.alphasparse_destroy(A)
