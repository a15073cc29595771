"""An analysed csrmv only launches kernels on the handle's stream (no allocation, no memset, no
synchronisation), so it can be recorded into a HIP graph and replayed.  Every replay is checked
against the eager result, with eager work and synchronisations between replays."""
import ctypes
from ctypes import byref, c_void_p

import numpy as np
import pytest

from alsparse_amd import capi, hiprt, workloads as wl
from helpers import ALGOS, TOL, DeviceCsr, announce, check_spmv
from oracle import oracle as orc

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("shape", ["powerlaw_merge", "laplace_ell", "uniform_tiled", "transposed"])
def test_analysed_csrmv_replays_from_a_hip_graph(gpu, shape):
    lib, hip = capi.load(), hiprt.lib()
    dtype = np.float64 if shape == "laplace_ell" else np.float32
    if shape == "powerlaw_merge":
        a = wl.powerlaw_rmat(15, 200000, dtype)
    elif shape == "laplace_ell":
        a = wl.laplace2d(700, 600, dtype)
    else:
        a = wl.uniform_rows(1 << 19, 1 << 22, 12, dtype)   # x = 16 MiB: the tiled copy is built and timed
    trans = capi.ALPHA_SPARSE_OPERATION_TRANSPOSE if shape == "transposed" else 0
    xlen, ylen = (a.rows, a.cols) if trans else (a.cols, a.rows)
    x, y0 = wl.uniform(xlen, dtype, 3), wl.uniform(ylen, dtype, 4)
    T, p = capi.scalar_type(dtype), capi.prefix(dtype)
    da = DeviceCsr(a)
    dx, dy = hiprt.DeviceArray.from_numpy(x), hiprt.DeviceArray.from_numpy(y0)
    stream, graph, gexec = c_void_p(), c_void_p(), c_void_p()
    hiprt.check(hip.hipStreamCreate(byref(stream)), "hipStreamCreate")
    h = capi.Handle()
    info = capi.alphasparse_dcu_mat_info_t()
    assert lib.alphasparse_dcu_create_mat_info(byref(info)) == 0
    descr = capi.make_descr()
    al, be = T(1.25), T(0.5)
    csrmv = getattr(lib, "alphasparse_dcu_%s_csrmv" % p)

    def multiply():
        return csrmv(h.h, trans, a.rows, a.cols, a.nnz, byref(al), byref(descr), da.val.c_ptr(), da.row_ptr.c_ptr(),
                     da.col.c_ptr(), info, dx.c_ptr(), byref(be), dy.c_ptr())
    try:
        assert lib.asamd_handle_set_stream(h.h, stream) == 0
        announce("graph capture: analysis", shape)
        assert getattr(lib, "alphasparse_dcu_%s_csrmv_analysis" % p)(
            h.h, trans, a.rows, a.cols, a.nnz, byref(descr), da.val.c_ptr(), da.row_ptr.c_ptr(), da.col.c_ptr(), info) == 0
        stats = lib.asamd_analysis_stats(info).contents
        announce("graph capture: analysis chose", capi.ALGO_NAMES[stats.algo])
        assert multiply() == 0                                   # eager, on the stream
        hiprt.check(hip.hipStreamSynchronize(stream), "sync")
        eager = dy.to_numpy()

        def verify(y, what):
            if trans:
                ref = orc.csrmv_trans_plain(a, 1.25, x, 0.5, y0)
                err = orc.csrmv_err(orc.transpose(a), 1.25, x, 0.5, y0, y, ref)
                assert err.zero_den_mismatch == 0 and err.full <= TOL[a.dtype], (what, err)
            else:
                check_spmv(a, 1.25, x, 0.5, y0, y, what)
        verify(eager, "eager " + shape)
        # the plan that runs the multiply: the transposed copy has an analysis of its own
        running = lib.asamd_analysis_transpose_stats(info).contents if trans else stats
        announce("graph capture: record", shape)
        hiprt.check(hip.hipStreamBeginCapture(stream, 0), "hipStreamBeginCapture")
        st = multiply()
        hiprt.check(hip.hipStreamEndCapture(stream, byref(graph)), "hipStreamEndCapture")
        assert st == 0
        hiprt.check(hip.hipGraphInstantiate(byref(gexec), graph, None, None, ctypes.c_size_t(0)), "hipGraphInstantiate")
        for replay in range(3):
            dy.copy_from(y0)                                     # eager work between the replays
            hiprt.synchronize()
            announce("graph capture: replay", shape, replay)
            hiprt.check(hip.hipGraphLaunch(gexec, stream), "hipGraphLaunch")
            hiprt.check(hip.hipStreamSynchronize(stream), "sync")
            got = dy.to_numpy()
            if running.tiled_built:  # checked against the oracle like the eager result
                verify(got, "replay %d" % replay)
            else:
                assert np.array_equal(got, eager), "replay %d differs from the eager result" % replay
    finally:
        if gexec:
            hip.hipGraphExecDestroy(gexec)
        if graph:
            hip.hipGraphDestroy(graph)
        lib.alphasparse_dcu_destroy_mat_info(info)
        h.close()
        hip.hipStreamDestroy(stream)
        for d in (dx, dy):
            d.free()
        da.free()


CAPTURE_CASES = [(algo, "uniform") for algo in ("vector", "rowconst", "merge", "scalar", "tiled", "stream", "ell", "hot",
                                                "binned")]
CAPTURE_CASES += [("xlds", "narrow")]  # x fits the LDS: 20 000 columns, read as 16-bit numbers
CAPTURE_CASES += [("xlds", "uniform")]  # 50 000 columns: two slices over a copy of the entries, behind the value guard
# heavy-tailed rows: the tiled copy's third phase, the bins' chunked long rows, merge blocks inside one row
CAPTURE_CASES += [(algo, "powerlaw") for algo in ("merge", "tiled", "hot", "binned")]


@pytest.mark.parametrize("algo,shape", CAPTURE_CASES, ids=["%s-%s" % c for c in CAPTURE_CASES])
def test_every_kernel_family_replays_from_a_hip_graph(gpu, algo, shape):
    """The thin kernel ABI with a forced family, recorded on a caller's stream."""
    lib, hip = capi.load(), hiprt.lib()
    a = (wl.uniform_rows(60000, 50000, 16, np.float32) if shape == "uniform" else
         wl.uniform_rows(60000, 20000, 16, np.float32) if shape == "narrow" else wl.powerlaw_rmat(15, 200000, np.float32))
    x, y0 = wl.uniform(a.cols, a.dtype, 5), wl.uniform(a.rows, a.dtype, 6)
    da = DeviceCsr(a)
    dx, dy = hiprt.DeviceArray.from_numpy(x), hiprt.DeviceArray.from_numpy(y0)
    stream, graph, gexec, plan = c_void_p(), c_void_p(), c_void_p(), c_void_p()
    hiprt.check(hip.hipStreamCreate(byref(stream)), "hipStreamCreate")
    try:
        announce("graph capture: plan", algo)
        assert lib.asamd_csr_plan_create(stream, a.rows, a.cols, a.nnz, da.row_ptr.c_ptr(), da.col.c_ptr(),
                                         da.val.c_ptr(), a.base, a.dtype.itemsize, 2, byref(plan)) == 0
        assert lib.asamd_csr_plan_set_algo(plan, ALGOS[algo]) == 0, "this matrix can run every family"

        ws = capi.Workspace(lib, plan)

        def multiply():
            return capi.plan_csrmv(lib, stream, plan, 0, ctypes.c_float(-0.75), da.val.c_ptr(), da.row_ptr.c_ptr(),
                                   da.col.c_ptr(), dx.c_ptr(), ctypes.c_float(2.0), dy.c_ptr(), ws)
        assert multiply() == 0
        hiprt.check(hip.hipStreamSynchronize(stream), "sync")
        eager = dy.to_numpy()
        check_spmv(a, -0.75, x, 2.0, y0, eager, "eager " + algo)
        hiprt.check(hip.hipStreamBeginCapture(stream, 0), "hipStreamBeginCapture")
        st = multiply()
        hiprt.check(hip.hipStreamEndCapture(stream, byref(graph)), "hipStreamEndCapture")
        assert st == 0
        hiprt.check(hip.hipGraphInstantiate(byref(gexec), graph, None, None, ctypes.c_size_t(0)), "hipGraphInstantiate")
        for replay in range(3):
            dy.copy_from(y0)
            hiprt.synchronize()
            announce("graph capture: replay", algo, replay)
            hiprt.check(hip.hipGraphLaunch(gexec, stream), "hipGraphLaunch")
            hiprt.check(hip.hipStreamSynchronize(stream), "sync")
            got = dy.to_numpy()
            assert np.array_equal(got, eager), "replay %d differs from the eager result" % replay
    finally:
        if gexec:
            hip.hipGraphExecDestroy(gexec)
        if graph:
            hip.hipGraphDestroy(graph)
        if plan:
            lib.asamd_csr_plan_destroy(plan)
        hip.hipStreamDestroy(stream)
        for d in (dx, dy):
            d.free()
        da.free()


def test_first_transposed_multiply_of_a_mirror_can_be_captured(gpu):
    """A library-built mirror lays out its copy of the transpose on the first transposed multiply -- which
    allocates and waits, so a call under stream capture scatters with atomics instead (kernels only); the
    copy is laid out by the first transposed multiply outside a capture."""
    from ctypes import POINTER, cast, c_float
    lib, hip = capi.load(), hiprt.lib()
    a = wl.powerlaw_rmat(13, 3000, np.float32)
    x, y0 = wl.uniform(a.rows, a.dtype, 3), wl.uniform(a.cols, a.dtype, 4)
    A = capi.alphasparse_matrix_t()
    rs, re = np.ascontiguousarray(a.row_ptr[:-1]), np.ascontiguousarray(a.row_ptr[1:])
    assert lib.alphasparse_s_create_csr(byref(A), a.base, a.rows, a.cols, capi.ptr(rs), capi.ptr(re), capi.ptr(a.col_ind),
                                        capi.ptr(a.values)) == 0
    dx, dy = hiprt.DeviceArray.from_numpy(x), hiprt.DeviceArray.from_numpy(y0)
    stream, graph, gexec = c_void_p(), c_void_p(), c_void_p()
    hiprt.check(hip.hipStreamCreate(byref(stream)), "hipStreamCreate")
    h = capi.Handle()
    descr = capi.make_descr()
    al, be = c_float(1.25), c_float(0.5)
    T = capi.ALPHA_SPARSE_OPERATION_TRANSPOSE

    def multiply():
        return lib.alphasparse_s_mv_dcu(h.h, T, byref(al), A, byref(descr), dx.c_ptr(), byref(be), dy.c_ptr())

    def verify(y, what):
        ref = orc.csrmv_trans_plain(a, 1.25, x, 0.5, y0)
        err = orc.csrmv_err(orc.transpose(a), 1.25, x, 0.5, y0, y, ref)
        assert err.zero_den_mismatch == 0 and err.full <= TOL[a.dtype], (what, err)
    try:
        assert lib.host2device_s_csr(A) == 0
        key = cast(A.contents.mat, POINTER(capi.spmat_csr_s_t)).contents.d_row_ptr
        assert lib.asamd_handle_set_stream(h.h, stream) == 0
        announce("graph capture: first transposed multiply of a mirror")
        hiprt.check(hip.hipStreamBeginCapture(stream, 0), "hipStreamBeginCapture")
        st = multiply()
        hiprt.check(hip.hipStreamEndCapture(stream, byref(graph)), "hipStreamEndCapture")
        assert st == 0
        assert not lib.asamd_analysis_transpose_stats(key), "no copy may be laid out under capture"
        hiprt.check(hip.hipGraphInstantiate(byref(gexec), graph, None, None, ctypes.c_size_t(0)), "hipGraphInstantiate")
        for replay in range(3):
            dy.copy_from(y0)
            hiprt.synchronize()
            hiprt.check(hip.hipGraphLaunch(gexec, stream), "hipGraphLaunch")
            hiprt.check(hip.hipStreamSynchronize(stream), "sync")
            verify(dy.to_numpy(), "replay %d" % replay)
        dy.copy_from(y0)
        assert multiply() == 0                                   # eager: lays out the copy and uses it
        hiprt.check(hip.hipStreamSynchronize(stream), "sync")
        verify(dy.to_numpy(), "eager after the capture")
        assert lib.asamd_analysis_transpose_stats(key), "the eager call lays out the copy of the transpose"
    finally:
        if gexec:
            hip.hipGraphExecDestroy(gexec)
        if graph:
            hip.hipGraphDestroy(graph)
        h.close()
        hip.hipStreamDestroy(stream)
        lib.alphasparse_destroy(A)
        for d in (dx, dy):
            d.free()


def test_first_row_major_csrmm_of_a_matrix_can_be_captured(gpu):
    """With a dense operand of 48 to 384 MiB the first row-major csrmm of a matrix looks at the matrix to choose
    its kernel, which needs a synchronisation -- not under stream capture: there it only launches.  The replays
    and an eager call afterwards (which does look) are checked against the oracle."""
    from ctypes import c_float
    lib, hip = capi.load(), hiprt.lib()
    a = wl.stencil3d(64, 60, 56, np.float32)
    n = 64
    B = wl.uniform(a.cols * n, np.float32, 5).reshape(a.cols, n)
    C0 = wl.uniform(a.rows * n, np.float32, 6).reshape(a.rows, n)
    assert 48 << 20 < B.nbytes <= 384 << 20
    ref = orc.csrmm_plain(a, 1.25, B, 0.5, C0)
    da = DeviceCsr(a)
    dB, dC = hiprt.DeviceArray.from_numpy(B), hiprt.DeviceArray.from_numpy(C0)
    stream, graph, gexec = c_void_p(), c_void_p(), c_void_p()
    hiprt.check(hip.hipStreamCreate(byref(stream)), "hipStreamCreate")
    h = capi.Handle()
    descr = capi.make_descr()
    al, be = c_float(1.25), c_float(0.5)

    def multiply():
        return lib.alphasparse_dcu_s_csrmm(h.h, 0, 0, capi.ALPHA_SPARSE_LAYOUT_ROW_MAJOR, a.rows, n, a.cols, a.nnz, byref(al),
                                           byref(descr), da.val.c_ptr(), da.row_ptr.c_ptr(), da.col.c_ptr(), dB.c_ptr(), n,
                                           byref(be), dC.c_ptr(), n)

    def verify(what):
        err = orc.csrmm_err(a, 1.25, B, 0.5, C0, dC.to_numpy().reshape(a.rows, n), ref)
        assert err.zero_den_mismatch == 0 and err.full <= TOL[a.dtype], (what, err)
    try:
        assert lib.asamd_handle_set_stream(h.h, stream) == 0
        announce("graph capture: first row-major csrmm of a matrix")
        hiprt.check(hip.hipStreamBeginCapture(stream, 0), "hipStreamBeginCapture")
        st = multiply()
        hiprt.check(hip.hipStreamEndCapture(stream, byref(graph)), "hipStreamEndCapture")
        assert st == 0
        hiprt.check(hip.hipGraphInstantiate(byref(gexec), graph, None, None, ctypes.c_size_t(0)), "hipGraphInstantiate")
        for replay in range(3):
            dC.copy_from(C0)
            hiprt.synchronize()
            hiprt.check(hip.hipGraphLaunch(gexec, stream), "hipGraphLaunch")
            hiprt.check(hip.hipStreamSynchronize(stream), "sync")
            verify("replay %d" % replay)
        dC.copy_from(C0)
        assert multiply() == 0                                   # eager: looks at the matrix first
        hiprt.check(hip.hipStreamSynchronize(stream), "sync")
        verify("eager after the capture")
    finally:
        if gexec:
            hip.hipGraphExecDestroy(gexec)
        if graph:
            hip.hipGraphDestroy(graph)
        h.close()
        hip.hipStreamDestroy(stream)
        for d in (dB, dC):
            d.free()
        da.free()
