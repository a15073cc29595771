"""Multiplies WITHOUT analysis (info == NULL, as the reference's own programs call csrmv,
test/dcu/level2/mv_csr_s_dcu_test.cpp:220-222) on arrays that keep coming back.  The reference reads the caller's
arrays on every call, so whatever the caller does to them between calls must show in the next result.  The
library may by then multiply through a tiled copy -- but only behind fingerprints of every byte of row_ptr,
col_ind and csr_val, taken on the device in front of every multiply.  Every result is compared with the CPU oracle
on what the arrays hold at that moment."""
import ctypes
from ctypes import byref, c_float, c_void_p

import numpy as np
import pytest

from alsparse_amd import capi, hiprt, workloads as wl
from helpers import DeviceCsr, announce, check_spmv

pytestmark = pytest.mark.gpu


def _with(a, values=None, col_ind=None):
    """The matrix a with other values and / or column indices (the arrays are not shared with a)."""
    return wl.Csr(a.rows, a.cols, a.row_ptr, a.col_ind.copy() if col_ind is None else col_ind,
                  a.values.copy() if values is None else values, a.base, a.name)


def _multiply(lib, h, descr, da, dx, dy, alpha, beta):
    a = da.a
    T = capi.scalar_type(a.dtype)
    al, be = T(alpha), T(beta)
    st = getattr(lib, "alphasparse_dcu_%s_csrmv" % capi.prefix(a.dtype))(
        h.h, 0, a.rows, a.cols, a.nnz, byref(al), byref(descr), da.val.c_ptr(), da.row_ptr.c_ptr(), da.col.c_ptr(),
        None, dx.c_ptr(), byref(be), dy.c_ptr())
    assert st == 0, "csrmv status %d" % st


def _promoted(lib, h, da):
    return lib.asamd_registry_lazy_promoted(h.h, da.row_ptr.c_ptr())


@pytest.mark.parametrize("base", [0, 1])
def test_returning_matrix_goes_through_a_watched_copy_and_every_edit_shows(gpu, base):
    lib = capi.load()
    a = wl.uniform_rows(1 << 21, 1 << 21, 16, np.float32, base=base)  # 8 MiB of x, scattered columns: the tiled copy's case
    x, y0 = wl.uniform(a.cols, a.dtype, 3), wl.uniform(a.rows, a.dtype, 4)
    da = DeviceCsr(a)
    dx, dy = hiprt.DeviceArray.from_numpy(x), hiprt.DeviceArray.from_numpy(y0)
    h = capi.Handle()
    descr = capi.make_descr(base=base)
    try:
        announce("no analysis: the same arrays four times, base", base)
        for call in range(1, 7):
            dy.copy_from(y0)
            _multiply(lib, h, descr, da, dx, dy, 1.5, 0.5)
            hiprt.synchronize()
            check_spmv(a, 1.5, x, 0.5, y0, dy.to_numpy(), "call %d" % call)
            assert _promoted(lib, h, da) == (1 if call >= 4 else 0), "call %d" % call

        announce("no analysis: ONE value poked in place under the watched copy")
        b = _with(a)
        b.values[12345677] = np.float32(37.25)
        da.val.copy_from(b.values)
        dy.copy_from(y0)
        _multiply(lib, h, descr, da, dx, dy, 1.5, 0.5)
        hiprt.synchronize()
        check_spmv(b, 1.5, x, 0.5, y0, dy.to_numpy(), "one value changed")
        assert _promoted(lib, h, da) == 1

        announce("no analysis: one column index changed in place under the watched copy")
        c = _with(b)
        row = 777777
        k = int(c.row_ptr[row]) - c.base
        taken = set(int(v) for v in c.col_ind[k:int(c.row_ptr[row + 1]) - c.base])
        new_col = next(v for v in range(c.base, c.base + c.cols) if v not in taken)
        c.col_ind[k] = new_col
        order = np.argsort(c.col_ind[k:k + 16], kind="stable")  # keep the row's columns ascending
        c.col_ind[k:k + 16] = c.col_ind[k:k + 16][order]
        c.values[k:k + 16] = c.values[k:k + 16][order]
        da.col.copy_from(c.col_ind)
        da.val.copy_from(c.values)
        for again in range(2):
            dy.copy_from(y0)
            _multiply(lib, h, descr, da, dx, dy, 1.5, 0.5)
            hiprt.synchronize()
            check_spmv(c, 1.5, x, 0.5, y0, dy.to_numpy(), "one column changed, call %d" % again)
        # the verdicts travel to the host behind the multiplies: after two of them the copy is given up
        dy.copy_from(y0)
        _multiply(lib, h, descr, da, dx, dy, 1.5, 0.5)
        hiprt.synchronize()
        check_spmv(c, 1.5, x, 0.5, y0, dy.to_numpy(), "after the copy was given up")
        assert _promoted(lib, h, da) == 0
    finally:
        h.close()
        for d in (dx, dy):
            d.free()
        da.free()


def test_watched_multiply_can_be_captured_and_replayed_over_changing_values(gpu):
    lib, hip = capi.load(), hiprt.lib()
    a = wl.uniform_rows(1 << 21, 1 << 21, 16, np.float32)
    x, y0 = wl.uniform(a.cols, a.dtype, 5), wl.uniform(a.rows, a.dtype, 6)
    da = DeviceCsr(a)
    dx, dy = hiprt.DeviceArray.from_numpy(x), hiprt.DeviceArray.from_numpy(y0)
    stream, graph, gexec = c_void_p(), c_void_p(), c_void_p()
    hiprt.check(hip.hipStreamCreate(byref(stream)), "hipStreamCreate")
    h = capi.Handle()
    descr = capi.make_descr()
    try:
        assert lib.asamd_handle_set_stream(h.h, stream) == 0
        for call in range(4):
            _multiply(lib, h, descr, da, dx, dy, 1.0, 0.0)
        hiprt.synchronize()
        assert _promoted(lib, h, da) == 1
        announce("graph capture: a multiply without analysis through the watched copy")
        hiprt.check(hip.hipStreamBeginCapture(stream, 0), "hipStreamBeginCapture")
        _multiply(lib, h, descr, da, dx, dy, 1.0, 0.0)
        hiprt.check(hip.hipStreamEndCapture(stream, byref(graph)), "hipStreamEndCapture")
        hiprt.check(hip.hipGraphInstantiate(byref(gexec), graph, None, None, ctypes.c_size_t(0)), "hipGraphInstantiate")
        cur = a
        for replay in range(3):
            if replay:  # new values at the same address between the replays, with the program's own work
                cur = _with(a, values=wl.uniform(a.nnz, a.dtype, 40 + replay))
                da.val.copy_from(cur.values)
            dy.fill_bytes(0)
            hiprt.check(hip.hipGraphLaunch(gexec, stream), "hipGraphLaunch")
            hiprt.check(hip.hipStreamSynchronize(stream), "hipStreamSynchronize")
            check_spmv(cur, 1.0, x, 0.0, y0, dy.to_numpy(), "replay %d" % replay)
    finally:
        if gexec:
            hip.hipGraphExecDestroy(gexec)
        if graph:
            hip.hipGraphDestroy(graph)
        h.close()
        hip.hipStreamDestroy(stream)
        for d in (dx, dy):
            d.free()
        da.free()


def test_matrices_that_a_copy_would_not_help_stay_on_their_own_arrays(gpu):
    lib = capi.load()
    h = capi.Handle()
    descr = capi.make_descr()
    try:
        for name, a in (("laplace", wl.laplace2d(2048, 2048, np.float64)),
                        ("small", wl.uniform_rows(1 << 16, 1 << 16, 16, np.float32))):
            x, y0 = wl.uniform(a.cols, a.dtype, 7), wl.uniform(a.rows, a.dtype, 8)
            da = DeviceCsr(a)
            dx, dy = hiprt.DeviceArray.from_numpy(x), hiprt.DeviceArray.from_numpy(y0)
            announce("no analysis, no copy:", name)
            for call in range(6):
                dy.copy_from(y0)
                _multiply(lib, h, descr, da, dx, dy, 2.0, 1.0)
            hiprt.synchronize()
            check_spmv(a, 2.0, x, 1.0, y0, dy.to_numpy(), name)
            assert _promoted(lib, h, da) == 0, name
            for d in (dx, dy):
                d.free()
            da.free()
    finally:
        h.close()


def test_alternating_value_arrays_are_never_promoted(gpu):
    lib = capi.load()
    a = wl.uniform_rows(1 << 21, 1 << 21, 16, np.float32)
    b = _with(a, values=wl.uniform(a.nnz, a.dtype, 90))
    x, y0 = wl.uniform(a.cols, a.dtype, 9), wl.uniform(a.rows, a.dtype, 10)
    da = DeviceCsr(a)
    other_val = hiprt.DeviceArray.from_numpy(b.values)
    dx, dy = hiprt.DeviceArray.from_numpy(x), hiprt.DeviceArray.from_numpy(y0)
    h = capi.Handle()
    descr = capi.make_descr()
    T = capi.scalar_type(a.dtype)
    try:
        announce("no analysis: two value arrays in turn over one structure")
        for call in range(8):
            which, vals = (a, da.val) if call % 2 == 0 else (b, other_val)
            dy.copy_from(y0)
            al, be = T(1.0), T(0.5)
            st = lib.alphasparse_dcu_s_csrmv(h.h, 0, a.rows, a.cols, a.nnz, byref(al), byref(descr), vals.c_ptr(),
                                             da.row_ptr.c_ptr(), da.col.c_ptr(), None, dx.c_ptr(), byref(be), dy.c_ptr())
            assert st == 0
            hiprt.synchronize()
            check_spmv(which, 1.0, x, 0.5, y0, dy.to_numpy(), "call %d" % call)
            assert _promoted(lib, h, da) == 0
    finally:
        h.close()
        for d in (dx, dy, other_val):
            d.free()
        da.free()
