"""asamd_s_csrmv_noalloc: the multiply that allocates nothing (its merge-path scratch is a fixed device
array) against the existing entry points, through the C-ABI.

Bar: y within 1e-4 per row of the plain-kernel oracle (normalised by |alpha| sum|a x| + |beta y0|; by the products alone when beta == 0),
and bit-equal to asamd_csr_plan_csrmv running the same merge-path kernels in a caller-provided workspace.
Two calls in a row share the array; the second is smaller, so slots the first call wrote stay behind."""
from ctypes import byref, c_float, c_void_p

import numpy as np
import pytest

from alsparse_amd import capi, hiprt, workloads as wl
from helpers import DeviceCsr, announce, check_spmv, csr_from_lengths, run_csrmv, run_plan_csrmv

pytestmark = pytest.mark.gpu

MAX_ITEMS = 536868864  # ASAMD_CSRMV_NOALLOC_MAX_ITEMS


def _noalloc(da, alpha, x, beta, y0):
    a = da.a
    lib = capi.load()
    dx = hiprt.DeviceArray.from_numpy(np.ascontiguousarray(x, dtype=np.float32))
    dy = hiprt.DeviceArray.from_numpy(np.ascontiguousarray(y0, dtype=np.float32))
    hiprt.synchronize()
    free_before, _ = hiprt.mem_info()
    e = lib.asamd_s_csrmv_noalloc(None, a.rows, a.cols, a.nnz, a.base, c_float(alpha), da.val.c_ptr(),
                                  da.row_ptr.c_ptr(), da.col.c_ptr(), dx.c_ptr(), c_float(beta), dy.c_ptr())
    assert e == 0, "asamd_s_csrmv_noalloc hip error %d" % e
    hiprt.synchronize()
    free_after, _ = hiprt.mem_info()
    y = dy.to_numpy()
    dx.free()
    dy.free()
    return y, free_before - free_after


def test_noalloc_matches_existing_entry_points_on_two_calls_in_a_row(gpu):
    big = wl.powerlaw_rmat(15, 200000, np.float32)           # skewed rows, rows spanning many workgroups
    small = csr_from_lengths([0, 0, 5, 0, 3000, 0, 0, 1, 1, 0, 64, 65, 0] * 3, 5000, np.float32, base=1)
    tiny = csr_from_lengths([3], 10, np.float32)              # a single workgroup: no fix-up launch
    grew = []
    for k, (a, alpha, beta) in enumerate(((big, 1.25, 0.5), (small, -0.75, 3.0), (tiny, 2.0, 0.0), (big, 1.0, 0.0))):
        x = wl.uniform(a.cols, a.dtype, 3)
        y0 = wl.uniform(a.rows, a.dtype, 4)
        da = DeviceCsr(a)
        try:
            announce("noalloc", k, a.name, alpha, beta)
            y, used = _noalloc(da, alpha, x, beta, y0)
            grew.append(used)
            check_spmv(a, alpha, x, beta, y0, y, "noalloc/%s" % a.name)
            # the same kernels from a plan's own buffers: bit for bit
            y_plan = run_plan_csrmv(da, "merge", alpha, x, beta, y0)
            assert np.array_equal(y.view(np.uint32), y_plan.view(np.uint32)), "call %d differs from the planned merge path" % k
            # and the public raw-pointer entry point (whatever kernel it picks) to the parity tolerance
            y_api = run_csrmv(gpu, da, alpha, x, beta, y0)
            check_spmv(a, alpha, x, beta, y0, y_api, "api/%s" % a.name)
        finally:
            da.free()
    # after the first call (code objects loaded) the device's free memory does not move across a call
    assert all(u == 0 for u in grew[1:]), grew


def test_noalloc_zero_entries_scales_y(gpu):
    a = csr_from_lengths([0] * 777, 50, np.float32)
    y0 = wl.uniform(a.rows, a.dtype, 4)
    x = wl.uniform(a.cols, a.dtype, 3)
    da = DeviceCsr(a)
    try:
        announce("noalloc nnz=0")
        y, _ = _noalloc(da, 2.0, x, 0.5, y0)
        assert np.array_equal(y, y0 * np.float32(0.5))
        y, _ = _noalloc(da, 2.0, x, 0.0, np.full(a.rows, np.nan, np.float32))
        assert np.array_equal(y, np.zeros(a.rows, np.float32))
    finally:
        da.free()


def test_noalloc_refuses_what_the_fixed_array_cannot_hold(gpu):
    lib = capi.load()
    d = hiprt.DeviceArray((16,), np.float32)
    p = d.c_ptr()
    # rejected before anything is read or launched: the pointers only have to be non-null
    m, nnz = 2 ** 29, 2 ** 29
    assert m + nnz > MAX_ITEMS
    assert lib.asamd_s_csrmv_noalloc(None, m, m, nnz, 0, c_float(1), p, p, p, p, c_float(0), p) == 2  # hipErrorOutOfMemory
    # bad arguments
    assert lib.asamd_s_csrmv_noalloc(None, 0, 4, 4, 0, c_float(1), p, p, p, p, c_float(0), p) == 1   # hipErrorInvalidValue
    assert lib.asamd_s_csrmv_noalloc(None, 4, 4, 4, 2, c_float(1), p, p, p, p, c_float(0), p) == 1
    assert lib.asamd_s_csrmv_noalloc(None, 4, 4, 4, 0, c_float(1), p, None, p, p, c_float(0), p) == 1
    hiprt.synchronize()
    d.free()
