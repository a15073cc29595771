"""Device memory over a plan's life: whatever a plan lays out (tiled copy, hot-column table, ELL copy, binned rows,
column-slice offsets and copy, 16-bit column numbers and distances, the transposed copy) goes back to the device when the plan is destroyed, and a second analysis
of the same arrays replaces the first one's memory instead of adding to it.  The reference frees its analysis in
alphasparse_dcu_csrmv_clear (src/util_cpp/alphasparse_dcu_x_csrmv_analysis.cpp:393-414)."""
from ctypes import byref, c_void_p

import numpy as np
import pytest

from alsparse_amd import capi, hiprt, workloads as wl
from helpers import ALGOS, DeviceCsr, announce, check_spmv

pytestmark = pytest.mark.gpu

SLACK = 4 << 20  # bytes the runtime may keep for itself between two readings
ROUNDS = 8


def _no_growth(free_after_round, what):
    """The runtime hands freed memory back with some delay, so a single reading may be low; a leak, though, lowers
    EVERY later reading: the best of the last three rounds is compared with the best of the first three."""
    early, late = max(free_after_round[:3]), max(free_after_round[-3:])
    assert early - late < SLACK, "%s: %d bytes of device memory gone over %d rounds (free after each: %s)" % (
        what, early - late, len(free_after_round), free_after_round)


_best_free = [0]


def _free_bytes():
    """Free device memory once the runtime has caught up: it hands freed blocks back with some delay (a reading taken
    right after a free can be hundreds of MB low and recover by itself), so a reading below the best one seen is
    taken again for up to two seconds, with a small allocation in between to make the runtime look at its lists."""
    import time
    free = 0
    for _ in range(40):
        hiprt.synchronize()
        free = max(free, hiprt.mem_info()[0])
        if free >= _best_free[0] - SLACK:
            break
        hiprt.DeviceArray(256, "uint8").free()
        time.sleep(0.05)
    return free


def _cycle(lib, da, algo, x, y0, check):
    a = da.a
    plan = c_void_p()
    assert lib.asamd_csr_plan_create(None, a.rows, a.cols, a.nnz, da.row_ptr.c_ptr(), da.col.c_ptr(), da.val.c_ptr(),
                                     a.base, a.dtype.itemsize, 2, byref(plan)) == 0
    try:
        if lib.asamd_csr_plan_set_algo(plan, ALGOS[algo.split("_")[0]]) != 0:
            return False
        T = capi.scalar_type(a.dtype)
        dx, dy = hiprt.DeviceArray.from_numpy(x), hiprt.DeviceArray.from_numpy(y0)
        ws = capi.Workspace(lib, plan)
        for trans in (0, 1):
            if trans and a.rows != a.cols:
                continue
            assert capi.plan_csrmv(lib, None, plan, trans, T(1.0), da.val.c_ptr(), da.row_ptr.c_ptr(), da.col.c_ptr(),
                                   dx.c_ptr(), T(0.0), dy.c_ptr(), ws) == 0
            hiprt.synchronize()
            if check and not trans:
                check_spmv(a, 1.0, x, 0.0, y0, dy.to_numpy(), algo)
        for d in (dx, dy, ws.buf):
            d.free()
        return True
    finally:
        lib.asamd_csr_plan_destroy(plan)


CASES = [
    ("tiled", lambda: wl.uniform_rows(1 << 20, 1 << 20, 16, np.float32)),
    ("hot", lambda: wl.uniform_rows(1 << 20, 1 << 20, 16, np.float32)),
    ("ell", lambda: wl.uniform_rows(1 << 20, 1 << 20, 8, np.float64)),
    ("binned", lambda: wl.uniform_rows(1 << 20, 1 << 20, 8, np.float32)),
    ("xlds", lambda: wl.uniform_rows(1 << 18, 1 << 17, 64, np.float32)),  # four column slices (512 KB of x)
    ("merge", lambda: wl.uniform_rows(1 << 20, 1 << 20, 16, np.float32)),
    ("xlds_one_slice", lambda: wl.uniform_rows(1 << 20, 1 << 15, 16, np.float32)),  # 16-bit column numbers
    ("stream", lambda: wl.stencil3d(96, 96, 96, np.float32)),  # 16-bit column distances
]


@pytest.mark.parametrize("algo,make", CASES, ids=[c[0] for c in CASES])
def test_destroyed_plans_give_their_memory_back(gpu, algo, make):
    lib = capi.load()
    a = make()
    x, y0 = wl.uniform(a.cols, a.dtype, 3), wl.uniform(a.rows, a.dtype, 4)
    da = DeviceCsr(a)
    try:
        announce("lifecycle: first plan", algo)
        if not _cycle(lib, da, algo, x, y0, check=True):
            pytest.skip("this structure cannot run " + algo)
        readings = []
        _best_free[0] = _free_bytes()
        for i in range(ROUNDS):
            announce("lifecycle: plan", i + 2, algo)
            _cycle(lib, da, algo, x, y0, check=False)
            readings.append(_free_bytes())
        _no_growth(readings, algo)
    finally:
        da.free()


def test_analysing_again_and_clearing_returns_the_memory(gpu):
    """The reference's calls: analysis, multiply, analysis again on the same arrays, clear -- four times over."""
    lib = capi.load()
    a = wl.uniform_rows(1 << 20, 1 << 20, 16, np.float32)
    x, y0 = wl.uniform(a.cols, a.dtype, 3), wl.uniform(a.rows, a.dtype, 4)
    da = DeviceCsr(a)
    descr = capi.make_descr(base=a.base)
    T = capi.scalar_type(a.dtype)
    al, be = T(1.0), T(0.0)
    dx, dy = hiprt.DeviceArray.from_numpy(x), hiprt.DeviceArray.from_numpy(y0)

    def round_trip(check):
        info = capi.alphasparse_dcu_mat_info_t()
        assert lib.alphasparse_dcu_create_mat_info(byref(info)) == 0
        for _ in range(2):
            assert lib.alphasparse_dcu_s_csrmv_analysis(gpu.h, 0, a.rows, a.cols, a.nnz, byref(descr), da.val.c_ptr(),
                                                        da.row_ptr.c_ptr(), da.col.c_ptr(), info) == 0
            assert lib.alphasparse_dcu_s_csrmv(gpu.h, 0, a.rows, a.cols, a.nnz, byref(al), byref(descr),
                                               da.val.c_ptr(), da.row_ptr.c_ptr(), da.col.c_ptr(), info, dx.c_ptr(),
                                               byref(be), dy.c_ptr()) == 0
            hiprt.synchronize()
            if check:
                check_spmv(a, 1.0, x, 0.0, y0, dy.to_numpy(), "analysed")
        assert lib.alphasparse_dcu_csrmv_clear(gpu.h, info) == 0
        assert lib.alphasparse_dcu_destroy_mat_info(info) == 0

    try:
        announce("lifecycle: analysis twice, clear")
        round_trip(True)
        readings = []
        _best_free[0] = _free_bytes()
        for i in range(ROUNDS):
            announce("lifecycle: analysis twice, clear; round", i + 2)
            round_trip(False)
            readings.append(_free_bytes())
        _no_growth(readings, "analysis twice, clear")
    finally:
        for d in (dx, dy):
            d.free()
        da.free()
