"""The staged row-block kernel reading 16-bit column distances: for a structure that stays (an analysis) and a matrix
whose entries all lie within 32 767 columns of the first row of their workgroup -- discretisations, bands -- the
columns are kept once as distances from that row, 2 instead of 4 index bytes per entry.  The reference has one kernel
for every shape (src/kernel/dcu/level2/mv/csrmv/dcu_gemv_vector.h:14-57); results are compared with the CPU oracle."""
from ctypes import byref, c_void_p

import numpy as np
import pytest

from alsparse_amd import capi, hiprt, workloads as wl
from helpers import ALGOS, DeviceCsr, announce, check_spmv, run_csrmv
from helpers_shapes import csr_from_lengths

pytestmark = pytest.mark.gpu


def _forced_stream(da, x, y0, alpha, beta):
    """(y, device bytes the plan keeps): a plan that lays out everything it can, the staged kernel forced."""
    a = da.a
    lib = capi.load()
    plan = c_void_p()
    assert lib.asamd_csr_plan_create(None, a.rows, a.cols, a.nnz, da.row_ptr.c_ptr(), da.col.c_ptr(), da.val.c_ptr(),
                                     a.base, a.dtype.itemsize, 2, byref(plan)) == 0
    try:
        if lib.asamd_csr_plan_set_algo(plan, ALGOS["stream"]) != 0:
            return None, 0
        kept = lib.asamd_csr_plan_stats(plan).contents.device_bytes
        T = capi.scalar_type(a.dtype)
        dx, dy = hiprt.DeviceArray.from_numpy(x), hiprt.DeviceArray.from_numpy(y0)
        ws = capi.Workspace(lib, plan)
        assert capi.plan_csrmv(lib, None, plan, 0, T(alpha), da.val.c_ptr(), da.row_ptr.c_ptr(), da.col.c_ptr(),
                               dx.c_ptr(), T(beta), dy.c_ptr(), ws) == 0
        hiprt.synchronize()
        y = dy.to_numpy()
        for d in (dx, dy, ws.buf):
            d.free()
        return y, kept
    finally:
        lib.asamd_csr_plan_destroy(plan)


def _band(m, n, lengths, reach, dtype, seed, base):
    """Rows of the given lengths whose columns lie within `reach` of the row number (clipped to the matrix)."""
    rng = np.random.default_rng(seed)
    row_ptr = np.zeros(m + 1, dtype=np.int64)
    np.cumsum(lengths, out=row_ptr[1:])
    cols = np.empty(int(row_ptr[-1]), dtype=np.int64)
    for r in range(m):
        lo, hi = max(0, r - reach), min(n, r + reach + 1)
        k = int(lengths[r])
        cols[row_ptr[r]:row_ptr[r + 1]] = np.sort(rng.choice(np.arange(lo, hi), size=k, replace=False))
    return wl.Csr(m, n, (row_ptr + base).astype(np.int32), (cols + base).astype(np.int32),
                  wl.uniform(int(row_ptr[-1]), dtype, 7, seed), base, "band")


@pytest.mark.parametrize("dtype", [np.float32, np.float64], ids=["f32", "f64"])
@pytest.mark.parametrize("base", [0, 1])
@pytest.mark.parametrize("longest", [3, 14, 40, 120])
def test_bands_of_every_row_length_through_the_distances(gpu, dtype, base, longest, monkeypatch):
    """Rows of 0 .. longest entries (one lane per row up to sixteen lanes per row), columns on both sides of the
    diagonal, a last workgroup that ends inside the matrix, both index bases; with the distances and (the same
    matrix, ALSPARSE_AMD_STREAM_NARROW=0) without."""
    rng = np.random.default_rng(longest * 7 + base)
    m = 5000 + longest
    lengths = rng.integers(0, longest + 1, size=m)
    lengths[:4] = [0, longest, 1, longest]
    a = _band(m, m + 37, lengths, 300, dtype, 11 + longest, base)
    x, y0 = wl.uniform(a.cols, a.dtype, 3), wl.uniform(a.rows, a.dtype, 4)
    da = DeviceCsr(a)
    try:
        for alpha, beta in ((1.0, 0.0), (-1.5, 0.5)):
            announce("stream, 16-bit distances:", np.dtype(dtype).name, "base", base, "longest", longest, alpha, beta)
            y, kept = _forced_stream(da, x, y0, alpha, beta)
            assert y is not None
            check_spmv(a, alpha, x, beta, y0, y, "distances %s" % ((alpha, beta),))
        monkeypatch.setenv("ALSPARSE_AMD_STREAM_NARROW", "0")
        y, kept_without = _forced_stream(da, x, y0, 1.0, 0.0)
        check_spmv(a, 1.0, x, 0.0, y0, y, "column numbers")
        assert kept - kept_without >= 2 * a.nnz, "the plan kept no 16-bit distances"
    finally:
        da.free()


def test_an_entry_too_far_from_its_row_keeps_the_column_numbers(gpu):
    """One entry 40 000 columns from its row: no distances (they would not fit 16 bits), same results."""
    m = 60000
    a = _band(m, m, np.full(m, 5), 50, np.float32, 3, 0)
    cols = a.col_ind.copy()
    k = int(a.row_ptr[100])  # row 100's first entry moves far to the right, behind the row's other entries
    row = np.sort(np.concatenate([cols[k + 1:k + 5], [40100]]))
    cols[k:k + 5] = row
    b = wl.Csr(m, m, a.row_ptr, cols, a.values, 0, "one far entry")
    x, y0 = wl.uniform(m, np.float32, 3), wl.uniform(m, np.float32, 4)
    da, db = DeviceCsr(a), DeviceCsr(b)
    try:
        announce("stream: all entries near")
        ya, kept_near = _forced_stream(da, x, y0, 1.0, 0.0)
        announce("stream: one entry too far")
        yb, kept_far = _forced_stream(db, x, y0, 1.0, 0.0)
        check_spmv(a, 1.0, x, 0.0, y0, ya, "near")
        check_spmv(b, 1.0, x, 0.0, y0, yb, "far")
        assert kept_near - kept_far >= 2 * a.nnz, (kept_near, kept_far)
    finally:
        da.free()
        db.free()


def test_analysed_stencil_beyond_the_cache_reads_distances(gpu, monkeypatch):
    """27-point stencil on 128^3 points, fp64 (56 M entries, 0.7 GB): the analysis keeps the staged kernel and makes
    the distances by itself; new values in place need nothing (the values are read from the caller's array)."""
    lib = capi.load()
    a = wl.stencil3d(128, 128, 128, np.float64)
    x, y0 = wl.uniform(a.cols, a.dtype, 3), wl.uniform(a.rows, a.dtype, 4)
    da = DeviceCsr(a)
    descr = capi.make_descr(base=a.base)

    def analysed():
        info = capi.alphasparse_dcu_mat_info_t()
        assert lib.alphasparse_dcu_create_mat_info(byref(info)) == 0
        assert lib.alphasparse_dcu_d_csrmv_analysis(gpu.h, 0, a.rows, a.cols, a.nnz, byref(descr), da.val.c_ptr(),
                                                    da.row_ptr.c_ptr(), da.col.c_ptr(), info) == 0
        return info

    info = None
    try:
        announce("stream, 16-bit distances: analysed stencil")
        info = analysed()
        st = lib.asamd_analysis_stats(info).contents
        assert st.algo == capi.ASAMD_SPMV_STREAM, st.algo
        assert 2 * a.nnz <= st.device_bytes < 3 * a.nnz, "distances, and no copy of the values"
        check_spmv(a, 1.5, x, 0.5, y0, run_csrmv(gpu, da, 1.5, x, 0.5, y0, info=info), "stencil")
        b = wl.Csr(a.rows, a.cols, a.row_ptr, a.col_ind, wl.uniform(a.nnz, a.dtype, 21), a.base, a.name)
        da.val.copy_from(b.values)
        check_spmv(b, 1.0, x, 0.0, y0, run_csrmv(gpu, da, 1.0, x, 0.0, y0, info=info), "stencil, new values in place")
        lib.alphasparse_dcu_destroy_mat_info(info)
        info = None
        monkeypatch.setenv("ALSPARSE_AMD_STREAM_NARROW", "0")
        info = analysed()
        assert lib.asamd_analysis_stats(info).contents.device_bytes < 2 * a.nnz or \
            lib.asamd_analysis_stats(info).contents.algo != capi.ASAMD_SPMV_STREAM
    finally:
        if info is not None:
            lib.alphasparse_dcu_destroy_mat_info(info)
        da.free()


@pytest.mark.parametrize("dtype", [np.float32, np.float64], ids=["f32", "f64"])
def test_large_laplacian_takes_the_non_temporal_forms(gpu, dtype):
    """5-point Laplacian on 4096 x 4096 points (84 M entries): large enough for the cache policies that small
    matrices never see -- 4-byte values and their distances past the caches, 8-byte values with y past the caches."""
    lib = capi.load()
    a = wl.laplace2d(4096, 4096, dtype)
    x, y0 = wl.uniform(a.cols, a.dtype, 3), wl.uniform(a.rows, a.dtype, 4)
    da = DeviceCsr(a)
    descr = capi.make_descr(base=a.base)
    info = capi.alphasparse_dcu_mat_info_t()
    assert lib.alphasparse_dcu_create_mat_info(byref(info)) == 0
    try:
        announce("stream, 16-bit distances: large Laplacian", np.dtype(dtype).name)
        assert getattr(lib, "alphasparse_dcu_%s_csrmv_analysis" % capi.prefix(a.dtype))(
            gpu.h, 0, a.rows, a.cols, a.nnz, byref(descr), da.val.c_ptr(), da.row_ptr.c_ptr(), da.col.c_ptr(), info) == 0
        st = lib.asamd_analysis_stats(info).contents
        assert st.algo == capi.ASAMD_SPMV_STREAM and st.device_bytes >= 2 * a.nnz, (st.algo, st.device_bytes)
        for alpha, beta in ((1.0, 0.0), (1.5, 0.5)):
            check_spmv(a, alpha, x, beta, y0, run_csrmv(gpu, da, alpha, x, beta, y0, info=info), "laplace %s" % ((alpha, beta),))
    finally:
        lib.alphasparse_dcu_destroy_mat_info(info)
        da.free()
