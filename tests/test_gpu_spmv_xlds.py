"""Matrices of few columns: x larger than the 32 KB L1 and small enough for a compute unit's LDS (160 KB at most).
The library then multiplies with one persistent workgroup per compute unit that holds x in LDS and reads the CSR
arrays in place -- with or without an analysis, since nothing is kept.  The reference has one kernel for every
shape (src/kernel/dcu/level2/mv/csrmv/dcu_gemv_vector.h:14-57); results are compared with the CPU oracle."""
from ctypes import byref, c_void_p

import numpy as np
import pytest

from alsparse_amd import capi, hiprt, workloads as wl
from helpers import DeviceCsr, announce, check_spmv, run_csrmv
from helpers_shapes import csr_from_lengths

pytestmark = pytest.mark.gpu


def _plan_algo(lib, da, trusted=1):
    a = da.a
    plan = c_void_p()
    assert lib.asamd_csr_plan_create(None, a.rows, a.cols, a.nnz, da.row_ptr.c_ptr(), da.col.c_ptr(), da.val.c_ptr(),
                                     a.base, a.dtype.itemsize, trusted, byref(plan)) == 0
    algo = lib.asamd_csr_plan_stats(plan).contents.algo
    lib.asamd_csr_plan_destroy(plan)
    return algo


@pytest.mark.parametrize("dtype,cols", [(np.float32, 20000), (np.float32, 32768), (np.float64, 16384)],
                         ids=["f32_20000", "f32_32768", "f64_16384"])
def test_tall_matrix_is_multiplied_with_x_in_lds(gpu, dtype, cols, monkeypatch):
    lib = capi.load()
    a = wl.uniform_rows(300000, cols, 16, dtype)  # 4.8 M entries, scattered columns
    x, y0 = wl.uniform(a.cols, a.dtype, 3), wl.uniform(a.rows, a.dtype, 4)
    da = DeviceCsr(a)
    try:
        announce("x in LDS: the analysis' choice", np.dtype(dtype).name, cols)
        assert _plan_algo(lib, da) == capi.ASAMD_SPMV_XLDS
        monkeypatch.setenv("ALSPARSE_AMD_XLDS", "0")
        assert _plan_algo(lib, da) != capi.ASAMD_SPMV_XLDS
        monkeypatch.delenv("ALSPARSE_AMD_XLDS")
        announce("x in LDS: multiply without analysis", np.dtype(dtype).name, cols)
        for alpha, beta in ((1.0, 0.0), (-0.5, 2.0)):
            y = run_csrmv(gpu, da, alpha, x, beta, y0)
            check_spmv(a, alpha, x, beta, y0, y, "no analysis %s" % ((alpha, beta),))
        assert lib.asamd_analysis_stats(da.row_ptr.c_ptr()).contents.algo == capi.ASAMD_SPMV_XLDS
    finally:
        da.free()


def test_columns_that_neighbours_share_keep_the_plain_kernel(gpu):
    """A band: the gathers of a wave fall into a few cache lines, and the row kernels are as fast from the caches."""
    lib = capi.load()
    m, n, per_row = 300000, 30000, 16
    rows = np.repeat(np.arange(m, dtype=np.int64), per_row)
    cols = (rows * n // m + np.tile(np.arange(per_row, dtype=np.int64), m)) % n
    order = np.lexsort((cols, rows))
    a = wl.Csr(m, n, np.arange(0, m * per_row + 1, per_row, dtype=np.int32), cols[order].astype(np.int32),
               wl.uniform(m * per_row, np.float32, 9), 0, "band")
    da = DeviceCsr(a)
    try:
        announce("x in LDS: a banded matrix keeps its row kernel")
        assert _plan_algo(lib, da) != capi.ASAMD_SPMV_XLDS
    finally:
        da.free()


def test_rows_of_every_length_and_both_bases(gpu):
    """Rows for the lane groups, rows for the whole wave (more than eight entries per lane), empty rows, a last
    trip that ends inside the matrix, index base one; the family forced on a matrix below its size threshold."""
    from helpers import run_plan_csrmv
    rng = np.random.default_rng(77)
    lengths = rng.integers(0, 40, size=9000)
    lengths[rng.integers(0, 9000, size=60)] = rng.integers(129, 6000, size=60)
    lengths[:17] = [0, 1, 127, 128, 129, 5999, 0, 0, 64, 65, 1023, 1024, 1025, 16, 17, 15, 6000]
    for dtype in (np.float32, np.float64):
        for base in (0, 1):
            a = csr_from_lengths(list(lengths), 6000, dtype, seed=5 + base, base=base)
            x, y0 = wl.uniform(a.cols, a.dtype, 3), wl.uniform(a.rows, a.dtype, 4)
            da = DeviceCsr(a)
            try:
                for alpha, beta in ((1.0, 0.0), (2.0, -1.0)):
                    announce("x in LDS: ragged rows", np.dtype(dtype).name, "base", base, alpha, beta)
                    y = run_plan_csrmv(da, "xlds", alpha, x, beta, y0)
                    assert y is not None
                    check_spmv(a, alpha, x, beta, y0, y, "ragged base %d %s" % (base, (alpha, beta)))
            finally:
                da.free()


SLICED = {
    # 2 slices of fp32 columns, pieces of 150 entries; 20 M entries (the slices carry a fixed cost of some 20 us per
    # multiply: smaller matrices keep merge-path)
    "f32_70000": lambda: wl.uniform_rows(65536, 70000, 300, np.float32),
    # 4 slices of fp64 columns, index base one
    "f64_80000_base1": lambda: wl.uniform_rows(100000, 80000, 250, np.float64, base=1),
}


@pytest.mark.parametrize("copy", ["copy", "in_place"])
@pytest.mark.parametrize("shape", sorted(SLICED))
def test_long_rows_over_several_lds_fills_of_x_go_slice_by_slice(gpu, shape, copy, monkeypatch):
    """x of 280 / 640 KB (two / four LDS fills) under rows of hundreds of entries: the analysis lays out a table of offsets (where every
    row's piece of every column slice begins) and the multiply runs a row of workgroups per slice -- over a copy of
    the entries slice by slice, which the value guard brings up to date when the caller's values change in place,
    or (ALSPARSE_AMD_XLDS_COPY=0) over the caller's arrays."""
    if copy == "in_place":
        monkeypatch.setenv("ALSPARSE_AMD_XLDS_COPY", "0")
    lib = capi.load()
    a = SLICED[shape]()
    x, y0 = wl.uniform(a.cols, a.dtype, 3), wl.uniform(a.rows, a.dtype, 4)
    da = DeviceCsr(a)
    info = capi.alphasparse_dcu_mat_info_t()
    assert lib.alphasparse_dcu_create_mat_info(byref(info)) == 0
    descr = capi.make_descr(base=a.base)
    p = capi.prefix(a.dtype)
    try:
        announce("x in LDS, sliced: analysis", shape)
        assert getattr(lib, "alphasparse_dcu_%s_csrmv_analysis" % p)(
            gpu.h, 0, a.rows, a.cols, a.nnz, byref(descr), da.val.c_ptr(), da.row_ptr.c_ptr(), da.col.c_ptr(), info) == 0
        st = lib.asamd_analysis_stats(info).contents
        assert st.algo == capi.ASAMD_SPMV_XLDS and st.xlds_slices >= 2, (st.algo, st.xlds_slices)
        table = (st.xlds_slices + 1) * a.rows * 4
        if copy == "copy":
            assert st.device_bytes > table + a.nnz * (a.dtype.itemsize + 2), "no copy of the entries was laid out"
        else:
            assert st.device_bytes < table + a.nnz, "a copy was laid out against ALSPARSE_AMD_XLDS_COPY=0"
        for alpha, beta in ((1.0, 0.0), (-0.5, 2.0)):
            announce("x in LDS, sliced: multiply", shape, copy, alpha, beta)
            y = run_csrmv(gpu, da, alpha, x, beta, y0, info=info)
            check_spmv(a, alpha, x, beta, y0, y, "%s %s" % (shape, (alpha, beta)))
        announce("x in LDS, sliced: new values in place", shape)
        b = wl.Csr(a.rows, a.cols, a.row_ptr, a.col_ind, wl.uniform(a.nnz, a.dtype, 21), a.base, a.name)
        da.val.copy_from(b.values)
        y = run_csrmv(gpu, da, 2.0, x, 0.0, y0, info=info)
        check_spmv(b, 2.0, x, 0.0, y0, y, "%s new values" % shape)
        monkeypatch.setenv("ALSPARSE_AMD_XLDS", "0")
        assert _plan_algo(lib, da) != capi.ASAMD_SPMV_XLDS
    finally:
        lib.alphasparse_dcu_destroy_mat_info(info)
        da.free()


def test_rows_whose_columns_do_not_ascend_get_no_slices(gpu):
    lib = capi.load()
    a = wl.uniform_rows(65536, 70000, 300, np.float32)
    da = DeviceCsr(a)
    try:
        announce("x in LDS, sliced: the same matrix with ascending columns")
        assert _plan_algo(lib, da) == capi.ASAMD_SPMV_XLDS
    finally:
        da.free()
    cols = a.col_ind.copy()
    cols[5:7] = cols[5:7][::-1]  # one pair out of order in row 0
    b = wl.Csr(a.rows, a.cols, a.row_ptr, cols, a.values, a.base, "unsorted")
    da = DeviceCsr(b)
    try:
        announce("x in LDS, sliced: unsorted columns")
        assert _plan_algo(lib, da) != capi.ASAMD_SPMV_XLDS
        x, y0 = wl.uniform(b.cols, b.dtype, 3), wl.uniform(b.rows, b.dtype, 4)
        y = run_csrmv(gpu, da, 1.0, x, 0.0, y0)
        check_spmv(b, 1.0, x, 0.0, y0, y, "unsorted")
    finally:
        da.free()


@pytest.mark.parametrize("copy", ["copy", "in_place"])
@pytest.mark.parametrize("seed", range(10))
def test_random_structures_slice_by_slice(gpu, seed, copy, monkeypatch):
    """Seeded random structures over 2 .. 7 column slices: empty rows, rows that miss whole slices, rows of thousands
    of entries, both index bases, both real types, val / col_ind off their 16-byte alignment; over the copy of the
    entries slice by slice and over the caller's arrays."""
    from helpers import run_plan_csrmv
    if copy == "in_place":
        monkeypatch.setenv("ALSPARSE_AMD_XLDS_COPY", "0")
    rng = np.random.default_rng(4200 + seed)
    dtype = (np.float32, np.float64)[seed % 2]
    fill = 163840 // np.dtype(dtype).itemsize
    cols = int(rng.integers(fill + 1, 7 * fill))
    m = int(rng.integers(1, 4000))
    law = seed % 3
    if law == 0:
        lengths = rng.integers(0, 200, size=m)
    elif law == 1:
        lengths = rng.geometric(1.0 / 40.0, size=m) - 1
    else:
        lengths = rng.integers(0, 12, size=m)
        lengths[rng.integers(0, m, size=max(1, m // 100))] = rng.integers(1000, 9000)
    base = int(rng.integers(0, 2))
    a = csr_from_lengths(list(np.minimum(lengths, cols)), cols, dtype, seed=int(rng.integers(1, 1 << 30)), base=base)
    if a.nnz < 4:
        pytest.skip("drew a matrix of fewer than four entries")
    x, y0 = wl.uniform(a.cols, a.dtype, 3, seed), wl.uniform(a.rows, a.dtype, 4, seed)
    da = DeviceCsr(a, shift=int(rng.integers(0, 4)))
    try:
        for alpha, beta in ((1.0, 0.0), (2.0, 3.0)):
            announce("x in LDS, sliced: random structure", seed, copy, np.dtype(dtype).name, "cols", cols, "base", base,
                     alpha, beta)
            y = run_plan_csrmv(da, "xlds", alpha, x, beta, y0)
            assert y is not None, "no slice table for a matrix with ascending columns"
            check_spmv(a, alpha, x, beta, y0, y, "seed %d %s" % (seed, (alpha, beta)))
    finally:
        da.free()


def test_the_copy_follows_the_values(gpu):
    """The slice-by-slice copy holds values: a multiply with ANOTHER value array (same structure) must not see them
    (it runs over that array through the table of offsets), asamd_csr_plan_refresh_values re-bases the copy on the
    new array, and pieces of every length -- none, one entry, more than a lane group's loads -- come out right."""
    lib = capi.load()
    rng = np.random.default_rng(99)
    m, cols = 3000, 100000  # three fp32 slices
    lengths = rng.integers(0, 60, size=m)
    lengths[:8] = [0, 1, 2, 3, 4, 5, 20000, 9000]
    a = csr_from_lengths(list(lengths), cols, np.float32, seed=8, base=1)
    x, y0 = wl.uniform(a.cols, a.dtype, 3), wl.uniform(a.rows, a.dtype, 4)
    da = DeviceCsr(a)
    other = wl.uniform(a.nnz, a.dtype, 31)
    b = wl.Csr(a.rows, a.cols, a.row_ptr, a.col_ind, other, a.base, "other values")
    d_other = hiprt.DeviceArray.from_numpy(other)
    plan = c_void_p()
    assert lib.asamd_csr_plan_create(None, a.rows, a.cols, a.nnz, da.row_ptr.c_ptr(), da.col.c_ptr(), da.val.c_ptr(),
                                     a.base, a.dtype.itemsize, 2, byref(plan)) == 0
    T = capi.scalar_type(a.dtype)
    dx, dy = hiprt.DeviceArray.from_numpy(x), hiprt.DeviceArray.from_numpy(y0)
    try:
        assert lib.asamd_csr_plan_set_algo(plan, capi.ASAMD_SPMV_XLDS) == 0
        assert lib.asamd_csr_plan_stats(plan).contents.device_bytes > a.nnz * 6, "no copy of the entries"
        ws = capi.Workspace(lib, plan)

        def multiply(val, want, what):
            announce("x in LDS, sliced copy:", what)
            dy.copy_from(y0)
            assert capi.plan_csrmv(lib, None, plan, 0, T(1.5), val.c_ptr(), da.row_ptr.c_ptr(), da.col.c_ptr(),
                                   dx.c_ptr(), T(0.5), dy.c_ptr(), ws) == 0
            hiprt.synchronize()
            check_spmv(want, 1.5, x, 0.5, y0, dy.to_numpy(), what)

        multiply(da.val, a, "the array the copy was taken from")
        multiply(d_other, b, "another value array")
        multiply(da.val, a, "the first array again")
        assert lib.asamd_csr_plan_refresh_values(None, plan, da.row_ptr.c_ptr(), da.col.c_ptr(), d_other.c_ptr()) == 0
        multiply(d_other, b, "the copy re-based on the other array")
        multiply(da.val, a, "the first array, now the foreign one")
        ws.buf.free()
    finally:
        lib.asamd_csr_plan_destroy(plan)
        for d in (dx, dy, d_other):
            d.free()
        da.free()


@pytest.mark.parametrize("dtype,cols,base", [(np.float32, 32768, 0), (np.float32, 21001, 1), (np.float64, 16384, 1)],
                         ids=["f32_32768", "f32_21001_base1", "f64_16384_base1"])
def test_analysed_tall_matrix_reads_sixteen_bit_columns(gpu, dtype, cols, base, monkeypatch):
    """With an analysis (a structure that stays) the kernel that holds x in LDS reads the column numbers from a 16-bit
    copy made once; the values stay in the caller's array, so new values in place need nothing."""
    lib = capi.load()
    a = wl.uniform_rows(300000, cols, 16, dtype, base=base)
    x, y0 = wl.uniform(a.cols, a.dtype, 3), wl.uniform(a.rows, a.dtype, 4)
    da = DeviceCsr(a)
    descr = capi.make_descr(base=a.base)
    p = capi.prefix(a.dtype)

    def analysed():
        info = capi.alphasparse_dcu_mat_info_t()
        assert lib.alphasparse_dcu_create_mat_info(byref(info)) == 0
        assert getattr(lib, "alphasparse_dcu_%s_csrmv_analysis" % p)(
            gpu.h, 0, a.rows, a.cols, a.nnz, byref(descr), da.val.c_ptr(), da.row_ptr.c_ptr(), da.col.c_ptr(), info) == 0
        return info

    try:
        announce("x in LDS, 16-bit columns: analysis", np.dtype(dtype).name, cols)
        info = analysed()
        st = lib.asamd_analysis_stats(info).contents
        assert st.algo == capi.ASAMD_SPMV_XLDS and st.xlds_slices == 0
        assert st.device_bytes >= 2 * a.nnz, "no 16-bit copy of the columns"
        for alpha, beta in ((1.0, 0.0), (-0.5, 2.0)):
            announce("x in LDS, 16-bit columns: multiply", alpha, beta)
            check_spmv(a, alpha, x, beta, y0, run_csrmv(gpu, da, alpha, x, beta, y0, info=info), "narrow %s" % ((alpha, beta),))
        b = wl.Csr(a.rows, a.cols, a.row_ptr, a.col_ind, wl.uniform(a.nnz, a.dtype, 21), a.base, a.name)
        da.val.copy_from(b.values)
        check_spmv(b, 2.0, x, 0.0, y0, run_csrmv(gpu, da, 2.0, x, 0.0, y0, info=info), "narrow, new values in place")
        lib.alphasparse_dcu_destroy_mat_info(info)
        monkeypatch.setenv("ALSPARSE_AMD_XLDS_NARROW", "0")
        info = analysed()
        st = lib.asamd_analysis_stats(info).contents
        assert st.algo == capi.ASAMD_SPMV_XLDS and st.device_bytes < 2 * a.nnz
        check_spmv(b, 1.0, x, 0.0, y0, run_csrmv(gpu, da, 1.0, x, 0.0, y0, info=info), "32-bit columns")
    finally:
        lib.alphasparse_dcu_destroy_mat_info(info)
        da.free()


def test_rows_far_longer_than_the_mean_keep_the_balanced_kernels(gpu):
    """Rows of 4 entries and, every eighth, 256 (nine tenths of the entries in rows of seven times the mean): the
    kernel that holds x in LDS would walk the long rows load by load; the library keeps merge-path, with all of x in
    that kernel's LDS table once analysed.  A milder mix (12 and 24 entries) still takes the x-in-LDS kernel."""
    lib = capi.load()
    for short, long_, every, takes_xlds in ((4, 256, 8, False), (12, 24, 2, True)):
        a = wl.bimodal_rows(300000, 16384, short, long_, every, np.float32)
        assert a.nnz >= 1 << 22
        da = DeviceCsr(a)
        try:
            announce("x in LDS: row-length mix", short, long_, every)
            algo = _plan_algo(lib, da)
            assert (algo == capi.ASAMD_SPMV_XLDS) == takes_xlds, (short, long_, every)
            x, y0 = wl.uniform(a.cols, a.dtype, 3), wl.uniform(a.rows, a.dtype, 4)
            check_spmv(a, 1.0, x, 0.0, y0, run_csrmv(gpu, da, 1.0, x, 0.0, y0), "mix %d/%d" % (short, long_))
            if not takes_xlds:
                # an analysis balances the rows with merge-path and keeps all of x in that kernel's LDS table
                assert algo == capi.ASAMD_SPMV_MERGE_HOT, capi.ALGO_NAMES[algo]
                info = capi.alphasparse_dcu_mat_info_t()
                assert lib.alphasparse_dcu_create_mat_info(byref(info)) == 0
                descr = capi.make_descr(base=a.base)
                try:
                    assert lib.alphasparse_dcu_s_csrmv_analysis(gpu.h, 0, a.rows, a.cols, a.nnz, byref(descr),
                                                                da.val.c_ptr(), da.row_ptr.c_ptr(), da.col.c_ptr(),
                                                                info) == 0
                    assert lib.asamd_analysis_stats(info).contents.algo == capi.ASAMD_SPMV_MERGE_HOT
                    check_spmv(a, -0.5, x, 2.0, y0, run_csrmv(gpu, da, -0.5, x, 2.0, y0, info=info), "mix, analysed")
                finally:
                    lib.alphasparse_dcu_destroy_mat_info(info)
        finally:
            da.free()


def test_few_very_long_rows_keep_the_balanced_kernels(gpu):
    """2 048 rows of 2 048 entries under 16 384 columns: the kernel that holds x in LDS gives a lane group four rows per
    trip and rows beyond 512 entries to single waves, so eight of its 256 workgroups would work; the library keeps
    merge-path.  32 768 rows of 256 entries take it."""
    lib = capi.load()
    for rows, cols, per_row, takes_xlds in ((2048, 16384, 2048, False), (32768, 32768, 256, True)):
        a = wl.uniform_rows(rows, cols, per_row, np.float32)
        assert a.nnz >= 1 << 22
        da = DeviceCsr(a)
        try:
            announce("x in LDS: rows", rows, "of", per_row)
            assert (_plan_algo(lib, da) == capi.ASAMD_SPMV_XLDS) == takes_xlds, (rows, per_row)
            x, y0 = wl.uniform(a.cols, a.dtype, 3), wl.uniform(a.rows, a.dtype, 4)
            check_spmv(a, 1.0, x, 0.5, y0, run_csrmv(gpu, da, 1.0, x, 0.5, y0), "%d rows of %d" % (rows, per_row))
        finally:
            da.free()
