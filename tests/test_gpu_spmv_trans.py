"""Transposed CSR SpMV on the GPU, y = alpha*A^T*x + beta*y, through every route of the C API:
no analysis (atomic scatter), an analysis asked for the transposed operation (CSR copy of A^T,
ordinary kernels), and a library-owned mirror (copy built on first use).  Checked against the
oracle's restatement of the reference's plain transposed kernel; the per-column error is
normalised by sum_i |a_ij x_i| (+ |beta y0_j|), rows of A^T without entries must be exact."""
from ctypes import byref

import numpy as np
import pytest

from alsparse_amd import capi, hiprt, workloads as wl
from oracle import oracle as orc
from helpers import DeviceCsr, TOL, announce, check_beta_rows
from helpers_shapes import csr_from_lengths

pytestmark = pytest.mark.gpu
DT = [np.float32, np.float64]
IDS = ["f32", "f64"]
TRANS = capi.ALPHA_SPARSE_OPERATION_TRANSPOSE

SHAPES = {
    "uniform16_tall": lambda dt: wl.uniform_rows(9000, 700, 16, dt),
    "uniform16_wide": lambda dt: wl.uniform_rows(700, 9000, 16, dt),
    "powerlaw": lambda dt: wl.powerlaw_rmat(13, 3000, dt),
    "laplace": lambda dt: wl.laplace2d(64, 48, dt),
    "empty_rows_and_columns": lambda dt: csr_from_lengths([0, 0, 5, 0, 3000, 0, 0, 1, 1, 0, 64, 65, 0], 50000, dt),
    "one_row": lambda dt: csr_from_lengths([7000], 10000, dt),
    "one_column": lambda dt: csr_from_lengths([1] * 5000, 1, dt),
    "single_entry": lambda dt: csr_from_lengths([1], 1, dt),
    "base_one": lambda dt: wl.uniform_rows(3000, 2500, 16, dt, base=1),
}


def check_trans(a, alpha, x, beta, y0, y, what):
    at = orc.transpose(a)
    ref = orc.csrmv_trans_plain(a, alpha, x, beta, y0)
    err = orc.csrmv_err(at, alpha, x, beta, y0, y, ref)
    tol = TOL[a.dtype]
    assert err.zero_den_mismatch == 0, "%s: %d columns without entries differ" % (what, err.zero_den_mismatch)
    assert err.full <= tol, "%s: error %.3e at column %d exceeds %g" % (what, err.full, err.row, tol)
    if beta == 0:
        assert err.strict <= tol, "%s: strict error %.3e exceeds %g" % (what, err.strict, tol)
    else:
        check_beta_rows(at, alpha, x, beta, y0, y, ref, tol, what)


def run_csrmv_trans(h, da, alpha, x, beta, y0, info=None):
    a = da.a
    lib = capi.load()
    T = capi.scalar_type(a.dtype)
    descr = capi.make_descr(base=a.base)
    dx, dy = hiprt.DeviceArray.from_numpy(x), hiprt.DeviceArray.from_numpy(y0)
    al, be = T(alpha), T(beta)
    st = getattr(lib, "alphasparse_dcu_%s_csrmv" % capi.prefix(a.dtype))(
        h.h, TRANS, a.rows, a.cols, a.nnz, byref(al), byref(descr), da.val.c_ptr(), da.row_ptr.c_ptr(),
        da.col.c_ptr(), info, dx.c_ptr(), byref(be), dy.c_ptr())
    assert st == 0, "csrmv(trans) status %d" % st
    hiprt.synchronize()
    y = dy.to_numpy()
    dx.free()
    dy.free()
    return y


@pytest.mark.parametrize("dtype", DT, ids=IDS)
@pytest.mark.parametrize("shape", sorted(SHAPES))
def test_transposed_csrmv_scatter_and_analysed(gpu, shape, dtype):
    lib = capi.load()
    a = SHAPES[shape](dtype)
    x, y0 = wl.uniform(a.rows, dtype, 3), wl.uniform(a.cols, dtype, 4)
    da = DeviceCsr(a)
    info = capi.alphasparse_dcu_mat_info_t()
    assert lib.alphasparse_dcu_create_mat_info(byref(info)) == 0
    try:
        for alpha, beta in ((1.0, 0.0), (2.0, 3.0), (-0.75, 1.0)):
            announce("csrmv trans scatter", shape, np.dtype(dtype).name, alpha, beta)
            y = run_csrmv_trans(gpu, da, alpha, x, beta, y0)
            check_trans(a, alpha, x, beta, y0, y, "%s scatter" % shape)
        descr = capi.make_descr(base=a.base)
        announce("csrmv trans analysis", shape, np.dtype(dtype).name)
        assert getattr(lib, "alphasparse_dcu_%s_csrmv_analysis" % capi.prefix(dtype))(
            gpu.h, TRANS, a.rows, a.cols, a.nnz, byref(descr), da.val.c_ptr(), da.row_ptr.c_ptr(), da.col.c_ptr(), info) == 0
        st = lib.asamd_analysis_stats(info).contents
        assert st.transpose_built == 1
        runs = []
        for alpha, beta in ((1.0, 0.0), (2.0, 3.0), (-0.75, 1.0)):
            announce("csrmv trans analysed", shape, np.dtype(dtype).name, alpha, beta)
            y = run_csrmv_trans(gpu, da, alpha, x, beta, y0, info)
            check_trans(a, alpha, x, beta, y0, y, "%s analysed" % shape)
            runs.append(y)
        # the copy of A^T is multiplied by the ordinary kernels: reproducible
        assert np.array_equal(runs[1], run_csrmv_trans(gpu, da, 2.0, x, 3.0, y0, info))
        # another value array on the analysed structure: the copy holds the old values and must not be used
        b = wl.Csr(a.rows, a.cols, a.row_ptr, a.col_ind, (a.values * dtype(-2.0)).astype(dtype), a.base, "new values")
        old_val = da.val
        da.a, da.val = b, hiprt.DeviceArray.from_numpy(b.values)
        try:
            announce("csrmv trans analysed, other value array", shape, np.dtype(dtype).name)
            y = run_csrmv_trans(gpu, da, 2.0, x, 3.0, y0, info)
            check_trans(b, 2.0, x, 3.0, y0, y, "%s other values" % shape)
        finally:
            da.val.free()
            da.a, da.val = a, old_val
    finally:
        lib.alphasparse_dcu_destroy_mat_info(info)
        da.free()


@pytest.mark.parametrize("dtype", DT, ids=IDS)
def test_transposed_copy_matches_the_oracle_transpose_bit_for_bit(gpu, dtype):
    """The CSR copy of A^T (stable sort by column) is exactly the matrix orc.transpose builds;
    checked through its analysis statistics and a product with integer data (exact sums)."""
    lib = capi.load()
    from ctypes import c_void_p
    rng = np.random.default_rng(9)
    a = wl.powerlaw_rmat(12, 2000, dtype)
    a = wl.Csr(a.rows, a.cols, a.row_ptr, a.col_ind, rng.integers(-4, 5, a.nnz).astype(dtype), 0, a.name)
    x, y0 = rng.integers(-4, 5, a.rows).astype(dtype), rng.integers(-4, 5, a.cols).astype(dtype)
    da = DeviceCsr(a)
    plan = c_void_p()
    try:
        announce("transpose copy", np.dtype(dtype).name)
        assert lib.asamd_csr_plan_create(None, a.rows, a.cols, a.nnz, da.row_ptr.c_ptr(), da.col.c_ptr(), da.val.c_ptr(),
                                         0, a.dtype.itemsize, 1, byref(plan)) == 0
        assert lib.asamd_csr_plan_build_transpose(None, plan, da.row_ptr.c_ptr(), da.col.c_ptr(), da.val.c_ptr()) == 0
        st = lib.asamd_csr_plan_transpose_stats(plan).contents
        at = orc.transpose(a)
        lens = np.diff(at.row_ptr)
        assert (st.m, st.n, st.nnz) == (a.cols, a.rows, a.nnz)
        assert (st.min_len, st.max_len) == (int(lens.min()), int(lens.max()))
        want_hist = [0] * capi.ASAMD_HIST_BINS
        for n_ in lens:
            want_hist[0 if n_ == 0 else int(n_).bit_length()] += 1
        assert list(st.hist) == want_hist
        T = capi.scalar_type(dtype)
        dx, dy = hiprt.DeviceArray.from_numpy(x), hiprt.DeviceArray.from_numpy(y0)
        ws = capi.Workspace(lib, plan)
        assert capi.plan_csrmv(lib, None, plan, 1, T(2.0), da.val.c_ptr(), da.row_ptr.c_ptr(), da.col.c_ptr(), dx.c_ptr(),
                               T(3.0), dy.c_ptr(), ws) == 0
        hiprt.synchronize()
        assert np.array_equal(dy.to_numpy(), orc.csrmv_trans_plain(a, 2.0, x, 3.0, y0))
        dx.free()
        dy.free()
    finally:
        lib.asamd_csr_plan_destroy(plan)
        da.free()


@pytest.mark.parametrize("dtype", DT, ids=IDS)
def test_handle_api_transposed(gpu, dtype):
    """create_csr -> alphasparse_?_mv (host vectors) and host2device -> alphasparse_?_mv_dcu with
    op(A) = A^T on a rectangular matrix; the conjugate of a real matrix is refused."""
    lib = capi.load()
    p, T = capi.prefix(dtype), capi.scalar_type(dtype)
    a = wl.uniform_rows(4000, 1500, 12, dtype)
    x, y0 = wl.uniform(a.rows, dtype, 3), wl.uniform(a.cols, dtype, 4)
    A = capi.alphasparse_matrix_t()
    rs, re = np.ascontiguousarray(a.row_ptr[:-1]), np.ascontiguousarray(a.row_ptr[1:])
    assert getattr(lib, "alphasparse_%s_create_csr" % p)(byref(A), 0, a.rows, a.cols, capi.ptr(rs), capi.ptr(re),
                                                          capi.ptr(a.col_ind), capi.ptr(a.values)) == 0
    try:
        gen = capi.alpha_matrix_descr(0, 0, 0)
        mv = getattr(lib, "alphasparse_%s_mv" % p)
        announce("host api mv trans", np.dtype(dtype).name)
        y = y0.copy()
        assert mv(TRANS, T(1.5), A, gen, capi.ptr(x), T(0.5), capi.ptr(y)) == 0
        check_trans(a, 1.5, x, 0.5, y0, y, "alphasparse_mv trans")
        y2 = y0.copy()
        assert mv(TRANS, T(1.5), A, gen, capi.ptr(x), T(0.5), capi.ptr(y2)) == 0
        assert np.array_equal(y, y2)
        assert mv(2, T(1.5), A, gen, capi.ptr(x), T(0.5), capi.ptr(y2)) == capi.ALPHA_SPARSE_STATUS_INVALID_VALUE
        announce("mv_dcu trans", np.dtype(dtype).name)
        dx, dy = hiprt.DeviceArray.from_numpy(x), hiprt.DeviceArray.from_numpy(y0)
        al, be = T(-2.0), T(1.0)
        descr = capi.make_descr()
        mv_dcu = getattr(lib, "alphasparse_%s_mv_dcu" % p)
        assert mv_dcu(gpu.h, TRANS, byref(al), A, byref(descr), dx.c_ptr(), byref(be), dy.c_ptr()) == 0
        hiprt.synchronize()
        check_trans(a, -2.0, x, 1.0, y0, dy.to_numpy(), "mv_dcu trans")
        assert mv_dcu(gpu.h, 2, byref(al), A, byref(descr), dx.c_ptr(), byref(be), dy.c_ptr()) == capi.ALPHA_SPARSE_STATUS_NOT_SUPPORTED
        # the non-transposed product of the same handle is unaffected
        xn, yn = wl.uniform(a.cols, dtype, 5), wl.uniform(a.rows, dtype, 6)
        yh = yn.copy()
        assert mv(0, T(1.0), A, gen, capi.ptr(xn), T(0.0), capi.ptr(yh)) == 0
        ref = orc.csrmv_plain(a, 1.0, xn, 0.0, yn)
        e = orc.csrmv_err(a, 1.0, xn, 0.0, yn, yh, ref)
        assert e.strict <= TOL[np.dtype(dtype)] and e.zero_den_mismatch == 0
        dx.free()
        dy.free()
    finally:
        assert lib.alphasparse_destroy(A) == 0


def test_transposed_full_size_configuration_3(gpu):
    """A^T of benchmark configuration 3 (16.7 M columns of ~16 entries each) through an analysis
    asked for the transposed operation; strict criterion, and linearity in alpha (bit-exact for a
    power of two with beta = 0: the copy's kernels are deterministic)."""
    lib = capi.load()
    a, _, _, _, _, _ = wl.config(3)
    x, y0 = wl.uniform(a.rows, np.float32, 3), wl.uniform(a.cols, np.float32, 4)
    da = DeviceCsr(a)
    info = capi.alphasparse_dcu_mat_info_t()
    assert lib.alphasparse_dcu_create_mat_info(byref(info)) == 0
    try:
        descr = capi.make_descr()
        announce("full size config 3 transposed: analysis")
        assert lib.alphasparse_dcu_s_csrmv_analysis(gpu.h, TRANS, a.rows, a.cols, a.nnz, byref(descr), da.val.c_ptr(),
                                                    da.row_ptr.c_ptr(), da.col.c_ptr(), info) == 0
        announce("full size config 3 transposed: multiply")
        y = run_csrmv_trans(gpu, da, 1.0, x, 0.5, y0, info)
        ref = orc.csrmv_trans_plain(a, 1.0, x, 0.5, y0)
        # per-column sum |a_ij x_i| by the same scatter on absolute values (cheaper than transposing 268 M entries
        # on the host); every product is non-negative, so fp32 accumulation is accurate to a few ulps
        absa = wl.Csr(a.rows, a.cols, a.row_ptr, a.col_ind, np.abs(a.values), 0)
        den = orc.csrmv_trans_plain(absa, 1.0, np.abs(x), 0.0, np.zeros(a.cols, np.float32)).astype(np.float64)
        diff = np.abs(y.astype(np.float64) - ref.astype(np.float64))
        assert np.all(diff[den == 0] == 0)
        assert np.max(diff[den > 0] / den[den > 0]) <= 1e-4
        y1 = run_csrmv_trans(gpu, da, 1.0, x, 0.0, y0, info)
        y4 = run_csrmv_trans(gpu, da, 4.0, x, 0.0, y0, info)
        assert np.array_equal(y4, 4 * y1)
    finally:
        lib.alphasparse_dcu_destroy_mat_info(info)
        da.free()


TALL = {
    # >= 2^20 entries and a y (n elements) that fits a compute unit's LDS: the unanalysed transposed multiply adds
    # up in LDS, a workgroup per compute unit, instead of scattering with global atomics
    "uniform16_f32": lambda: wl.uniform_rows(100000, 20000, 16, np.float32),
    "uniform40_f64_base1": lambda: wl.uniform_rows(40000, 15000, 40, np.float64, base=1),
    "ragged_f32": lambda: csr_from_lengths(list((np.arange(60000) * 7) % 45), 30000, np.float32, seed=3),
}


@pytest.mark.parametrize("shape", sorted(TALL))
def test_transposed_csrmv_without_analysis_on_tall_matrices(gpu, shape, monkeypatch):
    a = TALL[shape]()
    assert a.nnz >= 1 << 20
    x, y0 = wl.uniform(a.rows, a.dtype, 3), wl.uniform(a.cols, a.dtype, 4)
    da = DeviceCsr(a)
    try:
        for alpha, beta in ((1.0, 0.0), (-0.5, 2.0), (2.0, 1.0)):
            announce("transposed csrmv, y in LDS", shape, alpha, beta)
            y = run_csrmv_trans(gpu, da, alpha, x, beta, y0)
            check_trans(a, alpha, x, beta, y0, y, "%s y in LDS %s" % (shape, (alpha, beta)))
        monkeypatch.setenv("ALSPARSE_AMD_XLDS", "0")  # the scatter with global atomics, same inputs
        y = run_csrmv_trans(gpu, da, 1.0, x, 0.0, y0)
        check_trans(a, 1.0, x, 0.0, y0, y, "%s global atomics" % shape)
    finally:
        da.free()


def test_analysed_tall_transpose_runs_slice_by_slice_and_follows_the_values(gpu):
    """19 M entries in 1 200 000 rows of 20 000 columns: the analysed transposed multiply runs on a CSR copy of the
    transpose (20 000 rows of 960 entries, an x of 1 200 000 elements: thirty LDS fills, cut into 32 slices), which the analysis of that copy
    multiplies slice by slice over its own copy of the entries.  New values written into the caller's array travel
    through both copies before the next multiply."""
    lib = capi.load()
    a = wl.uniform_rows(1200000, 20000, 16, np.float32)
    x, y0 = wl.uniform(a.rows, a.dtype, 3), wl.uniform(a.cols, a.dtype, 4)
    da = DeviceCsr(a)
    info = capi.alphasparse_dcu_mat_info_t()
    assert lib.alphasparse_dcu_create_mat_info(byref(info)) == 0
    descr = capi.make_descr(base=a.base)
    try:
        announce("tall transpose: analysis")
        assert lib.alphasparse_dcu_s_csrmv_analysis(gpu.h, TRANS, a.rows, a.cols, a.nnz, byref(descr), da.val.c_ptr(),
                                                    da.row_ptr.c_ptr(), da.col.c_ptr(), info) == 0
        st = lib.asamd_analysis_stats(info).contents
        assert st.transpose_built == 1
        tst = lib.asamd_analysis_transpose_stats(info).contents
        assert tst.algo == capi.ASAMD_SPMV_XLDS and tst.xlds_slices == 32, (tst.algo, tst.xlds_slices)
        assert tst.device_bytes > a.nnz * 6, "the transpose's analysis kept no copy slice by slice"
        for alpha, beta in ((1.0, 0.0), (2.0, 3.0)):
            announce("tall transpose: multiply", alpha, beta)
            check_trans(a, alpha, x, beta, y0, run_csrmv_trans(gpu, da, alpha, x, beta, y0, info), "tall analysed")
        for seed in (41, 42):
            announce("tall transpose: new values in place", seed)
            b = wl.Csr(a.rows, a.cols, a.row_ptr, a.col_ind, wl.uniform(a.nnz, a.dtype, seed), a.base, "new values")
            da.val.copy_from(b.values)
            check_trans(b, 1.5, x, 0.5, y0, run_csrmv_trans(gpu, da, 1.5, x, 0.5, y0, info), "tall, new values %d" % seed)
    finally:
        lib.alphasparse_dcu_destroy_mat_info(info)
        da.free()
