"""GPU SpMV on the converters' output formats (alphasparse_dcu_?_ellmv / _coomv) against
the CPU oracle: per-row error within 1e-4 (fp32) / 1e-12 (fp64) of sum|a x| (+ |beta y0|),
rows without entries exact, and the pipeline csr2ell -> ellmv / csr2coo -> coomv on the GPU
agreeing with csrmv on the same matrix."""
from ctypes import byref, c_int32

import numpy as np
import pytest

from alsparse_amd import capi, hiprt, workloads as wl
from oracle import oracle as orc
from helpers import DeviceCsr, TOL, announce, check_beta_rows, run_csrmv
from helpers_shapes import csr_from_lengths

pytestmark = pytest.mark.gpu
DT = [np.float32, np.float64]
IDS = ["f32", "f64"]


def dev(a):
    return hiprt.DeviceArray.from_numpy(np.ascontiguousarray(a))


def run_coomv(h, m, n, vals, rows, cols, base, alpha, x, beta, y0):
    lib = capi.load()
    T = capi.scalar_type(vals.dtype)
    d = capi.make_descr(base=base)
    bufs = [dev(vals), dev(rows.astype(np.int32)), dev(cols.astype(np.int32)), dev(x), dev(y0)]
    al, be = T(alpha), T(beta)
    st = getattr(lib, "alphasparse_dcu_%s_coomv" % capi.prefix(vals.dtype))(
        h.h, 0, m, n, vals.size, byref(al), byref(d), bufs[0].c_ptr(), bufs[1].c_ptr(), bufs[2].c_ptr(),
        bufs[3].c_ptr(), byref(be), bufs[4].c_ptr())
    assert st == 0, "coomv status %d" % st
    hiprt.synchronize()
    y = bufs[4].to_numpy()
    for b in bufs:
        b.free()
    return y


def run_ellmv(h, m, n, ev, ec, width, base, alpha, x, beta, y0):
    lib = capi.load()
    T = capi.scalar_type(ev.dtype)
    d = capi.make_descr(base=base)
    pad = lambda v: v if v.size else np.zeros(1, v.dtype)  # noqa: E731  (no zero-byte allocations)
    bufs = [dev(pad(ev)), dev(pad(ec.astype(np.int32))), dev(x), dev(y0)]
    al, be = T(alpha), T(beta)
    st = getattr(lib, "alphasparse_dcu_%s_ellmv" % capi.prefix(ev.dtype))(
        h.h, 0, m, n, byref(al), byref(d), bufs[0].c_ptr(), bufs[1].c_ptr(), width, bufs[2].c_ptr(), byref(be),
        bufs[3].c_ptr())
    assert st == 0, "ellmv status %d" % st
    hiprt.synchronize()
    y = bufs[3].to_numpy()
    for b in bufs:
        b.free()
    return y


def check(a, alpha, x, beta, y0, y, ref, what):
    err = orc.csrmv_err(a, alpha, x, beta, y0, y, ref)
    tol = TOL[a.dtype]
    assert err.zero_den_mismatch == 0, "%s: %d rows with zero denominator differ" % (what, err.zero_den_mismatch)
    assert err.full <= tol, "%s: per-row error %.3e at row %d exceeds %g" % (what, err.full, err.row, tol)
    if beta == 0:
        assert err.strict <= tol, "%s: strict per-row error %.3e exceeds %g" % (what, err.strict, tol)
    else:
        check_beta_rows(a, alpha, x, beta, y0, y, ref, tol, what)


SHAPES = {
    "uniform16": lambda dt: wl.uniform_rows(70000, 50000, 16, dt),
    "powerlaw": lambda dt: wl.powerlaw_rmat(14, 20000, dt),
    "laplace": lambda dt: wl.laplace2d(300, 177, dt),
    # one row longer than a wave's run of 1024 entries and than a workgroup's 4096, empty runs around it
    "long_and_empty": lambda dt: csr_from_lengths([0] * 600 + [9000] + [0] * 300 + [2, 4097, 4095, 0, 0, 1, 63, 64, 65],
                                                  20000, dt),
    "single_row": lambda dt: csr_from_lengths([5000], 6000, dt),
    "ones": lambda dt: csr_from_lengths([1] * 9001, 9001, dt),
    "tiny": lambda dt: csr_from_lengths([2, 0, 1], 5, dt),
}
SCALARS = [(1.0, 0.0), (2.0, 3.0), (-0.5, 1.0)]


@pytest.mark.parametrize("dtype", DT, ids=IDS)
@pytest.mark.parametrize("shape", sorted(SHAPES))
def test_coomv_matches_oracle(gpu, shape, dtype):
    a = SHAPES[shape](dtype)
    x, y0 = wl.uniform(a.cols, dtype, 3), wl.uniform(a.rows, dtype, 4)
    rows = orc.csr2coo(a)
    for alpha, beta in SCALARS:
        for base in (0, 1):
            announce("coomv", shape, np.dtype(dtype).name, alpha, beta, base)
            y = run_coomv(gpu, a.rows, a.cols, a.values, rows + base, a.col_ind + base, base, alpha, x, beta, y0)
            check(a, alpha, x, beta, y0, y, orc.coomv_plain(a, rows, alpha, x, beta, y0), "coomv %s" % shape)


@pytest.mark.parametrize("shape", ["powerlaw", "long_and_empty", "single_row"])
def test_coomv_grouped_by_row_is_the_same_every_run(gpu, shape):
    """Rows that several waves share (every row of more than a thousand entries, and any row across a wave
    boundary) are summed in wave order: entries grouped by row give the same bits from run to run."""
    a = SHAPES[shape](np.float32)
    x, y0 = wl.uniform(a.cols, np.float32, 3), wl.uniform(a.rows, np.float32, 4)
    rows = orc.csr2coo(a)
    announce("coomv determinism", shape)
    runs = [run_coomv(gpu, a.rows, a.cols, a.values, rows, a.col_ind, 0, 1.5, x, 0.5, y0) for _ in range(4)]
    for y in runs[1:]:
        assert np.array_equal(runs[0], y)


@pytest.mark.parametrize("dtype", DT, ids=IDS)
def test_coomv_any_entry_order_and_out_of_range_entries(gpu, dtype):
    """Entries need not be grouped by row; entries whose row or column is out of range are skipped."""
    a = wl.powerlaw_rmat(12, 5000, dtype)
    x, y0 = wl.uniform(a.cols, dtype, 3), wl.uniform(a.rows, dtype, 4)
    rows = orc.csr2coo(a)
    perm = np.random.default_rng(3).permutation(a.nnz)
    ref = orc.coomv_plain(a, rows, 2.0, x, 3.0, y0)
    announce("coomv shuffled", np.dtype(dtype).name)
    y = run_coomv(gpu, a.rows, a.cols, a.values[perm], rows[perm], a.col_ind[perm], 0, 2.0, x, 3.0, y0)
    check(a, 2.0, x, 3.0, y0, y, ref, "coomv shuffled")
    # plant bad entries: they must change nothing
    r2 = np.concatenate([rows, [-1, a.rows, 5, 7]]).astype(np.int32)
    c2 = np.concatenate([a.col_ind, [3, 3, -1, a.cols]]).astype(np.int32)
    v2 = np.concatenate([a.values, np.full(4, 1e6, dtype)])
    announce("coomv out of range", np.dtype(dtype).name)
    y = run_coomv(gpu, a.rows, a.cols, v2, r2, c2, 0, 2.0, x, 3.0, y0)
    check(a, 2.0, x, 3.0, y0, y, ref, "coomv with out-of-range entries")


@pytest.mark.parametrize("dtype", DT, ids=IDS)
@pytest.mark.parametrize("shape", ["uniform16", "laplace", "long_and_empty", "single_row", "ones", "tiny"])
def test_ellmv_matches_oracle(gpu, shape, dtype):
    a = SHAPES[shape](dtype)
    x, y0 = wl.uniform(a.cols, dtype, 3), wl.uniform(a.rows, dtype, 4)
    w = orc.csr2ell_width(a)
    ev, ec = orc.csr2ell(a)
    for alpha, beta in SCALARS:
        for base in (0, 1):
            announce("ellmv", shape, np.dtype(dtype).name, alpha, beta, base)
            y = run_ellmv(gpu, a.rows, a.cols, ev, ec + base, w, base, alpha, x, beta, y0)
            check(a, alpha, x, beta, y0, y, orc.ellmv(a.rows, a.cols, ev, ec, w, alpha, x, beta, y0), "ellmv %s" % shape)


@pytest.mark.parametrize("dtype", DT, ids=IDS)
def test_ellmv_skips_slots_outside_the_matrix(gpu, dtype):
    """Index >= n (dcu_gemv_x_ell.cpp:33) or < 0: the slot does not count, whatever its value."""
    a = csr_from_lengths([3, 0, 5, 1, 2, 0, 4], 50, dtype)
    x, y0 = wl.uniform(a.cols, dtype, 3), wl.uniform(a.rows, dtype, 4)
    w = orc.csr2ell_width(a)
    ev, ec = orc.csr2ell(a)
    ref = orc.ellmv(a.rows, a.cols, ev, ec, w, 1.5, x, 0.5, y0)
    pad = np.flatnonzero(ev == 0)
    ev2, ec2 = ev.copy(), ec.copy()
    ev2[pad[::2]], ec2[pad[::2]] = 1e6, a.cols
    ev2[pad[1::2]], ec2[pad[1::2]] = np.nan, -1
    announce("ellmv skipped slots", np.dtype(dtype).name)
    y = run_ellmv(gpu, a.rows, a.cols, ev2, ec2, w, 0, 1.5, x, 0.5, y0)
    check(a, 1.5, x, 0.5, y0, y, ref, "ellmv skipped slots")


@pytest.mark.parametrize("dtype", DT, ids=IDS)
def test_beta_zero_never_reads_y(gpu, dtype):
    a = wl.uniform_rows(5000, 4000, 8, dtype)
    x = wl.uniform(a.cols, dtype, 3)
    y0 = np.full(a.rows, np.nan, dtype)
    rows = orc.csr2coo(a)
    w = orc.csr2ell_width(a)
    ev, ec = orc.csr2ell(a)
    zeros = np.zeros(a.rows, dtype)
    announce("beta=0 NaN y", np.dtype(dtype).name)
    y = run_coomv(gpu, a.rows, a.cols, a.values, rows, a.col_ind, 0, 1.0, x, 0.0, y0)
    check(a, 1.0, x, 0.0, zeros, y, orc.coomv_plain(a, rows, 1.0, x, 0.0, zeros), "coomv beta=0")
    y = run_ellmv(gpu, a.rows, a.cols, ev, ec, w, 0, 1.0, x, 0.0, y0)
    check(a, 1.0, x, 0.0, zeros, y, orc.ellmv(a.rows, a.cols, ev, ec, w, 1.0, x, 0.0, zeros), "ellmv beta=0")


@pytest.mark.parametrize("dtype", DT, ids=IDS)
@pytest.mark.parametrize("shape", ["uniform16", "laplace", "powerlaw"])
def test_conversion_pipelines_agree_with_csrmv(gpu, shape, dtype):
    """csr2coo -> coomv and csr2ell -> ellmv, all on the device, against csrmv on the same CSR arrays."""
    a = SHAPES[shape](dtype) if shape != "powerlaw" else wl.powerlaw_rmat(12, 700, dtype)
    lib = capi.load()
    x, y0 = wl.uniform(a.cols, dtype, 3), wl.uniform(a.rows, dtype, 4)
    da = DeviceCsr(a)
    T = capi.scalar_type(dtype)
    al, be = T(2.0), T(3.0)
    d = capi.make_descr(base=0)
    try:
        announce("pipeline", shape, np.dtype(dtype).name)
        y_csr = run_csrmv(gpu, da, 2.0, x, 3.0, y0)
        ref = orc.csrmv_plain(a, 2.0, x, 3.0, y0)
        check(a, 2.0, x, 3.0, y0, y_csr, ref, "csrmv")
        dx = dev(x)
        # COO
        d_rows = hiprt.DeviceArray((a.nnz,), np.int32)
        assert lib.alphasparse_dcu_csr2coo(gpu.h, da.row_ptr.c_ptr(), a.nnz, a.rows, d_rows.c_ptr(), 0) == 0
        dy = dev(y0)
        assert getattr(lib, "alphasparse_dcu_%s_coomv" % capi.prefix(dtype))(
            gpu.h, 0, a.rows, a.cols, a.nnz, byref(al), byref(d), da.val.c_ptr(), d_rows.c_ptr(), da.col.c_ptr(),
            dx.c_ptr(), byref(be), dy.c_ptr()) == 0
        hiprt.synchronize()
        check(a, 2.0, x, 3.0, y0, dy.to_numpy(), ref, "csr2coo -> coomv")
        dy.free()
        d_rows.free()
        # ELL
        w = c_int32(-1)
        assert lib.alphasparse_dcu_csr2ell_width(gpu.h, a.rows, byref(d), da.row_ptr.c_ptr(), byref(d), byref(w)) == 0
        ev = hiprt.DeviceArray((w.value * a.rows,), dtype)
        ec = hiprt.DeviceArray((w.value * a.rows,), np.int32)
        conv = lib.alphasparse_dcu_scsr2ell if dtype == np.float32 else lib.alphasparse_dcu_dcsr2ell
        assert conv(gpu.h, a.rows, byref(d), da.val.c_ptr(), da.row_ptr.c_ptr(), da.col.c_ptr(), byref(d), w.value,
                    ev.c_ptr(), ec.c_ptr()) == 0
        dy = dev(y0)
        assert getattr(lib, "alphasparse_dcu_%s_ellmv" % capi.prefix(dtype))(
            gpu.h, 0, a.rows, a.cols, byref(al), byref(d), ev.c_ptr(), ec.c_ptr(), w.value, dx.c_ptr(), byref(be),
            dy.c_ptr()) == 0
        hiprt.synchronize()
        check(a, 2.0, x, 3.0, y0, dy.to_numpy(), ref, "csr2ell -> ellmv")
        for b in (dy, ev, ec, dx):
            b.free()
    finally:
        da.free()


@pytest.mark.parametrize("dtype", DT, ids=IDS)
def test_handle_api_coo_and_ell(gpu, dtype):
    """create_coo -> host2device_?_coo -> alphasparse_?_mv_dcu, and convert_ell -> host2device_?_ell ->
    alphasparse_?_mv_dcu: the route of the reference's spmv_coo / spmv_ell programs."""
    lib = capi.load()
    p, T = capi.prefix(dtype), capi.scalar_type(dtype)
    a = wl.powerlaw_rmat(12, 150, dtype)
    x, y0 = wl.uniform(a.cols, dtype, 3), wl.uniform(a.rows, dtype, 4)
    perm = np.random.default_rng(1).permutation(a.nnz)
    rows, cols, vals = orc.csr2coo(a)[perm].copy(), a.col_ind[perm].copy(), a.values[perm].copy()
    coo, ell = capi.alphasparse_matrix_t(), capi.alphasparse_matrix_t()
    assert getattr(lib, "alphasparse_%s_create_coo" % p)(byref(coo), 0, a.rows, a.cols, a.nnz, capi.ptr(rows), capi.ptr(cols), capi.ptr(vals)) == 0
    assert lib.alphasparse_convert_ell(coo, 0, byref(ell)) == 0
    al, be = T(2.0), T(3.0)
    descr = capi.make_descr()
    mv_dcu = getattr(lib, "alphasparse_%s_mv_dcu" % p)
    dx = dev(x)
    ref = orc.csrmv_plain(a, 2.0, x, 3.0, y0)
    try:
        for name, h, upload in (("coo", coo, "host2device_%s_coo" % p), ("ell", ell, "host2device_%s_ell" % p)):
            dy = dev(y0)
            announce("mv_dcu on a %s handle" % name, np.dtype(dtype).name)
            assert mv_dcu(gpu.h, 0, byref(al), h, byref(descr), dx.c_ptr(), byref(be), dy.c_ptr()) == capi.ALPHA_SPARSE_STATUS_NOT_INITIALIZED
            assert getattr(lib, upload)(h) == 0
            assert getattr(lib, upload)(h) == 0   # a second upload replaces the mirror
            assert mv_dcu(gpu.h, 0, byref(al), h, byref(descr), dx.c_ptr(), byref(be), dy.c_ptr()) == 0
            hiprt.synchronize()
            check(a, 2.0, x, 3.0, y0, dy.to_numpy(), ref, "mv_dcu %s" % name)
            dy.free()
        other = "d" if p == "s" else "s"
        assert getattr(lib, "host2device_%s_coo" % other)(coo) == capi.ALPHA_SPARSE_STATUS_INVALID_VALUE
        assert getattr(lib, "host2device_%s_ell" % p)(coo) == capi.ALPHA_SPARSE_STATUS_INVALID_VALUE
    finally:
        dx.free()
        assert lib.alphasparse_destroy(coo) == 0 and lib.alphasparse_destroy(ell) == 0
