"""GPU parity of CSR SpMV against the CPU oracle, through the C-ABI.

Tolerance (north star): per row |y - y_ref| / (|alpha| * sum_j |a_ij x_j|)
<= 1e-4 for fp32 and <= 1e-12 for fp64; rows with a zero denominator must match
exactly."""
from ctypes import byref, c_float, c_void_p

import numpy as np
import pytest

from alsparse_amd import capi, hiprt, workloads as wl
from oracle import oracle as orc
from helpers import (ALGOS, TOL, DeviceCsr, announce, check_spmv, csr_from_lengths, plan_stats, run_csrmv,
                     run_plan_csrmv)

pytestmark = pytest.mark.gpu


def _vectors(a, seed=3):
    return wl.uniform(a.cols, a.dtype, 3, seed), wl.uniform(a.rows, a.dtype, 4, seed)


SHAPES = {
    "points_1000": lambda dt: wl.random_points(1000, 1000, 5000, dt),
    "laplace_64x48": lambda dt: wl.laplace2d(64, 48, dt),
    "uniform16_5000": lambda dt: wl.uniform_rows(5000, 7000, 16, dt),
    "uniform32_3000": lambda dt: wl.uniform_rows(3000, 3000, 32, dt),
    "uniform5_4099": lambda dt: wl.uniform_rows(4099, 999, 5, dt),
    "powerlaw_2^13": lambda dt: wl.powerlaw_rmat(13, 3000, dt),
    "powerlaw_2^15_long": lambda dt: wl.powerlaw_rmat(15, 200000, dt),
    "one_row_70000": lambda dt: csr_from_lengths([70000], 100000, dt),
    "empty_rows_mixed": lambda dt: csr_from_lengths([0, 0, 5, 0, 3000, 0, 0, 1, 1, 0, 64, 65, 0], 5000, dt),
    "all_rows_length_1": lambda dt: csr_from_lengths([1] * 10000, 10000, dt),
    "many_empty_then_long": lambda dt: csr_from_lengths([0] * 5000 + [9000] + [0] * 3000 + [2, 2049, 2047], 20000, dt),
    "single_entry": lambda dt: csr_from_lengths([1], 1, dt),
    "ragged_tail": lambda dt: csr_from_lengths(list(range(0, 300)), 4000, dt),
    "length_class_edges": lambda dt: csr_from_lengths([8, 9, 0, 64, 65, 2048, 2049, 1, 4096, 4097, 8193, 7, 63], 9000, dt),
    "wide_few_rows": lambda dt: csr_from_lengths([4096, 4095, 4097, 1, 0, 8192], 10000, dt),
    # rows of similar lengths: the staged row-block kernel with 2, 4, 8 and 16 lanes per row
    "stencil3d_12x10x9": lambda dt: wl.stencil3d(12, 10, 9, dt),
    "regular_40_60": lambda dt: csr_from_lengths(list(40 + (np.arange(1500) * 7) % 21), 3000, dt),
    "regular_90_128": lambda dt: csr_from_lengths(list(90 + (np.arange(700) * 5) % 39), 3000, dt),
    "regular_200_256": lambda dt: csr_from_lengths(list(200 + (np.arange(300) * 11) % 57), 3000, dt),
}


@pytest.mark.parametrize("dtype", [np.float32, np.float64], ids=["f32", "f64"])
@pytest.mark.parametrize("shape", sorted(SHAPES))
def test_every_kernel_family_matches_oracle(gpu, shape, dtype):
    a = SHAPES[shape](dtype)
    x, y0 = _vectors(a)
    da = DeviceCsr(a)
    try:
        for algo in ("vector", "merge", "scalar", "rowconst", "stream", "tiled", "ell", "hot", "binned", "xlds", "auto"):
            for alpha, beta in ((1.0, 0.0), (2.0, 3.0), (-0.75, 1.0)):
                announce("spmv", shape, np.dtype(dtype).name, algo, alpha, beta)
                y = run_plan_csrmv(da, algo, alpha, x, beta, y0)
                if y is None:
                    continue
                check_spmv(a, alpha, x, beta, y0, y, "%s/%s/%s" % (shape, algo, (alpha, beta)))
    finally:
        da.free()


def _random_structure(rng, dtype):
    """A seeded random CSR structure: row count, column count, a row-length law (constant, narrow band, wide band,
    geometric with some empty rows, a few very long rows among short ones), index base and the element offset of
    val / col_ind inside their allocations."""
    m = int(rng.integers(1, 3000))
    cols = int(rng.integers(1, 5000))
    law = int(rng.integers(0, 5))
    if law == 0:
        lengths = np.full(m, int(rng.integers(1, 70)))
    elif law == 1:
        lo = int(rng.integers(1, 120))
        lengths = rng.integers(lo, lo + int(rng.integers(1, 12)) + 1, size=m)
    elif law == 2:
        lengths = rng.integers(0, int(rng.integers(2, 300)) + 1, size=m)
    elif law == 3:
        lengths = rng.geometric(1.0 / float(rng.integers(2, 30)), size=m) - 1
    else:
        lengths = rng.integers(0, 6, size=m)
        lengths[rng.integers(0, m, size=max(1, m // 200))] = int(rng.integers(300, 4500))
    base = int(rng.integers(0, 2))
    a = csr_from_lengths(list(np.minimum(lengths, cols)), cols, dtype, seed=int(rng.integers(1, 1 << 30)), base=base)
    return a, int(rng.integers(0, 4))


@pytest.mark.parametrize("dtype", [np.float32, np.float64], ids=["f32", "f64"])
@pytest.mark.parametrize("seed", range(24))
def test_random_structures_every_family(gpu, seed, dtype):
    rng = np.random.default_rng(1000 + seed)
    a, shift = _random_structure(rng, dtype)
    if a.nnz == 0:
        pytest.skip("drew a matrix without entries")
    x, y0 = _vectors(a)
    da = DeviceCsr(a, shift=shift)
    try:
        for algo in ("vector", "merge", "scalar", "rowconst", "stream", "tiled", "ell", "binned", "xlds", "auto"):
            alpha, beta = ((1.0, 0.0), (2.0, 3.0), (-0.75, 1.0))[int(rng.integers(0, 3))]
            announce("spmv random structure", seed, a.name, "base", a.base, "shift", shift, np.dtype(dtype).name, algo, alpha, beta)
            y = run_plan_csrmv(da, algo, alpha, x, beta, y0)
            if y is None:
                continue
            check_spmv(a, alpha, x, beta, y0, y, "seed %d/%s/%s" % (seed, algo, (alpha, beta)))
        y = run_csrmv(gpu, da, 1.5, x, 0.25, y0)
        check_spmv(a, 1.5, x, 0.25, y0, y, "seed %d/api without analysis" % seed)
    finally:
        da.free()


@pytest.mark.parametrize("dtype", [np.float32, np.float64], ids=["f32", "f64"])
@pytest.mark.parametrize("shift", [1, 3], ids=["shift1", "shift3"])
def test_streams_off_16_byte_alignment(gpu, dtype, shift):
    """val and col_ind that are element-aligned only: the kernels with 128-bit loads (constant row length,
    staged row blocks, ELL pairs) must take their narrow forms, not fault and not read other bytes."""
    for maker in (lambda: wl.stencil3d(12, 10, 9, dtype), lambda: wl.uniform_rows(3000, 2500, 16, dtype),
                  lambda: wl.laplace2d(40, 30, dtype), lambda: csr_from_lengths(list(40 + (np.arange(1500) * 7) % 21), 3000, dtype)):
        a = maker()
        x, y0 = _vectors(a)
        da = DeviceCsr(a, shift=shift)
        try:
            for algo in ("vector", "merge", "rowconst", "stream", "binned", "xlds", "auto"):
                announce("spmv shifted streams", a.name, np.dtype(dtype).name, algo, shift)
                y = run_plan_csrmv(da, algo, 1.5, x, 0.25, y0)
                if y is None:
                    continue
                check_spmv(a, 1.5, x, 0.25, y0, y, "%s/%s/shift%d" % (a.name, algo, shift))
        finally:
            da.free()


@pytest.mark.parametrize("dtype", [np.float32, np.float64], ids=["f32", "f64"])
def test_index_base_one(gpu, dtype):
    for maker in (lambda: wl.uniform_rows(3000, 2500, 16, dtype, base=1),
                  lambda: wl.stencil3d(9, 8, 7, dtype, base=1),
                  lambda: wl.powerlaw_rmat(12, 2000, dtype, base=1),
                  lambda: wl.laplace2d(40, 30, dtype, base=1)):
        a = maker()
        x, y0 = _vectors(a)
        da = DeviceCsr(a)
        try:
            for algo in ("vector", "merge", "scalar", "stream", "tiled", "ell", "hot", "binned", "xlds", "auto"):
                announce("spmv base1", a.name, algo)
                y = run_plan_csrmv(da, algo, 1.5, x, 0.25, y0)
                if y is None:
                    continue
                check_spmv(a, 1.5, x, 0.25, y0, y, a.name + "/" + algo)
            y = run_csrmv(gpu, da, 1.5, x, 0.25, y0)
            check_spmv(a, 1.5, x, 0.25, y0, y, a.name + "/api")
        finally:
            da.free()


def test_beta_zero_ignores_nan_in_y(gpu):
    """beta == 0 must not read y: NaN / Inf in the output buffer may not leak
    (the bytes model counts y once in that case)."""
    a = wl.powerlaw_rmat(12, 2000, np.float32)
    x, _ = _vectors(a)
    y0 = np.full(a.rows, np.nan, dtype=np.float32)
    da = DeviceCsr(a)
    try:
        for algo in ("vector", "merge", "scalar", "tiled", "hot", "binned", "xlds"):
            announce("spmv beta0 nan", algo)
            y = run_plan_csrmv(da, algo, 1.0, x, 0.0, y0)
            assert np.isfinite(y).all()
            check_spmv(a, 1.0, x, 0.0, np.zeros_like(y0), y, algo)
    finally:
        da.free()


def test_ell_copy_is_built_only_for_short_even_rows(gpu):
    lib = capi.load()
    from ctypes import byref, c_void_p
    for a, want in ((wl.laplace2d(64, 48, np.float64), 1), (wl.uniform_rows(3000, 3000, 32, np.float32), 1),
                    (wl.powerlaw_rmat(13, 3000, np.float32), 0), (csr_from_lengths([1] * 900 + [30] * 100, 500, np.float32), 0)):
        da = DeviceCsr(a)
        plan = c_void_p()
        try:
            announce("ell eligibility", a.name)
            assert lib.asamd_csr_plan_create(None, a.rows, a.cols, a.nnz, da.row_ptr.c_ptr(), da.col.c_ptr(), da.val.c_ptr(),
                                             a.base, a.dtype.itemsize, 2, byref(plan)) == 0
            st = lib.asamd_csr_plan_stats(plan).contents
            assert st.ell_built == want, a.name
            if want:
                assert st.ell_width == int(np.diff(a.row_ptr).max())
            assert (lib.asamd_csr_plan_set_algo(plan, capi.ASAMD_SPMV_ELL) == 0) == bool(want)
        finally:
            lib.asamd_csr_plan_destroy(plan)
            da.free()


def test_deterministic_across_runs(gpu):
    a = wl.powerlaw_rmat(15, 200000, np.float32)
    x, y0 = _vectors(a)
    da = DeviceCsr(a)
    try:
        # the families that sum every row in a fixed order (no floating-point atomics)
        # (the tiled copy of this matrix has tiles too long for its second phase: the third phase runs)
        for algo in ("merge", "hot", "binned", "vector", "tiled", "xlds"):
            announce("spmv determinism", algo)
            runs = [run_plan_csrmv(da, algo, 1.0, x, 0.5, y0) for _ in range(3)]
            assert np.array_equal(runs[0], runs[1]) and np.array_equal(runs[0], runs[2]), algo
        lib, plan = capi.load(), c_void_p()
        assert lib.asamd_csr_plan_create(None, a.rows, a.cols, a.nnz, da.row_ptr.c_ptr(), da.col.c_ptr(), da.val.c_ptr(),
                                         a.base, a.dtype.itemsize, 2, byref(plan)) == 0
        st = lib.asamd_csr_plan_stats(plan).contents
        built, long_blocks = st.tiled_built, st.tile_long_blocks
        lib.asamd_csr_plan_destroy(plan)
        assert built and long_blocks > 0, "the tiled copy was meant to have long tiles"
    finally:
        da.free()


def test_analysis_statistics(gpu):
    lengths = [0, 1, 2, 3, 4, 7, 8, 100, 1024, 0, 5]
    a = csr_from_lengths(lengths, 5000, np.float32)
    da = DeviceCsr(a)
    try:
        announce("analysis stats")
        st = plan_stats(da)
        assert st["min_len"] == 0 and st["max_len"] == 1024 and st["const_len"] == -1
        want = [0] * capi.ASAMD_HIST_BINS
        for n in lengths:
            want[0 if n == 0 else int(n).bit_length()] += 1
        assert st["hist"] == want
        assert sum(st["hist"]) == a.rows
    finally:
        da.free()
    a = wl.uniform_rows(2048, 2048, 16, np.float32)
    da = DeviceCsr(a)
    try:
        st = plan_stats(da)
        assert st["const_len"] == 16 and st["algo"] == capi.ASAMD_SPMV_ROWCONST
        st = plan_stats(da, trusted=0)
        assert st["algo"] != capi.ASAMD_SPMV_ROWCONST  # untrusted structure never skips row_ptr
    finally:
        da.free()


@pytest.mark.parametrize("dtype", [np.float32, np.float64], ids=["f32", "f64"])
def test_explicit_analysis_and_garbage_info(gpu, dtype):
    """csrmv with (a) info == NULL, (b) an analysed info, (c) a hand-allocated info
    full of garbage (as the reference's own fp64 test passes), (d) after clear."""
    lib = capi.load()
    a = wl.powerlaw_rmat(13, 4000, dtype)
    x, y0 = _vectors(a)
    da = DeviceCsr(a)
    descr = capi.make_descr()
    p = capi.prefix(dtype)
    try:
        announce("csrmv info NULL")
        check_spmv(a, 2.0, x, 3.0, y0, run_csrmv(gpu, da, 2.0, x, 3.0, y0), "null info")
        info = capi.alphasparse_dcu_mat_info_t()
        assert lib.alphasparse_dcu_create_mat_info(byref(info)) == 0
        st = getattr(lib, "alphasparse_dcu_%s_csrmv_analysis" % p)(
            gpu.h, 0, a.rows, a.cols, a.nnz, byref(descr), da.val.c_ptr(), da.row_ptr.c_ptr(), da.col.c_ptr(), info)
        assert st == 0
        assert info.contents.csrmv_info.contents.m == a.rows and info.contents.csrmv_info.contents.nnz == a.nnz
        announce("csrmv analysed info")
        check_spmv(a, 2.0, x, 3.0, y0, run_csrmv(gpu, da, 2.0, x, 3.0, y0, info), "analysed info")
        assert lib.alphasparse_dcu_csrmv_clear(gpu.h, info) == 0
        announce("csrmv cleared info")
        check_spmv(a, 2.0, x, 3.0, y0, run_csrmv(gpu, da, 2.0, x, 3.0, y0, info), "cleared info")
        assert lib.alphasparse_dcu_destroy_mat_info(info) == 0
        garbage = (capi._alphasparse_dcu_mat_info * 1)()
        np.frombuffer(garbage, dtype=np.uint8)[:] = 0xA5
        announce("csrmv garbage info")
        check_spmv(a, 2.0, x, 3.0, y0, run_csrmv(gpu, da, 2.0, x, 3.0, y0, garbage), "garbage info")
    finally:
        da.free()


def test_lazy_cache_survives_structure_change_at_same_address(gpu):
    """Two different structures with equal (m, nnz) living at the same device
    address one after the other: the cached lazy plan may be stale, results may not."""
    lens1 = [1] * 4000 + [4000]
    lens2 = [4000] + [1] * 4000
    a1 = csr_from_lengths(lens1, 9000, np.float32, seed=1)
    a2 = csr_from_lengths(lens2, 9000, np.float32, seed=2)
    assert a1.nnz == a2.nnz and a1.rows == a2.rows
    da = DeviceCsr(a1)
    try:
        x, y0 = _vectors(a1)
        announce("lazy plan structure 1")
        check_spmv(a1, 1.0, x, 0.5, y0, run_csrmv(gpu, da, 1.0, x, 0.5, y0), "structure 1")
        da.row_ptr.copy_from(a2.row_ptr)
        da.col.copy_from(a2.col_ind)
        da.val.copy_from(a2.values)
        da.a = a2
        announce("lazy plan structure 2 at the same address")
        check_spmv(a2, 1.0, x, 0.5, y0, run_csrmv(gpu, da, 1.0, x, 0.5, y0), "structure 2")
    finally:
        da.free()


@pytest.mark.parametrize("dtype", [np.float32, np.float64], ids=["f32", "f64"])
def test_handle_api_host_and_device(gpu, dtype):
    """create_csr -> host2device -> mv_dcu (device vectors) and alphasparse_?_mv
    (host vectors, computed on the GPU) -> export -> destroy."""
    lib = capi.load()
    p = capi.prefix(dtype)
    T = capi.scalar_type(dtype)
    for base, maker in ((0, lambda: wl.powerlaw_rmat(12, 3000, dtype)), (1, lambda: wl.uniform_rows(2000, 1500, 16, dtype, base=1))):
        a = maker()
        x, y0 = _vectors(a)
        A = capi.alphasparse_matrix_t()
        rs = np.ascontiguousarray(a.row_ptr[:-1])
        re = np.ascontiguousarray(a.row_ptr[1:])
        st = getattr(lib, "alphasparse_%s_create_csr" % p)(byref(A), base, a.rows, a.cols, capi.ptr(rs), capi.ptr(re),
                                                           capi.ptr(a.col_ind), capi.ptr(a.values))
        assert st == 0
        a0 = wl.Csr(a.rows, a.cols, (a.row_ptr - base).astype(np.int32), (a.col_ind - base).astype(np.int32), a.values, 0, a.name)
        announce("host api mv", a.name)
        y = y0.copy()
        st = getattr(lib, "alphasparse_%s_mv" % p)(0, T(1.5), A, capi.alpha_matrix_descr(0, 0, 0), capi.ptr(x), T(0.5), capi.ptr(y))
        assert st == 0
        check_spmv(a0, 1.5, x, 0.5, y0, y, "alphasparse_mv host")
        announce("mv_dcu", a.name)
        dx, dy = hiprt.DeviceArray.from_numpy(x), hiprt.DeviceArray.from_numpy(y0)
        al, be = T(-2.0), T(1.0)
        descr = capi.make_descr()
        st = getattr(lib, "alphasparse_%s_mv_dcu" % p)(gpu.h, 0, byref(al), A, byref(descr), dx.c_ptr(), byref(be), dy.c_ptr())
        assert st == 0
        hiprt.synchronize()
        check_spmv(a0, -2.0, x, 1.0, y0, dy.to_numpy(), "mv_dcu")
        assert lib.alphasparse_destroy(A) == 0
        dx.free()
        dy.free()


@pytest.mark.parametrize("seed", range(48))
def test_random_structures_every_family(gpu, seed):
    """Seeded sweep over odd shapes: tiny and lopsided dimensions, mixtures of empty, short and very
    long rows, both index bases and precisions, through every kernel family (the tiled and ELL copies
    are forced so that they see shapes their size thresholds would never give them)."""
    rng = np.random.default_rng(1000 + seed)
    dtype = [np.float32, np.float64][seed % 2]
    base = (seed // 2) % 2
    m = int(rng.choice([1, 2, 63, 64, 65, 257, 1000, 4097]))
    n = int(rng.choice([1, 2, 255, 256, 257, 1000, 33000, 70001]))
    kind = seed % 4
    if kind == 0:
        lens = rng.integers(0, min(n, 6) + 1, m)
    elif kind == 1:
        lens = np.minimum(rng.geometric(0.08, m) - 1, n)
    elif kind == 2:
        lens = np.where(rng.random(m) < 0.7, 0, rng.integers(1, min(n, 40) + 1, m))
    else:
        lens = np.minimum(rng.zipf(1.5, m), n)
    if m > 2:
        lens[rng.integers(0, m)] = min(n, 9000)       # one long row
    a = csr_from_lengths([int(v) for v in lens], n, dtype, seed=seed + 1, base=base)
    if a.nnz == 0:
        a = csr_from_lengths([min(n, 3)] + [0] * (m - 1), n, dtype, seed=seed + 1, base=base)
    x, y0 = _vectors(a, seed)
    da = DeviceCsr(a)
    try:
        for algo in ("vector", "merge", "scalar", "rowconst", "stream", "tiled", "ell", "hot", "binned", "xlds", "auto"):
            for alpha, beta in ((1.5, 0.0), (-2.0, 0.5)):
                announce("spmv random", seed, m, n, a.nnz, np.dtype(dtype).name, base, algo, alpha, beta)
                y = run_plan_csrmv(da, algo, alpha, x, beta, y0)
                if y is None:
                    continue
                check_spmv(a, alpha, x, beta, y0, y, "seed %d %dx%d %s" % (seed, m, n, algo))
        announce("spmv random api", seed)
        check_spmv(a, 1.0, x, 1.0, y0, run_csrmv(gpu, da, 1.0, x, 1.0, y0), "seed %d api" % seed)
    finally:
        da.free()


@pytest.mark.parametrize("dtype", [np.float32, np.float64], ids=["f32", "f64"])
def test_unsorted_and_duplicate_columns_and_non_finite_values(gpu, dtype):
    """CSR does not promise sorted or distinct columns inside a row (alphasparse_convert_csr keeps
    duplicates): every family must sum such rows like the plain kernel does.  Infinities and NaNs
    travel to exactly the rows whose entries hold or meet them."""
    rng = np.random.default_rng(77)
    m, n = 3000, 2000
    lens = np.minimum(rng.geometric(0.1, m), 60)
    lens[5] = 5000
    rp = np.zeros(m + 1, dtype=np.int32)
    np.cumsum(lens, out=rp[1:])
    col = rng.integers(0, n, int(rp[-1])).astype(np.int32)          # unsorted, with repeats
    val = rng.uniform(-1, 1, col.size).astype(dtype)
    a = wl.Csr(m, n, rp, col, val, 0, "unsorted-duplicates")
    x, y0 = _vectors(a, 5)
    da = DeviceCsr(a)
    try:
        for algo in ("vector", "merge", "scalar", "stream", "tiled", "ell", "hot", "binned", "xlds", "auto"):
            announce("spmv unsorted", np.dtype(dtype).name, algo)
            y = run_plan_csrmv(da, algo, 1.5, x, 0.5, y0)
            if y is not None:
                check_spmv(a, 1.5, x, 0.5, y0, y, "unsorted %s" % algo)
    finally:
        da.free()
    # non-finite values: row 7 holds +inf, row 9 meets a NaN in x, row 11 has inf - inf
    val2 = val.copy()
    x2 = x.copy()
    val2[rp[7]] = np.inf
    x2[col[rp[7]]] = 1.0
    x2[col[rp[9]]] = np.nan
    val2[rp[11]], val2[rp[11] + 1] = np.inf, -np.inf
    x2[col[rp[11]]], x2[col[rp[11] + 1]] = 1.0, 1.0
    b = wl.Csr(m, n, rp, col, val2, 0, "non-finite")
    with np.errstate(invalid="ignore", over="ignore"):
        ref = orc.csrmv_plain(b, 1.0, x2, 0.0, y0)
    db = DeviceCsr(b)
    try:
        for algo in ("vector", "merge", "scalar", "tiled", "hot", "binned", "xlds", "auto"):
            announce("spmv non-finite", np.dtype(dtype).name, algo)
            y = run_plan_csrmv(db, algo, 1.0, x2, 0.0, y0)
            assert np.array_equal(np.isnan(y), np.isnan(ref)), algo
            assert np.array_equal(np.isinf(y), np.isinf(ref)) and np.array_equal(np.sign(y[np.isinf(y)]), np.sign(ref[np.isinf(ref)])), algo
            finite = np.isfinite(ref)
            assert np.isnan(ref[9]) and np.isnan(ref[11]) and np.isinf(ref[7]) and finite.sum() >= m - 300
    finally:
        db.free()


@pytest.mark.parametrize("algo", ["tiled", "ell"])
def test_copy_is_not_used_for_another_value_array(gpu, algo):
    """The tiled and ELL copies hold the values they were built from.  A multiply that passes a different
    value array (same structure, new numbers) must be computed from the new numbers."""
    from ctypes import c_void_p
    lib = capi.load()
    a = wl.uniform_rows(6000, 5000, 8, np.float32)
    x, y0 = wl.uniform(a.cols, a.dtype, 3), wl.uniform(a.rows, a.dtype, 4)
    da = DeviceCsr(a)
    new_vals = (a.values * np.float32(-3.0) + np.float32(0.25)).astype(np.float32)
    b = wl.Csr(a.rows, a.cols, a.row_ptr, a.col_ind, new_vals, a.base, "new values")
    d_new = hiprt.DeviceArray.from_numpy(new_vals)
    plan = c_void_p()
    try:
        assert lib.asamd_csr_plan_create(None, a.rows, a.cols, a.nnz, da.row_ptr.c_ptr(), da.col.c_ptr(), da.val.c_ptr(),
                                         a.base, 4, 2, byref(plan)) == 0
        assert lib.asamd_csr_plan_set_algo(plan, ALGOS[algo]) == 0
        for vals, mat in ((da.val, a), (d_new, b), (da.val, a)):
            announce("value array", algo, mat.name)
            dx, dy = hiprt.DeviceArray.from_numpy(x), hiprt.DeviceArray.from_numpy(y0)
            ws = capi.Workspace(lib, plan)
            assert capi.plan_csrmv(lib, None, plan, 0, c_float(1.5), vals.c_ptr(), da.row_ptr.c_ptr(), da.col.c_ptr(),
                                   dx.c_ptr(), c_float(0.5), dy.c_ptr(), ws) == 0
            hiprt.synchronize()
            y = dy.to_numpy()
            dx.free()
            dy.free()
            err = orc.csrmv_err(mat, 1.5, x, 0.5, y0, y, orc.csrmv_plain(mat, 1.5, x, 0.5, y0))
            assert err.full <= TOL[a.dtype] and err.zero_den_mismatch == 0, (mat.name, err)
    finally:
        lib.asamd_csr_plan_destroy(plan)
        da.free()
        d_new.free()


@pytest.mark.parametrize("tune", ["model", "timed"])
def test_analysis_choices(gpu, tune, monkeypatch):
    """What the analysis decides and what it skips: a banded matrix runs the staged row-block kernel on the
    caller's arrays, or the ELL copy if that is at least 5 % faster by the analysis' model (or, with
    ALSPARSE_AMD_TUNE=timed, by its timing run), the value guard's launches in front of the copy counted, and never
    lays out the tiled copy (slower than either); a matrix small enough to be launch-bound takes the
    single-kernel path however skewed its rows are."""
    monkeypatch.setenv("ALSPARSE_AMD_TUNE", tune)
    lib = capi.load()
    a, x, y0, alpha, beta, _ = wl.config(2)
    da = DeviceCsr(a)
    info = capi.alphasparse_dcu_mat_info_t()
    assert lib.alphasparse_dcu_create_mat_info(byref(info)) == 0
    descr = capi.make_descr(base=a.base)
    try:
        announce("analysis choices", a.name)
        assert lib.alphasparse_dcu_d_csrmv_analysis(gpu.h, 0, a.rows, a.cols, a.nnz, byref(descr), da.val.c_ptr(),
                                                    da.row_ptr.c_ptr(), da.col.c_ptr(), info) == 0
        st = lib.asamd_analysis_stats(info).contents
        assert st.algo in (capi.ASAMD_SPMV_ELL, capi.ASAMD_SPMV_STREAM), capi.ALGO_NAMES[st.algo]
        assert st.ell_built == (1 if st.algo == capi.ASAMD_SPMV_ELL else 0) and st.tiled_built == 0
        assert st.tune_ms_ell > 0 and st.tune_ms_base > 0
        # timed: the tiled copy was not even tried; model: its estimate is there, and slower
        assert st.tune_ms_tiled == 0 if tune == "timed" else st.tune_ms_tiled > st.tune_ms_base
        # (the model's estimate of a copy that holds values counts the value guard's launches, 0.022 ms; the timing
        # run times the kernels alone and adds them before it compares)
        ell_cost = st.tune_ms_ell + (0.022 if tune == "timed" else 0.0)
        assert (st.algo == capi.ASAMD_SPMV_ELL) == (ell_cost < 0.95 * st.tune_ms_base), (st.tune_ms_ell, st.tune_ms_base)
        check_spmv(a, alpha, x, beta, y0, run_csrmv(gpu, da, alpha, x, beta, y0, info), "config 2 analysed")
    finally:
        lib.alphasparse_dcu_destroy_mat_info(info)
        da.free()
    b = csr_from_lengths([0, 1, 700, 3, 0, 2, 2, 9] * 40, 5000, np.float32)
    db = DeviceCsr(b)
    try:
        xb, yb = wl.uniform(b.cols, b.dtype, 3), wl.uniform(b.rows, b.dtype, 4)
        announce("analysis choices", b.name)
        check_spmv(b, 1.0, xb, 0.0, yb, run_csrmv(gpu, db, 1.0, xb, 0.0, yb), "small skewed, lazy")
        st = lib.asamd_analysis_stats(db.row_ptr.c_ptr()).contents
        assert st.algo == capi.ASAMD_SPMV_VECTOR, capi.ALGO_NAMES[st.algo]
    finally:
        db.free()


@pytest.mark.parametrize("dtype", [np.float32, np.float64], ids=["f32", "f64"])
@pytest.mark.parametrize("per_row", [1, 2, 5])
def test_tiled_second_phase_in_both_forms(gpu, dtype, per_row, monkeypatch):
    """The tiled copy's second phase takes one or two entries per lane and tile.  Both forms, forced and as
    the analysis picks them, on structures whose tiles hold around 32, 64 and 128+ entries (2048 rows x one
    column block each): tiles too long for the form in use must reach the long-tile kernel instead."""
    from ctypes import c_void_p
    lib = capi.load()
    a = wl.uniform_rows(3 * 2048 + 77, 1 << 20, per_row, dtype)
    x, y0 = _vectors(a)
    da = DeviceCsr(a)
    T = capi.scalar_type(a.dtype)
    # what the analysis must pick where the tile sizes leave no doubt (blocks are cut to even entry counts,
    # so tiles hold somewhat under 2048 rows x per_row x block width / columns: mean about 25: hardly a tile
    # above 64; about 100: most entries in tiles of 65..128)
    clear = {("float64", 1): 1, ("float32", 2): 2}
    try:
        for forced in (None, "1", "2"):
            if forced is None:
                monkeypatch.delenv("ALSPARSE_AMD_TILED_HALVES", raising=False)
            else:
                monkeypatch.setenv("ALSPARSE_AMD_TILED_HALVES", forced)
            plan = c_void_p()
            announce("tiled forms", np.dtype(dtype).name, per_row, forced)
            assert lib.asamd_csr_plan_create(None, a.rows, a.cols, a.nnz, da.row_ptr.c_ptr(), da.col.c_ptr(),
                                             da.val.c_ptr(), a.base, a.dtype.itemsize, 2, byref(plan)) == 0
            try:
                st = lib.asamd_csr_plan_stats(plan).contents
                assert st.tiled_built == 1
                if forced is None:  # few entries in tiles of 65..128 entries <=> one entry per lane
                    want = clear.get((np.dtype(dtype).name, per_row))
                    assert st.tile_entries_per_lane in ((1, 2) if want is None else (want,)), st.tile_entries_per_lane
                else:
                    assert st.tile_entries_per_lane == int(forced)
                assert lib.asamd_csr_plan_set_algo(plan, ALGOS["tiled"]) == 0
                ws = capi.Workspace(lib, plan)
                for alpha, beta in ((1.0, 0.0), (-1.5, 0.5)):
                    dx, dy = hiprt.DeviceArray.from_numpy(x), hiprt.DeviceArray.from_numpy(y0)
                    assert capi.plan_csrmv(lib, None, plan, 0, T(alpha), da.val.c_ptr(), da.row_ptr.c_ptr(), da.col.c_ptr(),
                                           dx.c_ptr(), T(beta), dy.c_ptr(), ws) == 0
                    hiprt.synchronize()
                    y = dy.to_numpy()
                    dx.free()
                    dy.free()
                    check_spmv(a, alpha, x, beta, y0, y, "tiled form %s, %d per row" % (forced, per_row))
            finally:
                lib.asamd_csr_plan_destroy(plan)
    finally:
        da.free()


@pytest.mark.parametrize("m,n,per_row", [(1 << 21, 1 << 21, 16), (1 << 19, 1 << 21, 128)], ids=["16_per_row", "128_per_row"])
def test_tiled_row_blocks_follow_the_tile_population(gpu, m, n, per_row):
    """2 M x 2 M with 16 entries per row: 52 column blocks (40 960 columns each), so a 2 048-row block would put
    630 entries into every tile and leave them all to the long-tile kernel.  The analysis cuts the blocks to
    about 200 rows (about 60 entries per tile), and the tiled pair then wins its timing run against the row
    kernels.  With 128 entries per row even the shortest row block (64 rows) would overfill its tiles: the
    column blocks are made narrower as well (about 128 of them instead of 52)."""
    lib = capi.load()
    a = wl.uniform_rows(m, n, per_row, np.float32)
    x, y0 = _vectors(a)
    da = DeviceCsr(a)
    info = capi.alphasparse_dcu_mat_info_t()
    assert lib.alphasparse_dcu_create_mat_info(byref(info)) == 0
    descr = capi.make_descr(base=a.base)
    try:
        announce("tile population", a.name)
        assert lib.alphasparse_dcu_s_csrmv_analysis(gpu.h, 0, a.rows, a.cols, a.nnz, byref(descr), da.val.c_ptr(),
                                                    da.row_ptr.c_ptr(), da.col.c_ptr(), info) == 0
        st = lib.asamd_analysis_stats(info).contents
        assert st.tiled_built == 1 and st.algo == capi.ASAMD_SPMV_TILED, capi.ALGO_NAMES[st.algo]
        assert 6000 <= st.tile_row_blocks <= 12000, st.tile_row_blocks
        mean_tile = a.nnz / (st.tile_row_blocks * st.tile_col_blocks)
        assert 40 <= mean_tile <= 80, mean_tile
        assert 0 < st.tune_ms_tiled < st.tune_ms_base
        assert (st.tile_col_blocks > 100) == (per_row == 128), st.tile_col_blocks
        check_spmv(a, 1.5, x, 0.5, y0, run_csrmv(gpu, da, 1.5, x, 0.5, y0, info), "%d per row analysed" % per_row)
    finally:
        lib.alphasparse_dcu_destroy_mat_info(info)
        da.free()


@pytest.mark.parametrize("maker", [lambda: wl.powerlaw_rmat(13, 3000, np.float32), lambda: wl.uniform_rows(5000, 7000, 16, np.float32),
                                   lambda: wl.laplace2d(64, 48, np.float32)], ids=["powerlaw", "uniform16", "laplace"])
def test_row_ptr_into_the_middle_of_larger_arrays(gpu, maker):
    """row_ptr[0] > base: the matrix is a row slice of a larger one whose col / val arrays are passed whole.
    The reference's kernel indexes with the absolute offsets (dcu_gemv_vector.h:38-45); every path here must
    see the same entries: un-analysed, analysed (no merge-path, no re-ordered copy) and transposed."""
    lib = capi.load()
    a = maker()
    lead = 777
    rng = np.random.default_rng(5)
    big = wl.Csr(a.rows, a.cols, (a.row_ptr + lead).astype(np.int32),
                 np.concatenate([rng.integers(0, a.cols, lead).astype(np.int32), a.col_ind]),
                 np.concatenate([rng.uniform(-9, 9, lead).astype(a.dtype), a.values]), a.base, a.name + "+lead")
    assert big.nnz == a.nnz + lead
    x, y0 = _vectors(a)
    xt, yt0 = wl.uniform(a.rows, a.dtype, 5), wl.uniform(a.cols, a.dtype, 6)
    da = DeviceCsr(big)
    da.a = wl.Csr(a.rows, a.cols, big.row_ptr, big.col_ind, big.values, a.base, big.name)
    da.a.nnz = a.nnz  # what the caller passes as nnz: the entries of these rows
    info = capi.alphasparse_dcu_mat_info_t()
    assert lib.alphasparse_dcu_create_mat_info(byref(info)) == 0
    descr = capi.make_descr(base=a.base)
    try:
        announce("row_ptr[0] > base", a.name)
        check_spmv(a, 1.5, x, 0.5, y0, run_csrmv(gpu, da, 1.5, x, 0.5, y0), "un-analysed")
        assert lib.alphasparse_dcu_s_csrmv_analysis(gpu.h, 1, a.rows, a.cols, a.nnz, byref(descr), da.val.c_ptr(),
                                                    da.row_ptr.c_ptr(), da.col.c_ptr(), info) == 0
        st = lib.asamd_analysis_stats(info).contents
        assert st.first_offset == lead
        assert st.algo in (capi.ASAMD_SPMV_VECTOR, capi.ASAMD_SPMV_STREAM), capi.ALGO_NAMES[st.algo]
        assert st.tiled_built == 0 and st.ell_built == 0 and st.transpose_built == 0
        check_spmv(a, 1.5, x, 0.5, y0, run_csrmv(gpu, da, 1.5, x, 0.5, y0, info), "analysed")
        # transposed: the scatter route
        dx, dy = hiprt.DeviceArray.from_numpy(xt), hiprt.DeviceArray.from_numpy(yt0)
        al, be = c_float(1.5), c_float(0.5)
        assert lib.alphasparse_dcu_s_csrmv(gpu.h, 1, a.rows, a.cols, a.nnz, byref(al), byref(descr), da.val.c_ptr(),
                                           da.row_ptr.c_ptr(), da.col.c_ptr(), info, dx.c_ptr(), byref(be), dy.c_ptr()) == 0
        hiprt.synchronize()
        got = dy.to_numpy()
        ref = orc.csrmv_trans_plain(a, 1.5, xt, 0.5, yt0)
        err = orc.csrmv_err(orc.transpose(a), 1.5, xt, 0.5, yt0, got, ref)
        assert err.zero_den_mismatch == 0 and err.full <= TOL[a.dtype], err
        dx.free()
        dy.free()
    finally:
        lib.alphasparse_dcu_destroy_mat_info(info)
        da.free()


@pytest.mark.parametrize("dtype", [np.float32, np.float64], ids=["f32", "f64"])
def test_structure_swapped_under_an_unanalysed_plan(gpu, dtype):
    """Un-analysed calls remember row statistics per row_ptr address and pick the staged row-block kernel for
    short rows.  Another matrix of the same m, n and nnz written over the arrays in place is multiplied with
    those stale statistics: workgroups whose rows no longer fit the staging area must take them straight from
    the arrays (the result is right whatever the statistics said), and nothing may be written out of bounds."""
    lib = capi.load()
    m, cols = 4096, 3000
    a1 = csr_from_lengths([5] * m, cols, dtype)
    lengths = np.zeros(m, dtype=np.int64)
    lengths[0:6] = 3000
    lengths[300:300 + 496] = 5
    a2 = csr_from_lengths(list(lengths), cols, dtype, seed=11)
    assert a1.nnz == a2.nnz == 5 * m
    x, y0 = _vectors(a1)
    da = DeviceCsr(a1)
    try:
        announce("structure swapped under a lazy plan", np.dtype(dtype).name, "first structure")
        check_spmv(a1, 1.5, x, 0.5, y0, run_csrmv(gpu, da, 1.5, x, 0.5, y0), "first structure")
        st = lib.asamd_analysis_stats(da.row_ptr.c_ptr()).contents
        assert st.algo == capi.ASAMD_SPMV_STREAM and st.trusted == 0, capi.ALGO_NAMES[st.algo]
        da.row_ptr.copy_from(a2.row_ptr)
        da.col.copy_from(a2.col_ind)
        da.val.copy_from(a2.values)
        da.a = a2
        announce("structure swapped under a lazy plan", np.dtype(dtype).name, "second structure, stale statistics")
        check_spmv(a2, 1.5, x, 0.5, y0, run_csrmv(gpu, da, 1.5, x, 0.5, y0), "second structure")
        st = lib.asamd_analysis_stats(da.row_ptr.c_ptr()).contents
        assert st.algo == capi.ASAMD_SPMV_STREAM and st.max_len == 5, "the statistics were meant to be stale"
    finally:
        da.free()


def test_lazy_analyses_are_bounded(gpu):
    """10 000 un-analysed matrices at distinct row_ptr addresses multiplied one after the other: the library
    remembers at most 64 lazy analyses (least recently used goes), device memory stays put, a matrix whose
    record was evicted still multiplies correctly, and a handle's records go with the handle."""
    lib = capi.load()
    a = csr_from_lengths([3, 0, 5, 1, 7, 2, 0, 4], 40, np.float32)
    x, y0 = _vectors(a)
    count = 10000
    stride = 16  # ints per copy of row_ptr: 64 bytes apart
    pool = np.zeros(count * stride, dtype=np.int32)
    for k in range(count):
        pool[k * stride:k * stride + a.rows + 1] = a.row_ptr
    d_pool = hiprt.DeviceArray.from_numpy(pool)
    d_col, d_val = hiprt.DeviceArray.from_numpy(a.col_ind), hiprt.DeviceArray.from_numpy(a.values)
    dx, dy = hiprt.DeviceArray.from_numpy(x), hiprt.DeviceArray.from_numpy(y0)
    h = capi.Handle()
    descr = capi.make_descr()
    al, be = c_float(1.0), c_float(0.0)

    def multiply(k):
        rp = c_void_p(d_pool.ptr + 4 * stride * k)
        assert lib.alphasparse_dcu_s_csrmv(h.h, 0, a.rows, a.cols, a.nnz, byref(al), byref(descr), d_val.c_ptr(), rp,
                                           d_col.c_ptr(), None, dx.c_ptr(), byref(be), dy.c_ptr()) == 0
    try:
        announce("lazy analyses bounded")
        before = lib.asamd_registry_lazy_count()
        for k in range(200):
            multiply(k)
        hiprt.synchronize()
        free_mid, _ = hiprt.mem_info()
        assert lib.asamd_registry_lazy_count() <= 64
        for k in range(200, count):
            multiply(k)
        hiprt.synchronize()
        free_end, _ = hiprt.mem_info()
        assert lib.asamd_registry_lazy_count() <= 64
        assert free_mid - free_end <= 8 << 20, "device memory grew by %d bytes over 9 800 more matrices" % (free_mid - free_end)
        multiply(0)  # evicted long ago
        hiprt.synchronize()
        check_spmv(a, 1.0, x, 0.0, y0, dy.to_numpy(), "evicted matrix")
        h.close()
        assert lib.asamd_registry_lazy_count() <= before, "a handle's lazy analyses go with the handle"
    finally:
        h.close()
        for d in (d_pool, d_col, d_val, dx, dy):
            d.free()
