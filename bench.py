#!/usr/bin/env python3
"""Benchmark of the CSR SpMV hot path on one MI355X.

A "step" is one y <- alpha*A*x + beta*y through the C API
(alphasparse_dcu_?_csrmv after alphasparse_dcu_?_csrmv_analysis) on a synthetic
matrix that is resident in HBM before the timed region starts.  The default
workload is benchmark configuration 3 (fp32, 16 777 216 rows x 16 entries per
row, beta = 0.5), the one the bandwidth target is stated on; --config selects
2 (fp64 Laplacian), 4 (fp32 power-law) or 5 (fp32 SpMM, n = 64) instead and
--all appends their figures under "others".

Prints ONE JSON line: metric/value (effective GB/s under the algorithmic bytes
model), roofline (against 8 TB/s HBM3E) and cpu_baseline (the reference's
OpenMP kernel, or its restatement, on the host cores -- reported, not a target).
"""
import argparse
import json
import os
import sys
import time
from ctypes import byref, c_void_p

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0
NO_ANALYSIS = False  # --no-analysis

# HBM bytes per multiply measured with rocprofv3 in separate counter runs (FETCH_SIZE x 2.000 + WRITE_SIZE x 1.000,
# factors from a 1 GiB copy kernel) -- a table of earlier measurements, not an in-run reading; each entry names the
# summary under profiles/ it comes from.  Keyed by (configuration, kernel family); anything else reports null.
MEASURED_TRAFFIC_BYTES = {
    (3, "tiled two-phase"): (5.17e9, "profiles/spmv_tiled_C3.txt"),
    (3, "rowconst"): (34.6e9, "profiles/spmv_tiled_C3.txt"),
    (4, "merge-path"): (3.19e9, "profiles/spmv_merge_C4.txt"),
    (4, "merge-path, hot columns in LDS"): (2.85e9, "profiles/spmv_merge_hot_C4.txt"),
    (2, "ell copy"): (356.6e6, "profiles/spmv_ell_copy_C2.txt"),
    (2, "row-block stream"): (338.8e6, "profiles/spmv_stream_C2.txt"),
    (5, "spmm row-major"): (9.27e9, "profiles/spmm_rowmajor_C5.txt"),
}


def measured_traffic(cfg, kernel):
    """(bytes, source file) of the counter measurement recorded for this configuration and kernel, or (None, None)."""
    return MEASURED_TRAFFIC_BYTES.get((cfg, kernel), (None, None))


WORKLOAD_NAMES = {
    2: "C2: CSR SpMV fp64, 5-point Laplacian 2048x2048 (4194304 rows, 20963328 nnz), alpha=1 beta=0",
    3: "C3: CSR SpMV fp32, 16777216 rows x 16 nnz/row uniform random sorted columns (268435456 nnz), alpha=1 beta=0.5",
    4: "C4: CSR SpMV fp32, power-law rows (Zipf 2, <=200000) x R-MAT columns, 8388608 rows, alpha=1 beta=0",
    5: "C5: CSR SpMM fp32, 1048576 rows x 32 nnz/row, B/C 1048576x64 row-major, alpha=1.5 beta=0.5",
}


def log(*a):
    print(*a, file=sys.stderr, flush=True)


def time_steps(fn, steps, warmup, hiprt):
    """HIP-event timing on the stream the library launches on (the handle's stream is the
    null stream), bracketed by device synchronisation.  The K steps are timed once
    back to back between two events (avg_ms: what a caller's loop sees) and once
    more with an event after every step (min / median; each event costs a few
    microseconds of gap, which shows on the 60 us kernels)."""
    for _ in range(warmup):
        fn()
    hiprt.synchronize()
    e0, e1 = hiprt.Event(), hiprt.Event()
    t0 = time.perf_counter()
    e0.record()
    for _ in range(steps):
        fn()
    e1.record()
    e1.synchronize()
    hiprt.synchronize()
    wall_ms = (time.perf_counter() - t0) * 1e3
    avg = e0.elapsed_ms(e1) / steps
    evs = [hiprt.Event() for _ in range(steps + 1)]
    evs[0].record()
    for i in range(steps):
        fn()
        evs[i + 1].record()
    evs[-1].synchronize()
    hiprt.synchronize()
    per = [evs[i].elapsed_ms(evs[i + 1]) for i in range(steps)]
    return {"avg_ms": float(avg), "min_ms": float(np.min(per)), "median_ms": float(np.median(per)),
            "per_step_events_avg_ms": float(np.mean(per)), "wall_ms_per_step": wall_ms / steps}


ROCSPARSE = "/opt/rocm/lib/librocsparse.so"


def vendor_spmv(a, x, y0, alpha, beta, nbytes, steps, warmup, transpose=False):
    """rocSPARSE's csrmv (with its analysis) on the same device arrays' contents, timed the same
    way: the vendor library that the reference's own tests compare against
    (test/dcu/level2/mv_csr_s_dcu_test.cpp:41-147).  A reported comparison, never part of the
    product; None when the library is not installed."""
    if not os.path.exists(ROCSPARSE):
        return None
    import ctypes
    from ctypes import c_double, c_float, c_int
    from alsparse_amd import hiprt
    R = ctypes.CDLL(ROCSPARSE)
    f32 = a.dtype == np.float32
    T, p = (c_float, "s") if f32 else (c_double, "d")
    h, descr, info = c_void_p(), c_void_p(), c_void_p()
    if R.rocsparse_create_handle(byref(h)) or R.rocsparse_create_mat_descr(byref(descr)) or R.rocsparse_create_mat_info(byref(info)):
        return None
    a0 = a
    d = [hiprt.DeviceArray.from_numpy(np.ascontiguousarray(v)) for v in (a0.values, a0.row_ptr - a0.base, a0.col_ind - a0.base, x, y0)]
    mv, an = getattr(R, "rocsparse_%scsrmv" % p), getattr(R, "rocsparse_%scsrmv_analysis" % p)
    P = c_void_p
    mv.argtypes = [P, c_int, c_int, c_int, c_int, P, P, P, P, P, P, P, P, P]
    an.argtypes = [P, c_int, c_int, c_int, c_int, P, P, P, P, P]
    op = 112 if transpose else 111  # rocsparse_operation_transpose / _none
    al, be = T(alpha), T(beta)
    t0 = time.perf_counter()
    st = an(h, op, a.rows, a.cols, a.nnz, descr, d[0].c_ptr(), d[1].c_ptr(), d[2].c_ptr(), info)
    hiprt.synchronize()
    analysis_ms = (time.perf_counter() - t0) * 1e3
    if st != 0:
        return None

    def step():
        s_ = mv(h, op, a.rows, a.cols, a.nnz, byref(al), descr, d[0].c_ptr(), d[1].c_ptr(), d[2].c_ptr(), info,
                d[3].c_ptr(), byref(be), d[4].c_ptr())
        if s_ != 0:
            raise RuntimeError("rocsparse csrmv status %d" % s_)
    t = time_steps(step, steps, warmup, hiprt)
    for v in d:
        v.free()
    R.rocsparse_destroy_mat_info(info)
    R.rocsparse_destroy_mat_descr(descr)
    R.rocsparse_destroy_handle(h)
    return {"library": "rocSPARSE csrmv after csrmv_analysis", "value": nbytes / t["avg_ms"] / 1e6, "unit": "GB/s",
            "ms": t["avg_ms"], "analysis_ms": analysis_ms}


def run_spmv(cfg, steps, warmup, cpu_baseline, check, transpose=False, vendor=False, cx=False, conjugate=False,
             analyse=None, structure_only=False, cold_copies=0, tune=None):
    """cx: the configuration's structure with complex values (complex64 for the fp32 configurations,
    complex128 for the fp64 one), complex x, y, alpha and beta; conjugate: A^H instead of A^T.
    structure_only: the analysis keeps no copy of the values (ALSPARSE_AMD_ANALYSIS=structure, what the reference's
    analysis keeps).  cold_copies = K > 1: the multiply is also timed rotating over K copies of the matrix and its
    vectors, each with an analysis of its own, so that no step finds anything of its operands in the 256 MB
    memory-side cache ("cold").  tune: "timed" makes the analysis time its candidates instead of deciding from its model (ALSPARSE_AMD_TUNE)."""
    from alsparse_amd import capi, hiprt, workloads as wl
    lib = capi.load()
    t0 = time.time()
    if isinstance(cfg, tuple) and cfg[0] == "bimodal":  # ("bimodal", rows, cols, short, long, every, dtype)
        _, um, un, ks, kl, every, udt = cfg
        a = wl.bimodal_rows(um, un, ks, kl, every, udt)
        x, y0, alpha, beta = wl.uniform(a.cols, udt, 3), wl.uniform(a.rows, udt, 4), 1.0, 0.5
        workload_name = ("two row lengths: CSR SpMV %s, %d rows x %d columns, every %d-th row %d entries, the others %d, "
                         "uniform random sorted columns, alpha=1 beta=0.5" % (np.dtype(udt).name, um, un, every, kl, ks))
    elif isinstance(cfg, tuple) and cfg[0] == "stencil3d":  # ("stencil3d", nx, ny, nz, dtype)
        _, gx, gy, gz, udt = cfg
        a = wl.stencil3d(gx, gy, gz, udt)
        x, y0, alpha, beta = wl.uniform(a.cols, udt, 3), wl.uniform(a.rows, udt, 4), 1.0, 0.5
        workload_name = "27-point stencil: CSR SpMV %s, %d x %d x %d grid (%d rows, %d nnz), alpha=1 beta=0.5" % (
            np.dtype(udt).name, gx, gy, gz, a.rows, a.nnz)
    elif isinstance(cfg, tuple) and cfg[0] == "laplace2d":  # ("laplace2d", nx, ny, dtype)
        _, gx, gy, udt = cfg
        a = wl.laplace2d(gx, gy, udt)
        x, y0, alpha, beta = wl.uniform(a.cols, udt, 3), wl.uniform(a.rows, udt, 4), 1.0, 0.5
        workload_name = "5-point Laplacian: CSR SpMV %s, %d x %d grid (%d rows, %d nnz), alpha=1 beta=0.5" % (
            np.dtype(udt).name, gx, gy, a.rows, a.nnz)
    elif isinstance(cfg, tuple):  # ("uniform", rows, cols, entries per row, dtype): not a benchmark configuration
        _, um, un, uk, udt = cfg
        a = wl.uniform_rows(um, un, uk, udt)
        x, y0, alpha, beta = wl.uniform(a.cols, udt, 3), wl.uniform(a.rows, udt, 4), 1.0, 0.5
        workload_name = "uniform rows: CSR SpMV %s, %d rows x %d columns, %d nnz/row uniform random sorted columns, alpha=1 beta=0.5" % (
            np.dtype(udt).name, um, un, uk)
    else:
        a, x, y0, alpha, beta, _ = wl.config(cfg)
        workload_name = WORKLOAD_NAMES[cfg]
    if cx:
        cdt = np.complex64 if a.dtype == np.float32 else np.complex128
        a = wl.complexify(a, cdt)
        x, y0 = wl.complex_vector(a.cols, cdt, 3), wl.complex_vector(a.rows, cdt, 4)
        alpha, beta = complex(alpha, -0.5), complex(beta, 0.25)
        cpu_baseline = vendor = False
    log("[bench] generated %s: %d rows, %d nnz in %.1f s" % (a.name, a.rows, a.nnz, time.time() - t0))
    T, p = capi.scalar_type(a.dtype), capi.prefix(a.dtype)
    h = capi.Handle()
    descr = capi.make_descr()
    d_val, d_rp, d_ci = (hiprt.DeviceArray.from_numpy(v) for v in (a.values, a.row_ptr, a.col_ind))
    op = capi.ALPHA_SPARSE_OPERATION_TRANSPOSE if transpose else capi.ALPHA_SPARSE_OPERATION_NON_TRANSPOSE
    if transpose and conjugate and cx:
        op = capi.ALPHA_SPARSE_OPERATION_CONJUGATE_TRANSPOSE
    if transpose:  # y = alpha*A^T*x + beta*y: x has `rows` entries, y has `cols`
        x, y0 = ((wl.complex_vector(a.rows, a.dtype, 3), wl.complex_vector(a.cols, a.dtype, 4)) if cx else
                 (wl.uniform(a.rows, a.dtype, 3), wl.uniform(a.cols, a.dtype, 4)))
    d_x, d_y = hiprt.DeviceArray.from_numpy(x), hiprt.DeviceArray.from_numpy(y0)

    info = capi.alphasparse_dcu_mat_info_t()
    assert lib.alphasparse_dcu_create_mat_info(byref(info)) == 0
    al, be = T(alpha), T(beta)
    csrmv = getattr(lib, "alphasparse_dcu_%s_csrmv" % p)
    # analyse=False: without alphasparse_dcu_?_csrmv_analysis (info = NULL); None: as --no-analysis says
    analysed = not (NO_ANALYSIS if analyse is None else not analyse)

    def step():
        s = csrmv(h.h, op, a.rows, a.cols, a.nnz, byref(al), byref(descr), d_val.c_ptr(), d_rp.c_ptr(),
                  d_ci.c_ptr(), info if analysed else None, d_x.c_ptr(), byref(be), d_y.c_ptr())
        if s != 0:
            raise RuntimeError("csrmv status %d" % s)

    env_set = {}
    if structure_only:
        env_set["ALSPARSE_AMD_ANALYSIS"] = "structure"
    if tune:
        env_set["ALSPARSE_AMD_TUNE"] = tune
    env_old = {k: os.environ.get(k) for k in env_set}
    os.environ.update(env_set)
    hiprt.synchronize()
    t0 = time.perf_counter()
    if analysed:
        st = getattr(lib, "alphasparse_dcu_%s_csrmv_analysis" % p)(
            h.h, op, a.rows, a.cols, a.nnz, byref(descr), d_val.c_ptr(), d_rp.c_ptr(), d_ci.c_ptr(), info)
        assert st == 0, "analysis status %d" % st
    else:
        step()  # the first call without analysis looks at row_ptr once and remembers what it saw
    hiprt.synchronize()
    analysis_ms = (time.perf_counter() - t0) * 1e3
    early_calls_ms = None
    if not analysed and not transpose:
        # Calls 2 to 5 on the same arrays, one at a time: the library counts them, and where its model expects a
        # tiled copy to pay even behind fingerprints of all three arrays it lays one out in the fourth call.
        early_calls_ms = []
        for _ in range(4):
            t1 = time.perf_counter()
            step()
            hiprt.synchronize()
            early_calls_ms.append((time.perf_counter() - t1) * 1e3)
    stats = lib.asamd_analysis_stats(info if analysed else d_rp.c_ptr()).contents
    if transpose and analysed:
        assert stats.transpose_built != 0, "no room for the transposed copy"
        stats = lib.asamd_analysis_transpose_stats(info).contents
    algo = capi.ALGO_NAMES.get(stats.algo, "?")
    if stats.algo == capi.ASAMD_SPMV_VECTOR:
        algo += "(W=%d)" % stats.vector_width
    if transpose and not analysed:
        algo = "scatter with atomics (no copy of the transpose; in LDS where y fits it)"
    watched = bool(not analysed and not transpose and lib.asamd_registry_lazy_promoted(h.h, d_rp.c_ptr()))
    if watched:
        algo = "tiled two-phase behind fingerprints of row_ptr, col_ind and csr_val (laid out by the 4th call)"

    parity = None
    if check and cx and transpose:
        log("[bench] parity of the complex transposed operations is covered by tests/test_gpu_complex.py, not here")
    elif check:
        from oracle import oracle as orc
        d_y.copy_from(y0)
        step()
        hiprt.synchronize()
        y = d_y.to_numpy()
        t0 = time.time()
        tol = 1e-4 if a.dtype.itemsize // (2 if cx else 1) == 4 else 1e-12
        if transpose:
            ref = orc.csrmv_trans_plain(a, alpha, x, beta, y0)
            absa = wl.Csr(a.rows, a.cols, a.row_ptr, a.col_ind, np.abs(a.values), a.base)
            den = abs(alpha) * orc.csrmv_trans_plain(absa, 1.0, np.abs(x), 0.0, np.zeros(a.cols, a.dtype)).astype(np.float64)
            diff = np.abs(y.astype(np.float64) - ref.astype(np.float64))
            zbad = int(np.count_nonzero(diff[den == 0]))
            strict = float(np.max(diff[den > 0] / den[den > 0])) if np.any(den > 0) else 0.0
            parity = {"max_row_err": strict, "tol": tol, "zero_den_mismatch": zbad, "ok": bool(strict <= tol and zbad == 0)}
        else:
            ref = orc.csrmv_plain(a, alpha, x, beta, y0)
            err = orc.csrmv_err(a, alpha, x, beta, y0, y, ref)
            parity = {"max_row_err": err.strict, "max_row_err_with_beta_y": err.full, "tol": tol,
                      "zero_den_mismatch": err.zero_den_mismatch, "reference_check_ratio": err.ref_ratio,
                      "ok": bool(err.strict <= tol and err.zero_den_mismatch == 0)}
        log("[bench] parity vs plain-kernel oracle: %s (oracle %.1f s)" % (parity, time.time() - t0))
        d_y.copy_from(y0)

    t = time_steps(step, steps, warmup, hiprt)
    cold = None
    if cold_copies > 1 and analysed and not transpose:
        # K copies of everything a multiply touches, used in turn: with K * footprint well beyond the 256 MB
        # memory-side cache every step reads its operands from HBM
        copies = []
        for _ in range(cold_copies):
            arrs = [hiprt.DeviceArray.from_numpy(v) for v in (a.values, a.row_ptr, a.col_ind, x, y0)]
            inf = capi.alphasparse_dcu_mat_info_t()
            assert lib.alphasparse_dcu_create_mat_info(byref(inf)) == 0
            assert getattr(lib, "alphasparse_dcu_%s_csrmv_analysis" % p)(
                h.h, op, a.rows, a.cols, a.nnz, byref(descr), arrs[0].c_ptr(), arrs[1].c_ptr(), arrs[2].c_ptr(), inf) == 0
            copies.append((arrs, inf))
        turn = [0]

        def cold_step():
            arrs, inf = copies[turn[0] % cold_copies]
            turn[0] += 1
            s = csrmv(h.h, op, a.rows, a.cols, a.nnz, byref(al), byref(descr), arrs[0].c_ptr(), arrs[1].c_ptr(),
                      arrs[2].c_ptr(), inf, arrs[3].c_ptr(), byref(be), arrs[4].c_ptr())
            if s != 0:
                raise RuntimeError("csrmv status %d" % s)
        cold = time_steps(cold_step, steps, warmup, hiprt)
        cold["copies"] = cold_copies
        cold["kernel"] = capi.ALGO_NAMES.get(lib.asamd_analysis_stats(copies[0][1]).contents.algo, "?")
        for arrs, inf in copies:
            lib.alphasparse_dcu_destroy_mat_info(inf)
            for d in arrs:
                d.free()
    # A second matrix info analysed from scratch on the same arrays: what an analysis costs once the process has
    # launched every kernel of the pass before (the first one above also pays for loading them).
    analysis_again_ms = None
    if analysed:
        inf2 = capi.alphasparse_dcu_mat_info_t()
        assert lib.alphasparse_dcu_create_mat_info(byref(inf2)) == 0
        hiprt.synchronize()
        t0 = time.perf_counter()
        st = getattr(lib, "alphasparse_dcu_%s_csrmv_analysis" % p)(
            h.h, op, a.rows, a.cols, a.nnz, byref(descr), d_val.c_ptr(), d_rp.c_ptr(), d_ci.c_ptr(), inf2)
        hiprt.synchronize()
        analysis_again_ms = (time.perf_counter() - t0) * 1e3
        assert st == 0, "second analysis status %d" % st
        lib.alphasparse_dcu_destroy_mat_info(inf2)
    # the analysis repeated on the same arrays, as a caller does after rewriting csr_val in place: the structure
    # is fingerprinted, found unchanged, and only the values of the plan's copies are gathered again
    hiprt.synchronize()
    t0 = time.perf_counter()
    if analysed:
        st = getattr(lib, "alphasparse_dcu_%s_csrmv_analysis" % p)(
            h.h, op, a.rows, a.cols, a.nnz, byref(descr), d_val.c_ptr(), d_rp.c_ptr(), d_ci.c_ptr(), info)
        assert st == 0, "repeated analysis status %d" % st
    hiprt.synchronize()
    reanalysis_ms = (time.perf_counter() - t0) * 1e3 if analysed else None
    if analysed:  # the repeated analysis replaced the record that `stats` looked into
        stats = (lib.asamd_analysis_transpose_stats(info) if transpose else lib.asamd_analysis_stats(info)).contents
    for k, v in env_old.items():
        if v is None:
            os.environ.pop(k, None)
        else:
            os.environ[k] = v
    nbytes = (wl.spmv_bytes(a.cols, a.rows, a.nnz, a.dtype.itemsize, beta) if transpose
              else wl.spmv_bytes(a.rows, a.cols, a.nnz, a.dtype.itemsize, beta))
    opname = "" if not transpose else (" -- CONJUGATE-TRANSPOSED operation" if op == 2 else " -- TRANSPOSED operation")
    mode = "" if analysed else " -- WITHOUT analysis (info = NULL)"
    if structure_only:
        mode = " -- analysis keeps STRUCTURE ONLY (no copy of the values, as the reference's)"
    res = {"workload": workload_name + (" -- COMPLEX values (%s)" % a.dtype.name if cx else "") + opname + mode, "rows": a.rows, "nnz": a.nnz, "algorithmic_bytes": int(nbytes),
           "flops": 2 * a.nnz, "kernel": algo, "analysis_ms": analysis_ms, "analysis_again_ms": analysis_again_ms,
           "reanalysis_ms": reanalysis_ms, "timing": t,
           "gbs": nbytes / t["avg_ms"] / 1e6, "gflops": 2 * a.nnz / t["avg_ms"] / 1e6,
           "dtype": {"float32": "f32", "float64": "f64", "complex64": "c64", "complex128": "c128"}[a.dtype.name],
           "parity": parity}
    # what the analysis measured when it chose the kernel (one multiply each on scratch vectors; 0 = not tried)
    res["analysis_timings_ms"] = {k: round(float(getattr(stats, "tune_ms_" + k)), 4) for k in ("base", "tiled", "ell", "hot", "binned")}
    if cx:  # a complex multiply-add is 8 real flops
        res["flops"], res["gflops"] = 8 * a.nnz, 8 * a.nnz / t["avg_ms"] / 1e6
    res["hbm_frac"] = res["gbs"] / HBM_PEAK_GBS
    res["traffic"], res["traffic_source"] = (None, None) if (transpose or cx or isinstance(cfg, tuple)) else measured_traffic(cfg, algo)
    if watched and not (cx or isinstance(cfg, tuple)):
        tiled_traffic, src = measured_traffic(cfg, "tiled two-phase")
        if tiled_traffic:
            # the pair's measured traffic plus one read of each of the three arrays for their fingerprints (computed)
            res["traffic"] = tiled_traffic + a.nnz * (4 + a.dtype.itemsize) + (a.rows + 1) * 4
            res["traffic_source"] = src + " + one read of row_ptr, col_ind and csr_val (computed)"
    # device memory that the analysis holds beside the caller's CSR arrays, and the per-call scratch in the handle
    res["analysis_bytes"] = int(stats.device_bytes)
    res["workspace_bytes"] = int(stats.workspace_bytes)
    res["value_check"] = {0: "off", 1: "sampled fingerprint of csr_val before every multiply that uses a copy",
                          2: "full fingerprint"}[int(stats.value_check)]
    res["tune_mode"] = "model" if stats.tune_mode else "timed"
    if early_calls_ms is not None:
        res["calls_2_to_5_ms"] = [round(v, 4) for v in early_calls_ms]
        res["watched_copy"] = watched
    res["locality_probe"] = {"lines_per_entry_wave": float(stats.lines_per_entry_wave),
                             "lines_per_entry_segment": float(stats.lines_per_entry_segment)}
    if cold:
        res["cold"] = {"ms": cold["avg_ms"], "min_ms": cold["min_ms"], "gbs": nbytes / cold["avg_ms"] / 1e6,
                       "frac_of_8TBps": nbytes / cold["avg_ms"] / 1e6 / HBM_PEAK_GBS, "copies_rotated": cold["copies"],
                       "kernel": cold["kernel"]}

    if cpu_baseline and not transpose:
        res["cpu_baseline"] = cpu_spmv(a, x, y0, alpha, beta, nbytes)
    if vendor:
        try:  # a comparison only: whatever goes wrong in the vendor library must not cost the measurement
            res["vendor_baseline"] = vendor_spmv(a, x, y0, alpha, beta, nbytes, steps, warmup, transpose)
        except Exception as e:  # noqa: BLE001
            log("[bench] vendor baseline skipped: %r" % (e,))
            res["vendor_baseline"] = None
    lib.alphasparse_dcu_destroy_mat_info(info)
    for d in (d_val, d_rp, d_ci, d_x, d_y):
        d.free()
    h.close()
    return res


def cpu_spmv(a, x, y0, alpha, beta, nbytes):
    """The reference's OpenMP CSR kernel (gemv_?_csr compiled from its own sources
    into oracle/_ref with its -Ofast flags) on all host cores; falls back to this
    repository's restatement when that library is absent."""
    from oracle import oracle as orc
    threads = int(os.environ.get("OMP_NUM_THREADS", "0")) or orc.num_procs()
    iters = 5
    times = []
    if orc.ref_available(fast=True):
        kind = "reference"
        fn, mat = orc.ref_call("gemv_{t}_csr", a, fast=True, threads=threads)
        from ctypes import c_double, c_float
        T = c_float if a.dtype == np.float32 else c_double
        fn.argtypes = [T, c_void_p, c_void_p, T, c_void_p]
        y = y0.copy()
        for i in range(iters + 1):
            t0 = time.perf_counter()
            fn(T(alpha), byref(mat.s), x.ctypes.data_as(c_void_p), T(beta), y.ctypes.data_as(c_void_p))
            if i:
                times.append(time.perf_counter() - t0)
    else:
        kind = "port"
        for i in range(iters + 1):
            t0 = time.perf_counter()
            orc.csrmv_omp(a, alpha, x, beta, y0, threads=threads, fast=True)
            if i:
                times.append(time.perf_counter() - t0)
    best = min(times)
    return {"value": nbytes / best / 1e9, "unit": "GB/s", "cores": threads, "kind": kind,
            "gflops": 2 * a.nnz / best / 1e9, "ms": best * 1e3, "median_ms": float(np.median(times)) * 1e3,
            "sample": "the full workload (%d rows, %d nnz), 1 warm-up + %d timed multiplies, best of %d"
                      % (a.rows, a.nnz, iters, iters)}


def run_host_pointer_spmv(cfg, steps):
    """alphasparse_?_mv with HOST x and y (the reference's CPU entry point): every call stages x and y
    to the device, multiplies there and copies y back, so this rate includes PCIe.  Reported beside
    the device-resident figure, never as `value`."""
    from alsparse_amd import capi, workloads as wl
    lib = capi.load()
    a, x, y0, alpha, beta, _ = wl.config(cfg)
    T, p = capi.scalar_type(a.dtype), capi.prefix(a.dtype)
    A = capi.alphasparse_matrix_t()
    rs, re = np.ascontiguousarray(a.row_ptr[:-1]), np.ascontiguousarray(a.row_ptr[1:])
    st = getattr(lib, "alphasparse_%s_create_csr" % p)(byref(A), a.base, a.rows, a.cols, capi.ptr(rs), capi.ptr(re),
                                                      capi.ptr(a.col_ind), capi.ptr(a.values))
    assert st == 0, "create_csr status %d" % st
    descr = capi.alpha_matrix_descr(0, 0, 0)
    mv = getattr(lib, "alphasparse_%s_mv" % p)
    y = y0.copy()
    t0 = time.perf_counter()
    assert mv(0, T(alpha), A, descr, capi.ptr(x), T(beta), capi.ptr(y)) == 0  # mirrors and analyses on first use
    first_ms = (time.perf_counter() - t0) * 1e3
    times = []
    for _ in range(steps):
        t0 = time.perf_counter()
        assert mv(0, T(alpha), A, descr, capi.ptr(x), T(beta), capi.ptr(y)) == 0
        times.append((time.perf_counter() - t0) * 1e3)
    lib.alphasparse_destroy(A)
    nbytes = wl.spmv_bytes(a.rows, a.cols, a.nnz, a.dtype.itemsize, beta)
    avg = sum(times) / len(times)
    return {"workload": WORKLOAD_NAMES[cfg] + " -- HOST x and y through alphasparse_%s_mv (PCIe-inclusive)" % p,
            "first_call_ms": first_ms, "avg_ms": avg, "min_ms": min(times), "gbs": nbytes / avg / 1e6,
            "staged_bytes_per_call": int(x.nbytes + y.nbytes * (2 if beta != 0 else 1))}


def run_conversions(cfg, steps, warmup):
    """alphasparse_dcu_csr2coo and alphasparse_dcu_?csr2ell on configuration `cfg`, device-resident:
    ms per conversion and GB/s of compulsory traffic (csr2coo reads row_ptr and writes nnz row
    indices; csr2ell reads the CSR arrays and writes m * width slots of value and index)."""
    from ctypes import c_int32
    from alsparse_amd import capi, hiprt, workloads as wl
    lib = capi.load()
    a, _, _, _, _, _ = wl.config(cfg)
    sz = a.dtype.itemsize
    h = capi.Handle()
    descr = capi.make_descr()
    d_val, d_rp, d_ci = (hiprt.DeviceArray.from_numpy(v) for v in (a.values, a.row_ptr, a.col_ind))
    d_rows = hiprt.DeviceArray((a.nnz,), np.int32)

    def coo_step():
        if lib.alphasparse_dcu_csr2coo(h.h, d_rp.c_ptr(), a.nnz, a.rows, d_rows.c_ptr(), 0) != 0:
            raise RuntimeError("csr2coo failed")
    t_coo = time_steps(coo_step, steps, warmup, hiprt)
    w = c_int32(-1)
    assert lib.alphasparse_dcu_csr2ell_width(h.h, a.rows, byref(descr), d_rp.c_ptr(), byref(descr), byref(w)) == 0
    ev, ec = hiprt.DeviceArray((w.value * a.rows,), a.dtype), hiprt.DeviceArray((w.value * a.rows,), np.int32)
    conv = lib.alphasparse_dcu_scsr2ell if a.dtype == np.float32 else lib.alphasparse_dcu_dcsr2ell

    def ell_step():
        if conv(h.h, a.rows, byref(descr), d_val.c_ptr(), d_rp.c_ptr(), d_ci.c_ptr(), byref(descr), w.value,
                ev.c_ptr(), ec.c_ptr()) != 0:
            raise RuntimeError("csr2ell failed")
    t_ell = time_steps(ell_step, steps, warmup, hiprt)
    coo_bytes = (a.rows + 1) * 4 + a.nnz * 4
    ell_bytes = a.nnz * (4 + sz) + (a.rows + 1) * 4 + a.rows * w.value * (4 + sz)
    for d in (d_val, d_rp, d_ci, d_rows, ev, ec):
        d.free()
    h.close()
    return {"workload": WORKLOAD_NAMES[cfg] + " -- conversions on the GPU",
            "rows": a.rows, "nnz": a.nnz, "dtype": "f32" if a.dtype == np.float32 else "f64",
            "csr2coo": {"avg_ms": t_coo["avg_ms"], "bytes": int(coo_bytes), "gbs": coo_bytes / t_coo["avg_ms"] / 1e6,
                        "timing": t_coo},
            "csr2ell": {"avg_ms": t_ell["avg_ms"], "width": w.value, "bytes": int(ell_bytes),
                        "gbs": ell_bytes / t_ell["avg_ms"] / 1e6, "timing": t_ell}}


def run_format_spmv(cfg, fmt, steps, warmup, check):
    """SpMV on the ELL or COO form of configuration `cfg`, converted on the GPU
    (alphasparse_dcu_csr2coo / _csr2ell) and multiplied by alphasparse_dcu_?_coomv / _ellmv."""
    from ctypes import c_int32
    from alsparse_amd import capi, hiprt, workloads as wl
    lib = capi.load()
    if isinstance(cfg, tuple):  # ("stencil3d", nx, ny, nz, dtype): not a benchmark configuration
        a = wl.stencil3d(cfg[1], cfg[2], cfg[3], cfg[4])
        x, y0, alpha, beta = wl.uniform(a.cols, a.dtype, 3), wl.uniform(a.rows, a.dtype, 4), 1.0, 0.5
    else:
        a, x, y0, alpha, beta, _ = wl.config(cfg)
    T, p, sz = capi.scalar_type(a.dtype), capi.prefix(a.dtype), a.dtype.itemsize
    h = capi.Handle()
    descr = capi.make_descr()
    d_val, d_rp, d_ci = (hiprt.DeviceArray.from_numpy(v) for v in (a.values, a.row_ptr, a.col_ind))
    d_x, d_y = hiprt.DeviceArray.from_numpy(x), hiprt.DeviceArray.from_numpy(y0)
    al, be = T(alpha), T(beta)
    extra = []
    if fmt == "coo":
        d_rows = hiprt.DeviceArray((a.nnz,), np.int32)
        extra.append(d_rows)
        assert lib.alphasparse_dcu_csr2coo(h.h, d_rp.c_ptr(), a.nnz, a.rows, d_rows.c_ptr(), 0) == 0
        fn = getattr(lib, "alphasparse_dcu_%s_coomv" % p)

        def step():
            s = fn(h.h, 0, a.rows, a.cols, a.nnz, byref(al), byref(descr), d_val.c_ptr(), d_rows.c_ptr(), d_ci.c_ptr(),
                   d_x.c_ptr(), byref(be), d_y.c_ptr())
            if s != 0:
                raise RuntimeError("coomv status %d" % s)
        nbytes = a.nnz * (8 + sz) + a.cols * sz + a.rows * sz * (2 if beta != 0 else 1)
        kernel = "coo segmented scan"
    else:
        w = c_int32(-1)
        assert lib.alphasparse_dcu_csr2ell_width(h.h, a.rows, byref(descr), d_rp.c_ptr(), byref(descr), byref(w)) == 0
        ev, ec = hiprt.DeviceArray((w.value * a.rows,), a.dtype), hiprt.DeviceArray((w.value * a.rows,), np.int32)
        extra += [ev, ec]
        conv = lib.alphasparse_dcu_scsr2ell if a.dtype == np.float32 else lib.alphasparse_dcu_dcsr2ell
        assert conv(h.h, a.rows, byref(descr), d_val.c_ptr(), d_rp.c_ptr(), d_ci.c_ptr(), byref(descr), w.value,
                    ev.c_ptr(), ec.c_ptr()) == 0
        fn = getattr(lib, "alphasparse_dcu_%s_ellmv" % p)

        def step():
            s = fn(h.h, 0, a.rows, a.cols, byref(al), byref(descr), ev.c_ptr(), ec.c_ptr(), w.value, d_x.c_ptr(),
                   byref(be), d_y.c_ptr())
            if s != 0:
                raise RuntimeError("ellmv status %d" % s)
        nbytes = a.rows * w.value * (4 + sz) + a.cols * sz + a.rows * sz * (2 if beta != 0 else 1)
        kernel = "ell, two rows per lane (width %d)" % w.value
    hiprt.synchronize()
    parity = None
    if check:
        from oracle import oracle as orc
        step()
        hiprt.synchronize()
        y = d_y.to_numpy()
        err = orc.csrmv_err(a, alpha, x, beta, y0, y, orc.csrmv_plain(a, alpha, x, beta, y0))
        tol = 1e-4 if a.dtype == np.float32 else 1e-12
        parity = {"max_row_err": err.strict, "max_row_err_with_beta_y": err.full, "tol": tol,
                  "zero_den_mismatch": err.zero_den_mismatch,
                  "ok": bool(err.strict <= tol and err.zero_den_mismatch == 0)}
        d_y.copy_from(y0)
    t = time_steps(step, steps, warmup, hiprt)
    wname = WORKLOAD_NAMES[cfg] if not isinstance(cfg, tuple) else (
        "27-point stencil: CSR SpMV %s, %d x %d x %d grid (%d rows, %d nnz), alpha=1 beta=0.5"
        % (a.dtype.name, cfg[1], cfg[2], cfg[3], a.rows, a.nnz))
    res = {"workload": wname.replace("CSR", fmt.upper() + " (from CSR on the GPU)"), "rows": a.rows,
           "nnz": a.nnz, "algorithmic_bytes": int(nbytes), "flops": 2 * a.nnz, "kernel": kernel, "timing": t,
           "gbs": nbytes / t["avg_ms"] / 1e6, "gflops": 2 * a.nnz / t["avg_ms"] / 1e6,
           "dtype": "f32" if a.dtype == np.float32 else "f64", "parity": parity}
    res["hbm_frac"] = res["gbs"] / HBM_PEAK_GBS
    for d in [d_val, d_rp, d_ci, d_x, d_y] + extra:
        d.free()
    h.close()
    return res


def run_spmm(steps, warmup, check, col_major=False, vendor=False, stencil=None, dense_cols=None):
    """stencil = (nx, ny, nz): instead of configuration 5's matrix, the 27-point stencil on that grid times a
    random dense matrix of dense_cols (default 64) columns."""
    from alsparse_amd import capi, hiprt, workloads as wl
    lib = capi.load()
    if stencil:
        a = wl.stencil3d(stencil[0], stencil[1], stencil[2], np.float32)
        n = dense_cols or 64
        B = wl.uniform(a.cols * n, np.float32, 3).reshape(a.cols, n)
        C0 = wl.uniform(a.rows * n, np.float32, 4).reshape(a.rows, n)
        alpha, beta = 1.0, 0.0
    else:
        a, B, C0, alpha, beta, extra = wl.config(5)
        n = dense_cols or extra["n"]
        if n != extra["n"]:
            B = wl.uniform(a.cols * n, np.float32, 3).reshape(a.cols, n)
            C0 = wl.uniform(a.rows * n, np.float32, 4).reshape(a.rows, n)
    h = capi.Handle()
    descr = capi.make_descr()
    from ctypes import c_float
    d_val, d_rp, d_ci = (hiprt.DeviceArray.from_numpy(v) for v in (a.values, a.row_ptr, a.col_ind))
    # column-major: the same B and C stored column by column (ldb = k, ldc = m)
    B_dev = np.ascontiguousarray(B.T) if col_major else B
    C_dev = np.ascontiguousarray(C0.T) if col_major else C0
    d_B, d_C = hiprt.DeviceArray.from_numpy(B_dev), hiprt.DeviceArray.from_numpy(C_dev)
    al, be = c_float(alpha), c_float(beta)
    layout = capi.ALPHA_SPARSE_LAYOUT_COLUMN_MAJOR if col_major else capi.ALPHA_SPARSE_LAYOUT_ROW_MAJOR
    ldb, ldc = (a.cols, a.rows) if col_major else (n, n)

    def step():
        s = lib.alphasparse_dcu_s_csrmm(h.h, 0, 0, layout, a.rows, n, a.cols, a.nnz,
                                        byref(al), byref(descr), d_val.c_ptr(), d_rp.c_ptr(), d_ci.c_ptr(),
                                        d_B.c_ptr(), ldb, byref(be), d_C.c_ptr(), ldc)
        if s != 0:
            raise RuntimeError("csrmm status %d" % s)

    parity = None
    if check:
        from oracle import oracle as orc
        step()
        hiprt.synchronize()
        C = d_C.to_numpy()
        if col_major:
            C = np.ascontiguousarray(C.reshape(n, a.rows).T)
        ref = orc.csrmm_plain(a, alpha, B, beta, C0, omp=True)
        err = orc.csrmm_err(a, alpha, B, beta, C0, C, ref)
        parity = {"max_elem_err": err.strict, "max_elem_err_with_beta_c": err.full, "tol": 1e-4,
                  "zero_den_mismatch": err.zero_den_mismatch, "ok": bool(err.strict <= 1e-4 and err.zero_den_mismatch == 0)}
        d_C.copy_from(C_dev)
    t = time_steps(step, steps, warmup, hiprt)
    nbytes = wl.spmm_bytes(a.rows, a.cols, n, a.nnz, 4, beta)
    wname = WORKLOAD_NAMES[5] if not stencil else (
        "27-point stencil SpMM: CSR fp32 %d x %d x %d grid (%d rows, %d nnz) times dense %d x %d row-major, alpha=1 beta=0"
        % (stencil[0], stencil[1], stencil[2], a.rows, a.nnz, a.cols, n))
    if not stencil and n != 64:
        wname += " -- with %d dense columns" % n
    res = {"workload": wname.replace("row-major", "column-major") if col_major else wname,
           "kernel": "spmm column-major (B transposed into scratch)" if col_major else "spmm row-major", "rows": a.rows, "nnz": a.nnz, "algorithmic_bytes": int(nbytes),
           "gather_upper_bound_bytes": int(a.nnz) * n * 4, "flops": 2 * a.nnz * n, "timing": t,
           "gbs": nbytes / t["avg_ms"] / 1e6, "gflops": 2 * a.nnz * n / t["avg_ms"] / 1e6, "dtype": "f32",
           "parity": parity}
    res["hbm_frac"] = res["gbs"] / HBM_PEAK_GBS
    res["traffic"], res["traffic_source"] = (None, None) if col_major else measured_traffic(5, "spmm row-major")
    if col_major and vendor and os.path.exists(ROCSPARSE):
        # rocSPARSE's legacy csrmm takes column-major operands only: compared on this layout
        import ctypes
        from ctypes import c_int
        R = ctypes.CDLL(ROCSPARSE)
        rh, rd = c_void_p(), c_void_p()
        if R.rocsparse_create_handle(byref(rh)) == 0 and R.rocsparse_create_mat_descr(byref(rd)) == 0:
            P = c_void_p
            R.rocsparse_scsrmm.argtypes = [P, c_int, c_int, c_int, c_int, c_int, c_int, P, P, P, P, P, P, c_int, P, P, c_int]

            def vstep():
                s_ = R.rocsparse_scsrmm(rh, 111, 111, a.rows, n, a.cols, a.nnz, byref(al), rd, d_val.c_ptr(), d_rp.c_ptr(),
                                        d_ci.c_ptr(), d_B.c_ptr(), ldb, byref(be), d_C.c_ptr(), ldc)
                if s_ != 0:
                    raise RuntimeError("rocsparse csrmm status %d" % s_)
            vt = time_steps(vstep, max(2, steps // 4), 1, hiprt)
            res["vendor_baseline"] = {"library": "rocSPARSE csrmm (column-major)", "value": nbytes / vt["avg_ms"] / 1e6,
                                      "unit": "GB/s", "ms": vt["avg_ms"]}
            R.rocsparse_destroy_mat_descr(rd)
            R.rocsparse_destroy_handle(rh)
    for d in (d_val, d_rp, d_ci, d_B, d_C):
        d.free()
    h.close()
    return res


def run_ceilings(steps, warmup, short=False):
    """What this GPU sustains with plain kernels (alsparse_amd/probes/ceilings.hip): 2 GiB read-only, write-only
    and copy streams, copies in short runs that one side reads or writes out of order (the product runs of the
    tiled SpMV's second phase), whole 256-byte rows gathered at random from 256 MiB (the B operand of configuration 5) and
    single floats gathered at random from 64 MiB / 4 MiB / 16 KiB (the x of configuration 3; an L2-sized x; an
    L1-sized x).  TB/s of useful bytes, and gathers per second.  short: only the ones that the configurations' figures
    are read against (the default line carries them)."""
    from ctypes import c_int64
    from alsparse_amd import capi, hiprt
    lib = capi.load_probes()
    big = 2 << 30
    a, b = hiprt.DeviceArray((big,), np.uint8), hiprt.DeviceArray((big,), np.uint8)
    sink = hiprt.DeviceArray((4,), np.uint8)
    a.fill_bytes(1)
    b.fill_bytes(2)
    moved = c_int64(0)
    out = {}

    def measure(name, kind, dst, src, nbytes, count):
        def step():
            e = lib.asamd_ceiling_kernel(None, kind, dst, src, nbytes, count, sink.c_ptr(), byref(moved))
            if e != 0:
                raise RuntimeError("asamd_ceiling_kernel(%s) hip error %d" % (name, e))
        t = time_steps(step, steps, warmup, hiprt)
        out[name] = {"avg_ms": t["avg_ms"], "min_ms": t["min_ms"], "useful_bytes": moved.value,
                     "tb_per_s": moved.value / t["avg_ms"] / 1e9}
        return out[name]
    measure("read_2GiB", 0, None, a.c_ptr(), big, 0)
    measure("read_2GiB_nontemporal", 5, None, a.c_ptr(), big, 0)
    if not short:
        measure("write_2GiB", 1, b.c_ptr(), None, big, 0)
    measure("copy_2GiB", 2, b.c_ptr(), a.c_ptr(), big, 0)
    if not short:
        measure("copy_2GiB_nontemporal", 6, b.c_ptr(), a.c_ptr(), big, 0)
    for runlen in ((80,) if short else (64, 80, 160)):
        measure("copy_1GiB_in_runs_of_%d_floats_gathered" % runlen, 7, b.c_ptr(), a.c_ptr(), 1 << 30, runlen)
        if not short:
            measure("copy_1GiB_in_runs_of_%d_floats_scattered" % runlen, 8, b.c_ptr(), a.c_ptr(), 1 << 30, runlen)
    r = measure("row_gather_256B_from_256MiB", 3, None, a.c_ptr(), 256 << 20, 1 << 25)
    r["rows_per_s"] = r["useful_bytes"] / 256 / r["avg_ms"] * 1e3
    if not short:
        r = measure("row_gather_256B_from_2GiB", 3, None, a.c_ptr(), big, 1 << 25)
        r["rows_per_s"] = r["useful_bytes"] / 256 / r["avg_ms"] * 1e3
    sizes = (("64MiB", 64 << 20), ("32MiB", 32 << 20), ("4MiB", 4 << 20), ("2MiB", 2 << 20), ("16KiB", 16 << 10))
    for label, nb in (sizes[:3] if short else sizes):
        r = measure("elem_gather_4B_from_" + label, 4, None, a.c_ptr(), nb, 1 << 28)
        r["gathers_per_s"] = r["useful_bytes"] / 4 / r["avg_ms"] * 1e3
    for d in (a, b, sink):
        d.free()
    return out


def against_ceiling(cfg, r, ceilings):
    """The measured ceiling that bounds the configuration's kernel, named, and how close the kernel runs to it.
    C2 streams its algorithmic bytes once: the non-temporal read rate.  C3's tiled pair moves its streams twice
    (products out and in again): its real traffic (counter measurement, `traffic`) against the copy rate.
    C4 and the row kernels on C3 gather single elements of x that miss the L1: entries per second against the
    4-byte gather rates from an L2-resident array and from one of x's size.  C5 fetches one 256-byte row of B per
    entry of A: rows per second against the random 256-byte row rate."""
    if not ceilings:
        return None
    ms = r["timing"]["avg_ms"]
    kernel = r.get("kernel") or ""
    if cfg == 5:
        c = ceilings["row_gather_256B_from_256MiB"]
        got = r["nnz"] / ms * 1e3
        return {"ceiling": "random 256-byte rows gathered from 256 MiB (probe kernel)", "ceiling_value": c["rows_per_s"],
                "achieved": got, "unit": "rows of B per second", "frac_of_ceiling": got / c["rows_per_s"]}
    if kernel.startswith("tiled") and r.get("traffic"):
        c = ceilings["copy_2GiB"]
        got = r["traffic"] / ms / 1e9
        return {"ceiling": "plain copy of 2 GiB (probe kernel); achieved = measured HBM traffic of the kernel pair / time",
                "ceiling_value": c["tb_per_s"], "achieved": got, "unit": "TB/s of real traffic",
                "frac_of_ceiling": got / c["tb_per_s"]}
    if cfg == 2 and (kernel.startswith("row-block stream") or kernel.startswith("ell")):
        c = ceilings["read_2GiB_nontemporal"]
        got = r["algorithmic_bytes"] / ms / 1e9
        return {"ceiling": "non-temporal read of 2 GiB (probe kernel)", "ceiling_value": c["tb_per_s"], "achieved": got,
                "unit": "TB/s", "frac_of_ceiling": got / c["tb_per_s"]}
    # gather-bound row kernels and merge-path
    foot = "64MiB" if cfg == 3 else "32MiB"
    c_l2, c_x = ceilings["elem_gather_4B_from_4MiB"], ceilings["elem_gather_4B_from_" + foot]
    got = r["nnz"] / ms * 1e3
    return {"ceiling": "random 4-byte gathers from an L2-sized array (4 MiB; probe kernel); also given: from an array "
                       "of x's size (%s)" % foot,
            "ceiling_value": c_l2["gathers_per_s"], "ceiling_value_at_x_size": c_x["gathers_per_s"], "achieved": got,
            "unit": "gathers of x per second", "frac_of_ceiling": got / c_l2["gathers_per_s"],
            "frac_of_ceiling_at_x_size": got / c_x["gathers_per_s"]}


def brief(r, cfg=None, ceilings=None):
    """The figures of one configuration that the default line carries under `others`."""
    t = r["timing"]
    out = {"workload": r["workload"], "kernel": r.get("kernel"), "dtype": r["dtype"], "ms": t["avg_ms"], "min_ms": t["min_ms"],
           "gbs": r["gbs"], "gflops": r["gflops"], "frac_of_8TBps": r["hbm_frac"], "algorithmic_bytes": r["algorithmic_bytes"],
           "analysis_ms": r.get("analysis_ms"), "analysis_again_ms": r.get("analysis_again_ms"),
           "reanalysis_ms": r.get("reanalysis_ms"), "parity": r["parity"], "traffic": r.get("traffic"),
           "traffic_source": r.get("traffic_source"), "analysis_bytes": r.get("analysis_bytes"),
           "workspace_bytes": r.get("workspace_bytes")}
    for k in ("calls_2_to_5_ms", "watched_copy"):
        if k in r:
            out[k] = r[k]
    if r.get("cold"):
        out["cold"] = r["cold"]
        out["note"] = ("ms / gbs: the same matrix multiplied back to back, as a solver does -- its values, x and y then come "
                       "from the 256 MB memory-side cache and only part of the bytes from HBM, so frac_of_8TBps is NOT a "
                       "fraction of HBM bandwidth; cold: rotating over copies so that every operand comes from HBM")
    if cfg is not None:
        out["against_ceiling"] = against_ceiling(cfg, r, ceilings)
    return out


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--config", type=int, default=3, choices=[2, 3, 4, 5])
    ap.add_argument("--format", default="csr", choices=["csr", "ell", "coo"],
                    help="multiply the ELL / COO form of configuration 2 or 3 (converted on the GPU) instead")
    ap.add_argument("--col-major", action="store_true", help="configuration 5 with column-major B and C")
    ap.add_argument("--transpose", action="store_true",
                    help="y = alpha*A^T*x + beta*y of configuration 2, 3 or 4 (analysis asked for the transposed operation)")
    ap.add_argument("--complex", action="store_true", dest="cx",
                    help="configuration 2, 3 or 4 with complex values (complex64 / complex128), complex x, y, alpha, beta")
    ap.add_argument("--conjugate", action="store_true", help="with --complex --transpose: A^H instead of A^T")
    ap.add_argument("--conversions", action="store_true",
                    help="measure alphasparse_dcu_csr2coo (the main line) and ?csr2ell on configuration 2 or 3")
    ap.add_argument("--uniform", nargs=3, type=int, metavar=("ROWS", "COLS", "PER_ROW"),
                    help="instead of a configuration: CSR SpMV on a matrix of that shape with PER_ROW uniform random "
                         "columns per row (fp32, --fp64 for fp64); same analysis, timing and parity check")
    ap.add_argument("--bimodal", nargs=5, type=int, metavar=("ROWS", "COLS", "SHORT", "LONG", "EVERY"),
                    help="instead of a configuration: CSR SpMV on a matrix whose every EVERY-th row has LONG entries "
                         "and the others SHORT (the workload of the row-length bins)")
    ap.add_argument("--stencil3d", nargs=3, type=int, metavar=("NX", "NY", "NZ"),
                    help="instead of a configuration: the 27-point stencil on an NX x NY x NZ grid (8 to 27 entries per row)")
    ap.add_argument("--laplace2d", nargs=2, type=int, metavar=("NX", "NY"),
                    help="not a benchmark configuration: the 5-point Laplacian of configuration 2 on an NX x NY grid (fp32; --fp64)")
    ap.add_argument("--dense-cols", type=int, default=None, metavar="N",
                    help="with --config 5: N dense columns instead of 64 (with --stencil3d too: the stencil as the sparse matrix)")
    ap.add_argument("--fp64", action="store_true", help="with --uniform / --bimodal / --stencil3d: fp64 values")
    ap.add_argument("--all", action="store_true", help="also measure the other configurations")
    ap.add_argument("--only", action="store_true",
                    help="measure the selected configuration alone (by default the line also carries brief figures of "
                         "configurations 2, 4 and 5 under `others`)")
    ap.add_argument("--stream-ceiling", action="store_true",
                    help="instead of a workload: time plain read / write / copy / gather kernels and print their TB/s")
    ap.add_argument("--no-analysis", action="store_true",
                    help="CSR SpMV without alphasparse_dcu_?_csrmv_analysis (info = NULL, as the reference's own tests call it): "
                         "analysis_ms is then the first call, which looks at row_ptr once")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-vendor-baseline", action="store_true",
                    help="skip timing rocSPARSE's csrmv on the same workload (reported as vendor_baseline)")
    ap.add_argument("--no-check", action="store_true")
    ap.add_argument("--calibrate-copy", type=int, default=0, metavar="MiB",
                    help="also launch one plain copy kernel of this many MiB (reads and writes that many "
                         "bytes each) so that a counter run can be scaled against a known transfer")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this build runs on exactly one GPU (rows would shard across GPUs with an "
                 "all-gather of x; that path is a design note only). Re-run with --gpus 1.")

    from alsparse_amd import hiprt
    if hiprt.device_count() < 1:
        sys.exit("bench.py: no GPU visible")
    hiprt.set_device(0)

    if args.calibrate_copy:
        from alsparse_amd import capi
        nb = args.calibrate_copy << 20
        src, dst = hiprt.DeviceArray((nb,), np.uint8), hiprt.DeviceArray((nb,), np.uint8)
        src.fill_bytes(1)
        for _ in range(2):
            assert capi.load_probes().asamd_copy_bytes(None, dst.c_ptr(), src.c_ptr(), nb) == 0
        hiprt.synchronize()
        src.free()
        dst.free()

    if args.stream_ceiling:
        print(json.dumps({"metric": "practical memory ceilings of this GPU (plain kernels, useful bytes / time)",
                          "unit": "TB/s", "steps": args.steps, "warmup": args.warmup, "hbm_peak_tb_per_s": HBM_PEAK_GBS / 1e3,
                          "ceilings": run_ceilings(args.steps, args.warmup)}), flush=True)
        return

    global NO_ANALYSIS
    NO_ANALYSIS = args.no_analysis
    check = not args.no_check
    conv = None
    if args.conversions:
        if args.config not in (2, 3):
            sys.exit("bench.py: --conversions is measured on configuration 2 or 3")
        conv = run_conversions(args.config, args.steps, args.warmup)
        main_res = {"workload": conv["workload"], "rows": conv["rows"], "nnz": conv["nnz"], "dtype": "int32",
                    "algorithmic_bytes": conv["csr2coo"]["bytes"], "gbs": conv["csr2coo"]["gbs"], "gflops": 0.0,
                    "hbm_frac": conv["csr2coo"]["gbs"] / HBM_PEAK_GBS, "timing": conv["csr2coo"]["timing"],
                    "kernel": "csr2coo", "parity": None}
    elif args.format != "csr":
        if args.config not in (2, 3) and not args.stencil3d:
            sys.exit("bench.py: --format ell|coo is measured on configuration 2 or 3 (or --stencil3d)")
        fcfg = (("stencil3d",) + tuple(args.stencil3d) + (np.float64 if args.fp64 else np.float32,)) if args.stencil3d else args.config
        main_res = run_format_spmv(fcfg, args.format, args.steps, args.warmup, check)
    elif args.config == 5:
        main_res = run_spmm(args.steps, args.warmup, check, args.col_major, not args.no_vendor_baseline,
                            args.stencil3d, args.dense_cols)
    else:
        cfg = args.config
        if args.uniform:
            cfg = ("uniform", args.uniform[0], args.uniform[1], args.uniform[2], np.float64 if args.fp64 else np.float32)
        if args.bimodal:
            cfg = ("bimodal",) + tuple(args.bimodal) + (np.float64 if args.fp64 else np.float32,)
        if args.stencil3d:
            cfg = ("stencil3d",) + tuple(args.stencil3d) + (np.float64 if args.fp64 else np.float32,)
        if args.laplace2d:
            cfg = ("laplace2d",) + tuple(args.laplace2d) + (np.float64 if args.fp64 else np.float32,)
        main_res = run_spmv(cfg, args.steps, args.warmup, not args.no_cpu_baseline, check, args.transpose,
                            not args.no_vendor_baseline, args.cx, args.conjugate)
    others = {}
    ceilings = None
    plain_default = (args.config == 3 and not (args.all or args.only or args.uniform or args.bimodal or args.stencil3d or args.laplace2d or args.no_analysis or args.transpose or args.cx or
                                               args.conversions or args.col_major) and args.format == "csr")
    if plain_default:
        # what this GPU sustains with plain kernels, measured in this very run: the figures below are read against it
        ceilings = run_ceilings(5, 1, short=True)
        # the default line is configuration 3; the other device configurations ride along, briefly
        for c in (2, 4, 5):
            r = (run_spmm(args.steps, args.warmup, check) if c == 5
                 else run_spmv(c, args.steps, args.warmup, False, check, False, False, cold_copies=5 if c == 2 else 0))
            others["C%d" % c] = brief(r, c, ceilings)
        # as a caller who never analyses sees them (info = NULL, as the reference's own tests call,
        # test/dcu/level2/mv_csr_s_dcu_test.cpp:220-222), and configuration 3 with an analysis that keeps structure
        # only, as the reference's does
        few = max(2, min(args.steps, 10))
        for c in (2, 3, 4):
            others["C%d_without_analysis" % c] = brief(run_spmv(c, args.steps if c != 3 else few, args.warmup if c != 3 else 1,
                                                               False, check, False, False, analyse=False), c, ceilings)
        others["C3_structure_only"] = brief(run_spmv(3, few, 1, False, check, False, False, structure_only=True), 3, ceilings)
        others["C3_timed_analysis"] = brief(run_spmv(3, few, 1, False, False, False, False, tune="timed"), 3, ceilings)
    if args.all:
        for c in (2, 3, 4, 5):
            if c == args.config and not args.transpose and args.format == "csr" and not args.col_major:
                continue
            r = (run_spmm(args.steps, args.warmup, check) if c == 5
                 else run_spmv(c, args.steps, args.warmup, False, check, False, not args.no_vendor_baseline))
            others["C%d" % c] = {k: r[k] for k in ("workload", "gbs", "gflops", "hbm_frac", "timing", "parity", "kernel",
                                                    "vendor_baseline") if k in r}
        if not (args.config == 5 and args.col_major):
            r = run_spmm(args.steps, args.warmup, check, True, not args.no_vendor_baseline)
            others["C5_column_major"] = {k: r[k] for k in ("workload", "gbs", "gflops", "hbm_frac", "timing", "parity", "kernel",
                                                            "vendor_baseline") if k in r}
        for c in (3, 4):
            if args.transpose and c == args.config:
                continue
            r = run_spmv(c, args.steps, args.warmup, False, check, True)
            others["C%d_transposed" % c] = {k: r[k] for k in ("workload", "gbs", "gflops", "hbm_frac", "timing", "parity", "kernel")}
        for c in (2, 3, 4):
            if args.cx and c == args.config and not args.transpose:
                continue
            r = run_spmv(c, args.steps, args.warmup, False, check, False, False, True)
            others["C%d_complex" % c] = {k: r[k] for k in ("workload", "gbs", "gflops", "hbm_frac", "timing", "parity", "kernel", "dtype")}
        for c, fmt in ((2, "ell"), (2, "coo"), (3, "ell"), (3, "coo")):
            if args.format == fmt and args.config == c:
                continue
            r = run_format_spmv(c, fmt, args.steps, args.warmup, check)
            others["C%d_%s" % (c, fmt)] = {k: r[k] for k in ("workload", "gbs", "gflops", "hbm_frac", "timing", "parity", "kernel")}

        others["C3_host_pointers"] = run_host_pointer_spmv(3, min(args.steps, 10))
        for c in (2, 3):
            others["C%d_conversions" % c] = run_conversions(c, min(args.steps, 10), 2)

    t = main_res["timing"]
    out = {
        "metric": "CSR -> COO conversion GB/s (row_ptr read + row indices written / time), 1 GPU" if conv else
                  ("CSR SpMV effective GB/s (algorithmic bytes / time), 1 GPU" if args.format == "csr"
                   else "%s SpMV effective GB/s (algorithmic bytes / time), 1 GPU" % args.format.upper())
                  if args.config != 5 else "CSR SpMM effective GB/s (algorithmic bytes / time), 1 GPU",
        "value": main_res["gbs"], "unit": "GB/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": t["avg_ms"], "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": main_res["dtype"], "data": "synthetic",
        "config": {"workload": main_res["workload"], "rows": main_res["rows"], "nnz": main_res["nnz"],
                   "kernel": main_res.get("kernel", "spmm row-major"), "analysis_ms": main_res.get("analysis_ms"),
                   "analysis_again_ms": main_res.get("analysis_again_ms"),
                   "reanalysis_ms": main_res.get("reanalysis_ms"), "analysis_timings_ms": main_res.get("analysis_timings_ms")},
        "gflops": main_res["gflops"], "pct_of_hbm_peak": 100.0 * main_res["hbm_frac"],
        "min_ms": t["min_ms"], "median_ms": t["median_ms"], "wall_ms_per_step": t["wall_ms_per_step"],
        "parity": main_res["parity"],
        "roofline": {"bound": "hbm", "achieved": main_res["gbs"], "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": main_res["hbm_frac"], "traffic": main_res.get("traffic"),
                     "traffic_source": main_res.get("traffic_source"),
                     "algorithmic_bytes_per_launch": main_res["algorithmic_bytes"]},
        "cpu_baseline": main_res.get("cpu_baseline"),
        "vendor_baseline": main_res.get("vendor_baseline"),
    }
    for k in ("analysis_bytes", "workspace_bytes", "value_check", "tune_mode", "locality_probe", "calls_2_to_5_ms", "watched_copy"):
        if main_res.get(k) is not None:
            out["config"][k] = main_res[k]
    if ceilings:
        out["ceilings"] = {k: {kk: vv for kk, vv in v.items() if kk != "useful_bytes"} for k, v in ceilings.items()}
        out["roofline"]["against_ceiling"] = against_ceiling(args.config, main_res, ceilings)
    if conv:
        others["csr2ell"] = {k: v for k, v in conv["csr2ell"].items() if k != "timing"}
    if others:
        out["others"] = others
    print(json.dumps(out), flush=True)


if __name__ == "__main__":
    main()
