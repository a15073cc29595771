"""The analysis decides from a model by default (row statistics, a deterministic locality probe of col_ind and
fixed constants), not from timing runs: the same matrix gets the same kernel family whatever else the GPU is doing.
ALSPARSE_AMD_TUNE=timed times the candidates instead, as the reference's `algo_tuning` flag intends
(include/alphasparse/handle.h:120-123).  On the shapes of the benchmark configurations both must agree."""
import os
from ctypes import byref, c_void_p

import numpy as np
import pytest

from alsparse_amd import capi, hiprt, workloads as wl
from helpers import DeviceCsr, announce, check_spmv, run_csrmv

pytestmark = pytest.mark.gpu

SHAPES = {
    # configuration 2 itself: 5-point Laplacian, fp64 -> the staged row-block kernel on the caller's arrays
    "laplace_c2": (lambda: wl.laplace2d(2048, 2048, np.float64), capi.ASAMD_SPMV_STREAM),
    # the same structure with complex128 values: the staged kernel moves 16-byte values at two thirds of its rate
    # with 8-byte ones, the ELL copy does not (0.145 against 0.110 ms, the value guard's launches included)
    "laplace_c2_complex": (lambda: wl.complexify(wl.laplace2d(2048, 2048, np.float64), np.complex128), capi.ASAMD_SPMV_ELL),
    # configuration 3's kind at an eighth of its size: scattered columns over 8 MiB of x -> the tiled copy
    "uniform_2M_16": (lambda: wl.uniform_rows(1 << 21, 1 << 21, 16, np.float32), capi.ASAMD_SPMV_TILED),
    # configuration 4's kind at half its size: power-law rows, R-MAT columns, 16 MiB of x -> merge-path
    "powerlaw_4M": (lambda: wl.powerlaw_rmat(22, 200000, np.float32), capi.ASAMD_SPMV_MERGE),
    # configuration 4 itself (32 MiB of x) -> merge-path with the popular columns' x in LDS
    "powerlaw_8M": (lambda: wl.powerlaw_rmat(23, 200000, np.float32), capi.ASAMD_SPMV_MERGE_HOT),
    # 27-point stencil, fp64: rows of 8..27 entries -> the staged row blocks (with 16-bit column distances: 0.68 GB)
    "stencil27_128": (lambda: wl.stencil3d(128, 128, 128, np.float64), capi.ASAMD_SPMV_STREAM),
}


def _analyse(lib, da, mode):
    a = da.a
    plan = c_void_p()
    old = os.environ.get("ALSPARSE_AMD_TUNE")
    if mode:
        os.environ["ALSPARSE_AMD_TUNE"] = mode
    try:
        assert lib.asamd_csr_plan_create_dtype(None, a.rows, a.cols, a.nnz, da.row_ptr.c_ptr(), da.col.c_ptr(),
                                               da.val.c_ptr(), a.base, capi.dtype_tag(a.dtype), 1, byref(plan)) == 0
    finally:
        if old is None:
            os.environ.pop("ALSPARSE_AMD_TUNE", None)
        else:
            os.environ["ALSPARSE_AMD_TUNE"] = old
    st = lib.asamd_csr_plan_stats(plan).contents
    out = {k: getattr(st, k) for k in ("algo", "tune_mode", "tune_ms_base", "tune_ms_tiled", "tune_ms_ell", "tiled_built",
                                        "ell_built", "binned_built", "lines_per_entry_wave", "lines_per_entry_segment",
                                        "device_bytes", "workspace_bytes")}
    lib.asamd_csr_plan_destroy(plan)
    return out


@pytest.mark.parametrize("shape", sorted(SHAPES))
def test_model_and_timing_choose_the_same_family(gpu, shape):
    lib = capi.load()
    make, want = SHAPES[shape]
    a = make()
    da = DeviceCsr(a)
    try:
        announce("analysis model vs timing", shape)
        default = _analyse(lib, da, None)
        assert default["tune_mode"] == 1, "the model is the default"
        model = [_analyse(lib, da, "model") for _ in range(3)]
        timed = _analyse(lib, da, "timed")
        assert timed["tune_mode"] == 0
        assert model[0]["algo"] == want, (shape, capi.ALGO_NAMES[model[0]["algo"]], model[0])
        # (a timing run may also keep the hot-column kernel at half of configuration 4's size, where it is 3 %
        # ahead of merge-path: the model lays it out only where the gain is beyond doubt)
        # and the ELL copy on the stencil, whose kernel is a few per cent ahead of the staged row blocks when timed
        # by itself: the model also counts the value guard's launches in front of a copy that holds values)
        near_ties = {"powerlaw_4M": capi.ASAMD_SPMV_MERGE_HOT, "stencil27_128": capi.ASAMD_SPMV_ELL}
        timed_ok = {want, near_ties[shape]} if shape in near_ties else {want}
        assert timed["algo"] in timed_ok, (shape, capi.ALGO_NAMES[timed["algo"]], timed)
        # the model's decision and every number behind it are the same on every analysis
        assert model[0] == model[1] == model[2] == default
        assert 0 < model[0]["lines_per_entry_wave"] <= 1 and 0 < model[0]["lines_per_entry_segment"] <= 1
        # its estimate of the kept family is within a third of what the timing run measured
        key = {capi.ASAMD_SPMV_TILED: "tune_ms_tiled", capi.ASAMD_SPMV_ELL: "tune_ms_ell"}.get(want, "tune_ms_base")
        if timed[key] > 0:  # (a copy that the timing run did not lay out has no measurement)
            # (the model's figure for a copy that holds values counts the value guard's launches, 0.022 ms; the timing
            # run launches the kernel alone)
            est = model[0][key] - (0.022 if key != "tune_ms_base" else 0.0)
            assert 0.66 * timed[key] <= est <= 1.5 * timed[key], (key, model[0][key], timed[key])
    finally:
        da.free()


def test_default_analysis_through_the_public_api_multiplies_correctly(gpu):
    """The public analysis call under default settings (model), followed by multiplies, on the tiled shape."""
    lib = capi.load()
    a = wl.uniform_rows(1 << 21, 1 << 21, 16, np.float32)
    x, y0 = wl.uniform(a.cols, a.dtype, 3), wl.uniform(a.rows, a.dtype, 4)
    da = DeviceCsr(a)
    info = capi.alphasparse_dcu_mat_info_t()
    assert lib.alphasparse_dcu_create_mat_info(byref(info)) == 0
    descr = capi.make_descr(base=a.base)
    try:
        announce("default analysis", a.name)
        assert lib.alphasparse_dcu_s_csrmv_analysis(gpu.h, 0, a.rows, a.cols, a.nnz, byref(descr), da.val.c_ptr(),
                                                    da.row_ptr.c_ptr(), da.col.c_ptr(), info) == 0
        st = lib.asamd_analysis_stats(info).contents
        assert st.tune_mode == 1 and st.algo == capi.ASAMD_SPMV_TILED
        assert st.ell_built == 0 and st.binned_built == 0, "the model lays out only the copy it keeps"
        check_spmv(a, 1.5, x, 0.5, y0, run_csrmv(gpu, da, 1.5, x, 0.5, y0, info), "model-chosen tiled copy")
    finally:
        lib.alphasparse_dcu_destroy_mat_info(info)
        da.free()
