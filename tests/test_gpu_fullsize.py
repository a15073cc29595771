"""The benchmark configurations at their full sizes on the GPU: parity against the
oracle (strict criterion: per-row error normalised by the row's sum |a_ij x_j|) and
size-independent properties (linearity in alpha, Laplacian times ones, sortedness and
row-count round trip of csr2coo, ELL round trip)."""
from ctypes import byref

import numpy as np
import pytest

from alsparse_amd import capi, hiprt, workloads as wl
from oracle import oracle as orc
from helpers import TOL, DeviceCsr, announce, check_spmv, run_csrmv

pytestmark = pytest.mark.gpu


def _analysed_csrmv(h, da, alpha, x, beta, y0):
    """explicit analysis, then csrmv with that info."""
    lib = capi.load()
    a = da.a
    p = capi.prefix(a.dtype)
    info = capi.alphasparse_dcu_mat_info_t()
    assert lib.alphasparse_dcu_create_mat_info(byref(info)) == 0
    descr = capi.make_descr(base=a.base)
    assert getattr(lib, "alphasparse_dcu_%s_csrmv_analysis" % p)(
        h.h, 0, a.rows, a.cols, a.nnz, byref(descr), da.val.c_ptr(), da.row_ptr.c_ptr(), da.col.c_ptr(), info) == 0
    y = run_csrmv(h, da, alpha, x, beta, y0, info)
    assert lib.alphasparse_dcu_destroy_mat_info(info) == 0
    return y


@pytest.mark.parametrize("cfg", [1, 2, 3, 4])
def test_spmv_configuration_full_size(gpu, cfg):
    a, x, y0, alpha, beta, _ = wl.config(cfg)
    da = DeviceCsr(a)
    try:
        announce("full size config", cfg, a.name, "analysed")
        y = _analysed_csrmv(gpu, da, alpha, x, beta, y0)
        check_spmv(a, alpha, x, beta, y0, y, "config %d analysed" % cfg, strict=True)
        announce("full size config", cfg, a.name, "info NULL")
        y2 = run_csrmv(gpu, da, alpha, x, beta, y0)
        check_spmv(a, alpha, x, beta, y0, y2, "config %d lazy" % cfg, strict=True)
        # linearity in alpha with a power of two: bit-exact scaling of A*x when beta = 0
        announce("full size config", cfg, "linearity")
        y1 = _analysed_csrmv(gpu, da, 1.0, x, 0.0, y0)
        y4 = _analysed_csrmv(gpu, da, 4.0, x, 0.0, y0)
        assert np.array_equal(y4, 4 * y1)
    finally:
        da.free()


def test_laplacian_times_ones_is_exact(gpu):
    """Row sums of the 5-point Laplacian: 4 - (#neighbours), exact in fp64 and fp32."""
    for dt in (np.float64, np.float32):
        a = wl.laplace2d(2048, 2048, dt)
        da = DeviceCsr(a)
        try:
            announce("laplacian times ones", np.dtype(dt).name)
            y = _analysed_csrmv(gpu, da, 1.0, np.ones(a.cols, dt), 0.0, np.zeros(a.rows, dt)).reshape(2048, 2048)
            want = np.zeros((2048, 2048), dt)
            want[0, :] += 1
            want[-1, :] += 1
            want[:, 0] += 1
            want[:, -1] += 1
            assert np.array_equal(y, want)
        finally:
            da.free()


def test_spmm_configuration_5_full_size(gpu):
    a, B, C0, alpha, beta, extra = wl.config(5)
    n = extra["n"]
    lib = capi.load()
    da = DeviceCsr(a)
    dB, dC = hiprt.DeviceArray.from_numpy(B), hiprt.DeviceArray.from_numpy(C0)
    try:
        from ctypes import c_float
        al, be = c_float(alpha), c_float(beta)
        descr = capi.make_descr()
        announce("full size config 5 spmm")
        assert lib.alphasparse_dcu_s_csrmm(gpu.h, 0, 0, 0, a.rows, n, a.cols, a.nnz, byref(al), byref(descr), da.val.c_ptr(),
                                           da.row_ptr.c_ptr(), da.col.c_ptr(), dB.c_ptr(), n, byref(be), dC.c_ptr(), n) == 0
        hiprt.synchronize()
        C = dC.to_numpy()
        ref = orc.csrmm_plain(a, alpha, B, beta, C0, omp=True)
        e = orc.csrmm_err(a, alpha, B, beta, C0, C, ref)
        assert e.zero_den_mismatch == 0 and e.strict <= 1e-4, e
    finally:
        da.free()
        dB.free()
        dC.free()


def test_conversions_full_size_properties(gpu):
    from test_gpu_convert import gpu_csr2coo, gpu_csr2ell
    lib = capi.load()
    # configuration 3: ELL of a matrix with exactly 16 entries per row is a pure transpose
    a = wl.uniform_rows(1 << 24, 1 << 24, 16, np.float32)
    da = DeviceCsr(a)
    try:
        announce("full size csr2coo config 3")
        rows = gpu_csr2coo(gpu, da)
        assert np.array_equal(rows, np.repeat(np.arange(a.rows, dtype=np.int32), 16))
        announce("full size csr2ell config 3")
        w, ev, ec = gpu_csr2ell(gpu, da)
        assert w == 16
        assert np.array_equal(ev.reshape(16, a.rows).T.reshape(-1), a.values)
        assert np.array_equal(ec.reshape(16, a.rows).T.reshape(-1), a.col_ind)
    finally:
        da.free()
    # configuration 4: sortedness + per-row counts of the COO rows; ELL must refuse (width * m >= 2^31)
    a = wl.powerlaw_rmat(23, 200000, np.float32)
    da = DeviceCsr(a)
    try:
        announce("full size csr2coo config 4")
        rows = gpu_csr2coo(gpu, da)
        assert np.all(np.diff(rows) >= 0)
        assert np.array_equal(np.bincount(rows, minlength=a.rows), np.diff(a.row_ptr))
        from ctypes import c_int32
        d = capi.make_descr()
        w = c_int32(0)
        assert lib.alphasparse_dcu_csr2ell_width(gpu.h, a.rows, byref(d), da.row_ptr.c_ptr(), byref(d), byref(w)) == 0
        assert w.value == int(np.diff(a.row_ptr).max())
        assert lib.alphasparse_dcu_scsr2ell(gpu.h, a.rows, byref(d), da.val.c_ptr(), da.row_ptr.c_ptr(), da.col.c_ptr(),
                                            byref(d), w.value, da.val.c_ptr(), da.col.c_ptr()) == capi.ALPHA_SPARSE_STATUS_INVALID_VALUE
    finally:
        da.free()
