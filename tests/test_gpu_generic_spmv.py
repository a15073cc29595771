"""alphasparse_dcu_spmv (descriptor API) on the GPU: the size-query call that also runs the CSR analysis,
then the multiply, for CSR / COO / ELL descriptors in fp32 and fp64, against the oracle."""
import ctypes
from ctypes import byref, c_size_t

import numpy as np
import pytest

from alsparse_amd import capi, hiprt, workloads as wl
from oracle import oracle as orc
from helpers import TOL, announce

pytestmark = pytest.mark.gpu
SM, DV = capi.alphasparse_dcu_spmat_descr, capi.alphasparse_dcu_dnvec_descr


def dev(a):
    return hiprt.DeviceArray.from_numpy(np.ascontiguousarray(a))


def check(a, alpha, x, beta, y0, y, what):
    err = orc.csrmv_err(a, alpha, x, beta, y0, y, orc.csrmv_plain(a, alpha, x, beta, y0))
    assert err.zero_den_mismatch == 0 and err.full <= TOL[a.dtype], (what, err)


@pytest.mark.parametrize("dtype", [np.float32, np.float64], ids=["f32", "f64"])
@pytest.mark.parametrize("shape", ["powerlaw", "laplace"])
def test_generic_spmv_csr_coo_ell(gpu, shape, dtype):
    lib = capi.load()
    a = wl.powerlaw_rmat(12, 300, dtype) if shape == "powerlaw" else wl.laplace2d(80, 60, dtype)
    x, y0 = wl.uniform(a.cols, dtype, 3), wl.uniform(a.rows, dtype, 4)
    T = capi.scalar_type(dtype)
    dt = capi.ALPHA_SPARSE_DATATYPE_FLOAT if dtype == np.float32 else capi.ALPHA_SPARSE_DATATYPE_DOUBLE
    I32 = capi.ALPHA_SPARSE_DCU_INDEXTYPE_I32
    d = capi.make_descr()
    info = capi.alphasparse_dcu_mat_info_t()
    assert lib.alphasparse_dcu_create_mat_info(byref(info)) == 0
    rows = orc.csr2coo(a)
    w = orc.csr2ell_width(a)
    ev, ec = orc.csr2ell(a)
    bufs = {k: dev(v) for k, v in (("val", a.values), ("rp", a.row_ptr), ("ci", a.col_ind), ("rows", rows),
                                    ("ev", ev), ("ec", ec), ("x", x))}
    al, be = T(1.5), T(0.5)
    size = c_size_t(0)
    tmp = hiprt.DeviceArray((16,), np.uint8)
    try:
        mats = {
            "csr": SM(True, False, a.rows, a.cols, a.nnz, bufs["rp"].c_ptr(), bufs["ci"].c_ptr(), None, bufs["val"].c_ptr(),
                      I32, I32, dt, 0, capi.ALPHA_SPARSE_FORMAT_CSR, ctypes.pointer(d), info),
            "coo": SM(True, False, a.rows, a.cols, a.nnz, bufs["rows"].c_ptr(), bufs["ci"].c_ptr(), None, bufs["val"].c_ptr(),
                      I32, I32, dt, 0, capi.ALPHA_SPARSE_FORMAT_COO, ctypes.pointer(d), None),
            "ell": SM(True, False, a.rows, a.cols, w, None, bufs["ec"].c_ptr(), None, bufs["ev"].c_ptr(),
                      I32, I32, dt, 0, capi.ALPHA_SPARSE_FORMAT_ELL, ctypes.pointer(d), None),
        }
        for fmt, m in mats.items():
            dy = dev(y0)
            xd, yd = DV(True, a.cols, bufs["x"].c_ptr(), dt), DV(True, a.rows, dy.c_ptr(), dt)
            announce("generic spmv", fmt, shape, np.dtype(dtype).name)
            # first call: size query (and, for CSR, the analysis)
            assert lib.alphasparse_dcu_spmv(gpu.h, 0, byref(al), byref(m), byref(xd), byref(be), byref(yd), dt,
                                            capi.ALPHA_SPARSE_DCU_SPMV_ALG_DEFAULT, byref(size), None) == 0
            assert size.value == 4
            assert m.analysed == (fmt == "csr")
            if fmt == "csr":
                assert lib.asamd_analysis_stats(info)  # the analysis is on record for this info
            hiprt.synchronize()
            assert np.array_equal(dy.to_numpy(), y0)   # the query multiplies nothing
            assert lib.alphasparse_dcu_spmv(gpu.h, 0, byref(al), byref(m), byref(xd), byref(be), byref(yd), dt,
                                            capi.ALPHA_SPARSE_DCU_SPMV_ALG_DEFAULT, byref(size), tmp.c_ptr()) == 0
            hiprt.synchronize()
            check(a, 1.5, x, 0.5, y0, dy.to_numpy(), "generic %s" % fmt)
            dy.free()
    finally:
        lib.alphasparse_dcu_destroy_mat_info(info)
        tmp.free()
        for b in bufs.values():
            b.free()
