"""Differential check against rocSPARSE on the GPU, the way the reference's own drivers check
their DCU kernels (test/dcu/level2/mv_csr_s_dcu_test.cpp:41-147, check_s at the end): the same
device arrays go through rocsparse_?csrmv / rocsparse_csr2coo and through this library.  Values
are compared with the per-row criterion, COO row indices bit for bit.  Skipped where rocSPARSE
is not installed; nothing in the product uses it."""
import ctypes
import os
from ctypes import byref, c_double, c_float, c_int, c_void_p

import numpy as np
import pytest

from alsparse_amd import capi, hiprt, workloads as wl
from oracle import oracle as orc
from helpers import DeviceCsr, TOL, announce, run_csrmv
from helpers_shapes import csr_from_lengths

ROCSPARSE = "/opt/rocm/lib/librocsparse.so"
pytestmark = [pytest.mark.gpu, pytest.mark.skipif(not os.path.exists(ROCSPARSE), reason="rocSPARSE is not installed")]
P = c_void_p


@pytest.fixture(scope="module")
def roc():
    R = ctypes.CDLL(ROCSPARSE)
    h = c_void_p()
    assert R.rocsparse_create_handle(byref(h)) == 0
    yield R, h
    R.rocsparse_destroy_handle(h)


def roc_csrmv(roc, da, op, alpha, x, beta, y0, analyse):
    R, h = roc
    a = da.a
    T, p = (c_float, "s") if a.dtype == np.float32 else (c_double, "d")
    descr, info = c_void_p(), c_void_p()
    assert R.rocsparse_create_mat_descr(byref(descr)) == 0
    assert R.rocsparse_set_mat_index_base(descr, a.base) == 0
    mv = getattr(R, "rocsparse_%scsrmv" % p)
    mv.argtypes = [P, c_int, c_int, c_int, c_int, P, P, P, P, P, P, P, P, P]
    if analyse:
        assert R.rocsparse_create_mat_info(byref(info)) == 0
        an = getattr(R, "rocsparse_%scsrmv_analysis" % p)
        an.argtypes = [P, c_int, c_int, c_int, c_int, P, P, P, P, P]
        assert an(h, op, a.rows, a.cols, a.nnz, descr, da.val.c_ptr(), da.row_ptr.c_ptr(), da.col.c_ptr(), info) == 0
    dx, dy = hiprt.DeviceArray.from_numpy(x), hiprt.DeviceArray.from_numpy(y0)
    al, be = T(alpha), T(beta)
    assert mv(h, op, a.rows, a.cols, a.nnz, byref(al), descr, da.val.c_ptr(), da.row_ptr.c_ptr(), da.col.c_ptr(),
              info if analyse else None, dx.c_ptr(), byref(be), dy.c_ptr()) == 0
    hiprt.synchronize()
    y = dy.to_numpy()
    dx.free()
    dy.free()
    if analyse:
        R.rocsparse_destroy_mat_info(info)
    R.rocsparse_destroy_mat_descr(descr)
    return y


SHAPES = {
    "uniform16": lambda dt: wl.uniform_rows(20000, 15000, 16, dt),
    "powerlaw": lambda dt: wl.powerlaw_rmat(14, 20000, dt),
    "laplace_base1": lambda dt: wl.laplace2d(120, 90, dt, base=1),
    "ragged": lambda dt: csr_from_lengths([0, 0, 5, 0, 3000, 0, 0, 1, 1, 0, 64, 65, 0], 5000, dt),
}


@pytest.mark.parametrize("dtype", [np.float32, np.float64], ids=["f32", "f64"])
@pytest.mark.parametrize("shape", sorted(SHAPES))
def test_csrmv_agrees_with_rocsparse(gpu, roc, shape, dtype):
    a = SHAPES[shape](dtype)
    x, y0 = wl.uniform(a.cols, dtype, 3), wl.uniform(a.rows, dtype, 4)
    da = DeviceCsr(a)
    try:
        for alpha, beta in ((2.0, 3.0), (1.0, 0.0)):   # 2 and 3 are the reference drivers' scalars
            announce("vs rocsparse csrmv", shape, np.dtype(dtype).name, alpha, beta)
            ours = run_csrmv(gpu, da, alpha, x, beta, y0)
            for analyse in (False, True):
                theirs = roc_csrmv(roc, da, 111, alpha, x, beta, y0, analyse)
                err = orc.csrmv_err(a, alpha, x, beta, y0, ours, theirs)
                assert err.zero_den_mismatch == 0 and err.full <= TOL[a.dtype], (shape, analyse, err)
                # the oracle sits between the two as well
                err = orc.csrmv_err(a, alpha, x, beta, y0, theirs, orc.csrmv_plain(a, alpha, x, beta, y0))
                assert err.zero_den_mismatch == 0 and err.full <= TOL[a.dtype], ("oracle vs rocsparse", shape, err)
    finally:
        da.free()


@pytest.mark.parametrize("dtype", [np.float32, np.float64], ids=["f32", "f64"])
def test_transposed_csrmv_agrees_with_rocsparse(gpu, roc, dtype):
    lib = capi.load()
    a = wl.powerlaw_rmat(13, 3000, dtype)
    x, y0 = wl.uniform(a.rows, dtype, 3), wl.uniform(a.cols, dtype, 4)
    at = orc.transpose(a)
    da = DeviceCsr(a)
    T = capi.scalar_type(dtype)
    try:
        announce("vs rocsparse csrmv transposed", np.dtype(dtype).name)
        theirs = roc_csrmv(roc, da, 112, 2.0, x, 3.0, y0, False)
        dx, dy = hiprt.DeviceArray.from_numpy(x), hiprt.DeviceArray.from_numpy(y0)
        al, be = T(2.0), T(3.0)
        d = capi.make_descr()
        assert getattr(lib, "alphasparse_dcu_%s_csrmv" % capi.prefix(dtype))(
            gpu.h, capi.ALPHA_SPARSE_OPERATION_TRANSPOSE, a.rows, a.cols, a.nnz, byref(al), byref(d), da.val.c_ptr(),
            da.row_ptr.c_ptr(), da.col.c_ptr(), None, dx.c_ptr(), byref(be), dy.c_ptr()) == 0
        hiprt.synchronize()
        err = orc.csrmv_err(at, 2.0, x, 3.0, y0, dy.to_numpy(), theirs)
        assert err.zero_den_mismatch == 0 and err.full <= TOL[a.dtype], err
        dx.free()
        dy.free()
    finally:
        da.free()


def test_csr2coo_agrees_with_rocsparse_bit_for_bit(gpu, roc):
    R, h = roc
    lib = capi.load()
    R.rocsparse_csr2coo.argtypes = [P, P, c_int, c_int, P, c_int]
    for base in (0, 1):
        a = wl.powerlaw_rmat(14, 20000, np.float32, base=base)
        da = DeviceCsr(a)
        ours, theirs = hiprt.DeviceArray((a.nnz,), np.int32), hiprt.DeviceArray((a.nnz,), np.int32)
        try:
            announce("vs rocsparse csr2coo", base)
            assert lib.alphasparse_dcu_csr2coo(gpu.h, da.row_ptr.c_ptr(), a.nnz, a.rows, ours.c_ptr(), base) == 0
            assert R.rocsparse_csr2coo(h, da.row_ptr.c_ptr(), a.nnz, a.rows, theirs.c_ptr(), base) == 0
            hiprt.synchronize()
            assert np.array_equal(ours.to_numpy(), theirs.to_numpy())
        finally:
            ours.free()
            theirs.free()
            da.free()
