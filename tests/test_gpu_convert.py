"""GPU csr2coo / csr2ell against the oracle and the reference's committed outputs: bit-exact."""
import os
from ctypes import byref, c_int32

import numpy as np
import pytest

from alsparse_amd import capi, hiprt, workloads as wl
from oracle import oracle as orc
from helpers import DeviceCsr, announce
from helpers_shapes import csr_from_lengths
from golden_cases import golden_matrices

pytestmark = pytest.mark.gpu
GOLD = np.load(os.path.join(os.path.dirname(__file__), "golden", "reference_kernels.npz"), allow_pickle=False)


def gpu_csr2coo(h, da):
    a = da.a
    out = hiprt.DeviceArray((a.nnz,), np.int32).fill_bytes(0xEE)
    st = capi.load().alphasparse_dcu_csr2coo(h.h, da.row_ptr.c_ptr(), a.nnz, a.rows, out.c_ptr(), a.base)
    assert st == 0
    hiprt.synchronize()
    r = out.to_numpy()
    out.free()
    return r


def gpu_csr2ell(h, da, ell_base=0):
    a = da.a
    lib = capi.load()
    d_csr, d_ell = capi.make_descr(base=a.base), capi.make_descr(base=ell_base)
    w = c_int32(-1)
    assert lib.alphasparse_dcu_csr2ell_width(h.h, a.rows, byref(d_csr), da.row_ptr.c_ptr(), byref(d_ell), byref(w)) == 0
    ev = hiprt.DeviceArray((max(w.value * a.rows, 1),), a.dtype).fill_bytes(0xEE)
    ec = hiprt.DeviceArray((max(w.value * a.rows, 1),), np.int32).fill_bytes(0xEE)
    f = lib.alphasparse_dcu_scsr2ell if a.dtype == np.float32 else lib.alphasparse_dcu_dcsr2ell
    assert f(h.h, a.rows, byref(d_csr), da.val.c_ptr(), da.row_ptr.c_ptr(), da.col.c_ptr(), byref(d_ell), w.value,
             ev.c_ptr(), ec.c_ptr()) == 0
    hiprt.synchronize()
    out = (w.value, ev.to_numpy()[: w.value * a.rows], ec.to_numpy()[: w.value * a.rows])
    ev.free()
    ec.free()
    return out


SHAPES = {
    "uniform16": lambda dt, b: wl.uniform_rows(70000, 50000, 16, dt, base=b),
    "powerlaw": lambda dt, b: wl.powerlaw_rmat(14, 20000, dt, base=b),
    "laplace": lambda dt, b: wl.laplace2d(100, 77, dt, base=b),
    "empty_runs": lambda dt, b: csr_from_lengths([0] * 6000 + [9000] + [0] * 3000 + [2, 4097, 4095, 0, 0, 1], 20000, dt, base=b),
    "single_row": lambda dt, b: csr_from_lengths([5000], 6000, dt, base=b),
    "ones": lambda dt, b: csr_from_lengths([1] * 9000, 9000, dt, base=b),
}


@pytest.mark.parametrize("shape", sorted(SHAPES))
def test_csr2coo_bit_exact(gpu, shape):
    for base in (0, 1):
        a = SHAPES[shape](np.float32, base)
        da = DeviceCsr(a)
        try:
            announce("csr2coo", shape, base)
            assert np.array_equal(gpu_csr2coo(gpu, da), orc.csr2coo(a))
        finally:
            da.free()


BOUNDARY_SHAPES = {
    # entries per workgroup chunk: 8192.  Rows that start exactly on chunk boundaries, a chunk that is one
    # row, empty rows around the boundaries, an entry count that is a whole number of chunks and one off it
    "rows_of_8192": [8192] * 3,
    "rows_of_4096": [4096] * 5,
    "empties_at_boundaries": [8192, 0, 0, 8191, 1, 0, 8192, 0],
    "one_short": [8192, 8191],
    "one_over": [8192, 8193],
    "long_row_over_chunks": [3, 30000, 0, 5],
    "many_empty_rows": [1] + [0] * 20000 + [1] + [0] * 20000 + [8190],
}


@pytest.mark.parametrize("shape", sorted(BOUNDARY_SHAPES))
def test_csr2coo_entry_points_and_chunk_boundaries(gpu, shape):
    """asamd_csr2coo (every workgroup searches its rows), asamd_csr2coo_ws (table of chunk rows), an output
    array that is not 16-byte aligned (no 128-bit stores), both index bases."""
    lib = capi.load()
    lens = BOUNDARY_SHAPES[shape]
    for base in (0, 1):
        a = csr_from_lengths(lens, max(max(lens), 8), np.float32, base=base)
        want = orc.csr2coo(a)
        d_rp = hiprt.DeviceArray.from_numpy(a.row_ptr)
        ws_bytes = lib.asamd_csr2coo_workspace_bytes(a.nnz)
        assert ws_bytes == 4 * ((a.nnz + 8191) // 8192 + 1)
        ws = hiprt.DeviceArray((ws_bytes,), np.uint8)
        out = hiprt.DeviceArray((a.nnz + 8,), np.int32)
        try:
            for shift in (0, 1, 3):                     # elements: 0 = aligned, 1 and 3 = misaligned for 128-bit stores
                for with_ws in (False, True):
                    announce("csr2coo raw", shape, base, shift, with_ws)
                    out.fill_bytes(0xEE)
                    ptr = out.c_ptr().value + 4 * shift
                    if with_ws:
                        st = lib.asamd_csr2coo_ws(None, d_rp.c_ptr(), a.nnz, a.rows, ptr, a.base, ws.c_ptr(), ws_bytes)
                    else:
                        st = lib.asamd_csr2coo(None, d_rp.c_ptr(), a.nnz, a.rows, ptr, a.base)
                    assert st == 0
                    hiprt.synchronize()
                    got = out.to_numpy()
                    assert np.array_equal(got[shift:shift + a.nnz], want)
                    guard = np.int32(-286331154)        # 0xEEEEEEEE: nothing outside [shift, shift + nnz) is written
                    assert np.all(got[:shift] == guard) and np.all(got[shift + a.nnz:] == guard)
        finally:
            for d in (d_rp, ws, out):
                d.free()


@pytest.mark.parametrize("dtype", [np.float32, np.float64], ids=["f32", "f64"])
@pytest.mark.parametrize("shape", ["uniform16", "laplace", "empty_runs", "single_row", "ones"])
def test_csr2ell_bit_exact(gpu, shape, dtype):
    for base, ell_base in ((0, 0), (1, 0), (0, 1), (1, 1)):
        a = SHAPES[shape](dtype, base)
        if shape in ("uniform16", "empty_runs") and (base, ell_base) != (0, 0):
            continue
        da = DeviceCsr(a)
        try:
            announce("csr2ell", shape, np.dtype(dtype).name, base, ell_base)
            w, ev, ec = gpu_csr2ell(gpu, da, ell_base)
            assert w == orc.csr2ell_width(a)
            rv, rc = orc.csr2ell(a, ell_base=ell_base)
            assert np.array_equal(ev.view(np.uint8), rv.view(np.uint8)) and np.array_equal(ec, rc)
        finally:
            da.free()


@pytest.mark.parametrize("key", sorted(golden_matrices()))
def test_against_reference_fixtures(gpu, key):
    """The same matrices whose outputs of the reference's own converters and plain
    kernels are committed: indices bit-exact, values within tolerance."""
    from helpers import TOL, run_csrmv
    a = golden_matrices()[key]
    da = DeviceCsr(a)
    try:
        announce("golden", key)
        assert np.array_equal(gpu_csr2coo(gpu, da), GOLD[key + ".coo_rows"])
        w, ev, ec = gpu_csr2ell(gpu, da)
        assert w == int(GOLD[key + ".ell_ld"][0])
        assert np.array_equal(ev, GOLD[key + ".ell_val"]) and np.array_equal(ec, GOLD[key + ".ell_col"])
        x, y0 = wl.uniform(a.cols, a.dtype, 3), wl.uniform(a.rows, a.dtype, 4)
        for (alpha, beta), name in (((2.0, 3.0), ".mv_plain"), ((1.0, 0.0), ".mv_plain_beta0")):
            y = run_csrmv(gpu, da, alpha, x, beta, y0)
            e = orc.csrmv_err(a, alpha, x, beta, y0, y, GOLD[key + name])
            assert e.zero_den_mismatch == 0 and e.full <= TOL[a.dtype], (key, name, e)
    finally:
        da.free()
