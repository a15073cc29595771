"""Shared helpers of the GPU parity tests: run the C-ABI entry points on device
buffers and compare with the CPU oracle on the same seeded inputs."""
import sys
from ctypes import byref

import numpy as np

from alsparse_amd import capi, hiprt, workloads as wl
from oracle import oracle as orc
from helpers_shapes import csr_from_lengths  # noqa: F401

TOL = {np.dtype(np.float32): 1e-4, np.dtype(np.float64): 1e-12}

ALGOS = {"auto": capi.ASAMD_SPMV_AUTO, "vector": capi.ASAMD_SPMV_VECTOR, "rowconst": capi.ASAMD_SPMV_ROWCONST,
         "merge": capi.ASAMD_SPMV_MERGE, "scalar": capi.ASAMD_SPMV_SCALAR, "tiled": capi.ASAMD_SPMV_TILED,
         "stream": capi.ASAMD_SPMV_STREAM, "ell": capi.ASAMD_SPMV_ELL, "hot": capi.ASAMD_SPMV_MERGE_HOT, "binned": capi.ASAMD_SPMV_BINNED,
         "xlds": capi.ASAMD_SPMV_XLDS}


def announce(*what):
    """Name the case before touching the GPU, flushed, so a fault can be attributed."""
    print("[gpu-case]", *what, flush=True)


class _ShiftedArray:
    """A device array that starts `shift` elements into its allocation (so that it is not 16-byte aligned)."""

    def __init__(self, host, shift):
        import ctypes
        self._ctypes = ctypes
        lead = np.zeros(shift, dtype=host.dtype)
        self.dev = hiprt.DeviceArray.from_numpy(np.concatenate([lead, host]))
        self.offset = shift * host.dtype.itemsize

    def c_ptr(self):
        return self._ctypes.c_void_p(self.dev.ptr + self.offset)

    def free(self):
        self.dev.free()


class DeviceCsr:
    def __init__(self, a, shift=0):
        """shift: elements by which val and col_ind are moved off their allocations' (256-byte) alignment"""
        self.a = a
        self.row_ptr = hiprt.DeviceArray.from_numpy(a.row_ptr)
        if shift:
            self.val, self.col = _ShiftedArray(a.values, shift), _ShiftedArray(a.col_ind, shift)
        else:
            self.val = hiprt.DeviceArray.from_numpy(a.values)
            self.col = hiprt.DeviceArray.from_numpy(a.col_ind)

    def free(self):
        for d in (self.val, self.row_ptr, self.col):
            d.free()


def run_csrmv(h, da, alpha, x, beta, y0, info=None):
    """alphasparse_dcu_?_csrmv on device copies of x, y0; returns y as numpy."""
    a = da.a
    lib = capi.load()
    T = capi.scalar_type(a.dtype)
    descr = capi.make_descr(base=a.base)
    dx = hiprt.DeviceArray.from_numpy(np.ascontiguousarray(x, dtype=a.dtype))
    dy = hiprt.DeviceArray.from_numpy(np.ascontiguousarray(y0, dtype=a.dtype))
    al, be = T(alpha), T(beta)
    st = getattr(lib, "alphasparse_dcu_%s_csrmv" % capi.prefix(a.dtype))(
        h.h, 0, a.rows, a.cols, a.nnz, byref(al), byref(descr), da.val.c_ptr(), da.row_ptr.c_ptr(),
        da.col.c_ptr(), info, dx.c_ptr(), byref(be), dy.c_ptr())
    assert st == 0, "csrmv status %d" % st
    hiprt.synchronize()
    y = dy.to_numpy()
    dx.free()
    dy.free()
    return y


def run_plan_csrmv(da, algo, alpha, x, beta, y0, trusted=1):
    """The thin kernel ABI directly, with a forced kernel family."""
    a = da.a
    lib = capi.load()
    from ctypes import c_void_p
    plan = c_void_p()
    if algo in ("tiled", "ell", "hot", "binned", "xlds"):
        trusted = 2  # build the copies whatever the size
    e = lib.asamd_csr_plan_create(None, a.rows, a.cols, a.nnz, da.row_ptr.c_ptr(), da.col.c_ptr(), da.val.c_ptr(),
                                  a.base, a.dtype.itemsize, trusted, byref(plan))
    assert e == 0, "plan_create hip error %d" % e
    try:
        e = lib.asamd_csr_plan_set_algo(plan, ALGOS[algo])
        if e != 0:
            assert algo in ("rowconst", "stream", "ell", "hot", "xlds"), algo
            return None  # this structure cannot run that family
        T = capi.scalar_type(a.dtype)
        dx = hiprt.DeviceArray.from_numpy(np.ascontiguousarray(x, dtype=a.dtype))
        dy = hiprt.DeviceArray.from_numpy(np.ascontiguousarray(y0, dtype=a.dtype))
        ws = capi.Workspace(lib, plan)
        e = capi.plan_csrmv(lib, None, plan, 0, T(alpha), da.val.c_ptr(), da.row_ptr.c_ptr(), da.col.c_ptr(), dx.c_ptr(),
                            T(beta), dy.c_ptr(), ws)
        assert e == 0, "asamd_csr_plan_csrmv hip error %d" % e
        hiprt.synchronize()
        y = dy.to_numpy()
        dx.free()
        dy.free()
        ws.buf.free()
        return y
    finally:
        lib.asamd_csr_plan_destroy(plan)


def plan_stats(da, trusted=1):
    a = da.a
    lib = capi.load()
    from ctypes import c_void_p
    plan = c_void_p()
    e = lib.asamd_csr_plan_create(None, a.rows, a.cols, a.nnz, da.row_ptr.c_ptr(), None, None, a.base,
                                  a.dtype.itemsize, trusted, byref(plan))
    assert e == 0
    st = lib.asamd_csr_plan_stats(plan).contents
    out = {k: getattr(st, k) for k, _ in st._fields_ if k != "hist"}
    out["hist"] = list(st.hist)
    lib.asamd_csr_plan_destroy(plan)
    return out


def check_beta_rows(a, alpha, x, beta, y0, y, ref, tol, what=""):
    """beta != 0: the strict criterion plus nothing but the rounding of the last addition.  Both sides form
    fl(fl(beta*y0) + fl(alpha*sum)): the first term rounds identically, the sum's error is the strict criterion's
    business (tol * |alpha| sum|a x|), and the addition rounds to within half an ulp of the result on each side
    (complex: each component, and the four-multiplication beta*y0 identically on both sides).  `a` is the matrix
    whose rows are the outputs (the transpose for the transposed operations)."""
    x64 = np.abs(np.asarray(x, dtype=np.complex128 if np.iscomplexobj(x) else np.float64))
    den = abs(complex(alpha)) * orc._row_abs_sums(a, x64)
    by = np.abs(complex(beta) * np.asarray(y0, dtype=np.complex128))
    real = {"f": np.float32, "d": np.float64, "F": np.float32, "D": np.float64}[np.dtype(a.dtype).char]
    u = float(np.finfo(real).eps) / 2
    diff = np.abs(np.asarray(y, dtype=np.complex128) - np.asarray(ref, dtype=np.complex128))
    allow = tol * den + 4 * u * (by + den)
    bad = np.flatnonzero(diff > allow)
    assert bad.size == 0, "%s: output %d off by %.3e, allowed %.3e (strict criterion + rounding of beta*y)" % (
        what, bad[0], diff[bad[0]], allow[bad[0]])


def check_spmv(a, alpha, x, beta, y0, y, what="", strict=False):
    """Compare y with the plain-kernel oracle.  Always: zero-denominator rows exact and
    the error relative to |alpha| sum|a x| + |beta y0| within tolerance.  beta == 0 (or strict=True): the
    north-star criterion, normalised by the products alone.  beta != 0: the same criterion with an allowance
    of four units of round-off of |beta y0| + |alpha| sum|a x| for the rounding of the final addition."""
    ref = orc.csrmv_plain(a, alpha, x, beta, y0)
    err = orc.csrmv_err(a, alpha, x, beta, y0, y, ref)
    tol = TOL[a.dtype]
    assert err.zero_den_mismatch == 0, "%s: %d rows with zero denominator differ" % (what, err.zero_den_mismatch)
    assert err.full <= tol, "%s: per-row error %.3e at row %d exceeds %g" % (what, err.full, err.row, tol)
    if strict or beta == 0:
        assert err.strict <= tol, "%s: strict per-row error %.3e exceeds %g" % (what, err.strict, tol)
    else:
        check_beta_rows(a, alpha, x, beta, y0, y, ref, tol, what)
    return err
