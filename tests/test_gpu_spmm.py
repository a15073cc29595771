"""GPU parity of CSR SpMM against the CPU oracle, through alphasparse_dcu_?_csrmm.
Tolerance per element as for SpMV (1e-4 fp32 / 1e-12 fp64)."""
from ctypes import byref

import numpy as np
import pytest

from alsparse_amd import capi, hiprt, workloads as wl
from oracle import oracle as orc
from helpers import TOL, DeviceCsr, announce
from helpers_shapes import csr_from_lengths

pytestmark = pytest.mark.gpu


def run_csrmm(h, da, layout, trans_b, alpha, B, ldb, beta, C0, ldc, n, k):
    a = da.a
    lib = capi.load()
    T = capi.scalar_type(a.dtype)
    descr = capi.make_descr(base=a.base)
    dB, dC = hiprt.DeviceArray.from_numpy(B), hiprt.DeviceArray.from_numpy(C0)
    al, be = T(alpha), T(beta)
    st = getattr(lib, "alphasparse_dcu_%s_csrmm" % capi.prefix(a.dtype))(
        h.h, 0, trans_b, layout, a.rows, n, k, a.nnz, byref(al), byref(descr), da.val.c_ptr(), da.row_ptr.c_ptr(),
        da.col.c_ptr(), dB.c_ptr(), ldb, byref(be), dC.c_ptr(), ldc)
    assert st == 0, "csrmm status %d" % st
    hiprt.synchronize()
    out = dC.to_numpy()
    dB.free()
    dC.free()
    return out


def check(a, alpha, B2, beta, C02, C2, what):
    ref = orc.csrmm_plain(a, alpha, np.ascontiguousarray(B2), beta, np.ascontiguousarray(C02))
    err = orc.csrmm_err(a, alpha, np.ascontiguousarray(B2), beta, np.ascontiguousarray(C02), np.ascontiguousarray(C2), ref)
    assert err.zero_den_mismatch == 0, what
    assert err.full <= TOL[a.dtype], "%s: %r" % (what, err)
    if beta == 0:
        assert err.strict <= TOL[a.dtype], "%s: %r" % (what, err)


MATS = {
    "uniform32": lambda dt, base: wl.uniform_rows(3000, 2500, 32, dt, base=base),
    "powerlaw": lambda dt, base: wl.powerlaw_rmat(11, 1500, dt, base=base),
    "ragged": lambda dt, base: csr_from_lengths([0, 1, 0, 130, 64, 65, 63, 2, 0, 300, 1, 1], 400, dt, base=base),
}


@pytest.mark.parametrize("dtype", [np.float32, np.float64], ids=["f32", "f64"])
@pytest.mark.parametrize("mat", sorted(MATS))
@pytest.mark.parametrize("n", [1, 2, 3, 7, 16, 17, 24, 31, 32, 64, 100, 128, 300])
def test_row_major(gpu, mat, n, dtype):
    for base in (0, 1):
        a = MATS[mat](dtype, base)
        da = DeviceCsr(a)
        try:
            for pad_b, pad_c in ((0, 0), (3, 5)):
                ldb, ldc = n + pad_b, n + pad_c
                Bfull = wl.uniform(a.cols * ldb, dtype, 5).reshape(a.cols, ldb)
                Cfull = wl.uniform(a.rows * ldc, dtype, 4).reshape(a.rows, ldc)
                for alpha, beta in ((1.5, 0.5), (1.0, 0.0)):
                    announce("spmm row-major", mat, n, np.dtype(dtype).name, base, ldb, ldc, alpha, beta)
                    out = run_csrmm(gpu, da, capi.ALPHA_SPARSE_LAYOUT_ROW_MAJOR, 0, alpha, Bfull, ldb, beta, Cfull, ldc, n, a.cols)
                    check(a, alpha, Bfull[:, :n], beta, Cfull[:, :n], out[:, :n], "%s n=%d" % (mat, n))
                    assert np.array_equal(out[:, n:], Cfull[:, n:]), "padding columns of C were touched"
        finally:
            da.free()


@pytest.mark.parametrize("dtype", [np.float32, np.float64], ids=["f32", "f64"])
@pytest.mark.parametrize("seed", range(12))
def test_random_structures_widths_and_layouts(gpu, seed, dtype):
    """Seeded random structures (row-length law, base), a random number of dense columns and random padding of the
    leading dimensions, row-major and column-major."""
    rng = np.random.default_rng(500 + seed)
    m, cols = int(rng.integers(1, 1500)), int(rng.integers(1, 2000))
    law = int(rng.integers(0, 4))
    if law == 0:
        lengths = np.full(m, int(rng.integers(1, 40)))
    elif law == 1:
        lengths = rng.integers(0, int(rng.integers(2, 120)) + 1, size=m)
    elif law == 2:
        lengths = rng.geometric(1.0 / float(rng.integers(2, 20)), size=m) - 1
    else:
        lengths = rng.integers(0, 5, size=m)
        lengths[rng.integers(0, m, size=max(1, m // 100))] = int(rng.integers(200, 1500))
    base = int(rng.integers(0, 2))
    a = csr_from_lengths(list(np.minimum(lengths, cols)), cols, dtype, seed=int(rng.integers(1, 1 << 30)), base=base)
    if a.nnz == 0:
        pytest.skip("drew a matrix without entries")
    n = int(rng.choice([1, 2, 3, 4, 5, 8, 12, 16, 17, 20, 31, 32, 33, 48, 64, 65, 96, 128, 130]))
    da = DeviceCsr(a)
    try:
        ldb, ldc = n + int(rng.integers(0, 4)), n + int(rng.integers(0, 4))
        B = wl.uniform(a.cols * ldb, dtype, 5).reshape(a.cols, ldb)
        C0 = wl.uniform(a.rows * ldc, dtype, 4).reshape(a.rows, ldc)
        alpha, beta = ((1.5, 0.5), (1.0, 0.0), (-2.0, 1.0))[int(rng.integers(0, 3))]
        announce("spmm random structure, row-major", seed, a.name, n, np.dtype(dtype).name, base, ldb, ldc, alpha, beta)
        out = run_csrmm(gpu, da, capi.ALPHA_SPARSE_LAYOUT_ROW_MAJOR, 0, alpha, B, ldb, beta, C0, ldc, n, a.cols)
        check(a, alpha, B[:, :n], beta, C0[:, :n], out[:, :n], "seed %d row-major n=%d" % (seed, n))
        assert np.array_equal(out[:, n:], C0[:, n:]), "padding columns of C were touched"
        # column-major: B is k x n with leading dimension ldbc >= k, C is m x n with ldcc >= m
        ldbc, ldcc = a.cols + int(rng.integers(0, 3)), a.rows + int(rng.integers(0, 3))
        Bc = wl.uniform(ldbc * n, dtype, 7).reshape(n, ldbc)
        Cc = wl.uniform(ldcc * n, dtype, 8).reshape(n, ldcc)
        announce("spmm random structure, column-major", seed, a.name, n, ldbc, ldcc)
        outc = run_csrmm(gpu, da, capi.ALPHA_SPARSE_LAYOUT_COLUMN_MAJOR, 0, alpha, Bc, ldbc, beta, Cc, ldcc, n, a.cols)
        check(a, alpha, Bc[:, :a.cols].T, beta, Cc[:, :a.rows].T, outc.reshape(n, ldcc)[:, :a.rows].T,
              "seed %d column-major n=%d" % (seed, n))
        assert np.array_equal(outc.reshape(n, ldcc)[:, a.rows:], Cc[:, a.rows:]), "padding rows of C were touched"
    finally:
        da.free()


@pytest.mark.parametrize("maker", [lambda: wl.stencil3d(64, 60, 56, np.float32), lambda: wl.uniform_rows(215040, 215040, 12, np.float32)],
                         ids=["stencil", "random_columns"])
def test_row_major_operand_of_the_middle_sizes(gpu, maker):
    """A dense operand of 48 to 384 MiB: which row-major kernel runs is decided by a look at the matrix (do
    neighbouring rows share columns?) on the first multiply.  Both answers, twice each (the second multiply
    reuses the first one's answer), against the oracle."""
    a = maker()
    n = 64
    assert 48 << 20 < a.cols * n * 4 <= 384 << 20
    B = wl.uniform(a.cols * n, np.float32, 5).reshape(a.cols, n)
    C0 = wl.uniform(a.rows * n, np.float32, 6).reshape(a.rows, n)
    da = DeviceCsr(a)
    try:
        for rep in range(2):
            announce("spmm row-major, operand of the middle sizes", a.name, rep)
            C = run_csrmm(gpu, da, capi.ALPHA_SPARSE_LAYOUT_ROW_MAJOR, 0, 1.25, B, n, 0.5, C0, n, n, a.cols)
            check(a, 1.25, B, 0.5, C0, C.reshape(a.rows, n), "%s rep %d" % (a.name, rep))
    finally:
        da.free()


@pytest.mark.parametrize("dtype", [np.float32, np.float64], ids=["f32", "f64"])
@pytest.mark.parametrize("n", [1, 5, 64, 70])
def test_column_major_and_transposed_b(gpu, n, dtype):
    a = wl.uniform_rows(1500, 1200, 16, dtype)
    da = DeviceCsr(a)
    try:
        ldc = a.rows + 3
        C0 = np.asfortranarray(wl.uniform(ldc * n, dtype, 4).reshape(n, ldc).T)          # (ldc, n) column-major
        # op(B) = B: B is k x n column-major with ldb >= k
        ldb = a.cols + 2
        B = np.asfortranarray(wl.uniform(ldb * n, dtype, 5).reshape(n, ldb).T)            # (ldb, n) column-major
        announce("spmm col-major N/N", n, np.dtype(dtype).name)
        out = run_csrmm(gpu, da, capi.ALPHA_SPARSE_LAYOUT_COLUMN_MAJOR, 0, 1.5, B.T.reshape(-1), ldb, 0.5,
                        C0.T.reshape(-1), ldc, n, a.cols)
        out = out.reshape(n, ldc).T
        check(a, 1.5, B[:a.cols, :], 0.5, C0[:a.rows, :], out[:a.rows, :], "col-major n=%d" % n)
        ref_col = orc.csrmm_plain(a, 1.5, np.asfortranarray(B[:a.cols, :]), 0.5, np.asfortranarray(C0[:a.rows, :]), layout="col")
        e = orc.csrmm_err(a, 1.5, np.asfortranarray(B[:a.cols, :]), 0.5, np.asfortranarray(C0[:a.rows, :]),
                          np.asfortranarray(out[:a.rows, :]), ref_col)
        assert e.full <= TOL[a.dtype]
        assert np.array_equal(out[a.rows:, :], C0[a.rows:, :])
        # op(B) = B^T: B is stored n x k column-major (ldb >= n), i.e. the memory of a row-major k x n matrix
        ldb = n + 1
        Bt = wl.uniform(a.cols * ldb, dtype, 5).reshape(a.cols, ldb)                       # row r of op(B) at Bt[r, :n]
        announce("spmm col-major N/T", n, np.dtype(dtype).name)
        out = run_csrmm(gpu, da, capi.ALPHA_SPARSE_LAYOUT_COLUMN_MAJOR, 1, 1.5, Bt.reshape(-1), ldb, 0.5,
                        C0.T.reshape(-1), ldc, n, a.cols)
        out = out.reshape(n, ldc).T
        check(a, 1.5, Bt[:, :n], 0.5, C0[:a.rows, :], out[:a.rows, :], "col-major transB n=%d" % n)
    finally:
        da.free()


@pytest.mark.parametrize("dtype", [np.float32, np.float64], ids=["f32", "f64"])
def test_host_pointer_mm(gpu, dtype):
    lib = capi.load()
    p, T = capi.prefix(dtype), capi.scalar_type(dtype)
    a = wl.uniform_rows(1000, 800, 16, dtype)
    A = capi.alphasparse_matrix_t()
    rs, re = np.ascontiguousarray(a.row_ptr[:-1]), np.ascontiguousarray(a.row_ptr[1:])
    assert getattr(lib, "alphasparse_%s_create_csr" % p)(byref(A), 0, a.rows, a.cols, capi.ptr(rs), capi.ptr(re),
                                                         capi.ptr(a.col_ind), capi.ptr(a.values)) == 0
    n = 10
    B = wl.uniform(a.cols * n, dtype, 5).reshape(a.cols, n)
    C0 = wl.uniform(a.rows * n, dtype, 4).reshape(a.rows, n)
    C = C0.copy()
    announce("host api mm row-major")
    st = getattr(lib, "alphasparse_%s_mm" % p)(0, T(1.5), A, capi.alpha_matrix_descr(0, 0, 0), 0, capi.ptr(B), n, n, T(0.5), capi.ptr(C), n)
    assert st == 0
    check(a, 1.5, B, 0.5, C0, C, "alphasparse_mm row-major")
    Bf, Cf0 = np.asfortranarray(B), np.asfortranarray(C0)
    Cf = Cf0.copy(order="F")
    announce("host api mm col-major")
    st = getattr(lib, "alphasparse_%s_mm" % p)(0, T(1.5), A, capi.alpha_matrix_descr(0, 0, 0), 1, capi.ptr(Bf), n, a.cols, T(0.5), capi.ptr(Cf), a.rows)
    assert st == 0
    check(a, 1.5, B, 0.5, C0, np.ascontiguousarray(Cf), "alphasparse_mm col-major")
    assert lib.alphasparse_destroy(A) == 0


@pytest.mark.parametrize("dtype", [np.float32, np.float64], ids=["f32", "f64"])
@pytest.mark.parametrize("mat", sorted(MATS))
def test_column_major_every_matrix_shape_and_scratch_growth(gpu, mat, dtype):
    """Column-major B and C on ragged / skewed / one-based matrices, with the dense width going up and
    down between calls on one handle (its scratch buffer grows, then is reused for smaller products),
    and beta = 0 over a C full of NaN."""
    for base in (0, 1):
        a = MATS[mat](dtype, base)
        da = DeviceCsr(a)
        try:
            for n in (2, 130, 3, 64, 65):
                ldb, ldc = a.cols + 1, a.rows + 2
                B = np.asfortranarray(wl.uniform(ldb * n, dtype, 5).reshape(n, ldb).T)
                C0 = np.asfortranarray(wl.uniform(ldc * n, dtype, 4).reshape(n, ldc).T)
                for alpha, beta in ((1.5, 0.5), (1.0, 0.0)):
                    Cin = C0 if beta != 0 else np.full_like(C0, np.nan)
                    announce("spmm col-major", mat, n, np.dtype(dtype).name, base, alpha, beta)
                    out = run_csrmm(gpu, da, capi.ALPHA_SPARSE_LAYOUT_COLUMN_MAJOR, 0, alpha, B.T.reshape(-1), ldb, beta,
                                    Cin.T.reshape(-1), ldc, n, a.cols).reshape(n, ldc).T
                    check(a, alpha, B[:a.cols, :], beta, np.zeros_like(C0[:a.rows, :]) if beta == 0 else C0[:a.rows, :],
                          out[:a.rows, :], "col-major %s n=%d" % (mat, n))
                    if beta != 0:
                        assert np.array_equal(out[a.rows:, :], C0[a.rows:, :]), "padding rows of C were touched"
        finally:
            da.free()


@pytest.mark.parametrize("dtype", [np.float32, np.float64], ids=["f32", "f64"])
def test_kernel_abi_with_and_without_workspace(gpu, dtype):
    """asamd_?_csrmm (no workspace: element-wise gathers of column-major B) and asamd_?_csrmm_ws
    (row-major copy of B in the workspace) agree with the oracle; a workspace that is too small is ignored."""
    lib = capi.load()
    a = wl.powerlaw_rmat(11, 1500, dtype)
    n = 37
    p, T = capi.prefix(dtype), capi.scalar_type(dtype)
    B = np.asfortranarray(wl.uniform(a.cols * n, dtype, 5).reshape(n, a.cols).T)
    C0 = np.asfortranarray(wl.uniform(a.rows * n, dtype, 4).reshape(n, a.rows).T)
    st = capi.asamd_dense_strides(1, a.cols, 1, a.rows)
    need = lib.asamd_csrmm_workspace_bytes(a.dtype.itemsize, a.rows, n, a.cols, byref(st))
    assert need >= a.cols * n * a.dtype.itemsize
    row_major = capi.asamd_dense_strides(n, 1, n, 1)
    assert lib.asamd_csrmm_workspace_bytes(a.dtype.itemsize, a.rows, n, a.cols, byref(row_major)) == 0
    da = DeviceCsr(a)
    dB = hiprt.DeviceArray.from_numpy(B.T.reshape(-1))
    ws = hiprt.DeviceArray((need,), np.uint8)
    try:
        outs = []
        for what, w, wb in (("none", None, 0), ("full", ws.c_ptr(), need), ("too small", ws.c_ptr(), need // 2)):
            announce("csrmm_ws workspace", what, np.dtype(dtype).name)
            dC = hiprt.DeviceArray.from_numpy(C0.T.reshape(-1))
            e = getattr(lib, "asamd_%s_csrmm_ws" % p)(None, a.rows, n, a.cols, a.nnz, T(1.5), da.val.c_ptr(), da.row_ptr.c_ptr(),
                                                     da.col.c_ptr(), 0, dB.c_ptr(), T(0.5), dC.c_ptr(), byref(st), w, wb)
            assert e == 0
            hiprt.synchronize()
            out = dC.to_numpy().reshape(n, a.rows).T
            dC.free()
            check(a, 1.5, B, 0.5, C0, out, "csrmm_ws %s" % what)
            outs.append(out)
        assert np.array_equal(outs[0], outs[2])   # both took the fallback
    finally:
        ws.free()
        dB.free()
        da.free()


def _band(rows, cols, width, dtype, base=0, seed=11):
    """Row r holds `width` consecutive columns starting near r * cols / rows: neighbouring rows share nearly all
    their columns."""
    rng = np.random.default_rng(seed)
    start = np.minimum((np.arange(rows, dtype=np.int64) * cols) // rows, cols - width)
    row_ptr = (np.arange(rows + 1, dtype=np.int64) * width + base).astype(np.int32)
    col = (start[:, None] + np.arange(width)[None, :] + base).astype(np.int32).reshape(-1)
    val = rng.uniform(-1, 1, size=rows * width).astype(dtype)
    return wl.Csr(rows, cols, row_ptr, col, val, base, "band(%d,%d,%d)" % (rows, cols, width))


SHARED = {
    # 27-point stencil: nine runs of three consecutive columns per row; 32 rows share their rows of B
    "stencil27": lambda dt, base: wl.stencil3d(20, 18, 16, dt, base=base),
    "laplace": lambda dt, base: wl.laplace2d(90, 70, dt, base=base),
    # 32 rows x 100 entries exceed the staged entries: the run is halved, then fits
    "band100": lambda dt, base: _band(3000, 2600, 100, dt, base),
    # rows whose own columns exceed the tile: halved down to one row, which one wave multiplies from global memory
    "band300": lambda dt, base: _band(700, 900, 300, dt, base),
    # a matrix with fewer rows than one workgroup takes, and one that ends inside a run
    "band_short": lambda dt, base: _band(19, 40, 7, dt, base),
    "band_tail": lambda dt, base: _band(32 * 5 + 3, 400, 9, dt, base),
}


@pytest.mark.parametrize("dtype", [np.float32, np.float64, np.complex64, np.complex128], ids=["f32", "f64", "c64", "c128"])
@pytest.mark.parametrize("mat", sorted(SHARED))
@pytest.mark.parametrize("n", [33, 64, 100, 128])
@pytest.mark.parametrize("kernel", ["chosen", "lds"])
def test_row_major_rows_that_share_columns(gpu, mat, n, dtype, kernel, monkeypatch):
    """Matrices whose neighbouring rows share columns.  "chosen": the kernel the library picks by itself (a
    device-side look at the structure where the size of B does not decide); "lds": the opt-in kernel that stages
    the distinct rows of B of a run of rows of A in LDS.  Aligned and padded leading dimensions (128-bit and
    element-wise loads), both bases, beta zero and not."""
    from helpers_shapes import complex_vector, complexify, real_dtype
    if kernel == "lds":
        monkeypatch.setenv("ALSPARSE_AMD_SPMM_LDS", "1")  # read by the library at every call
    else:
        monkeypatch.delenv("ALSPARSE_AMD_SPMM_LDS", raising=False)
    cx = np.iscomplexobj(np.zeros(1, dtype))
    tol = {4: 1e-4, 8: 1e-12}[np.dtype(real_dtype(dtype) if cx else dtype).itemsize]
    for base in (0, 1):
        a = SHARED[mat](real_dtype(dtype) if cx else dtype, base)
        if cx:
            a = complexify(a, dtype)
        da = DeviceCsr(a)
        try:
            for pad_b, pad_c in ((0, 0), (3, 5)):
                ldb, ldc = n + pad_b, n + pad_c
                if cx:
                    Bfull = complex_vector(a.cols * ldb, dtype, 5).reshape(a.cols, ldb)
                    Cfull = complex_vector(a.rows * ldc, dtype, 4).reshape(a.rows, ldc)
                else:
                    Bfull = wl.uniform(a.cols * ldb, dtype, 5).reshape(a.cols, ldb)
                    Cfull = wl.uniform(a.rows * ldc, dtype, 4).reshape(a.rows, ldc)
                for alpha, beta in ((1.5, 0.5), (1.0, 0.0)):
                    announce("spmm rows sharing columns", mat, n, np.dtype(dtype).name, base, ldb, ldc, alpha, beta)
                    out = run_csrmm(gpu, da, capi.ALPHA_SPARSE_LAYOUT_ROW_MAJOR, 0, alpha, Bfull, ldb, beta, Cfull, ldc, n, a.cols)
                    B2, C02, C2 = (np.ascontiguousarray(v) for v in (Bfull[:, :n], Cfull[:, :n], out[:, :n]))
                    ref = orc.csrmm_plain(a, alpha, B2, beta, C02)
                    err = orc.csrmm_err(a, alpha, B2, beta, C02, C2, ref)
                    assert err.zero_den_mismatch == 0 and err.full <= tol, "%s n=%d: %r" % (mat, n, err)
                    if beta == 0:
                        assert err.strict <= tol, "%s n=%d: %r" % (mat, n, err)
                    assert np.array_equal(out[:, n:], Cfull[:, n:]), "padding columns of C were touched"
                    # the same bits on a second run: sums are formed in CSR order whatever slot a column got
                    again = run_csrmm(gpu, da, capi.ALPHA_SPARSE_LAYOUT_ROW_MAJOR, 0, alpha, Bfull, ldb, beta, Cfull, ldc, n, a.cols)
                    assert np.array_equal(out.view(np.uint8), again.view(np.uint8))
        finally:
            da.free()
