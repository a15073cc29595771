"""The driver-side helpers (include/alphasparse_util.h) and the COO -> CSR route that the
reference's test programs take from a coordinate file to CSR arrays
(test/dcu/level2/mv_csr_s_dcu_test.cpp:268-292): reader against scipy.io, conversion against
scipy.sparse and -- where it is built -- the reference's own converter, flags, result check.
No GPU."""
import ctypes
import os
from ctypes import POINTER, byref, c_char_p, c_double, c_float, c_int32, c_void_p

import numpy as np
import pytest
import scipy.io
import scipy.sparse as sp

from alsparse_amd import capi, workloads as wl
from oracle import oracle as orc

S = capi


@pytest.fixture(scope="module")
def lib():
    return capi.load()


def argv(*flags):
    arr = (c_char_p * (len(flags) + 1))(b"prog", *[f.encode() for f in flags])
    return len(flags) + 1, arr


def read_coo(lib, path, double):
    m, n, nnz = c_int32(), c_int32(), c_int32()
    r, c, v = c_void_p(), c_void_p(), c_void_p()
    (lib.alpha_read_coo_d if double else lib.alpha_read_coo)(str(path).encode(), byref(m), byref(n), byref(nnz), byref(r), byref(c), byref(v))
    T = c_double if double else c_float
    rows = np.ctypeslib.as_array(ctypes.cast(r, POINTER(c_int32)), (nnz.value,)).copy()
    cols = np.ctypeslib.as_array(ctypes.cast(c, POINTER(c_int32)), (nnz.value,)).copy()
    vals = np.ctypeslib.as_array(ctypes.cast(v, POINTER(T)), (nnz.value,)).copy()
    for p in (r, c, v):
        lib.alpha_free(p)
    return m.value, n.value, rows, cols, vals


@pytest.mark.parametrize("double", [False, True], ids=["f32", "f64"])
def test_matrix_market_reader(lib, tmp_path, double):
    rng = np.random.default_rng(4)
    A = sp.random(37, 23, density=0.15, random_state=3, format="coo", dtype=np.float64)
    scipy.io.mmwrite(str(tmp_path / "general.mtx"), A, precision=17)
    m, n, rows, cols, vals = read_coo(lib, tmp_path / "general.mtx", double)
    assert (m, n, rows.size) == (37, 23, A.nnz)
    got = sp.coo_matrix((vals, (rows, cols)), shape=(m, n)).toarray()
    assert np.allclose(got, A.toarray(), rtol=1e-6 if not double else 1e-15, atol=0)
    # symmetric storage: lower triangle on file, both triangles in memory, diagonal once
    L = sp.tril(sp.random(30, 30, density=0.2, random_state=5, dtype=np.float64) + sp.eye(30)).tocoo()
    with open(tmp_path / "sym.mtx", "w") as f:
        f.write("%%%%MatrixMarket matrix coordinate real symmetric\n%% a comment line\n30 30 %d\n" % L.nnz)
        for r, c, v in zip(L.row, L.col, L.data):
            f.write("%d %d %.17g\n" % (r + 1, c + 1, v))
    m, n, rows, cols, vals = read_coo(lib, tmp_path / "sym.mtx", double)
    full = (L + sp.tril(L, -1).T).toarray()
    assert rows.size == 2 * L.nnz - 30
    assert np.allclose(sp.coo_matrix((vals, (rows, cols)), shape=(30, 30)).toarray(), full, rtol=1e-6 if not double else 1e-15)
    # pattern file: every value reads as 1
    with open(tmp_path / "pattern.mtx", "w") as f:
        f.write("%%MatrixMarket matrix coordinate pattern general\n4 5 3\n1 1\n4 5\n2 3\n")
    m, n, rows, cols, vals = read_coo(lib, tmp_path / "pattern.mtx", double)
    assert (m, n) == (4, 5) and rows.tolist() == [0, 3, 1] and cols.tolist() == [0, 4, 2] and vals.tolist() == [1, 1, 1]


def convert(lib, rows, cols, vals, m, n, base=0):
    p = "s" if vals.dtype == np.float32 else "d"
    coo, csr = capi.alphasparse_matrix_t(), capi.alphasparse_matrix_t()
    r, c = np.ascontiguousarray(rows + base, np.int32), np.ascontiguousarray(cols + base, np.int32)
    assert getattr(lib, "alphasparse_%s_create_coo" % p)(byref(coo), base, m, n, vals.size, capi.ptr(r), capi.ptr(c), capi.ptr(vals)) == 0
    assert lib.alphasparse_convert_csr(coo, 0, byref(csr)) == 0
    idx, rr, cc = ctypes.c_int(), c_int32(), c_int32()
    rs, re, ci, va = c_void_p(), c_void_p(), c_void_p(), c_void_p()
    assert getattr(lib, "alphasparse_%s_export_csr" % p)(csr, byref(idx), byref(rr), byref(cc), byref(rs), byref(re), byref(ci), byref(va)) == 0
    T = c_float if p == "s" else c_double
    row_start = np.ctypeslib.as_array(ctypes.cast(rs, POINTER(c_int32)), (m,)).copy()
    row_end = np.ctypeslib.as_array(ctypes.cast(re, POINTER(c_int32)), (m,)).copy()
    nnz = int(row_end[-1])
    col = np.ctypeslib.as_array(ctypes.cast(ci, POINTER(c_int32)), (max(nnz, 1),)).copy()[:nnz]
    val = np.ctypeslib.as_array(ctypes.cast(va, POINTER(T)), (max(nnz, 1),)).copy()[:nnz]
    assert lib.alphasparse_convert_csr(coo, 1, byref(capi.alphasparse_matrix_t())) == S.ALPHA_SPARSE_STATUS_NOT_SUPPORTED
    assert lib.alphasparse_convert_csr(csr, 0, byref(capi.alphasparse_matrix_t())) == S.ALPHA_SPARSE_STATUS_INVALID_VALUE
    assert lib.alphasparse_destroy(coo) == 0 and lib.alphasparse_destroy(csr) == 0
    return (idx.value, rr.value, cc.value), row_start, row_end, col, val


@pytest.mark.parametrize("dtype", [np.float32, np.float64], ids=["f32", "f64"])
def test_coo_to_csr_conversion(lib, dtype):
    rng = np.random.default_rng(8)
    for a in (wl.powerlaw_rmat(9, 200, dtype), wl.laplace2d(13, 7, dtype), wl.uniform_rows(50, 400, 8, dtype)):
        rows = orc.csr2coo(a)
        perm = rng.permutation(a.nnz)
        for base in (0, 1):
            hdr, rs, re, col, val = convert(lib, rows[perm], a.col_ind[perm], a.values[perm], a.rows, a.cols, base)
            assert hdr == (0, a.rows, a.cols)
            assert np.array_equal(rs, a.row_ptr[:-1]) and np.array_equal(re, a.row_ptr[1:])
            assert np.array_equal(col, a.col_ind) and np.array_equal(val, a.values)   # sorted columns, unique entries
    # duplicates are kept, in source order; empty rows at both ends
    rows = np.array([3, 1, 3, 1, 3], np.int32)
    cols = np.array([2, 0, 2, 0, 1], np.int32)
    vals = np.array([10, 20, 30, 40, 50], dtype)
    hdr, rs, re, col, val = convert(lib, rows, cols, vals, 6, 4)
    assert rs.tolist() == [0, 0, 2, 2, 5, 5] and re.tolist() == [0, 2, 2, 5, 5, 5]
    assert col.tolist() == [0, 0, 1, 2, 2] and val.tolist() == [20, 40, 50, 10, 30]
    # an entry outside the matrix is refused
    coo, csr = capi.alphasparse_matrix_t(), capi.alphasparse_matrix_t()
    bad = np.array([0, 6], np.int32)
    p = "s" if dtype == np.float32 else "d"
    assert getattr(lib, "alphasparse_%s_create_coo" % p)(byref(coo), 0, 6, 4, 2, capi.ptr(bad), capi.ptr(np.zeros(2, np.int32)), capi.ptr(np.ones(2, dtype))) == 0
    assert lib.alphasparse_convert_csr(coo, 0, byref(csr)) == S.ALPHA_SPARSE_STATUS_INVALID_VALUE
    assert lib.alphasparse_destroy(coo) == 0
    assert getattr(lib, "alphasparse_%s_create_coo" % p)(byref(coo), 0, 0, 4, 0, None, None, None) == S.ALPHA_SPARSE_STATUS_INVALID_VALUE
    assert getattr(lib, "alphasparse_%s_create_coo" % p)(byref(coo), 0, 6, 4, 2, None, capi.ptr(bad), capi.ptr(bad)) == S.ALPHA_SPARSE_STATUS_INVALID_POINTER


@pytest.mark.skipif(not orc.ref_available(), reason="oracle/_ref not built (reference tree absent)")
@pytest.mark.parametrize("dtype", [np.float32, np.float64], ids=["f32", "f64"])
def test_coo_to_csr_matches_the_reference_converter(lib, dtype):
    """convert_csr_?_coo compiled from the reference's source, on shuffled entries without duplicates."""
    from ctypes import Structure, c_bool
    t = "s" if dtype == np.float32 else "d"

    class Coo(Structure):  # include/alphasparse/spmat.h:73-86
        _fields_ = [("values", c_void_p), ("row_indx", c_void_p), ("col_indx", c_void_p), ("rows", c_int32), ("cols", c_int32),
                    ("nnz", c_int32), ("ordered", c_bool), ("d_rows_indx", c_void_p), ("d_cols_indx", c_void_p), ("d_values", c_void_p)]

    L = orc.ref_lib()
    f = getattr(L, "convert_csr_%s_coo" % t)
    f.argtypes = [POINTER(Coo), POINTER(c_void_p)]
    a = wl.powerlaw_rmat(10, 600, dtype)
    perm = np.random.default_rng(2).permutation(a.nnz)
    rows, cols, vals = orc.csr2coo(a)[perm].copy(), a.col_ind[perm].copy(), a.values[perm].copy()
    coo = Coo(vals.ctypes.data, rows.ctypes.data, cols.ctypes.data, a.rows, a.cols, a.nnz, False, None, None, None)
    out = c_void_p()
    assert f(byref(coo), byref(out)) == 0
    ref = ctypes.cast(out, POINTER(orc._ref_csr_struct(c_float if t == "s" else c_double))).contents
    ref_rs = np.ctypeslib.as_array(ctypes.cast(ref.rows_start, POINTER(c_int32)), (a.rows,))
    ref_re = np.ctypeslib.as_array(ctypes.cast(ref.rows_end, POINTER(c_int32)), (a.rows,))
    ref_ci = np.ctypeslib.as_array(ctypes.cast(ref.col_indx, POINTER(c_int32)), (a.nnz,))
    ref_v = np.ctypeslib.as_array(ctypes.cast(ref.values, POINTER(c_float if t == "s" else c_double)), (a.nnz,))
    _, rs, re, col, val = convert(lib, rows, cols, vals, a.rows, a.cols)
    assert np.array_equal(rs, ref_rs) and np.array_equal(re, ref_re) and np.array_equal(col, ref_ci) and np.array_equal(val, ref_v)


def test_command_line_flags(lib):
    n, av = argv("--data-file=/tmp/a.mtx", "--check", "--transA=T", "--layout=C", "--columns=17", "--iter=9", "--typeA=S",
                 "--fillA=U", "--diagA=U", "--thread-num=3")
    assert lib.args_get_data_file(n, av) == b"/tmp/a.mtx"
    assert lib.args_get_if_check(n, av) is True
    assert lib.alpha_args_get_transA(n, av) == S.ALPHA_SPARSE_OPERATION_TRANSPOSE
    assert lib.alpha_args_get_transB(n, av) == S.ALPHA_SPARSE_OPERATION_NON_TRANSPOSE
    assert lib.alpha_args_get_layout(n, av) == S.ALPHA_SPARSE_LAYOUT_COLUMN_MAJOR
    assert lib.args_get_columns(n, av, 5) == 17 and lib.args_get_iter(n, av) == 9 and lib.args_get_thread_num(n, av) == 3
    d = lib.alpha_args_get_matrix_descrA(n, av)
    assert (d.type, d.mode, d.diag) == (S.ALPHA_SPARSE_MATRIX_TYPE_SYMMETRIC, 1, 1)
    n, av = argv()
    assert lib.args_get_data_file(n, av) == b"" and lib.args_get_if_check(n, av) is False
    assert lib.args_get_columns(n, av, 5) == 5 and lib.args_get_iter(n, av) == 1
    assert lib.alpha_args_get_layout(n, av) == S.ALPHA_SPARSE_LAYOUT_ROW_MAJOR
    d = lib.alpha_args_get_matrix_descrA(n, av)
    assert (d.type, d.mode, d.diag) == (0, 0, 0)
    lib.args_help(n, av)   # no --help: returns


def test_result_check_and_fill(lib, capfd):
    a = np.array([1.0, -2.0, 3.0], np.float32)
    assert lib.check_s(capi.ptr(a), 3, capi.ptr(a.copy()), 3) == 0
    b = a.copy()
    b[1] += 1e-3
    assert lib.check_s(capi.ptr(a), 3, capi.ptr(b), 3) == -1
    assert lib.check_s(capi.ptr(a), 3, capi.ptr(b), 2) == -1
    d = a.astype(np.float64)
    e = d.copy()
    e[2] *= 1 + 1e-12
    assert lib.check_d(capi.ptr(d), 3, capi.ptr(e), 3) == 0
    e[2] *= 1 + 1e-8
    assert lib.check_d(capi.ptr(d), 3, capi.ptr(e), 3) == -1
    ctypes.CDLL(None).fflush(None)   # the library prints through C stdio
    out = capfd.readouterr().out
    assert "correct," in out and "error," in out
    x, y = np.empty(100, np.float32), np.empty(100, np.float32)
    lib.alpha_fill_random_s(capi.ptr(x), 7, 100)
    lib.alpha_fill_random_s(capi.ptr(y), 7, 100)
    assert np.array_equal(x, y) and x.min() >= 0 and x.max() <= 1 and np.unique(x).size > 50
    p = lib.alpha_memalign(100, 64)
    assert p % 64 == 0
    lib.alpha_free(p)


@pytest.mark.parametrize("dtype", [np.float32, np.float64], ids=["f32", "f64"])
def test_coo_to_ell_conversion(lib, dtype):
    """alphasparse_convert_ell + alphasparse_?_export_ell against the oracle's csr2ell (itself pinned
    bit for bit against the reference's converter) on shuffled entries."""
    p = "s" if dtype == np.float32 else "d"
    T = c_float if p == "s" else c_double
    a = wl.powerlaw_rmat(9, 60, dtype)
    perm = np.random.default_rng(6).permutation(a.nnz)
    rows, cols, vals = orc.csr2coo(a)[perm].copy(), a.col_ind[perm].copy(), a.values[perm].copy()
    coo, ell = capi.alphasparse_matrix_t(), capi.alphasparse_matrix_t()
    assert getattr(lib, "alphasparse_%s_create_coo" % p)(byref(coo), 0, a.rows, a.cols, a.nnz, capi.ptr(rows), capi.ptr(cols), capi.ptr(vals)) == 0
    assert lib.alphasparse_convert_ell(coo, 0, byref(ell)) == 0
    idx, rr, cc, w = ctypes.c_int(), c_int32(), c_int32(), c_int32()
    ci, va = c_void_p(), c_void_p()
    assert getattr(lib, "alphasparse_%s_export_ell" % p)(ell, byref(idx), byref(rr), byref(cc), byref(w), byref(ci), byref(va)) == 0
    assert (idx.value, rr.value, cc.value, w.value) == (0, a.rows, a.cols, orc.csr2ell_width(a))
    n = w.value * a.rows
    got_c = np.ctypeslib.as_array(ctypes.cast(ci, POINTER(c_int32)), (n,)).copy()
    got_v = np.ctypeslib.as_array(ctypes.cast(va, POINTER(T)), (n,)).copy()
    ev, ec = orc.csr2ell(a)
    assert np.array_equal(got_c, ec) and np.array_equal(got_v, ev)
    other = "d" if p == "s" else "s"
    assert getattr(lib, "alphasparse_%s_export_ell" % other)(ell, byref(idx), byref(rr), byref(cc), byref(w), byref(ci), byref(va)) == S.ALPHA_SPARSE_STATUS_INVALID_VALUE
    assert getattr(lib, "alphasparse_%s_export_ell" % p)(coo, byref(idx), byref(rr), byref(cc), byref(w), byref(ci), byref(va)) == S.ALPHA_SPARSE_STATUS_INVALID_VALUE
    assert lib.alphasparse_convert_ell(ell, 0, byref(capi.alphasparse_matrix_t())) == S.ALPHA_SPARSE_STATUS_INVALID_VALUE
    assert lib.alphasparse_destroy(coo) == 0 and lib.alphasparse_destroy(ell) == 0


def test_thread_count_is_kept_as_in_the_reference():
    """src/util/thread.c:22-38: 0 means every core, anything else is returned as set."""
    lib = capi.load()
    lib.alpha_set_thread_num(0)
    assert lib.alpha_get_thread_num() == lib.alpha_get_core_num() >= 1
    lib.alpha_set_thread_num(3)
    assert lib.alpha_get_thread_num() == 3
    lib.alpha_set_thread_num(0)


def test_operation_counts_and_timers():
    """src/util/analysis.c:8-56, :126-153 and src/util/timer.c of the reference."""
    import ctypes
    from ctypes import byref, c_int32
    lib = capi.load()
    rows = np.array([0, 1, 1, 2, 2, 2], dtype=np.int32)
    cols = np.array([0, 0, 1, 0, 2, 3], dtype=np.int32)
    lo, di, hi = c_int32(), c_int32(), c_int32()
    lib.alphasparse_nnz_counter_coo(capi.ptr(rows), capi.ptr(cols), 6, byref(lo), byref(di), byref(hi))
    assert (lo.value, di.value, hi.value) == (2, 3, 1)
    general = capi.alpha_matrix_descr(0, 0, 0)
    # real: 2 flops per entry + 3 per row; complex: 9 per entry + 16 per row; times the dense columns
    assert lib.alphasparse_operations_mv(3, 4, 2, 3, 1, 0, general, 0) == 6 * 2 + 3 * 3
    assert lib.alphasparse_operations_mm(3, 4, 2, 3, 1, 0, general, 5, 3) == (6 * 9 + 3 * 16) * 5
    lower_unit = capi.alpha_matrix_descr(capi.ALPHA_SPARSE_MATRIX_TYPE_SYMMETRIC, 0, 1)
    assert lib.alphasparse_operations_mv(3, 4, 2, 3, 1, 0, lower_unit, 0) == (2 + 3) * 2 + 3 * 3

    class Timer(ctypes.Structure):
        _fields_ = [("start", ctypes.c_double), ("end", ctypes.c_double)]
    t = Timer()
    lib.alpha_timing_start(byref(t))
    lib.alpha_timing_end(byref(t))
    assert 0 <= lib.alpha_timing_elapsed_time(byref(t)) < 1.0
    t.start, t.end = 1.0, 3.0
    assert lib.alpha_timing_gflops(byref(t), 4_000_000_000) == 2.0
    lib.alpha_clear_cache()


def test_level2_residual_check_accepts_rounding_and_rejects_errors(tmp_path, capfd):
    """check_s_l2 (src/util/check.c:7-57): resid = |d| / (|A|_1 |x| |y| 10 eps max(m, k)) against 50."""
    import ctypes
    lib = capi.load()
    path = tmp_path / "m.mtx"
    path.write_text("%%MatrixMarket matrix coordinate real general\n3 3 4\n1 1 2.0\n2 2 -3.0\n3 1 1.0\n3 3 0.5\n")
    argv = (ctypes.c_char_p * 2)(b"prog", ("--data-file=%s" % path).encode())
    x = np.array([1.0, 2.0, 3.0], dtype=np.float32)
    y = np.array([2.0, -6.0, 2.5], dtype=np.float32)
    near = y + np.float32(1e-6)
    far = y + np.float32(1e-2)
    assert lib.check_s_l2(capi.ptr(near), 3, capi.ptr(y), 3, capi.ptr(x), None, 1.0, 0.0, 2, argv) == 0
    assert lib.check_s_l2(capi.ptr(far), 3, capi.ptr(y), 3, capi.ptr(x), None, 1.0, 0.0, 2, argv) == -1
    assert lib.check_s_l2(capi.ptr(y), 3, capi.ptr(y), 2, capi.ptr(x), None, 1.0, 0.0, 2, argv) == -1   # size mismatch
    ctypes.CDLL(None).fflush(None)
    out = capfd.readouterr().out
    assert "correct," in out and "error," in out and "normA : 3.0" in out
