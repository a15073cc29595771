"""The C-ABI library loads and exports every symbol that include/*.h declares;
enum values and struct layouts are those of the reference headers.  No GPU."""
import ctypes
import os
import re
import subprocess

import pytest

from alsparse_amd import capi
from alsparse_amd.build import LIB_PATH, ROOT

HEADERS = ["alphasparse.h", "alphasparse_util.h", "alpha_spblas_dcu.h", "alsparse_amd_kernels.h", "alsparse_amd_plan.h"]


def declared_functions():
    names = set()
    for h in HEADERS:
        text = open(os.path.join(ROOT, "include", h)).read()
        text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
        for m in re.finditer(r"\b([A-Za-z_][A-Za-z0-9_]*)\s*\(", text):
            n = m.group(1)
            if n.startswith(("alphasparse_", "asamd_", "host2device_", "init_handle", "get_alphasparse", "alpha_malloc",
                             "alpha_memalign", "alpha_free", "alpha_fill_", "alpha_read_", "alpha_args_", "args_", "check_",
                             "alpha_get_core_num", "alpha_set_thread_num", "alpha_get_thread_num", "alpha_timing_",
                             "alpha_clear_cache",
                             "get_time_us")):
                names.add(n)
    return names


def test_library_exports_every_declared_symbol():
    lib = ctypes.CDLL(LIB_PATH)
    declared = declared_functions()
    assert len(declared) >= 45
    missing = [n for n in sorted(declared) if not hasattr(lib, n)]
    assert not missing, "declared in include/*.h but not exported: %s" % missing


def test_python_bindings_cover_every_declared_symbol():
    lib = capi.load()
    protos = capi.prototypes()
    for n in declared_functions():
        assert n in protos, "no ctypes prototype for %s" % n
        assert getattr(lib, n).argtypes is not None


def test_headers_compile_as_c_and_cxx(tmp_path):
    src = tmp_path / "t.c"
    src.write_text('#include "alpha_spblas_dcu.h"\n#include "alsparse_amd_kernels.h"\n#include "alsparse_amd_plan.h"\n'
                   "int main(void){ alphasparse_dcu_handle h; (void)h; return sizeof(struct _alphasparse_dcu_mat_info) == 0; }\n")
    inc = ["-I" + os.path.join(ROOT, "include"), "-I/opt/rocm/include"]
    subprocess.check_call(["gcc", "-std=c11", "-Wall", "-Werror", "-fsyntax-only", str(src)] + inc)
    subprocess.check_call(["g++", "-std=c++14", "-Wall", "-fsyntax-only", "-x", "c++", str(src)] + inc)


def test_enum_values_are_the_reference_abi():
    # include/alphasparse/spdef.h:8-19, :22-27, :32-41, :46-50, :73-77, :120-143 of the reference
    assert (capi.ALPHA_SPARSE_STATUS_SUCCESS, capi.ALPHA_SPARSE_STATUS_NOT_INITIALIZED,
            capi.ALPHA_SPARSE_STATUS_ALLOC_FAILED, capi.ALPHA_SPARSE_STATUS_INVALID_VALUE,
            capi.ALPHA_SPARSE_STATUS_EXECUTION_FAILED, capi.ALPHA_SPARSE_STATUS_INTERNAL_ERROR,
            capi.ALPHA_SPARSE_STATUS_NOT_SUPPORTED, capi.ALPHA_SPARSE_STATUS_INVALID_POINTER,
            capi.ALPHA_SPARSE_STATUS_INVALID_HANDLE) == tuple(range(9))
    text = open(os.path.join(ROOT, "include", "alphasparse.h")).read()
    for name, value in (("ALPHA_SPARSE_FORMAT_CSR", 1), ("ALPHA_SPARSE_FORMAT_ELL", 6), ("ALPHA_SPARSE_FORMAT_CSR5", 10),
                        ("ALPHA_SPARSE_DATATYPE_DOUBLE", 1), ("ALPHA_SPARSE_LAYOUT_COLUMN_MAJOR", 1),
                        ("ALPHA_SPARSE_OPERATION_CONJUGATE_TRANSPOSE", 2), ("ALPHA_SPARSE_INDEX_BASE_ONE", 1),
                        ("ALPHA_SPARSE_MATRIX_TYPE_GENERAL", 0), ("ALPHA_SPARSE_STATUS_INVALID_HANDLE", 8)):
        assert re.search(r"\b%s\s*=\s*%d\b" % (name, value), text), name


def test_struct_layouts_match_c(tmp_path):
    """sizeof / offsetof as the C compiler sees them == what the ctypes mirrors use."""
    src = tmp_path / "layout.c"
    src.write_text(r'''
#include <stdio.h>
#include <stddef.h>
#include "alpha_spblas_dcu.h"
#include "alsparse_amd_plan.h"
int main(void) {
  printf("%zu %zu %zu %zu\n", sizeof(alphasparse_matrix), offsetof(alphasparse_matrix, format),
         offsetof(alphasparse_matrix, inspector), offsetof(alphasparse_matrix, dcu_info));
  printf("%zu %zu %zu %zu %zu\n", sizeof(spmat_csr_s_t), offsetof(spmat_csr_s_t, rows),
         offsetof(spmat_csr_s_t, ordered), offsetof(spmat_csr_s_t, d_values), offsetof(spmat_csr_d_t, d_col_indx));
  printf("%zu %zu %zu\n", sizeof(struct _alphasparse_dcu_csrmv_info), offsetof(struct _alphasparse_dcu_csrmv_info, m),
         offsetof(struct _alphasparse_dcu_csrmv_info, csr_row_ptr));
  printf("%zu %zu %zu\n", sizeof(struct _alphasparse_dcu_mat_info), offsetof(struct _alphasparse_dcu_mat_info, csrmv_info),
         offsetof(struct _alphasparse_dcu_mat_info, boost_enable));
  printf("%zu %zu\n", sizeof(asamd_csr_stats), offsetof(asamd_csr_stats, hist));
  printf("%zu %zu\n", sizeof(struct alpha_dcu_matrix_descr), sizeof(struct alpha_matrix_descr));
  printf("%zu %zu %zu %zu %zu\n", sizeof(struct _alphasparse_dcu_spmat_descr), offsetof(struct _alphasparse_dcu_spmat_descr, rows),
         offsetof(struct _alphasparse_dcu_spmat_descr, val_data), offsetof(struct _alphasparse_dcu_spmat_descr, format),
         offsetof(struct _alphasparse_dcu_spmat_descr, info));
  printf("%zu %zu %zu\n", sizeof(struct _alphasparse_dcu_dnvec_descr), offsetof(struct _alphasparse_dcu_dnvec_descr, values),
         offsetof(struct _alphasparse_dcu_dnvec_descr, data_type));
  return 0;
}''')
    exe = tmp_path / "layout"
    subprocess.check_call(["gcc", "-std=c11", str(src), "-o", str(exe), "-I" + os.path.join(ROOT, "include"), "-I/opt/rocm/include"])
    out = subprocess.check_output([str(exe)], text=True).split("\n")
    nums = [[int(v) for v in line.split()] for line in out if line]
    M, S, D = capi.alphasparse_matrix, capi.spmat_csr_s_t, capi.spmat_csr_d_t
    CI, MI, ST = capi._alphasparse_dcu_csrmv_info, capi._alphasparse_dcu_mat_info, capi.asamd_csr_stats
    assert nums[0] == [ctypes.sizeof(M), M.format.offset, M.inspector.offset, M.dcu_info.offset]
    assert nums[1] == [ctypes.sizeof(S), S.rows.offset, S.ordered.offset, S.d_values.offset, D.d_col_indx.offset]
    assert nums[2] == [ctypes.sizeof(CI), CI.m.offset, CI.csr_row_ptr.offset]
    assert nums[3] == [ctypes.sizeof(MI), MI.csrmv_info.offset, MI.boost_enable.offset]
    assert nums[4] == [ctypes.sizeof(ST), ST.hist.offset]
    assert nums[5] == [ctypes.sizeof(capi.alpha_dcu_matrix_descr), ctypes.sizeof(capi.alpha_matrix_descr)]
    SM, DV = capi.alphasparse_dcu_spmat_descr, capi.alphasparse_dcu_dnvec_descr
    assert nums[6] == [ctypes.sizeof(SM), SM.rows.offset, SM.val_data.offset, SM.format.offset, SM.info.offset]
    assert nums[7] == [ctypes.sizeof(DV), DV.values.offset, DV.data_type.offset]


def test_no_product_code_touches_the_oracle():
    """The shipped library and package must not import, link or call anything under oracle/."""
    bad = []
    for base, _, files in os.walk(os.path.join(ROOT, "alsparse_amd")):
        for f in files:
            if f.endswith((".py", ".c", ".h", ".hip", ".hpp", ".inc")) or f == "Makefile":
                text = open(os.path.join(base, f), errors="ignore").read()
                if re.search(r"\boracle\b", text) and not f == "build.py":
                    bad.append(os.path.join(base, f))
    assert not bad, bad
    out = subprocess.check_output(["ldd", LIB_PATH], text=True)
    assert "oracle" not in out
