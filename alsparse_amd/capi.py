"""ctypes bindings of ``libalpha_spblas.so``: the same names, argument order and
status codes as the reference's C API (``include/alphasparse.h`` and
``include/alpha_spblas_dcu.h`` of this repository list each entry with the
reference declaration it replaces).

There is no fallback: if the library has not been built, :func:`load` raises.
"""
import ctypes
import os
from ctypes import POINTER, Structure, byref, c_bool, c_double, c_float, c_int, c_int32, c_int64, c_size_t, c_void_p

from .build import LIB_PATH, PROBES_PATH

# ---- enums (values are ABI) -------------------------------------------------
ALPHA_SPARSE_STATUS_SUCCESS = 0
ALPHA_SPARSE_STATUS_NOT_INITIALIZED = 1
ALPHA_SPARSE_STATUS_ALLOC_FAILED = 2
ALPHA_SPARSE_STATUS_INVALID_VALUE = 3
ALPHA_SPARSE_STATUS_EXECUTION_FAILED = 4
ALPHA_SPARSE_STATUS_INTERNAL_ERROR = 5
ALPHA_SPARSE_STATUS_NOT_SUPPORTED = 6
ALPHA_SPARSE_STATUS_INVALID_POINTER = 7
ALPHA_SPARSE_STATUS_INVALID_HANDLE = 8

ALPHA_SPARSE_OPERATION_NON_TRANSPOSE = 0
ALPHA_SPARSE_OPERATION_TRANSPOSE = 1
ALPHA_SPARSE_OPERATION_CONJUGATE_TRANSPOSE = 2

ALPHA_SPARSE_MATRIX_TYPE_GENERAL = 0
ALPHA_SPARSE_MATRIX_TYPE_SYMMETRIC = 1

ALPHA_SPARSE_INDEX_BASE_ZERO = 0
ALPHA_SPARSE_INDEX_BASE_ONE = 1

ALPHA_SPARSE_LAYOUT_ROW_MAJOR = 0
ALPHA_SPARSE_LAYOUT_COLUMN_MAJOR = 1

ALPHA_SPARSE_FORMAT_COO, ALPHA_SPARSE_FORMAT_CSR, ALPHA_SPARSE_FORMAT_BSR = 0, 1, 3
ALPHA_SPARSE_FORMAT_ELL, ALPHA_SPARSE_FORMAT_COO_AOS = 6, 9
ALPHA_SPARSE_DATATYPE_FLOAT = 0
ALPHA_SPARSE_DATATYPE_DOUBLE = 1
ALPHA_SPARSE_DATATYPE_FLOAT_COMPLEX, ALPHA_SPARSE_DATATYPE_DOUBLE_COMPLEX = 2, 3

# kernel families of the thin kernel ABI (include/alsparse_amd_kernels.h)
(ASAMD_SPMV_AUTO, ASAMD_SPMV_VECTOR, ASAMD_SPMV_ROWCONST, ASAMD_SPMV_MERGE, ASAMD_SPMV_SCALAR, ASAMD_SPMV_TILED,
 ASAMD_SPMV_STREAM, ASAMD_SPMV_ELL, ASAMD_SPMV_MERGE_HOT, ASAMD_SPMV_BINNED, ASAMD_SPMV_XLDS) = range(11)
ASAMD_HIST_BINS = 33


# ---- structs ------------------------------------------------------------------
class alphasparse_matrix(Structure):
    _fields_ = [("mat", c_void_p), ("format", c_int), ("datatype", c_int),
                ("inspector", c_void_p), ("dcu_info", c_void_p)]


alphasparse_matrix_t = POINTER(alphasparse_matrix)


class alpha_matrix_descr(Structure):
    _fields_ = [("type", c_int), ("mode", c_int), ("diag", c_int)]


class alpha_dcu_matrix_descr(Structure):
    _fields_ = [("type", c_int), ("mode", c_int), ("diag", c_int), ("base", c_int)]


alpha_dcu_matrix_descr_t = POINTER(alpha_dcu_matrix_descr)


def _csr_struct(ctype):
    class _S(Structure):
        _fields_ = [("values", POINTER(ctype)), ("rows_start", POINTER(c_int32)),
                    ("rows_end", POINTER(c_int32)), ("col_indx", POINTER(c_int32)),
                    ("rows", c_int32), ("cols", c_int32), ("ordered", c_bool),
                    ("d_values", c_void_p), ("d_row_ptr", c_void_p), ("d_col_indx", c_void_p)]
    return _S


spmat_csr_s_t = _csr_struct(c_float)
spmat_csr_d_t = _csr_struct(c_double)


class _alphasparse_dcu_csrmv_info(Structure):
    _fields_ = [("algo_tuning", c_bool), ("algo", c_int), ("iter", c_int32), ("size", c_size_t),
                ("row_blocks", c_void_p), ("csr_adaptive_has_tuned", c_bool), ("trans", c_int),
                ("m", c_int32), ("n", c_int32), ("nnz", c_int32), ("descr", c_void_p),
                ("csr_row_ptr", c_void_p), ("csr_col_ind", c_void_p)]


class _alphasparse_dcu_mat_info(Structure):
    _fields_ = ([(n, c_void_p) for n in (
        "bsrsv_upper_info", "bsrsv_lower_info", "bsrsvt_upper_info", "bsrsvt_lower_info",
        "bsric0_info", "bsrilu0_info")] +
        [("csrmv_info", POINTER(_alphasparse_dcu_csrmv_info))] +
        [(n, c_void_p) for n in (
            "csric0_info", "csrilu0_info", "csrsv_upper_info", "csrsv_lower_info",
            "csrsvt_upper_info", "csrsvt_lower_info", "csrsm_upper_info", "csrsm_lower_info",
            "csrsmt_upper_info", "csrsmt_lower_info", "csrgemm_info", "zero_pivot")] +
        [("boost_enable", c_int), ("use_double_prec_tol", c_int),
         ("boost_tol", c_void_p), ("boost_val", c_void_p)])


alphasparse_dcu_mat_info_t = POINTER(_alphasparse_dcu_mat_info)
alphasparse_dcu_handle_t = c_void_p  # opaque from Python: holds a hipDeviceProp_t


class alphasparse_dcu_spmat_descr(Structure):  # include/alphasparse/handle.h:272-295 of the reference
    _fields_ = [("init", c_bool), ("analysed", c_bool), ("rows", c_int64), ("cols", c_int64), ("nnz", c_int64),
                ("row_data", c_void_p), ("col_data", c_void_p), ("ind_data", c_void_p), ("val_data", c_void_p),
                ("row_type", c_int), ("col_type", c_int), ("data_type", c_int), ("idx_base", c_int), ("format", c_int),
                ("descr", POINTER(alpha_dcu_matrix_descr)), ("info", alphasparse_dcu_mat_info_t)]


class alphasparse_dcu_dnvec_descr(Structure):  # include/alphasparse/handle.h:297-304
    _fields_ = [("init", c_bool), ("size", c_int64), ("values", c_void_p), ("data_type", c_int)]


ALPHA_SPARSE_DCU_INDEXTYPE_U16, ALPHA_SPARSE_DCU_INDEXTYPE_I32, ALPHA_SPARSE_DCU_INDEXTYPE_I64 = 1, 2, 3
(ALPHA_SPARSE_DCU_SPMV_ALG_DEFAULT, ALPHA_SPARSE_DCU_SPMV_ALG_COO, ALPHA_SPARSE_DCU_SPMV_ALG_CSR_ADAPTIVE,
 ALPHA_SPARSE_DCU_SPMV_ALG_CSR_STREAM, ALPHA_SPARSE_DCU_SPMV_ALG_ELL) = range(5)


class asamd_csr_stats(Structure):
    _fields_ = [("m", c_int32), ("n", c_int32), ("nnz", c_int32), ("base", c_int32),
                ("min_len", c_int32), ("max_len", c_int32), ("const_len", c_int32),
                ("first_offset", c_int32), ("algo", c_int32), ("vector_width", c_int32),
                ("merge_blocks", c_int32), ("trusted", c_int32), ("tiled_built", c_int32),
                ("tile_col_blocks", c_int32), ("tile_row_blocks", c_int32),
                ("tune_ms_base", c_float), ("tune_ms_tiled", c_float), ("tune_ms_ell", c_float),
                ("ell_built", c_int32), ("ell_width", c_int32), ("transpose_built", c_int32),
                ("tile_entries_per_lane", c_int32),
                ("hist", ctypes.c_int64 * ASAMD_HIST_BINS),
                ("hot_built", c_int32), ("hot_cols_lds", c_int32), ("hot_cols", c_int32),
                ("hot_share_lds", c_float), ("tune_ms_hot", c_float),
                ("binned_built", c_int32), ("bin_rows", c_int32 * 4), ("tune_ms_binned", c_float),
                ("tile_long_blocks", c_int32), ("value_check", c_int32), ("tune_mode", c_int32),
                ("device_bytes", c_int64), ("workspace_bytes", c_int64),
                ("lines_per_entry_wave", c_float), ("lines_per_entry_segment", c_float),
                ("xlds_slices", c_int32)]


class asamd_spmv_args(Structure):  # include/alsparse_amd_kernels.h
    _fields_ = [("dtype", c_int32), ("m", c_int32), ("n", c_int32), ("nnz", c_int32), ("base", c_int32),
                ("alpha", c_void_p), ("beta", c_void_p), ("val", c_void_p), ("row_ptr", c_void_p),
                ("col_ind", c_void_p), ("x", c_void_p), ("y", c_void_p)]


class asamd_xlds_layout(Structure):  # include/alsparse_amd_kernels.h
    _fields_ = [("seg", c_void_p), ("slices", c_int32), ("slice_cols", c_int32), ("m", c_int32),
                ("device_bytes", ctypes.c_int64), ("off", c_void_p), ("val", c_void_p), ("col", c_void_p),
                ("dtype", c_int32), ("nnz", c_int32), ("base", c_int32)]


class asamd_dense_strides(Structure):
    _fields_ = [("b_row_stride", ctypes.c_int64), ("b_col_stride", ctypes.c_int64),
                ("c_row_stride", ctypes.c_int64), ("c_col_stride", ctypes.c_int64)]


_I, _P = c_int32, c_void_p


class ALPHA_Complex8(Structure):  # include/alphasparse/types.h:42-47 of the reference
    _fields_ = [("real", c_float), ("imag", c_float)]

    def __init__(self, v=0):
        v = complex(v)
        super().__init__(v.real, v.imag)


class ALPHA_Complex16(Structure):  # include/alphasparse/types.h:50-55
    _fields_ = [("real", c_double), ("imag", c_double)]

    def __init__(self, v=0):
        v = complex(v)
        super().__init__(v.real, v.imag)


ASAMD_DTYPE_FLOAT, ASAMD_DTYPE_DOUBLE, ASAMD_DTYPE_FLOAT_COMPLEX, ASAMD_DTYPE_DOUBLE_COMPLEX = range(4)


def _per_type(ctype):
    """Public entry points that exist once per value type (s, d, c, z); T is the scalar ctype."""
    T, PT = ctype, POINTER(ctype)
    return {
        "alphasparse_{s}_create_csr": [POINTER(alphasparse_matrix_t), c_int, _I, _I, _P, _P, _P, _P],
        "alphasparse_{s}_create_coo": [POINTER(alphasparse_matrix_t), c_int, _I, _I, _I, _P, _P, _P],
        "alphasparse_{s}_export_ell": [alphasparse_matrix_t, POINTER(c_int), POINTER(_I), POINTER(_I), POINTER(_I),
                                       POINTER(_P), POINTER(_P)],
        "alphasparse_{s}_export_csr": [alphasparse_matrix_t, POINTER(c_int), POINTER(_I), POINTER(_I),
                                       POINTER(_P), POINTER(_P), POINTER(_P), POINTER(_P)],
        "alphasparse_{s}_mv": [c_int, T, alphasparse_matrix_t, alpha_matrix_descr, _P, T, _P],
        "alphasparse_{s}_mm": [c_int, T, alphasparse_matrix_t, alpha_matrix_descr, c_int, _P, _I, _I, T, _P, _I],
        "alphasparse_{s}_mv_plain": [c_int, T, alphasparse_matrix_t, alpha_matrix_descr, _P, T, _P],
        "alphasparse_{s}_mm_plain": [c_int, T, alphasparse_matrix_t, alpha_matrix_descr, c_int, _P, _I, _I, T, _P, _I],
        "check_{s}_l2": [_P, c_size_t, _P, c_size_t, _P, _P, T, T, c_int, POINTER(ctypes.c_char_p)],
        "check_{s}_l3": [_P, _I, c_size_t, _P, _I, c_size_t, _P, _P, _I, _P, _I, T, T, c_int, POINTER(ctypes.c_char_p)],
        "asamd_{s}_csrmv_plain": [_P, _I, _I, _I, _I, T, _P, _P, _P, _P, T, _P],
        "asamd_{s}_csrmm_plain": [_P, _I, _I, T, _P, _P, _P, _I, _P, T, _P, POINTER(asamd_dense_strides)],
        "host2device_{s}_csr": [alphasparse_matrix_t],
        "host2device_{s}_coo": [alphasparse_matrix_t],
        "host2device_{s}_ell": [alphasparse_matrix_t],
        "alphasparse_{s}_mv_dcu": [alphasparse_dcu_handle_t, c_int, PT, alphasparse_matrix_t,
                                   alpha_dcu_matrix_descr_t, _P, PT, _P],
        "alphasparse_dcu_{s}_csrmv_analysis": [alphasparse_dcu_handle_t, c_int, _I, _I, _I,
                                               alpha_dcu_matrix_descr_t, _P, _P, _P, _P],
        "alphasparse_dcu_{s}_csrmv": [alphasparse_dcu_handle_t, c_int, _I, _I, _I, PT,
                                      alpha_dcu_matrix_descr_t, _P, _P, _P, _P, _P, PT, _P],
        "alphasparse_dcu_{s}_csrmm": [alphasparse_dcu_handle_t, c_int, c_int, c_int, _I, _I, _I, _I, PT,
                                      alpha_dcu_matrix_descr_t, _P, _P, _P, _P, _I, PT, _P, _I],
        "alphasparse_dcu_{s}csr2ell": [alphasparse_dcu_handle_t, _I, alpha_dcu_matrix_descr_t, _P, _P, _P,
                                       alpha_dcu_matrix_descr_t, _I, _P, _P],
        "alphasparse_dcu_{s}_coomv": [alphasparse_dcu_handle_t, c_int, _I, _I, _I, PT, alpha_dcu_matrix_descr_t,
                                      _P, _P, _P, _P, PT, _P],
        "alphasparse_dcu_{s}_ellmv": [alphasparse_dcu_handle_t, c_int, _I, _I, PT, alpha_dcu_matrix_descr_t,
                                      _P, _P, _I, _P, PT, _P],
    }


def _per_real_type(ctype):
    """Thin kernel ABI of the real value types."""
    T = ctype
    return {
        "asamd_{s}_ellmv": [_P, _I, _I, T, _P, _P, _I, _I, _P, T, _P],
        "asamd_{s}_coomv": [_P, _I, _I, c_int64, T, _P, _P, _P, _I, _P, T, _P, _P, c_size_t],
        "asamd_{s}_csrmm": [_P, _I, _I, _I, _I, T, _P, _P, _P, _I, _P, T, _P, POINTER(asamd_dense_strides)],
        "asamd_{s}_csrmm_ws": [_P, _I, _I, _I, _I, T, _P, _P, _P, _I, _P, T, _P, POINTER(asamd_dense_strides), _P,
                               c_size_t],
        "asamd_{s}_csr2ell": [_P, _I, _P, _P, _P, _I, _I, _I, _P, _P],
    }


def _per_complex_type(ctype):
    """Prototypes that exist for the complex value types only; T is passed by value."""
    T = ctype
    return {
        # thin kernel ABI
        "asamd_{s}_ellmv": [_P, _I, _I, T, _P, _P, _I, _I, _P, T, _P],
        "asamd_{s}_coomv": [_P, _I, _I, c_int64, T, _P, _P, _P, _I, _P, T, _P, _P, c_size_t],
        "asamd_{s}_csrmm_ws": [_P, _I, _I, _I, _I, T, _P, _P, _P, _I, _P, T, _P, POINTER(asamd_dense_strides), _P,
                               c_size_t],
        "asamd_{s}_csr2ell": [_P, _I, _P, _P, _P, _I, _I, _I, _P, _P],
    }


_COMMON = {
    "alphasparse_destroy": [alphasparse_matrix_t],
    "alphasparse_convert_csr": [alphasparse_matrix_t, c_int, POINTER(alphasparse_matrix_t)],
    "alphasparse_convert_ell": [alphasparse_matrix_t, c_int, POINTER(alphasparse_matrix_t)],
    # driver helpers (include/alphasparse_util.h)
    "alpha_malloc": [c_size_t],
    "alpha_memalign": [c_size_t, c_size_t],
    "alpha_free": [_P],
    "alpha_fill_random_s": [_P, ctypes.c_uint, c_size_t],
    "alpha_fill_random_d": [_P, ctypes.c_uint, c_size_t],
    "alpha_fill_random_c": [_P, ctypes.c_uint, c_size_t],
    "alpha_fill_random_z": [_P, ctypes.c_uint, c_size_t],
    "alpha_read_coo_c": [ctypes.c_char_p, POINTER(_I), POINTER(_I), POINTER(_I), POINTER(_P), POINTER(_P), POINTER(_P)],
    "alpha_read_coo_z": [ctypes.c_char_p, POINTER(_I), POINTER(_I), POINTER(_I), POINTER(_P), POINTER(_P), POINTER(_P)],
    "check_c": [_P, c_size_t, _P, c_size_t],
    "check_z": [_P, c_size_t, _P, c_size_t],
    "alpha_read_coo": [ctypes.c_char_p, POINTER(_I), POINTER(_I), POINTER(_I), POINTER(_P), POINTER(_P), POINTER(_P)],
    "alpha_read_coo_d": [ctypes.c_char_p, POINTER(_I), POINTER(_I), POINTER(_I), POINTER(_P), POINTER(_P), POINTER(_P)],
    "check_s": [_P, c_size_t, _P, c_size_t],
    "check_d": [_P, c_size_t, _P, c_size_t],
    "args_help": [c_int, POINTER(ctypes.c_char_p)],
    "args_get_if_check": [c_int, POINTER(ctypes.c_char_p)],
    "args_get_thread_num": [c_int, POINTER(ctypes.c_char_p)],
    "args_get_columns": [c_int, POINTER(ctypes.c_char_p), c_int],
    "args_get_iter": [c_int, POINTER(ctypes.c_char_p)],
    "args_get_data_file": [c_int, POINTER(ctypes.c_char_p)],
    "args_get_data_fileA": [c_int, POINTER(ctypes.c_char_p)],
    "args_get_data_fileB": [c_int, POINTER(ctypes.c_char_p)],
    "alpha_args_get_layout": [c_int, POINTER(ctypes.c_char_p)],
    "alpha_args_get_layoutB": [c_int, POINTER(ctypes.c_char_p)],
    "alpha_args_get_layoutC": [c_int, POINTER(ctypes.c_char_p)],
    "alpha_args_get_matrix_descrA": [c_int, POINTER(ctypes.c_char_p)],
    "alpha_args_get_matrix_descrB": [c_int, POINTER(ctypes.c_char_p)],
    "alpha_args_get_transA": [c_int, POINTER(ctypes.c_char_p)],
    "alpha_args_get_transB": [c_int, POINTER(ctypes.c_char_p)],
    "get_time_us": [],
    "alpha_timing_wtime": [],
    "alpha_timing_start": [_P],
    "alpha_timing_end": [_P],
    "alpha_timing_elapsed_time": [_P],
    "alpha_timing_gflops": [_P, c_int64],
    "alpha_timing_elaped_time_print": [_P, ctypes.c_char_p],
    "alpha_timing_gflops_print": [_P, c_int64, ctypes.c_char_p],
    "alpha_clear_cache": [],
    "alphasparse_nnz_counter_coo": [_P, _P, _I, POINTER(_I), POINTER(_I), POINTER(_I)],
    "alphasparse_operations_mm": [_I, _I, _I, _I, _I, c_int, alpha_matrix_descr, _I, c_int],
    "alphasparse_operations_mv": [_I, _I, _I, _I, _I, c_int, alpha_matrix_descr, c_int],
    "alpha_get_core_num": [],
    "alpha_set_thread_num": [c_int],
    "alpha_get_thread_num": [],
    "init_handle": [POINTER(alphasparse_dcu_handle_t)],
    "alphasparse_dcu_get_handle": [POINTER(alphasparse_dcu_handle_t)],
    "alphasparse_dcu_destory_handle": [alphasparse_dcu_handle_t],
    "alphasparse_dcu_create_mat_descr": [POINTER(alpha_dcu_matrix_descr_t)],
    "alphasparse_dcu_destroy_mat_descr": [alpha_dcu_matrix_descr_t],
    "alphasparse_dcu_create_mat_info": [POINTER(alphasparse_dcu_mat_info_t)],
    "alphasparse_dcu_destroy_mat_info": [alphasparse_dcu_mat_info_t],
    "alphasparse_dcu_create_csrmv_info": [POINTER(POINTER(_alphasparse_dcu_csrmv_info)), c_bool],
    "alphasparse_dcu_destroy_csrmv_info": [POINTER(_alphasparse_dcu_csrmv_info)],
    "get_alphasparse_dcu_status_for_hip_status": [c_int],
    "alphasparse_dcu_csrmv_clear": [alphasparse_dcu_handle_t, _P],
    "alphasparse_dcu_spmv": [alphasparse_dcu_handle_t, c_int, _P, POINTER(alphasparse_dcu_spmat_descr),
                             POINTER(alphasparse_dcu_dnvec_descr), _P, POINTER(alphasparse_dcu_dnvec_descr), c_int, c_int,
                             POINTER(c_size_t), _P],
    "alphasparse_dcu_csr2coo": [alphasparse_dcu_handle_t, _P, _I, _I, _P, c_int],
    "alphasparse_dcu_csr2ell_width": [alphasparse_dcu_handle_t, _I, alpha_dcu_matrix_descr_t, _P,
                                      alpha_dcu_matrix_descr_t, POINTER(_I)],
    # thin kernel ABI
    "asamd_csr_plan_create": [_P, _I, _I, _I, _P, _P, _P, _I, _I, _I, POINTER(_P)],
    "asamd_csr_plan_create_dtype": [_P, _I, _I, _I, _P, _P, _P, _I, _I, _I, POINTER(_P)],
    "asamd_csr_plan_build_conj_transpose": [_P, _P, _P, _P, _P],
    "asamd_csr_plan_destroy": [_P],
    "asamd_csr_plan_stats": [_P],
    "asamd_csr_plan_set_algo": [_P, _I],
    "asamd_csr_plan_refresh_values": [_P, _P, _P, _P, _P],
    "asamd_csr_structure_hash": [_P, _I, _I, _P, _P, _P, POINTER(ctypes.c_uint64)],
    "asamd_csr_plan_workspace_bytes": [_P],
    "asamd_csr_plan_csrmv": [_P, _P, _I, _P, _P, _P, _P, _P, _P, _P, _P, c_size_t],
    "asamd_handle_reserve": [_P, c_size_t],
    "asamd_csr_plan_watched_workspace_bytes": [_P],
    "asamd_csr_plan_watch_begin": [_P, _P, _P, _P, _P, _P, _P, c_size_t],
    "asamd_csr_plan_csrmv_watched": [_P, _P, _P, _P, _P, _P, _P, _P, _P, _P, _P, c_size_t, _P],
    # stateless launchers and layout builders (records are passed as opaque pointers here)
    "asamd_spmv_vector": [_P, POINTER(asamd_spmv_args), _I],
    "asamd_spmv_vector_if": [_P, POINTER(asamd_spmv_args), _I, _P],
    "asamd_value_guard_any": [_P, _P, _P, _P],
    "asamd_spmv_scalar": [_P, POINTER(asamd_spmv_args)],
    "asamd_spmv_rowconst": [_P, POINTER(asamd_spmv_args), _I],
    "asamd_spmv_stream": [_P, POINTER(asamd_spmv_args), _I, _I, _I],
    "asamd_merge_partition": [_P, _I, _I, _P, _I, _I, _I, _P],
    "asamd_spmv_merge": [_P, POINTER(asamd_spmv_args), _I, _P, _P, _P, _P],
    "asamd_spmv_trans_scatter": [_P, POINTER(asamd_spmv_args), _I, _I],
    "asamd_spmv_trans_ylds_bytes": [_I, _I, _I],
    "asamd_spmv_trans_ylds": [_P, POINTER(asamd_spmv_args), _I, _I, _P],
    "asamd_tiled_fits": [_I, _I, _I, _I],
    "asamd_tiled_build": [_P, _I, _I, _I, _I, _I, _P, _P, _P, _I, _I, _P],
    "asamd_tiled_free": [_P],
    "asamd_tiled_gather_values": [_P, _P, _P, _P],
    "asamd_spmv_tiled": [_P, POINTER(asamd_spmv_args), _P, _P, _P, _P],
    "asamd_hot_build": [_P, _I, _I, _I, _I, _I, _P, _P, _I, _I, _I, _P],
    "asamd_hot_free": [_P],
    "asamd_spmv_hot": [_P, POINTER(asamd_spmv_args), _P, _P, _P, _P, _P],
    "asamd_binned_build": [_P, _I, _I, _P, _P],
    "asamd_binned_free": [_P],
    "asamd_spmv_binned": [_P, POINTER(asamd_spmv_args), _P, _P],
    "asamd_transpose_build": [_P, _I, _I, _I, _I, _I, _I, _P, _P, _P, _P],
    "asamd_transpose_free": [_P],
    "asamd_csr_row_stats": [_P, _I, _P, _P, _P],
    "asamd_csr_locality_probe": [_P, _I, _I, _I, _P, _I, _P, POINTER(c_float)],
    "asamd_value_guard_run": [c_size_t],
    "asamd_value_guard": [_P, _P, c_size_t, _I, _P, _P],
    "asamd_value_guard_commit": [_P, _P, _P],
    "asamd_gather_values": [_P, _I, _I, _I, _P, _P, _P, _P],
    "asamd_spmv_xlds": [_P, _P, _I],
    "asamd_spmv_xlds_fits": [_I, _I],
    "asamd_narrow_columns": [_P, _I, _I, _P, _P],
    "asamd_narrow_rel_columns": [_P, _I, _I, _I, _I, _P, _P, _P, _P],
    "asamd_spmv_stream_rel16": [_P, POINTER(asamd_spmv_args), _I, _I, _P],
    "asamd_spmv_xlds_narrow": [_P, POINTER(asamd_spmv_args), _I, _P],
    "asamd_xlds_slices": [_I, _I],
    "asamd_xlds_build": [_P, _I, _I, _I, _I, _I, _P, _P, _P, _P],
    "asamd_xlds_refresh_values": [_P, _P, _P, _P],
    "asamd_xlds_free": [_P],
    "asamd_spmv_xlds_sliced": [_P, POINTER(asamd_spmv_args), _I, _P, _P],
    "asamd_csr2ell_gated": [_P, _I, _I, _P, _P, _P, _I, _I, _I, _P, _P, _P],
    "asamd_csr_plan_build_transpose": [_P, _P, _P, _P, _P],
    "asamd_csr_plan_set_lazy_transpose": [_P, _I],
    "asamd_csr_plan_transpose_stats": [_P],
    "asamd_csr_plan_transpose_arrays": [_P, _I, POINTER(_P), POINTER(_P), POINTER(_P)],
    "asamd_csrmm_workspace_bytes": [_I, _I, _I, _I, POINTER(asamd_dense_strides)],
    "asamd_csr2coo_workspace_bytes": [_I],
    "asamd_csr2coo": [_P, _P, _I, _I, _P, _I],
    "asamd_csr2coo_ws": [_P, _P, _I, _I, _P, _I, _P, c_size_t],
    "asamd_csr2ell_width": [_P, _I, _P, POINTER(_I)],
    "asamd_warmup": [_P],
    "asamd_s_csrmv_noalloc": [_P, _I, _I, _I, _I, c_float, _P, _P, _P, _P, c_float, _P],
    "asamd_handle_set_stream": [_P, _P],
    "asamd_handle_get_stream": [_P],
    "asamd_registry_lazy_count": [],
    "asamd_registry_lazy_promoted": [_P, _P],
    "asamd_analysis_stats": [_P],
    "asamd_analysis_transpose_stats": [_P],
    "asamd_analysis_set_algo": [_P, _I],
}


def prototypes():
    """name -> argtypes for every symbol the public headers declare."""
    out = dict(_COMMON)
    for s, ct in (("s", c_float), ("d", c_double), ("c", ALPHA_Complex8), ("z", ALPHA_Complex16)):
        for k, v in _per_type(ct).items():
            out[k.format(s=s)] = v
        for k, v in (_per_real_type(ct) if s in "sd" else _per_complex_type(ct)).items():
            out[k.format(s=s)] = v
    return out


_RESTYPE = {"alpha_set_thread_num": None, "alpha_timing_wtime": c_double, "alpha_timing_start": None,
            "alpha_timing_end": None, "alpha_timing_elapsed_time": c_double, "alpha_timing_gflops": c_double,
            "alpha_timing_elaped_time_print": None, "alpha_timing_gflops_print": None, "alpha_clear_cache": None,
            "alphasparse_nnz_counter_coo": None, "alphasparse_operations_mm": c_int64, "alphasparse_operations_mv": c_int64, "asamd_csr_plan_destroy": None, "asamd_handle_get_stream": c_void_p, "alpha_malloc": c_void_p, "alpha_memalign": c_void_p, "alpha_free": None,
            "alpha_fill_random_s": None, "alpha_fill_random_d": None, "alpha_read_coo": None, "alpha_read_coo_d": None,
            "alpha_fill_random_c": None, "alpha_fill_random_z": None, "alpha_read_coo_c": None, "alpha_read_coo_z": None,
            "args_help": None, "args_get_if_check": c_bool, "args_get_data_file": ctypes.c_char_p,
            "args_get_data_fileA": ctypes.c_char_p, "args_get_data_fileB": ctypes.c_char_p,
            "alpha_args_get_matrix_descrA": alpha_matrix_descr, "alpha_args_get_matrix_descrB": alpha_matrix_descr,
            "get_time_us": c_double, "asamd_csrmm_workspace_bytes": c_size_t, "asamd_csr2coo_workspace_bytes": c_size_t, "asamd_csr_plan_workspace_bytes": c_size_t, "asamd_spmv_trans_ylds_bytes": c_size_t, "asamd_csr_plan_watched_workspace_bytes": c_size_t, "asamd_value_guard_run": c_size_t, "asamd_tiled_free": None, "asamd_xlds_free": None, "asamd_hot_free": None, "asamd_binned_free": None, "asamd_transpose_free": None, "asamd_csr_plan_stats": POINTER(asamd_csr_stats),
            "asamd_csr_plan_transpose_stats": POINTER(asamd_csr_stats),
            "asamd_analysis_transpose_stats": POINTER(asamd_csr_stats),
            "asamd_analysis_stats": POINTER(asamd_csr_stats)}

ALGO_NAMES = {ASAMD_SPMV_AUTO: "auto", ASAMD_SPMV_VECTOR: "vector", ASAMD_SPMV_ROWCONST: "rowconst",
              ASAMD_SPMV_MERGE: "merge-path", ASAMD_SPMV_SCALAR: "scalar", ASAMD_SPMV_TILED: "tiled two-phase",
              ASAMD_SPMV_STREAM: "row-block stream", ASAMD_SPMV_ELL: "ell copy",
              ASAMD_SPMV_MERGE_HOT: "merge-path, hot columns in LDS", ASAMD_SPMV_BINNED: "row-length bins",
              ASAMD_SPMV_XLDS: "x in LDS"}

_lib = None


def load():
    """Load libalpha_spblas.so and attach prototypes.  Raises if it is not built."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(
                "%s is missing: build it first (python -c 'import __graft_entry__ as g; g.build()' "
                "or make -C alsparse_amd/csrc). There is no CPU fallback." % LIB_PATH)
        lib = ctypes.CDLL(LIB_PATH, mode=ctypes.RTLD_GLOBAL)
        for name, args in prototypes().items():
            fn = getattr(lib, name)  # AttributeError if a declared symbol is not exported
            fn.argtypes = args
            fn.restype = _RESTYPE.get(name, c_int)
        _lib = lib
    return _lib


_probes = None


def load_probes():
    """The benchmark's plain memory kernels (libasamd_probes.so): stream / gather ceilings and the copy that
    calibrates the byte counters.  Not part of the product library."""
    global _probes
    if _probes is None:
        if not os.path.exists(PROBES_PATH):
            raise RuntimeError("%s is missing: build it first (python -c 'import __graft_entry__ as g; g.build()')"
                               % PROBES_PATH)
        lib = ctypes.CDLL(PROBES_PATH)
        lib.asamd_copy_bytes.argtypes = [_P, _P, _P, c_size_t]
        lib.asamd_copy_bytes.restype = c_int
        lib.asamd_ceiling_kernel.argtypes = [_P, _I, _P, _P, c_size_t, c_int64, _P, POINTER(c_int64)]
        lib.asamd_ceiling_kernel.restype = c_int
        _probes = lib
    return _probes


# ---- small conveniences used by tests and the benchmark -----------------------
def ptr(x):
    """Device pointer / numpy array / None -> c_void_p."""
    if x is None:
        return c_void_p(None)
    if hasattr(x, "ptr"):
        return c_void_p(x.ptr)
    if hasattr(x, "ctypes"):
        return x.ctypes.data_as(c_void_p)
    return c_void_p(x)


def scalar_type(dtype):
    import numpy as np
    return {np.dtype(np.float32): c_float, np.dtype(np.float64): c_double, np.dtype(np.complex64): ALPHA_Complex8,
            np.dtype(np.complex128): ALPHA_Complex16}[np.dtype(dtype)]


def prefix(dtype):
    import numpy as np
    return {np.dtype(np.float32): "s", np.dtype(np.float64): "d", np.dtype(np.complex64): "c",
            np.dtype(np.complex128): "z"}[np.dtype(dtype)]


def dtype_tag(dtype):
    """enum asamd_dtype / alphasparse_datatype_t of a numpy dtype."""
    return "sdcz".index(prefix(dtype))


class Handle:
    """alphasparse_dcu_get_handle / alphasparse_dcu_destory_handle."""

    def __init__(self):
        self.lib = load()
        self.h = alphasparse_dcu_handle_t(None)
        st = self.lib.alphasparse_dcu_get_handle(byref(self.h))
        if st != ALPHA_SPARSE_STATUS_SUCCESS:
            raise RuntimeError("alphasparse_dcu_get_handle -> %d" % st)

    def close(self):
        if self.h:
            self.lib.alphasparse_dcu_destory_handle(self.h)
            self.h = alphasparse_dcu_handle_t(None)


def make_descr(base=ALPHA_SPARSE_INDEX_BASE_ZERO, mtype=ALPHA_SPARSE_MATRIX_TYPE_GENERAL):
    d = alpha_dcu_matrix_descr(mtype, 0, 0, base)
    return d


class Workspace:
    """Per-call device scratch for asamd_csr_plan_csrmv, sized for a plan."""

    def __init__(self, lib, plan, extra=0):
        from . import hiprt
        self.bytes = int(lib.asamd_csr_plan_workspace_bytes(plan)) + extra
        self.buf = hiprt.DeviceArray(max(self.bytes, 256), "uint8")

    def c_ptr(self):
        return self.buf.c_ptr()


def plan_csrmv(lib, stream, plan, op, alpha, val, row_ptr, col_ind, x, beta, y, ws=None):
    """asamd_csr_plan_csrmv with ctypes scalars of the plan's element type (alpha, beta) and a Workspace (or none)."""
    return lib.asamd_csr_plan_csrmv(stream, plan, op, ctypes.cast(byref(alpha), c_void_p), val, row_ptr, col_ind, x,
                                    ctypes.cast(byref(beta), c_void_p), y, ws.c_ptr() if ws else None,
                                    ws.bytes if ws else 0)
