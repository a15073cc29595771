// The structure-only layouts (hot columns, row-length bins), the CSR copy of the transpose, and the
// launchers of the kernels that multiply with them (gfx950, wave64).  The reference has no counterpart
// for the first two; its transposed product always scatters
// (src/kernel/dcu/level2/mv/csrmv/dcu_gemv_x_csr_trans.cpp:11-68).

#include <hip/hip_runtime.h>

#include <vector>

#include "alsparse_amd_kernels.h"
#include "launch_utils.hpp"
#include "spmv_binned.hpp"
#include "spmv_hot.hpp"
#include "spmv_tiled.hpp"  // tile_bounds_kernel
#include "spmv_trans.hpp"
#include "spmv_xlds.hpp"
#include "tile_sort.hpp"

using namespace asamd;

// ---- hot columns ---------------------------------------------------------------------------------
// The kernel pays when x is far larger than an XCD's L2 and yet most entries fall into a few columns
// (power-law graphs).  Whether they do is only known after counting.
constexpr int kHotFrontBytes = 1 << 20;  // of every XCD's 4 MiB L2, beside the streams passing through
template <typename T>
struct HotKernel {
  // 4-byte values: 8 items per lane and 16 waves; 8-byte values: 4 items per lane (the staging areas of
  // 16 waves must leave room for the table)
  static constexpr int ipt = sizeof(T) == 4 ? 8 : 4;
  static constexpr int nw = 16;
  using Dims = HotDims<T, ipt, nw>;
};

// Counts the entries of every column, ranks the columns, rewrites the column stream as positions (LDS
// slot or column) and caches the merge coordinates of the wave-sized blocks.  Leaves the record empty (and
// no error) when the popular columns hold too few entries.
template <typename T>
static hipError_t build_hot(hipStream_t stream, asamd_hot_layout* L, int m, int n, int nnz_i, int base,
                            const int* row_ptr, const int* col_ind, bool force, int want_lds, int want_front) {
  using HK = HotKernel<T>;
  const size_t nnz = (size_t)nnz_i;
  int h1 = HK::Dims::lds_cols;
  if (want_lds > 0 && want_lds < h1) h1 = want_lds;
  if (h1 > n) h1 = n;
  // the compact front: the columns that share an XCD's L2 with the streams passing through
  int hc = (int)(((int64_t)kHotFrontBytes) / (int64_t)sizeof(T));
  if (want_front > 0) hc = want_front;
  if (hc > n) hc = n;
  if (hc < h1) hc = h1;
  const int64_t nb = ((int64_t)m + nnz_i + HK::Dims::items - 1) / HK::Dims::items;
  unsigned *d_cnt = nullptr, *d_key = nullptr, *d_key2 = nullptr, *d_idx = nullptr, *d_sorted = nullptr, *d_rank = nullptr;
  hipError_t e = hipMalloc(&d_cnt, (size_t)n * sizeof(unsigned));
  if (e == hipSuccess) e = hipMalloc(&d_key, (size_t)(n > 2 ? n : 2) * sizeof(unsigned));  // (also takes a 64-bit sum)
  if (e == hipSuccess) e = hipMalloc(&d_key2, (size_t)n * sizeof(unsigned));
  if (e == hipSuccess) e = hipMalloc(&d_idx, (size_t)n * sizeof(unsigned));
  if (e == hipSuccess) e = hipMalloc(&d_sorted, (size_t)n * sizeof(unsigned));
  if (e == hipSuccess) e = hipMemsetAsync(d_cnt, 0, (size_t)n * sizeof(unsigned), stream);
  // large matrices are counted through one chunk of entries in four (the ranking of the popular columns and the
  // share below are then estimates, good to a per cent or so)
  const int sample_shift = nnz_i >= (1 << 24) ? 2 : 0;
  if (e == hipSuccess) {
    col_count_kernel<<<256 * 32, 256, 0, stream>>>(nnz_i, col_ind, base, sample_shift, d_cnt);
    col_rank_keys_kernel<<<(unsigned)(((int64_t)n + 255) / 256), 256, 0, stream>>>(n, d_cnt, d_key, d_idx);
    e = hipGetLastError();
  }
  if (e == hipSuccess) e = sort_pairs_u32(stream, d_key, d_key2, d_idx, d_sorted, (size_t)n, 32);
  unsigned long long h_head = 0;
  if (e == hipSuccess) {
    // (d_key, the sort's input, is free again: its first words take the sum)
    col_rank_head_sum_kernel<<<1, 256, 0, stream>>>(h1, d_key2, (unsigned long long*)d_key);
    e = hipMemcpyAsync(&h_head, d_key, sizeof(h_head), hipMemcpyDeviceToHost, stream);
  }
  if (e == hipSuccess) e = hipStreamSynchronize(stream);
  if (e == hipSuccess) {
    const double in_lds = (double)h_head * (double)(1 << sample_shift);
    L->cols_lds = h1;
    L->cols_front = hc;
    L->share_lds = (float)(in_lds / (double)nnz);
    // worth laying out only if the LDS serves a good part of the gathers
    if (!force && L->share_lds < 0.3f) e = hipErrorNotSupported;
  }
  if (e == hipSuccess) e = hipMalloc(&d_rank, (size_t)n * sizeof(unsigned));
  if (e == hipSuccess) e = hipMalloc(&L->pcol, nnz * sizeof(unsigned));
  if (e == hipSuccess) e = hipMalloc(&L->hot_cols, (size_t)hc * sizeof(int));
  if (e == hipSuccess) e = hipMalloc(&L->block_row, ((size_t)nb + 1) * sizeof(int));
  if (e == hipSuccess) e = hipMemsetAsync(d_rank, 0xFF, (size_t)n * sizeof(unsigned), stream);
  if (e == hipSuccess) {
    col_rank_scatter_kernel<<<(unsigned)((hc + 255) / 256), 256, 0, stream>>>(hc, d_sorted, d_rank, L->hot_cols);
    hot_pcol_kernel<<<256 * 32, 256, 0, stream>>>(nnz_i, col_ind, base, hc, d_rank, L->pcol);
    merge_partition_kernel<<<(unsigned)((nb + 1 + 255) / 256), 256, 0, stream>>>(m, nnz_i, row_ptr, base, (int)nb,
                                                                                HK::Dims::items, L->block_row);
    e = hipGetLastError();
  }
  if (e == hipSuccess)
    e = hipFuncSetAttribute((const void*)spmv_merge_hot_kernel<T, HK::ipt, HK::nw>,
                            hipFuncAttributeMaxDynamicSharedMemorySize, HK::Dims::table_bytes + HK::Dims::stage_bytes);
  if (e == hipSuccess) e = hipStreamSynchronize(stream);
  free_all({d_cnt, d_key, d_key2, d_idx, d_sorted, d_rank});
  if (e != hipSuccess) {
    const int h1_kept = L->cols_lds, hc_kept = L->cols_front;
    const float share = L->share_lds;
    asamd_hot_free(L);
    if (e != hipErrorNotSupported) return e;
    // what the count found stays readable in the empty record
    L->cols_lds = h1_kept;
    L->cols_front = hc_kept;
    L->share_lds = share;
    return hipSuccess;
  }
  L->dtype = DtypeOf<T>::value;
  L->blocks = (int)nb;
  L->device_bytes = (int64_t)nnz * 4 + (int64_t)hc * 4 + (nb + 1) * 4;
  return hipSuccess;
}

extern "C" int asamd_hot_build(hipStream_t stream, int32_t dtype, int32_t m, int32_t n, int32_t nnz, int32_t base,
                               const int32_t* row_ptr, const int32_t* col_ind, int32_t force, int32_t cols_lds,
                               int32_t cols_front, asamd_hot_layout* out) {
  if (!out) return hipErrorInvalidValue;
  *out = asamd_hot_layout{};
  if (!row_ptr || !col_ind || m < 1 || n < 1 || nnz < 1) return hipErrorInvalidValue;
  // positions are 32-bit words, x is addressed through a buffer resource with 32-bit byte offsets
  if (((int64_t)n + (int64_t)kHotFrontBytes) >= (int64_t)UINT32_MAX) return hipErrorInvalidValue;
  if ((int64_t)m + nnz >= (int64_t)INT32_MAX / 2) return hipErrorInvalidValue;
  if (dtype == ASAMD_DTYPE_FLOAT)
    return build_hot<float>(stream, out, m, n, nnz, base, row_ptr, col_ind, force != 0, cols_lds, cols_front);
  if (dtype == ASAMD_DTYPE_DOUBLE)
    return build_hot<double>(stream, out, m, n, nnz, base, row_ptr, col_ind, force != 0, cols_lds, cols_front);
  if (dtype == ASAMD_DTYPE_FLOAT_COMPLEX)
    return build_hot<Cx<float>>(stream, out, m, n, nnz, base, row_ptr, col_ind, force != 0, cols_lds, cols_front);
  return hipErrorInvalidValue;  // 16-byte values: the staging areas leave no room for the table
}

extern "C" void asamd_hot_free(asamd_hot_layout* L) {
  if (!L) return;
  free_all({(void*)L->pcol, (void*)L->hot_cols, (void*)L->block_row});
  *L = asamd_hot_layout{};
}

template <typename T>
static int spmv_hot_impl(hipStream_t s, const asamd_spmv_args* a, const asamd_hot_layout* L, void* front,
                         int32_t* carry_row, void* carry_val, void* head_val) {
  using HK = HotKernel<T>;
  if (!a->alpha || !a->beta || !a->val || !a->row_ptr || !a->x || !a->y) return hipErrorInvalidValue;
  if (((uintptr_t)a->val | (uintptr_t)a->x | (uintptr_t)a->y | (uintptr_t)front | (uintptr_t)carry_val |
       (uintptr_t)head_val) % alignof(T))
    return hipErrorInvalidValue;
  const T alpha = scalar_of<T>(a->alpha), beta = scalar_of<T>(a->beta);
  const int nb = L->blocks, h1 = L->cols_lds, hc = L->cols_front;
  // x of the hot columns, then persistent workgroups, one per compute unit
  hot_prepare_kernel<T><<<(unsigned)((hc + 255) / 256), 256, 0, s>>>(hc, L->hot_cols, (const T*)a->x, (T*)front);
  static const int cus = device_cus();
  const int per_wg = (nb + HK::nw - 1) / HK::nw;
  const int grid = per_wg < cus ? per_wg : cus;
  spmv_merge_hot_kernel<T, HK::ipt, HK::nw>
      <<<grid, HK::Dims::threads, HK::Dims::table_bytes + HK::Dims::stage_bytes, s>>>(
          a->m, a->nnz, alpha, (const T*)a->val, a->row_ptr, L->pcol, (const T*)a->x, (const T*)front, h1, hc, beta,
          (T*)a->y, a->base, L->block_row, carry_row, (T*)carry_val, (T*)head_val, nb);
  if (nb > 1)
    merge_fixup_kernel<T><<<(nb + 255) / 256, 256, 0, s>>>(nb, a->m, alpha, beta, carry_row, (const T*)carry_val,
                                                           (const T*)head_val, (T*)a->y);
  return hipGetLastError();
}

extern "C" int asamd_spmv_hot(hipStream_t s, const asamd_spmv_args* a, const asamd_hot_layout* L, void* front,
                              int32_t* carry_row, void* carry_val, void* head_val) {
  if (!a || !L || !L->pcol || !front || !carry_row || !carry_val || !head_val || a->dtype != L->dtype)
    return hipErrorInvalidValue;
  if (a->dtype == ASAMD_DTYPE_FLOAT) return spmv_hot_impl<float>(s, a, L, front, carry_row, carry_val, head_val);
  if (a->dtype == ASAMD_DTYPE_DOUBLE) return spmv_hot_impl<double>(s, a, L, front, carry_row, carry_val, head_val);
  if (a->dtype == ASAMD_DTYPE_FLOAT_COMPLEX)
    return spmv_hot_impl<Cx<float>>(s, a, L, front, carry_row, carry_val, head_val);
  return hipErrorInvalidValue;
}

// ---- column slices for the kernel that holds x in LDS ----------------------------------------------
template <typename T>
static hipError_t xlds_copy_pieces(hipStream_t stream, const asamd_xlds_layout* L, const void* val, const int32_t* col_ind,
                                   const int32_t* gate) {
  const int64_t pieces = (int64_t)L->slices * L->m;
  // (a refresh behind the value guard is launched with every multiply and mostly returns at once: few workgroups)
  int64_t grid = (pieces + 31) / 32;
  if (grid > 4096) grid = 4096;
  xlds_copy_pieces_kernel<T><<<(unsigned)grid, 256, 0, stream>>>(pieces, L->m, L->slice_cols, L->base, L->seg, L->off,
                                                                (const T*)val, col_ind, (T*)L->val, L->col, gate);
  return hipGetLastError();
}
static hipError_t xlds_copy_pieces_dtype(hipStream_t stream, const asamd_xlds_layout* L, const void* val,
                                         const int32_t* col_ind, const int32_t* gate) {
  if (L->dtype == ASAMD_DTYPE_FLOAT) return xlds_copy_pieces<float>(stream, L, val, col_ind, gate);
  if (L->dtype == ASAMD_DTYPE_DOUBLE) return xlds_copy_pieces<double>(stream, L, val, col_ind, gate);
  return hipErrorInvalidValue;
}

// As few slices as hold x in ASAMD_XLDS_MAX_BYTES each -- or up to a quarter more if that count divides the 256
// compute units evenly: every slice then gets the same number of workgroups (7 slices of 36 workgroups leave four
// compute units idle and measured 0.217 ms on 262 144 x 262 144 x 400 where 8 slices of 32 take 0.200).
extern "C" int32_t asamd_xlds_slices(int32_t dtype, int32_t n) {
  const int vs = dtype_size(dtype);
  if (vs <= 0 || n < 1) return 0;
  const int64_t fill = (int64_t)ASAMD_XLDS_MAX_BYTES / vs;  // columns per LDS fill
  const int64_t need = ((int64_t)n + fill - 1) / fill;
  for (int64_t s = need; s * 4 <= need * 5 && s <= 256; ++s)
    if (256 % s == 0) return (int32_t)s;
  return need > INT32_MAX ? INT32_MAX : (int32_t)need;
}

// Slices of equal width (a multiple of 64 columns).
extern "C" int asamd_xlds_build(hipStream_t stream, int32_t dtype, int32_t m, int32_t n, int32_t nnz, int32_t base,
                                const int32_t* row_ptr, const int32_t* col_ind, const void* val, asamd_xlds_layout* L) {
  if (!L) return hipErrorInvalidValue;
  *L = asamd_xlds_layout{};
  const int vs = dtype_size(dtype);
  if (!row_ptr || !col_ind || m < 1 || n < 1 || nnz < 1 || vs <= 0) return hipErrorInvalidValue;
  if (val && dtype != ASAMD_DTYPE_FLOAT && dtype != ASAMD_DTYPE_DOUBLE) return hipErrorInvalidValue;
  const int64_t fill = (int64_t)ASAMD_XLDS_MAX_BYTES / vs;  // columns per LDS fill
  const int64_t slices = asamd_xlds_slices(dtype, n);
  if (slices < 2 || slices > 1024 || (slices + 1) * (int64_t)m >= (int64_t)INT32_MAX) return hipSuccess;  // no layout
  int64_t width = ((int64_t)n + slices - 1) / slices;
  width = (width + 63) / 64 * 64;
  if (width > fill) width = fill;
  int* d_flag = nullptr;
  int h_flag = 0;
  hipError_t e = hipMalloc(&d_flag, sizeof(int));
  if (e == hipSuccess) e = hipMemsetAsync(d_flag, 0, sizeof(int), stream);
  if (e == hipSuccess) {
    xlds_rows_ascend_kernel<<<(unsigned)(((int64_t)m + 3) / 4), 256, 0, stream>>>(m, row_ptr, col_ind, base, d_flag);
    e = hipMemcpyAsync(&h_flag, d_flag, sizeof(int), hipMemcpyDeviceToHost, stream);
  }
  if (e == hipSuccess) e = hipStreamSynchronize(stream);
  if (e == hipSuccess && h_flag == 0) {
    const int64_t count = (slices + 1) * (int64_t)m;
    e = hipMalloc(&L->seg, (size_t)count * sizeof(int));
    if (e == hipSuccess) {
      // rows long enough to keep a wave's lanes busy are walked once; short rows are searched, a lane per row and slice
      if ((int64_t)nnz >= 16 * (int64_t)m)
        xlds_slice_offsets_walk_kernel<<<(unsigned)(((int64_t)m + 3) / 4), 256, 0, stream>>>(m, (int)slices, (int)width,
                                                                                            row_ptr, col_ind, base, L->seg);
      else
        xlds_slice_offsets_kernel<<<(unsigned)((count + 255) / 256), 256, 0, stream>>>(m, (int)slices, (int)width,
                                                                                      row_ptr, col_ind, base, L->seg);
      e = hipGetLastError();
    }
    if (e == hipSuccess) e = hipStreamSynchronize(stream);
    if (e == hipSuccess) {
      L->slices = (int32_t)slices;
      L->slice_cols = (int32_t)width;
      L->m = m;
      L->dtype = dtype;
      L->nnz = nnz;
      L->base = base;
      L->device_bytes = count * (int64_t)sizeof(int);
    }
    if (e == hipSuccess && val) {
      // the copy: offsets (a running sum of the pieces' lengths, slice by slice), then the entries; four entries
      // of padding so that a 16-byte load of the last piece stays inside
      const int64_t pieces = slices * (int64_t)m;
      const size_t off_bytes = ((size_t)pieces + 1) * sizeof(int), val_bytes = ((size_t)nnz + 4) * (size_t)vs,
                   col_bytes = ((size_t)nnz + 4) * sizeof(uint16_t);
      hipError_t c = hipMalloc(&L->off, off_bytes);
      if (c == hipSuccess) c = hipMalloc(&L->val, val_bytes);
      if (c == hipSuccess) c = hipMalloc(&L->col, col_bytes);
      if (c == hipSuccess) c = hipMemsetAsync((char*)L->val + (size_t)nnz * vs, 0, 4 * (size_t)vs, stream);
      if (c == hipSuccess) c = hipMemsetAsync(L->col + nnz, 0, 4 * sizeof(uint16_t), stream);
      if (c == hipSuccess) c = scan_piece_lengths(stream, L->seg, m, pieces, L->off);
      if (c == hipSuccess) c = xlds_copy_pieces_dtype(stream, L, val, col_ind, nullptr);
      if (c == hipSuccess) c = hipStreamSynchronize(stream);
      if (c == hipSuccess) {
        L->device_bytes += (int64_t)(off_bytes + val_bytes + col_bytes);
      } else {
        // (no room for the copy, say: the table of offsets alone still serves)
        if (c == hipErrorOutOfMemory) (void)hipGetLastError();
        if (L->off) (void)hipFree(L->off);
        if (L->val) (void)hipFree(L->val);
        if (L->col) (void)hipFree(L->col);
        L->off = nullptr, L->val = nullptr, L->col = nullptr;
        if (c != hipErrorOutOfMemory) e = c;
      }
    }
  }
  if (d_flag) (void)hipFree(d_flag);
  if (e != hipSuccess) asamd_xlds_free(L);
  return e;
}

extern "C" int asamd_xlds_refresh_values(hipStream_t stream, const asamd_xlds_layout* L, const void* val,
                                         const int32_t* gate) {
  if (!L || !L->seg || !L->off || !L->val || !val) return hipErrorInvalidValue;
  return xlds_copy_pieces_dtype(stream, L, val, nullptr, gate);
}

extern "C" void asamd_xlds_free(asamd_xlds_layout* L) {
  if (!L) return;
  if (L->seg) (void)hipFree(L->seg);
  if (L->off) (void)hipFree(L->off);
  if (L->val) (void)hipFree(L->val);
  if (L->col) (void)hipFree(L->col);
  *L = asamd_xlds_layout{};
}

// ---- row-length bins -----------------------------------------------------------------------------
// Row numbers sorted by length class and the chunk table of the longest rows.
extern "C" int asamd_binned_build(hipStream_t stream, int32_t m, int32_t base, const int32_t* row_ptr,
                                  asamd_binned_layout* L) {
  if (!L) return hipErrorInvalidValue;
  *L = asamd_binned_layout{};
  if (!row_ptr || m < 1) return hipErrorInvalidValue;
  unsigned *d_key = nullptr, *d_key2 = nullptr, *d_idx = nullptr;
  int *d_count = nullptr, *d_bounds = nullptr;
  int h_count[kBinClasses] = {0, 0, 0, 0};
  hipError_t e = hipMalloc(&d_key, (size_t)m * sizeof(unsigned));
  if (e == hipSuccess) e = hipMalloc(&d_key2, (size_t)m * sizeof(unsigned));
  if (e == hipSuccess) e = hipMalloc(&d_idx, (size_t)m * sizeof(unsigned));
  if (e == hipSuccess) e = hipMalloc(&L->rows, (size_t)m * sizeof(int));
  if (e == hipSuccess) e = hipMalloc(&d_count, sizeof(h_count));
  if (e == hipSuccess) e = hipMemsetAsync(d_count, 0, sizeof(h_count), stream);
  if (e == hipSuccess) {
    bin_keys_kernel<<<(unsigned)(((int64_t)m + 255) / 256), 256, 0, stream>>>(m, row_ptr, d_key, d_idx, d_count);
    e = hipGetLastError();
  }
  if (e == hipSuccess) e = sort_pairs_u32(stream, d_key, d_key2, d_idx, (unsigned*)L->rows, (size_t)m, 2);
  if (e == hipSuccess) e = hipMemcpyAsync(h_count, d_count, sizeof(h_count), hipMemcpyDeviceToHost, stream);
  if (e == hipSuccess) e = hipStreamSynchronize(stream);
  const int nlong = h_count[kBinClasses - 1];
  std::vector<int> bounds, first;
  std::vector<BinChunk> chunks;
  if (e == hipSuccess && nlong > 0) {
    // the long rows' offsets come to the host, which cuts them into chunks
    bounds.resize((size_t)nlong * 2);
    e = hipMalloc(&d_bounds, bounds.size() * sizeof(int));
    if (e == hipSuccess) {
      bin_row_bounds_kernel<<<(unsigned)((nlong + 255) / 256), 256, 0, stream>>>(nlong, L->rows + (m - nlong), row_ptr,
                                                                               d_bounds);
      e = hipGetLastError();
    }
    if (e == hipSuccess) e = hipMemcpy(bounds.data(), d_bounds, bounds.size() * sizeof(int), hipMemcpyDeviceToHost);
    if (e == hipSuccess) {
      std::vector<int> rows((size_t)nlong);
      e = hipMemcpy(rows.data(), L->rows + (m - nlong), rows.size() * sizeof(int), hipMemcpyDeviceToHost);
      first.resize((size_t)nlong + 1);
      for (int i = 0; i < nlong && e == hipSuccess; ++i) {
        first[(size_t)i] = (int)chunks.size();
        const int64_t b = (int64_t)bounds[2 * (size_t)i] - base, en = (int64_t)bounds[2 * (size_t)i + 1] - base;
        for (int64_t c = b; c < en; c += kBinChunk)
          chunks.push_back(BinChunk{rows[(size_t)i], (int)c, (int)(c + kBinChunk < en ? c + kBinChunk : en)});
      }
      first[(size_t)nlong] = (int)chunks.size();
    }
    if (e == hipSuccess) e = hipMalloc(&L->chunk_list, chunks.size() * sizeof(BinChunk));
    if (e == hipSuccess) e = hipMalloc(&L->chunk_first, first.size() * sizeof(int));
    if (e == hipSuccess) e = hipMemcpy(L->chunk_list, chunks.data(), chunks.size() * sizeof(BinChunk), hipMemcpyHostToDevice);
    if (e == hipSuccess) e = hipMemcpy(L->chunk_first, first.data(), first.size() * sizeof(int), hipMemcpyHostToDevice);
  }
  free_all({d_key, d_key2, d_idx, d_count, d_bounds});
  if (e != hipSuccess) {
    asamd_binned_free(L);
    return e;
  }
  for (int c = 0; c < kBinClasses; ++c) L->count[c] = h_count[c];
  L->chunks = (int)chunks.size();
  L->device_bytes = (int64_t)m * 4 + (int64_t)chunks.size() * (int64_t)sizeof(BinChunk) + (int64_t)first.size() * 4;
  return hipSuccess;
}

extern "C" void asamd_binned_free(asamd_binned_layout* L) {
  if (!L) return;
  free_all({(void*)L->rows, L->chunk_list, (void*)L->chunk_first});
  *L = asamd_binned_layout{};
}

extern "C" int asamd_spmv_binned(hipStream_t s, const asamd_spmv_args* a, const asamd_binned_layout* L,
                                 void* partial) {
  if (!a || !L || !L->rows) return hipErrorInvalidValue;
  if (L->count[3] > 0 && !partial) return hipErrorInvalidValue;
  return by_dtype(a->dtype, [&](auto* tag) -> int {
    using T = std::remove_pointer_t<decltype(tag)>;
    if (!args_ok<T>(a) || (uintptr_t)partial % alignof(T)) return hipErrorInvalidValue;
    const T alpha = scalar_of<T>(a->alpha), beta = scalar_of<T>(a->beta);
    const T* val = (const T*)a->val;
    const T* x = (const T*)a->x;
    T* y = (T*)a->y;
    const int *rp = a->row_ptr, *ci = a->col_ind;
    // one launch per row-length class; the classes own disjoint rows, so the launches are independent
    const int* rows = L->rows;
    const int n0 = L->count[0], n1 = L->count[1], n2 = L->count[2], n3 = L->count[3];
    auto blocks = [](int count, int w) { return (unsigned)(((int64_t)count * w + kRowsBlock - 1) / kRowsBlock); };
    if (n0 > 0)
      spmv_bin_rows_kernel<T, 4><<<blocks(n0, 4), kRowsBlock, 0, s>>>(n0, rows, alpha, val, rp, ci, x, beta, y, a->base);
    if (n1 > 0)
      spmv_bin_rows_kernel<T, 16><<<blocks(n1, 16), kRowsBlock, 0, s>>>(n1, rows + n0, alpha, val, rp, ci, x, beta, y,
                                                                      a->base);
    if (n2 > 0)
      spmv_bin_rows_kernel<T, 64><<<blocks(n2, 64), kRowsBlock, 0, s>>>(n2, rows + n0 + n1, alpha, val, rp, ci, x, beta,
                                                                      y, a->base);
    if (n3 > 0) {
      spmv_bin_chunk_kernel<T><<<(unsigned)L->chunks, kRowsBlock, 0, s>>>(L->chunks, (const BinChunk*)L->chunk_list, val,
                                                                         ci, x, a->base, (T*)partial);
      spmv_bin_finish_kernel<T><<<(unsigned)((n3 + 255) / 256), 256, 0, s>>>(n3, rows + n0 + n1 + n2, L->chunk_first,
                                                                            (const T*)partial, alpha, beta, y);
    }
    return hipGetLastError();
  });
}

// ---- CSR of A^T ------------------------------------------------------------------------------------
// Sort (column, entry) pairs by column (stable: rows ascending inside a column), read the column offsets
// off the sorted keys, gather rows and values.
template <typename T>
static hipError_t build_transpose(hipStream_t stream, asamd_transpose_layout* t, bool conj, int m, int n, int nnz,
                                  int base, const int* row_ptr, const int* col_ind, const T* val) {
  int* d_coo = nullptr;
  unsigned *d_key = nullptr, *d_key2 = nullptr, *d_idx = nullptr;
  hipError_t e = hipMalloc(&d_coo, (size_t)nnz * sizeof(int));
  if (e == hipSuccess) e = hipMalloc(&d_key, (size_t)nnz * sizeof(unsigned));
  if (e == hipSuccess) e = hipMalloc(&d_key2, (size_t)nnz * sizeof(unsigned));
  if (e == hipSuccess) e = hipMalloc(&d_idx, (size_t)nnz * sizeof(unsigned));
  if (e == hipSuccess) e = hipMalloc(&t->perm, (size_t)nnz * sizeof(unsigned));
  if (e == hipSuccess) e = hipMalloc(&t->row_ptr, ((size_t)n + 1) * sizeof(int));
  if (e == hipSuccess) e = hipMalloc(&t->col_ind, (size_t)nnz * sizeof(int));
  if (e == hipSuccess) e = hipMalloc(&t->val, (size_t)nnz * sizeof(T));
  if (e == hipSuccess)  // d_key2 is free until the sort
    e = (hipError_t)asamd_csr2coo_ws(stream, row_ptr, nnz, m, d_coo, base, d_key2, (size_t)nnz * sizeof(unsigned));
  if (e == hipSuccess) {
    int64_t grid = ((int64_t)nnz + 255) / 256;
    if (grid > 256 * 32) grid = 256 * 32;
    transpose_keys_kernel<<<(unsigned)grid, 256, 0, stream>>>(nnz, col_ind, base, d_key, d_idx);
    e = hipGetLastError();
    unsigned bits = 1;
    while (bits < 32 && ((int64_t)1 << bits) < (int64_t)n) ++bits;
    if (e == hipSuccess) e = sort_pairs_u32(stream, d_key, d_key2, d_idx, t->perm, (size_t)nnz, bits);
    if (e == hipSuccess) {
      tile_bounds_kernel<<<(unsigned)(((int64_t)n + 1 + 255) / 256), 256, 0, stream>>>(nnz, d_key2, (int64_t)n,
                                                                                      t->row_ptr);
      if (conj)
        transpose_gather_kernel<T, true><<<grid, 256, 0, stream>>>(nnz, t->perm, d_coo, val, base, t->col_ind,
                                                                   (T*)t->val);
      else
        transpose_gather_kernel<T, false><<<grid, 256, 0, stream>>>(nnz, t->perm, d_coo, val, base, t->col_ind,
                                                                    (T*)t->val);
      e = hipGetLastError();
    }
    if (e == hipSuccess) e = hipStreamSynchronize(stream);
  }
  free_all({d_coo, d_key, d_key2, d_idx});
  if (e != hipSuccess) {
    asamd_transpose_free(t);
    return e;
  }
  t->device_bytes = (int64_t)nnz * (8 + (int64_t)sizeof(T)) + ((int64_t)n + 1) * 4;
  return hipSuccess;
}

extern "C" int asamd_transpose_build(hipStream_t stream, int32_t dtype, int32_t conj, int32_t m, int32_t n,
                                     int32_t nnz, int32_t base, const int32_t* row_ptr, const int32_t* col_ind,
                                     const void* val, asamd_transpose_layout* out) {
  if (!out) return hipErrorInvalidValue;
  *out = asamd_transpose_layout{};
  if (!row_ptr || !col_ind || !val || m < 1 || n < 1 || nnz < 1) return hipErrorInvalidValue;
  return by_dtype(dtype, [&](auto* tag) -> int {
    using T = std::remove_pointer_t<decltype(tag)>;
    if ((uintptr_t)val % alignof(T) || (conj && kIsReal<T>)) return hipErrorInvalidValue;
    return build_transpose<T>(stream, out, conj != 0, m, n, nnz, base, row_ptr, col_ind, (const T*)val);
  });
}

extern "C" void asamd_transpose_free(asamd_transpose_layout* t) {
  if (!t) return;
  free_all({(void*)t->row_ptr, (void*)t->col_ind, t->val, (void*)t->perm});
  *t = asamd_transpose_layout{};
}
