// CSR SpMM  C = alpha*A*B + beta*C  for gfx950 (wave64).
//
//   spmm_rowmajor_kernel<T, V>  unit stride along the dense columns (row-major
//       B and C, or column-major with op(B) = B^T read as row-major): one wave
//       per row of A and per chunk of 64*V dense columns; the row's
//       (col, alpha*val) pairs are read coalesced 64 at a time and broadcast
//       with v_readlane, so every B row is fetched with one wave-wide load of
//       64*V contiguous elements; C is read-modified-written once.
//       This is the layout the reference cannot run on the GPU at all
//       (dcu_gemm_?_csr_row returns NOT_SUPPORTED,
//       src/kernel/dcu/level3/mm/csrmm/dcu_gemm_x_csr_row.cpp:15-36).
//   spmm_rowmajor_group_kernel<T, G, V> / spmm_rowmajor_short_kernel<T, NV, W>
//       the same layout with at most 32 / at most 16 dense columns: several
//       rows of A per wave (described at the kernels).
//   dense_transpose_kernel<T> + spmm_colmajor_kernel<T>   column-major B and C
//       (the layout the reference's GPU path does run): B is first transposed
//       into a row-major workspace, 64 x 64 tiles through LDS, both sides
//       coalesced; then a workgroup takes 64 consecutive rows of A and 64 dense
//       columns, its waves form the rows' sums exactly as above (one wave-wide
//       load per B row), park them in an LDS tile and the workgroup writes the
//       tile to column-major C transposed: 64 consecutive rows of one column
//       per wave instruction.  Gathering column-major B directly costs one
//       128-byte line per ELEMENT instead of per row (44 ms against 1.3 ms on
//       a 2^20 x 2^20 matrix with 32 entries per row and 64 columns).
//   spmm_strided_kernel<T>      any strides: one lane per (row, dense column),
//       lanes of a wave on consecutive rows, so column-major C is written
//       coalesced and B(:, c) is gathered like an SpMV x.  Stands in for
//       csr_gemm_plain_device (dcu_gemm_csr_col_plain.h:9-39).
//
// Arithmetic follows the row-major plain kernel
// (src/plain/kernel/level3/mm/gemm/gemm_x_csr_row_plain.c:11-19): alpha is
// folded into each value, products are accumulated with fma in entry order,
// then C = beta*C + acc.  beta == 0 never reads C.

#include <hip/hip_runtime.h>

#include <cstdlib>
#include <mutex>

#include "alsparse_amd_kernels.h"
#include "device_utils.hpp"

using namespace asamd;

constexpr int kSpmmBlock = 256;
constexpr int kSpmmWaves = kSpmmBlock / kWave;

template <typename T, int V>
struct alignas(sizeof(T) * V) Vec {
  T e[V];
};

// N consecutive elements that are only known to be aligned like a single one: the compiler may
// still fetch them with one wide load (global memory takes unaligned wide accesses).
template <typename T, int N>
struct __attribute__((packed, aligned(alignof(T)))) Packed {
  T e[N];
};
template <typename T>
using Quad4 = Packed<T, 4>;

// The first `valid` (<= V) elements at p, zeros behind them: whole groups of four through one load each.
template <typename T, int V>
__device__ __forceinline__ Vec<T, V> load_short_row(const T* p, int valid) {
  Vec<T, V> r;
#pragma unroll
  for (int i = 0; i < V; i += 4) {
    if (V - i >= 4 && i + 4 <= valid) {
      const Quad4<T> q = *reinterpret_cast<const Quad4<T>*>(p + i);
#pragma unroll
      for (int u = 0; u < 4; ++u) r.e[i + u] = q.e[u];
    } else {
#pragma unroll
      for (int u = 0; u < 4 && i + u < V; ++u) r.e[i + u] = i + u < valid ? p[i + u] : T(0);
    }
  }
  return r;
}

template <typename T, int V>
__device__ __forceinline__ Vec<T, V> load_vec(const T* p, bool vector_ok, int valid) {
  Vec<T, V> r;
  if (vector_ok && valid == V) {
    r = *reinterpret_cast<const Vec<T, V>*>(p);
  } else if (valid == V) {
    const Packed<T, V> q = *reinterpret_cast<const Packed<T, V>*>(p);
#pragma unroll
    for (int i = 0; i < V; ++i) r.e[i] = q.e[i];
  } else {
#pragma unroll
    for (int i = 0; i < V; ++i) r.e[i] = i < valid ? p[i] : T(0);
  }
  return r;
}

__device__ __forceinline__ float readlane_t(float v, int l) {
  return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), l));
}
__device__ __forceinline__ double readlane_t(double v, int l) {
  const uint64_t b = __builtin_bit_cast(uint64_t, v);
  const uint32_t lo = (uint32_t)__builtin_amdgcn_readlane((int)(uint32_t)b, l);
  const uint32_t hi = (uint32_t)__builtin_amdgcn_readlane((int)(uint32_t)(b >> 32), l);
  return __builtin_bit_cast(double, ((uint64_t)hi << 32) | lo);
}

template <typename R>
__device__ __forceinline__ Cx<R> readlane_t(Cx<R> v, int l) {
  return Cx<R>(readlane_t(v.re, l), readlane_t(v.im, l));
}

// grid.x covers rows (one wave each), grid.y covers chunks of 64*V columns.
template <typename T, int V>
__global__ __launch_bounds__(kSpmmBlock) void spmm_rowmajor_kernel(
    int m, int n, T alpha, const T* __restrict__ val, const int* __restrict__ row_ptr,
    const int* __restrict__ col_ind, int base, const T* __restrict__ B, int64_t ldb, T beta,
    T* __restrict__ C, int64_t ldc, bool vector_ok, const int* __restrict__ gate, int gate_want) {
  if (gate && *gate != gate_want) return;  // the structure probe chose the other kernel
  const int lane = threadIdx.x % kWave;
  const int wave = threadIdx.x / kWave;
  const unsigned bid = xcd_contiguous_id(blockIdx.x, gridDim.x);
  const int64_t row = (int64_t)bid * kSpmmWaves + wave;
  if (row >= m) return;  // wave-uniform
  const int c0 = (blockIdx.y * kWave + lane) * V;  // first dense column of this lane
  int valid = n - c0;
  valid = valid > V ? V : (valid < 0 ? 0 : valid);

  const int64_t start = (int64_t)row_ptr[row] - base;
  const int64_t end = (int64_t)row_ptr[row + 1] - base;
  T acc[V];
#pragma unroll
  for (int i = 0; i < V; ++i) acc[i] = T(0);

  for (int64_t j0 = start; j0 < end; j0 += kWave) {
    const int64_t j = j0 + lane;
    int my_col = 0;
    T my_val = T(0);
    if (j < end) {
      // A and C are touched once: non-temporal, so that they do not push rows of B out of the caches
      my_col = nt_load(col_ind + j) - base;
      my_val = alpha * nt_load(val + j);
    }
    const int cnt = (int)(end - j0 < kWave ? end - j0 : kWave);
    int t = 0;
    constexpr int kU = 4;  // B rows in flight per wave (8 and 16 measured no faster)
    for (; t + kU <= cnt; t += kU) {
      Vec<T, V> b[kU];
      T a[kU];
#pragma unroll
      for (int u = 0; u < kU; ++u) {
        const int col = __builtin_amdgcn_readlane(my_col, t + u);
        a[u] = readlane_t(my_val, t + u);
        b[u] = load_vec<T, V>(B + (int64_t)col * ldb + c0, vector_ok, valid);
      }
#pragma unroll
      for (int u = 0; u < kU; ++u) {
#pragma unroll
        for (int i = 0; i < V; ++i) acc[i] = fma_t(a[u], b[u].e[i], acc[i]);
      }
    }
    for (; t < cnt; ++t) {
      const int col = __builtin_amdgcn_readlane(my_col, t);
      const T a = readlane_t(my_val, t);
      const Vec<T, V> b = load_vec<T, V>(B + (int64_t)col * ldb + c0, vector_ok, valid);
#pragma unroll
      for (int i = 0; i < V; ++i) acc[i] = fma_t(a, b.e[i], acc[i]);
    }
  }

  T* crow = C + row * ldc + c0;
  if (vector_ok && valid == V) {
    Vec<T, V> out;
    if (beta == T(0)) {
#pragma unroll
      for (int i = 0; i < V; ++i) out.e[i] = acc[i];
    } else {
      const Vec<T, V> old = *reinterpret_cast<const Vec<T, V>*>(crow);
#pragma unroll
      for (int i = 0; i < V; ++i) out.e[i] = old.e[i] * beta + acc[i];
    }
    *reinterpret_cast<Vec<T, V>*>(crow) = out;
  } else {
#pragma unroll
    for (int i = 0; i < V; ++i) {
      if (i < valid) {
        const T res = beta == T(0) ? acc[i] : nt_load(crow + i) * beta + acc[i];
        nt_store(res, crow + i);
      }
    }
  }
}

// Four entries of a row per wave instruction: the wave's lanes form four groups of 16, lane l of a group owns
// the E = 16 / sizeof(T) dense columns from (blockIdx.y * 16 + l) * E on and loads them with one 128-bit load,
// so one instruction fetches 16 * E contiguous elements of FOUR rows of B (group g takes the row's entries
// 4i + g), and all the loads of up to 32 entries are in flight at once: a 32-entry row waits for B once, not
// eight times in turn.  The four partial sums meet at the end (two exchanges across the groups).  Needs B and C
// rows that 128-bit loads can address: pointers and row strides multiples of 16 bytes, n a multiple of E.
// The entry loop carries no index arithmetic: each lane turns its entry's column into the byte offset of that
// row of B once, and the groups fetch offsets and values from the lanes that hold them with ds_bpermute at
// addresses that are constants of the unrolled loop.  NARROW: B spans less than 2 GiB, so the offset is one
// 32-bit word and the load is a buffer load (uniform base, per-lane 32-bit offset); otherwise two words and a
// 64-bit pointer.
template <typename T>
__device__ __forceinline__ T bperm(int byte_addr, T v) {
  if constexpr (sizeof(T) == 4) {
    return __builtin_bit_cast(T, __builtin_amdgcn_ds_bpermute(byte_addr, __builtin_bit_cast(int, v)));
  } else {
    static_assert(sizeof(T) % 4 == 0, "element size");
    struct Words { int w[sizeof(T) / 4]; };
    Words in = __builtin_bit_cast(Words, v), out;
#pragma unroll
    for (int i = 0; i < (int)(sizeof(T) / 4); ++i) out.w[i] = __builtin_amdgcn_ds_bpermute(byte_addr, in.w[i]);
    return __builtin_bit_cast(T, out);
  }
}

// One wave's 64 entries of a row: what the entry loop hands round.  The position of an entry's row of B is kept
// as a byte offset (NARROW: one word, with kNoRow for lanes past the row's end; else two words).
template <typename T>
struct QuadChunk {
  T val;
  unsigned off;
  int off_hi;
};
constexpr unsigned kNoRow = 0x80000000u;  // an offset the buffer's range check turns away (B spans less than 2 GiB)

// Requests the (up to 64) entries of [j0, end) -- nothing is waited for here.
template <typename T, bool NARROW>
__device__ __forceinline__ QuadChunk<T> quad_load_chunk(int64_t j0, int64_t end, int lane, T alpha,
                                                        const T* __restrict__ val, const int* __restrict__ col_ind,
                                                        int base, int64_t row_bytes) {
  QuadChunk<T> c;
  c.val = T(0);
  c.off = NARROW ? kNoRow : 0u;
  c.off_hi = 0;
  if (j0 < end) {  // wave-uniform
    const bool live = j0 + lane < end;
    const int64_t j = live ? j0 + lane : j0;
    // A and C are touched once: non-temporal, so that they do not push rows of B out of the caches
    const int col = nt_load(col_ind + j) - base;
    const T loaded = alpha * nt_load(val + j);
    const int64_t off64 = (int64_t)col * row_bytes;
    if constexpr (NARROW) {
      // lanes past the end hold (0, no row): a group that reads them adds 0 * 0, so nothing in the entry loop
      // depends on the row's length
      c.val = live ? loaded : T(0);
      c.off = live ? (unsigned)off64 : kNoRow;
    } else {
      c.val = loaded;  // (lanes past the end repeat the chunk's first entry, and are never summed)
      c.off = (unsigned)off64;
      c.off_hi = (int)(off64 >> 32);
    }
  }
  return c;
}

// PERSISTENT waves, each walking the rows w, w + W, w + 2W, ... (W = waves of the grid) with the loads of three rows
// in flight: the row offsets of the row after next, the entries of the next row, the rows of B of the current
// one -- a wave that handles one row and exits waits for those three in turn.
// What the kernel's time is (27-point stencil 128 x 128 x 64, n = 64, 0.51 ms): the path from the L1 to the
// registers, not the waves' waiting for memory.  A row of A brings 8 KB of B through that path (eight wave-wide
// 1 KB loads), and a load takes 24 clocks of its compute unit's time where the L1's 64 bytes per clock would
// allow 16.  Two forms that took the waiting out -- the next rows' entries and offsets parked in LDS by
// memory-to-LDS loads two rows ahead, and on top of that the rows of B of the next row of A requested before
// the sums of the current one (two sets of registers, four waves per SIMD) -- took 0.52 and 0.51 ms: their
// waves spend 60 % of their cycles waiting to ISSUE an instruction where this form's spend 75 % waiting for
// loads to complete.  With every load of B turned away by the range check and no store of C all forms take
// 0.31 ms: the LDS pipe (27 ds_bpermutes per row; 43 % of the wave cycles wait for it then).  Also without
// effect: a third of the loads of B turned away; the store of C delayed into the next row (0.57 ms); 7 or 8
// waves per SIMD, had only with spills (0.76 ms).
template <typename T, bool NARROW>
__global__ __launch_bounds__(kSpmmBlock) void spmm_rowmajor_quad_kernel(
    int m, int n, T alpha, const T* __restrict__ val, const int* __restrict__ row_ptr,
    const int* __restrict__ col_ind, int base, const T* __restrict__ B, int64_t ldb, unsigned b_bytes, T beta,
    T* __restrict__ C, int64_t ldc, const int* __restrict__ gate, int gate_want) {
  if (gate && *gate != gate_want) return;  // the structure probe chose the other kernel
  constexpr int E = 16 / (int)sizeof(T);
  constexpr int kU = 8;  // loads in flight per lane
  const int lane = threadIdx.x % kWave;
  const int wave = __builtin_amdgcn_readfirstlane((int)threadIdx.x / kWave);
  const int64_t stride = (int64_t)gridDim.x * kSpmmWaves;  // rows between a wave's consecutive rows
  int64_t row = (int64_t)blockIdx.x * kSpmmWaves + wave;   // wave-uniform
  if (row >= m) return;
  const int g = lane / 16;
  const int c0 = (blockIdx.y * 16 + lane % 16) * E;
  const bool owns = c0 < n;
  // lanes past the last dense column load what the group's first lane loads (the same cache line: no request
  // of their own) and add nothing
  const int my_c = owns ? c0 : blockIdx.y * 16 * E;
  const BufferRsrc brsrc = make_rsrc(B, (int)b_bytes);
  const int64_t row_bytes = ldb * (int64_t)sizeof(T);
  // ds_bpermute address of the lane that holds this group's entry g (entry 4u + g: 16 u further); kept as ONE
  // register and added to where it is used: registers decide how many waves, hence rows, a compute unit has in
  // flight, and that is what this kernel's speed hangs on
  const int from0 = g * 4;
  const unsigned my_c_bytes = (unsigned)my_c * (unsigned)sizeof(T);

  // prologue: this row's offsets and entries, the next row's offsets
  int64_t start = (int64_t)row_ptr[row] - base, end = (int64_t)row_ptr[row + 1] - base;
  QuadChunk<T> cur = quad_load_chunk<T, NARROW>(start, end, lane, alpha, val, col_ind, base, row_bytes);
  int64_t next = row + stride;
  int64_t n_start = 0, n_end = 0;
  if (next < m) {
    n_start = (int64_t)row_ptr[next] - base;
    n_end = (int64_t)row_ptr[next + 1] - base;
  }
  while (true) {
    // ---- requests for the rows to come ------------------------------------------------------------
    QuadChunk<T> nxt = quad_load_chunk<T, NARROW>(n_start, next < m ? n_end : n_start, lane, alpha, val, col_ind,
                                                  base, row_bytes);
    const int64_t after = next + stride;
    int64_t a_start = 0, a_end = 0;
    if (after < m) {
      a_start = (int64_t)row_ptr[after] - base;
      a_end = (int64_t)row_ptr[after + 1] - base;
    }
    // ---- the current row ----------------------------------------------------------------------------
    T acc[E];
#pragma unroll
    for (int i = 0; i < E; ++i) acc[i] = T(0);
    for (int64_t j0 = start; j0 < end; j0 += kWave) {
      // (rows of more than 64 entries fetch their further chunks here, unprepared)
      const QuadChunk<T> ch = j0 == start ? cur : quad_load_chunk<T, NARROW>(j0, end, lane, alpha, val, col_ind,
                                                                              base, row_bytes);
      const int cnt = (int)(end - j0 < kWave ? end - j0 : kWave);
      if constexpr (NARROW) {
#pragma unroll
        for (int half = 0; half < 2; ++half) {
          if (half * 4 * kU >= cnt) break;
          Vec<T, E> b[kU];
          T a[kU];
#pragma unroll
          for (int u = 0; u < kU; ++u) {
            a[u] = bperm(from0 + 16 * u + half * 16 * kU, ch.val);
            const unsigned off = (unsigned)__builtin_amdgcn_ds_bpermute(from0 + 16 * u + half * 16 * kU, (int)ch.off);
            b[u] = buffer_load<Vec<T, E>>(brsrc, (int)(off + my_c_bytes));
          }
#pragma unroll
          for (int u = 0; u < kU; ++u) {
#pragma unroll
            for (int i = 0; i < E; ++i) acc[i] = fma_t(a[u], b[u].e[i], acc[i]);
          }
        }
      } else {
        for (int t0 = 0; t0 < cnt; t0 += 4 * kU) {
          Vec<T, E> b[kU];
          T a[kU];
          // every load is issued whatever the group needs: loads under branches would wait for one another
#pragma unroll
          for (int u = 0; u < kU; ++u) {
            const int at = from0 + 16 * u + t0 * 4;
            a[u] = bperm(at, ch.val);
            const unsigned lo = (unsigned)__builtin_amdgcn_ds_bpermute(at, (int)ch.off);
            const int hi = __builtin_amdgcn_ds_bpermute(at, ch.off_hi);
            const int64_t off = ((int64_t)hi << 32) | lo;
            b[u] = *reinterpret_cast<const Vec<T, E>*>(reinterpret_cast<const char*>(B + my_c) + off);
          }
#pragma unroll
          for (int u = 0; u < kU; ++u) {
            if (t0 + 4 * u + g < cnt) {
#pragma unroll
              for (int i = 0; i < E; ++i) acc[i] = fma_t(a[u], b[u].e[i], acc[i]);
            }
          }
        }
      }
    }
#pragma unroll
    for (int i = 0; i < E; ++i) acc[i] = sum_with_lane_xor<16>(acc[i]);
#pragma unroll
    for (int i = 0; i < E; ++i) acc[i] = sum_with_lane_xor<32>(acc[i]);
    if (g == 0 && owns) {
      T* crow = C + row * ldc + c0;
      Vec<T, E> out;
      if (beta == T(0)) {
#pragma unroll
        for (int i = 0; i < E; ++i) out.e[i] = acc[i];
      } else {
        const Vec<T, E> old = *reinterpret_cast<const Vec<T, E>*>(crow);
#pragma unroll
        for (int i = 0; i < E; ++i) out.e[i] = old.e[i] * beta + acc[i];
      }
      *reinterpret_cast<Vec<T, E>*>(crow) = out;
    }
    // ---- on to the next row ---------------------------------------------------------------------------
    if (next >= m) break;
    row = next;
    start = n_start;
    end = n_end;
    cur = nxt;
    next = after;
    n_start = a_start;
    n_end = a_end;
  }
}

// Dense operands narrower than a wave, lane-group form: G lanes per row of A, 64 / G rows per wave,
// lane c of a group owns V consecutive dense columns.  The group walks its row four entries at a
// time; the entry loads are the same address for all lanes of a group (one request), each B row is
// one load of G*V contiguous elements, so one wave instruction fetches 64 / G rows of B.  A wave per
// row would leave 64 - n lanes idle and issue 64 / G times as many loads.
template <typename T, int G, int V>
__global__ __launch_bounds__(kSpmmBlock) void spmm_rowmajor_group_kernel(
    int m, int n, T alpha, const T* __restrict__ val, const int* __restrict__ row_ptr,
    const int* __restrict__ col_ind, int base, const T* __restrict__ B, int64_t ldb, T beta,
    T* __restrict__ C, int64_t ldc, bool vector_ok) {
  constexpr int kRowsPerBlock = kSpmmBlock / G;
  const unsigned bid = xcd_contiguous_id(blockIdx.x, gridDim.x);
  const int64_t row = (int64_t)bid * kRowsPerBlock + threadIdx.x / G;
  if (row >= m) return;
  const int c0 = (blockIdx.y * G + threadIdx.x % G) * V;  // first dense column of this lane
  int valid = n - c0;
  valid = valid > V ? V : (valid < 0 ? 0 : valid);
  const int64_t start = (int64_t)row_ptr[row] - base;
  const int64_t end = (int64_t)row_ptr[row + 1] - base;
  const T* bcol = B + c0;
  T acc[V];
#pragma unroll
  for (int i = 0; i < V; ++i) acc[i] = T(0);
  if constexpr (V == 1) {
    // four entries at a time, every lane of the group loading the same entry (one request per group):
    // measured faster than handing entries round when a lane has a single column (13 columns: 0.75 ms
    // against 0.81 ms on a 2^20 x 2^20 matrix with 32 entries per row)
    int64_t j = start;
    constexpr int kU = 4;
    for (; j + kU <= end; j += kU) {
      int col[kU];
      T a[kU], b[kU];
#pragma unroll
      for (int u = 0; u < kU; ++u) {
        col[u] = col_ind[j + u] - base;
        a[u] = alpha * val[j + u];
      }
#pragma unroll
      for (int u = 0; u < kU; ++u) b[u] = valid ? bcol[(int64_t)col[u] * ldb] : T(0);
#pragma unroll
      for (int u = 0; u < kU; ++u) acc[0] = fma_t(a[u], b[u], acc[0]);
    }
    for (; j < end; ++j)
      acc[0] = fma_t(alpha * val[j], valid ? bcol[(int64_t)(col_ind[j] - base) * ldb] : T(0), acc[0]);
  } else {
    const int gl = threadIdx.x % G;                  // lane inside the group
    const int g0 = (threadIdx.x % kWave) - gl;       // the group's first lane in the wave
    for (int64_t j0 = start; j0 < end; j0 += G) {
      // the group reads G entries of its row with one coalesced load, then hands them round
      const int64_t j = j0 + gl;
      int my_col = 0;
      T my_val = T(0);
      if (j < end) {
        my_col = nt_load(col_ind + j) - base;
        my_val = alpha * nt_load(val + j);
      }
      const int cnt = (int)(end - j0 < G ? end - j0 : G);
      int t = 0;
      constexpr int kU = 4;
      for (; t + kU <= cnt; t += kU) {
        T a[kU];
        Vec<T, V> b[kU];
#pragma unroll
        for (int u = 0; u < kU; ++u) {
          const int col = lane_get(my_col, g0 + t + u);
          a[u] = lane_get(my_val, g0 + t + u);
          b[u] = load_vec<T, V>(bcol + (int64_t)col * ldb, vector_ok, valid);
        }
#pragma unroll
        for (int u = 0; u < kU; ++u) {
#pragma unroll
          for (int i = 0; i < V; ++i) acc[i] = fma_t(a[u], b[u].e[i], acc[i]);
        }
      }
      for (; t < cnt; ++t) {
        const int col = lane_get(my_col, g0 + t);
        const T a = lane_get(my_val, g0 + t);
        const Vec<T, V> b = load_vec<T, V>(bcol + (int64_t)col * ldb, vector_ok, valid);
#pragma unroll
        for (int i = 0; i < V; ++i) acc[i] = fma_t(a, b.e[i], acc[i]);
      }
    }
  }
  T* out = C + row * ldc + c0;
#pragma unroll
  for (int i = 0; i < V; ++i)
    if (i < valid) out[i] = beta == T(0) ? acc[i] : out[i] * beta + acc[i];
}

template <typename T, int G, int V>
static void launch_group(hipStream_t s, int m, int n, T alpha, const T* val, const int* rp, const int* ci, int base,
                         const T* B, int64_t ldb, T beta, T* C, int64_t ldc) {
  constexpr int rows_per_block = kSpmmBlock / G;
  const dim3 grid((unsigned)(((int64_t)m + rows_per_block - 1) / rows_per_block), (unsigned)((n + G * V - 1) / (G * V)));
  const bool vector_ok = V > 1 && (uintptr_t)B % (V * sizeof(T)) == 0 && ldb % V == 0;
  spmm_rowmajor_group_kernel<T, G, V><<<grid, kSpmmBlock, 0, s>>>(m, n, alpha, val, rp, ci, base, B, ldb, beta, C, ldc,
                                                                  vector_ok);
}

// Narrow dense operands (n <= NV <= 16): W lanes share a row of A and read its entries coalesced, as
// in the lane-group SpMV kernel; every lane multiplies its entries with the whole (short) row of B
// -- one vector load of NV elements when B allows it -- and keeps NV partial sums; the group's sums
// meet through DPP and lane 0 writes the row of C.  Measured on a 2^20 x 2^20 matrix with 32 entries
// per row against the lane-group kernel above with a lane per column (n: ms -> ms): 1: 0.50 -> 0.21, 2: 0.68 -> 0.37,
// 4: 0.78 -> 0.48, 6: 0.82 -> 0.64, 8: 0.77 -> 0.55, 12: 0.73 -> 0.72, 16: 0.61 -> 0.60; 13: 0.75 -> 0.89,
// which is why widths above 8 that are not multiples of four stay with the kernel above.
template <typename T, int NV>
__device__ __forceinline__ Vec<T, NV> short_row(const T* p, bool vector_ok, int n) {
  if (vector_ok) return *reinterpret_cast<const Vec<T, NV>*>(p);  // n == NV and the row is aligned to its size
  return load_short_row<T, NV>(p, n);
}

template <typename T, int NV, int W>
__global__ __launch_bounds__(kSpmmBlock) void spmm_rowmajor_short_kernel(
    int m, int n, T alpha, const T* __restrict__ val, const int* __restrict__ row_ptr,
    const int* __restrict__ col_ind, int base, const T* __restrict__ B, int64_t ldb, T beta,
    T* __restrict__ C, int64_t c_row_stride, int64_t c_col_stride, bool vector_ok) {
  constexpr int kRowsPerBlock = kSpmmBlock / W;
  const unsigned bid = xcd_contiguous_id(blockIdx.x, gridDim.x);
  const int lane = threadIdx.x % W;
  const int64_t row = (int64_t)bid * kRowsPerBlock + threadIdx.x / W;
  if (row >= m) return;  // whole lane groups leave together
  const int64_t start = (int64_t)row_ptr[row] - base;
  const int64_t end = (int64_t)row_ptr[row + 1] - base;
  T acc[NV];
#pragma unroll
  for (int i = 0; i < NV; ++i) acc[i] = T(0);
  int64_t j = start + lane;
  // two entries per lane and trip keep two B rows in flight
  for (; j + W < end; j += 2 * W) {
    const T a0 = alpha * val[j], a1 = alpha * val[j + W];
    const int c0 = col_ind[j] - base, c1 = col_ind[j + W] - base;
    const Vec<T, NV> b0 = short_row<T, NV>(B + (int64_t)c0 * ldb, vector_ok, n);
    const Vec<T, NV> b1 = short_row<T, NV>(B + (int64_t)c1 * ldb, vector_ok, n);
#pragma unroll
    for (int i = 0; i < NV; ++i) acc[i] = fma_t(a0, b0.e[i], acc[i]);
#pragma unroll
    for (int i = 0; i < NV; ++i) acc[i] = fma_t(a1, b1.e[i], acc[i]);
  }
  if (j < end) {
    const T a0 = alpha * val[j];
    const Vec<T, NV> b0 = short_row<T, NV>(B + (int64_t)(col_ind[j] - base) * ldb, vector_ok, n);
#pragma unroll
    for (int i = 0; i < NV; ++i) acc[i] = fma_t(a0, b0.e[i], acc[i]);
  }
#pragma unroll
  for (int i = 0; i < NV; ++i) acc[i] = group_sum<W>(acc[i]);
  if (lane == 0) {
    // row-major C: n consecutive elements; column-major C: the lanes 0 of a wave's groups hold
    // consecutive rows, so every dense column is written as one contiguous run
    T* crow = C + row * c_row_stride;
#pragma unroll
    for (int i = 0; i < NV; ++i)
      if (i < n) crow[i * c_col_stride] = beta == T(0) ? acc[i] : crow[i * c_col_stride] * beta + acc[i];
  }
}

template <typename T, int NV, int W>
static void launch_short(hipStream_t s, int m, int n, T alpha, const T* val, const int* rp, const int* ci, int base,
                         const T* B, int64_t ldb, T beta, T* C, int64_t scr, int64_t scc) {
  constexpr int rows_per_block = kSpmmBlock / W;
  const unsigned grid = (unsigned)(((int64_t)m + rows_per_block - 1) / rows_per_block);
  const bool vector_ok = n == NV && ldb % NV == 0 && (uintptr_t)B % (NV * sizeof(T)) == 0;
  spmm_rowmajor_short_kernel<T, NV, W><<<grid, kSpmmBlock, 0, s>>>(m, n, alpha, val, rp, ci, base, B, ldb, beta, C,
                                                                     scr, scc, vector_ok);
}

// lanes per row from the mean row length
template <typename T, int NV>
static void launch_short_w(hipStream_t s, int m, int n, int64_t nnz, T alpha, const T* val, const int* rp,
                           const int* ci, int base, const T* B, int64_t ldb, T beta, T* C, int64_t scr,
                           int64_t scc) {
  const double mean = (double)nnz / (double)m;
  if (mean < 8) launch_short<T, NV, 4>(s, m, n, alpha, val, rp, ci, base, B, ldb, beta, C, scr, scc);
  else if (mean < 48) launch_short<T, NV, 16>(s, m, n, alpha, val, rp, ci, base, B, ldb, beta, C, scr, scc);
  else launch_short<T, NV, 64>(s, m, n, alpha, val, rp, ci, base, B, ldb, beta, C, scr, scc);
}

// B rows of n <= 16 contiguous elements, C with any two strides
template <typename T>
static void launch_short_n(hipStream_t s, int m, int n, int64_t nnz, T alpha, const T* val, const int* rp,
                           const int* ci, int base, const T* B, int64_t ldb, T beta, T* C, int64_t scr,
                           int64_t scc) {
  if (n <= 2) launch_short_w<T, 2>(s, m, n, nnz, alpha, val, rp, ci, base, B, ldb, beta, C, scr, scc);
  else if (n <= 4) launch_short_w<T, 4>(s, m, n, nnz, alpha, val, rp, ci, base, B, ldb, beta, C, scr, scc);
  else if (n <= 8) launch_short_w<T, 8>(s, m, n, nnz, alpha, val, rp, ci, base, B, ldb, beta, C, scr, scc);
  else launch_short_w<T, 16>(s, m, n, nnz, alpha, val, rp, ci, base, B, ldb, beta, C, scr, scc);
}

// out[r * out_ld + c] = in[r + c * in_ld] for r < rows, c < cols: 64 x 64 tiles, reads
// coalesced along r, writes along c.  grid = (ceil(rows/64), ceil(cols/64)).
template <typename T>
__global__ __launch_bounds__(kSpmmBlock) void dense_transpose_kernel(int rows, int cols, const T* __restrict__ in,
                                                                     int64_t in_ld, T* __restrict__ out,
                                                                     int64_t out_ld) {
  __shared__ T tile[kWave][kWave + 1];
  const int tx = threadIdx.x % kWave, ty = threadIdx.x / kWave;
  const int64_t r0 = (int64_t)blockIdx.x * kWave;
  const int c0 = blockIdx.y * kWave;
#pragma unroll 4
  for (int i = ty; i < kWave; i += kSpmmWaves) {
    const int64_t r = r0 + tx;
    const int c = c0 + i;
    tile[i][tx] = (r < rows && c < cols) ? nt_load(in + r + (int64_t)c * in_ld) : T(0);
  }
  __syncthreads();
#pragma unroll 4
  for (int i = ty; i < kWave; i += kSpmmWaves) {
    const int64_t r = r0 + i;
    const int c = c0 + tx;
    if (r < rows && c < cols) out[r * out_ld + c] = tile[tx][i];
  }
}

// C (column-major, element (r, c) at r + c*ldc) = alpha*A*Bt + beta*C with Bt row-major
// (element (r, c) at r*ldbt + c).  grid = (ceil(m/64), ceil(n/64)).
template <typename T>
__global__ __launch_bounds__(kSpmmBlock) void spmm_colmajor_kernel(
    int m, int n, T alpha, const T* __restrict__ val, const int* __restrict__ row_ptr,
    const int* __restrict__ col_ind, int base, const T* __restrict__ Bt, int64_t ldbt, T beta,
    T* __restrict__ C, int64_t ldc) {
  __shared__ T tile[kWave][kWave + 1];
  const int lane = threadIdx.x % kWave;
  const int wave = threadIdx.x / kWave;
  const unsigned bid = xcd_contiguous_id(blockIdx.x, gridDim.x);
  const int64_t row0 = (int64_t)bid * kWave;
  const int c0 = blockIdx.y * kWave;
  const bool col_ok = c0 + lane < n;
  const T* bcol = Bt + c0 + lane;
  for (int rr = wave; rr < kWave; rr += kSpmmWaves) {
    const int64_t row = row0 + rr;
    T acc = T(0);
    if (row < m) {  // wave-uniform
      const int64_t start = (int64_t)row_ptr[row] - base;
      const int64_t end = (int64_t)row_ptr[row + 1] - base;
      for (int64_t j0 = start; j0 < end; j0 += kWave) {
        const int64_t j = j0 + lane;
        int my_col = 0;
        T my_val = T(0);
        if (j < end) {
          my_col = nt_load(col_ind + j) - base;
          my_val = alpha * nt_load(val + j);
        }
        const int cnt = (int)(end - j0 < kWave ? end - j0 : kWave);
        int t = 0;
        constexpr int kU = 4;
        for (; t + kU <= cnt; t += kU) {
          T b[kU], a[kU];
#pragma unroll
          for (int u = 0; u < kU; ++u) {
            const int col = __builtin_amdgcn_readlane(my_col, t + u);
            a[u] = readlane_t(my_val, t + u);
            b[u] = col_ok ? bcol[(int64_t)col * ldbt] : T(0);
          }
#pragma unroll
          for (int u = 0; u < kU; ++u) acc = fma_t(a[u], b[u], acc);
        }
        for (; t < cnt; ++t) {
          const int col = __builtin_amdgcn_readlane(my_col, t);
          const T a = readlane_t(my_val, t);
          acc = fma_t(a, col_ok ? bcol[(int64_t)col * ldbt] : T(0), acc);
        }
      }
    }
    tile[rr][lane] = acc;
  }
  __syncthreads();
  const int64_t row = row0 + lane;
  if (row >= m) return;
  for (int cc = wave; cc < kWave; cc += kSpmmWaves) {
    const int c = c0 + cc;
    if (c >= n) break;
    T* out = C + row + (int64_t)c * ldc;
    const T acc = tile[lane][cc];
    const T res = beta == T(0) ? acc : nt_load(out) * beta + acc;
    nt_store(res, out);
  }
}

// One lane per (row, dense column); blockDim = (64 rows, 4 columns).
template <typename T>
__global__ __launch_bounds__(kSpmmBlock) void spmm_strided_kernel(
    int m, int n, T alpha, const T* __restrict__ val, const int* __restrict__ row_ptr,
    const int* __restrict__ col_ind, int base, const T* __restrict__ B, int64_t sbr, int64_t sbc,
    T beta, T* __restrict__ C, int64_t scr, int64_t scc) {
  const int64_t row = (int64_t)blockIdx.x * kWave + threadIdx.x;
  if (row >= m) return;
  const int64_t start = (int64_t)row_ptr[row] - base;
  const int64_t end = (int64_t)row_ptr[row + 1] - base;
  for (int64_t c = (int64_t)blockIdx.y * blockDim.y + threadIdx.y; c < n;
       c += (int64_t)gridDim.y * blockDim.y) {
    T acc = T(0);
    for (int64_t j = start; j < end; ++j) {
      const int64_t col = (int64_t)col_ind[j] - base;
      acc = fma_t(alpha * val[j], B[col * sbr + c * sbc], acc);
    }
    T* out = C + row * scr + c * scc;
    *out = beta == T(0) ? acc : *out * beta + acc;
  }
}

// column-major B (k x n) next to column-major C (m x n), more than one column:
// B has to be transposed into a workspace first
static bool colmajor_nn(const asamd_dense_strides* st, int n) {
  return n > 1 && st->b_row_stride == 1 && st->b_col_stride != 1 && st->c_row_stride == 1;
}

// ---- do neighbouring rows of A share columns? --------------------------------------------------
// Stencils and finite-element matrices do (a row of B fetched for one row of A is wanted again by the next
// rows), matrices with random columns do not, and which row-major kernel is faster depends on it.  csrmm has no
// analysis call, so every multiply whose operands make the question matter looks for itself, ON THE DEVICE: a
// small kernel samples kProbeRows rows scattered over the matrix and counts the share of their entries (the
// first 64 of each) whose column is in the next row as well; its last workgroup leaves the verdict (1: a
// quarter or more are shared; a 27-point stencil 0.67, a 5-point Laplacian 0.40, random columns 0.0003, R-MAT
// 0.006) in a word of the caller's workspace, and the two candidate kernels are both launched, each returning at
// once unless the word names it.  No host round trip, capturable.  The verdict is also copied to the host behind
// the multiply (never waited for): once it has arrived, later multiplies of the same arrays launch the one kernel.
constexpr int kProbeRows = 2048;
struct ProbeWords {
  unsigned shared, total, done;
  int verdict;
};
__global__ void spmm_probe_reset_kernel(ProbeWords* w) {
  w->shared = 0;
  w->total = 0;
  w->done = 0;
  w->verdict = 0;
}
constexpr int kProbeRowsPerBlock = kSpmmBlock / kWave;  // a wave per sampled row
__global__ __launch_bounds__(kSpmmBlock) void spmm_reuse_probe_kernel(int m, const int* __restrict__ row_ptr,
                                                                      const int* __restrict__ col_ind, int base,
                                                                      ProbeWords* __restrict__ out) {
  const int lane = threadIdx.x % kWave;
  const int t = blockIdx.x * kProbeRowsPerBlock + threadIdx.x / kWave;  // the sampled row's number
  unsigned shared = 0, total = 0;
  if (t < kProbeRows && m >= 2) {
    // scattered rows: evenly spaced ones fall on the same position of every grid line of a stencil
    const int64_t r = (int64_t)((((uint64_t)t + 1) * 0x9E3779B97F4A7C15ull >> 20) % (uint64_t)(m - 1));
    const int64_t b0 = (int64_t)row_ptr[r] - base, e0 = (int64_t)row_ptr[r + 1] - base, e1 = (int64_t)row_ptr[r + 2] - base;
    // lane l holds entry l of the row and entry l of the next row (the first 64 of each); every lane then
    // looks for its column among the next row's, which go round the wave
    const bool mine = b0 + lane < e0, theirs = e0 + lane < e1;
    const int c = mine ? col_ind[b0 + lane] : -1;
    const int d = theirs ? col_ind[e0 + lane] : -2;
    const int next_cnt = (int)(e1 - e0 < kWave ? e1 - e0 : kWave);
    bool found = false;
    for (int j = 0; j < next_cnt; ++j) found |= __builtin_amdgcn_readlane(d, j) == c;
    shared = (unsigned)__popcll(__ballot(mine && found));
    total = (unsigned)__popcll(__ballot(mine));
  }
  if (lane == 0 && total) {
    atomicAdd(&out->shared, shared);
    atomicAdd(&out->total, total);
  }
  // the workgroup that finishes last reads the totals and writes the verdict
  __shared__ bool last;
  __threadfence();
  __syncthreads();
  if (threadIdx.x == 0) last = atomicAdd(&out->done, 1u) == gridDim.x - 1;
  __syncthreads();
  if (last && threadIdx.x == 0) {
    const unsigned sh = atomicAdd(&out->shared, 0u), to = atomicAdd(&out->total, 0u);
    out->verdict = (to > 0 && 4ull * sh >= (unsigned long long)to) ? 1 : 0;
  }
}

// ---- rows of B shared through LDS ----------------------------------------------------------------
// Rows of B shared through LDS (opt-in, ALSPARSE_AMD_SPMM_LDS=1), for matrices whose neighbouring rows share
// columns.  The rows of A are cut into runs of consecutive rows, dealt round robin to persistent workgroups, one
// block of 64 dense columns each.  For every run a workgroup finds the distinct columns among the run's entries (a
// hash table in LDS), fetches each distinct row of B ONCE -- 128-bit loads, four rows of B per wave instruction
// for fp32 -- into an LDS tile, and its waves form the sums of the run's rows from the tile: lane groups own a
// row each, one 128-bit LDS read per product and group, C written once.  A 27-point stencil asks L1 for 27 rows
// of B per row of A in the one-wave-per-row kernels and for 10 here.
// The stages are software-pipelined: while run i is summed from the tile, the rows of B of run i + 1 are on
// their way into registers (they are written to the tile once run i is done with it), the entries of run i + 2
// are being read and the row offsets of run i + 3.  A run whose entries or distinct columns exceed the staging
// areas is multiplied straight from global memory, a wave per row.  Every sum is formed in CSR order: the same
// bits every run.
// Measured (27-point stencil 128 x 128 x 64, n = 64, fp32): 0.62 ms, against 0.51 ms for four rows of B per wave
// instruction without LDS.  The L1 requests fall as intended (62 per row of A instead of 147), but the stages'
// times add up instead of overlapping -- the sums alone take 0.28 ms: they read every entry's 256 bytes of B from
// LDS, 7 GB in all, and the LDS data path is busy half of the kernel's clocks -- and hashing the next run two
// iterations ahead, so that the rows of B travel for a whole iteration, changed nothing.  Not chosen by default.
template <typename T>
struct LdsSpmm {
  // rows of A per run, and rows of B that the tile holds (42 KiB; a 27-point stencil's 16 rows touch 9 x 18)
  static constexpr int run = sizeof(T) == 4 ? 16 : (sizeof(T) == 8 ? 8 : 4);
  static constexpr int cap = 168 * 4 / (int)sizeof(T);
  static constexpr int entries = 448;                      // entries of a run staged at most (three workgroups
                                                           // of fp32 then share a compute unit's 160 KiB)
  static constexpr int hash = 512;                         // slots of the column hash
  static constexpr int V = 16 / (int)sizeof(T);            // elements of a 128-bit load
  static constexpr int lpr = kWave / V;                    // lanes that cover the tile's 64 columns of one row of B
  static constexpr int rpi = kWave / lpr;                  // rows of B per wave instruction
  static constexpr int loads = (cap + kSpmmWaves * rpi - 1) / (kSpmmWaves * rpi);  // per lane, to fill the tile
  static constexpr int loads_one = (cap + kSpmmWaves - 1) / kSpmmWaves;            // ... element by element
  static constexpr int per_thread = (entries + kSpmmBlock - 1) / kSpmmBlock;  // entries a thread carries between stages
  static constexpr int row_bytes = kWave * (int)sizeof(T);  // of a tile row; byte offsets of rows fit 16 bits
  static constexpr int zero_row = cap;                     // one more tile row, all zero, for a wave's idle lanes
  static constexpr size_t val_off = (size_t)(cap + 1) * row_bytes;
  static constexpr size_t slot_off = val_off + 2 * (size_t)entries * sizeof(T);
  static constexpr size_t hkey_off = slot_off + 2 * (size_t)entries * sizeof(unsigned short);
  static constexpr size_t hslot_off = hkey_off + (size_t)hash * sizeof(int);
  static constexpr size_t ucol_off = hslot_off + (size_t)hash * sizeof(unsigned short);
  static constexpr size_t roff_off = ucol_off + (size_t)cap * sizeof(int);   // row offsets of both runs
  static constexpr size_t info_off = roff_off + 2 * (size_t)(run + 1) * sizeof(int);
  static constexpr size_t bytes = info_off + 64;
};

// what the stages hand on about a run (two copies: the run being summed and the one being prepared)
struct LdsRunInfo {
  int e_begin;   // first entry of the run, zero-based position in the CSR streams
  int cnt;       // entries
  int distinct;  // distinct columns (rows of the tile in use)
  int fits;      // 0: multiplied from global memory
};

// WIDE: B's rows can be addressed with 128-bit loads (pointer and row stride multiples of 16 bytes, n a
// multiple of the elements per load); otherwise a wave fetches one row of B per instruction, element by element.
template <typename T, bool WIDE>
__global__ __launch_bounds__(kSpmmBlock) void spmm_rowblock_lds_kernel(
    int m, int n, T alpha, const T* __restrict__ val, const int* __restrict__ row_ptr,
    const int* __restrict__ col_ind, int base, const T* __restrict__ B, int64_t ldb, T beta,
    T* __restrict__ C, int64_t ldc, int runs_total, bool c_wide) {
  using L = LdsSpmm<T>;
  constexpr int V = L::V;
  extern __shared__ __align__(16) unsigned char smem[];
  T* tile = reinterpret_cast<T*>(smem);
  T* s_val = reinterpret_cast<T*>(smem + L::val_off);                       // [2][entries]
  unsigned short* s_slot = reinterpret_cast<unsigned short*>(smem + L::slot_off);  // [2][entries]
  int* h_key = reinterpret_cast<int*>(smem + L::hkey_off);
  unsigned short* h_slot = reinterpret_cast<unsigned short*>(smem + L::hslot_off);
  int* u_col = reinterpret_cast<int*>(smem + L::ucol_off);
  int* s_roff = reinterpret_cast<int*>(smem + L::roff_off);                  // [2][run + 1], local to the run's first entry
  LdsRunInfo* info = reinterpret_cast<LdsRunInfo*>(smem + L::info_off);      // [2]
  int* s_count = reinterpret_cast<int*>(smem + L::info_off + 2 * sizeof(LdsRunInfo));  // [2]

  const int tid = threadIdx.x;
  const int lane = tid % kWave;
  const int wave = __builtin_amdgcn_readfirstlane(tid / kWave);
  // Runs are dealt round robin: at any time the grid works on one window of consecutive runs, so the rows of B
  // that neighbouring runs share are requested close together in time and are found in L2; run r always lands
  // on the same XCD (r modulo 8), so runs a multiple of 8 apart -- the neighbours across a grid line of a
  // discretisation whose lines are a multiple of 8 runs long -- share that XCD's L2.
  const int stride = (int)gridDim.x;
  const int first = (int)blockIdx.x;
  if (first >= runs_total) return;
  const int cnt = (runs_total - first + stride - 1) / stride;  // runs of this workgroup
  for (int q = tid; q < kWave; q += kSpmmBlock) tile[(size_t)L::zero_row * kWave + q] = T(0);  // (a barrier follows)
  const int c0 = blockIdx.y * kWave;  // first dense column of this workgroup
  const int my_c = c0 + lane;         // the dense column this lane sums
  const bool owns = my_c < n;
  // staging: lpr lanes x 16 bytes cover 64 columns of one row of B, rpi rows per wave instruction
  const int sg = lane / L::lpr, sl = lane % L::lpr;
  const int s_col_off = c0 + sl * V;
  const bool s_in = s_col_off < n;  // (n is a multiple of V on the wide path)

  // ---- stage E: the entries of a run into registers, in two steps ------------------------------
  // E1 reads the run's row offsets, E2 (an iteration later, when they have arrived) the entries themselves: no
  // stage waits for a load that it has issued itself
  int e_col[L::per_thread];
  T e_val[L::per_thread];
  int e_begin = 0, e_cnt = 0;  // of the run whose entries the registers hold
  int e_roff = 0;              // thread t <= run: offset of the run's row t
  int o_begin = 0, o_end = 0, o_row = 0;  // E1's loads: first and last offset of a run, and row t's
  auto load_offsets = [&](int run) __attribute__((always_inline)) {
    const int64_t r0 = (int64_t)run * L::run;
    const int64_t r1 = r0 + L::run < m ? r0 + L::run : m;
    o_begin = row_ptr[r0];
    o_end = row_ptr[r1];
    o_row = row_ptr[r0 + tid < r1 ? r0 + tid : r1];
  };
  auto load_values = [&]() __attribute__((always_inline)) {
    e_begin = o_begin - base;
    e_cnt = o_end - o_begin;
    e_roff = o_row - o_begin;
#pragma unroll
    for (int u = 0; u < L::per_thread; ++u) {
      const int i = tid + u * kSpmmBlock;
      const bool live = i < e_cnt && e_cnt <= L::entries;
      e_col[u] = live ? nt_load(col_ind + (int64_t)e_begin + i) - base : -1;
      e_val[u] = live ? alpha * nt_load(val + (int64_t)e_begin + i) : T(0);
    }
  };

  // rows of B of the run in preparation, on their way (raw 128-bit pieces: first-class values, so that the
  // array lives in registers)
  typedef int Raw128 __attribute__((ext_vector_type(4)));
  Raw128 b_reg[WIDE ? L::loads : 1];
  T b_one[WIDE ? 1 : L::loads_one];

  load_offsets(first);
  load_values();
  if (1 < cnt) load_offsets(first + stride);
  for (int k = -1; k < cnt; ++k) {
    const int i = first + k * stride;  // the run whose rows are summed in this iteration (none when k = -1)
    const int nb = (k + 1) & 1, cb = k & 1;
    const bool has_nxt = k + 1 < cnt;
    bool nxt_fits = false;
    int nxt_distinct = 0;
    if (has_nxt) {
      // ---- stage H: distinct columns of run nxt -> rows of the tile ----------------------------
      nxt_fits = e_cnt <= L::entries;
      if (nxt_fits) {
        for (int k = tid; k < L::hash; k += kSpmmBlock) h_key[k] = -1;
        if (tid == 0) {
          s_count[0] = 0;
          s_count[1] = 0;  // set when a column finds no place in the hash table
        }
        __syncthreads();
#pragma unroll
        for (int u = 0; u < L::per_thread; ++u) {
          const int k = tid + u * kSpmmBlock;
          if (k < e_cnt) {
            const int col = e_col[u];
            unsigned h = ((unsigned)col * 0x9E3779B1u) >> 23;  // 9 bits
            bool placed = false;
            for (int probe = 0; probe < L::hash && !placed; ++probe) {
              const int prev = atomicCAS(&h_key[h], -1, col);
              placed = prev == -1 || prev == col;
              if (!placed) h = (h + 1) & (L::hash - 1);
            }
            if (!placed) s_count[1] = 1;
            s_val[nb * L::entries + k] = e_val[u];
            s_slot[nb * L::entries + k] = (unsigned short)h;
          }
        }
        __syncthreads();
        for (int k = tid; k < L::hash; k += kSpmmBlock) {
          const int key = h_key[k];
          if (key >= 0) {
            const int slot = atomicAdd(&s_count[0], 1);
            h_slot[k] = (unsigned short)slot;
            if (slot < L::cap) u_col[slot] = key;
          }
        }
        __syncthreads();
        nxt_distinct = s_count[0];
        nxt_fits = nxt_distinct <= L::cap && s_count[1] == 0;
        if (nxt_fits) {
#pragma unroll
          for (int u = 0; u < L::per_thread; ++u) {
            const int k = tid + u * kSpmmBlock;
            if (k < e_cnt)
              s_slot[nb * L::entries + k] = (unsigned short)(h_slot[s_slot[nb * L::entries + k]] * L::row_bytes);
          }
        }
      }
      if (tid == 0) info[nb] = LdsRunInfo{e_begin, e_cnt, nxt_distinct, nxt_fits ? 1 : 0};
      if (tid <= L::run) s_roff[nb * (L::run + 1) + tid] = e_roff;
      // ---- stage L: the distinct rows of B of run nxt, requested ---------------------------------
      if (nxt_fits) {
        if constexpr (WIDE) {
#pragma unroll
          for (int u = 0; u < L::loads; ++u) {
            const int slot = (u * kSpmmWaves + wave) * L::rpi + sg;
            // lanes without a row of their own load the run's first row again (a line already requested)
            const int col = u_col[slot < nxt_distinct ? slot : 0];
            if (nxt_distinct > 0)
              b_reg[u] = *reinterpret_cast<const Raw128*>(B + (int64_t)col * ldb + (s_in ? s_col_off : c0));
          }
        } else {
#pragma unroll
          for (int u = 0; u < L::loads_one; ++u) {
            const int slot = u * kSpmmWaves + wave;
            const int col = u_col[slot < nxt_distinct ? slot : 0];
            b_one[u] = (owns && nxt_distinct > 0) ? B[(int64_t)col * ldb + my_c] : T(0);
          }
        }
      }
    }
    // ---- stage E: entries of the run after next, offsets of the one after that -------------------
    if (k + 2 < cnt) load_values();
    if (k + 3 < cnt) load_offsets(first + (k + 3) * stride);
    // ---- stage C: the rows of run i from the tile ---------------------------------------------------
    if (k >= 0) {
      const LdsRunInfo ri = info[cb];
      const int64_t r0 = (int64_t)i * L::run;
      const int r_cnt = (int)(r0 + L::run < m ? L::run : m - r0);
      if (ri.fits) {
        // rpi rows per wave at a time: lane group sg sums row rstep + sg, its lanes own V dense columns each;
        // per entry one read of (slot, value) -- the same address for the whole group -- and one 128-bit read
        // of the tile
        for (int rstep = wave * L::rpi; rstep < r_cnt; rstep += kSpmmWaves * L::rpi) {
          const int r = rstep + sg;
          const bool has = r < r_cnt;
          const int off = has ? s_roff[cb * (L::run + 1) + r] : 0;
          const int len = has ? s_roff[cb * (L::run + 1) + r + 1] - off : 0;
          int longest = len;
          if constexpr (L::rpi > 1) {
            for (int d = L::lpr; d < kWave; d <<= 1) {
              const int other = lane_xor(longest, d);
              longest = other > longest ? other : longest;
            }
          }
          const T* rv = s_val + cb * L::entries + off;
          const unsigned short* rs = s_slot + cb * L::entries + off;
          T acc[V];
#pragma unroll
          for (int q = 0; q < V; ++q) acc[q] = T(0);
          int shortest = len;
          if constexpr (L::rpi > 1) {
            for (int d = L::lpr; d < kWave; d <<= 1) {
              const int other = lane_xor(shortest, d);
              shortest = other < shortest ? other : shortest;
            }
          }
          const unsigned char* my_tile = reinterpret_cast<const unsigned char*>(tile) + sl * 16;
          // entries that every row of the wave has: no lane is masked
          int t0 = 0;
          for (; t0 + 4 <= shortest; t0 += 4) {
            T a4[4];
            Vec<T, V> b4[4];
#pragma unroll
            for (int u = 0; u < 4; ++u) {
              a4[u] = rv[t0 + u];
              b4[u] = *reinterpret_cast<const Vec<T, V>*>(my_tile + rs[t0 + u]);
            }
#pragma unroll
            for (int u = 0; u < 4; ++u) {
#pragma unroll
              for (int q = 0; q < V; ++q) acc[q] = fma_t(a4[u], b4[u].e[q], acc[q]);
            }
          }
          // the rest, row by row as long as any row of the wave has entries left
          for (; t0 < longest; ++t0) {
            if (t0 < len) {
              const T a = rv[t0];
              const Vec<T, V> b = *reinterpret_cast<const Vec<T, V>*>(my_tile + rs[t0]);
#pragma unroll
              for (int q = 0; q < V; ++q) acc[q] = fma_t(a, b.e[q], acc[q]);
            }
          }
          if (has && c_wide && s_col_off + V <= n) {
            // C's rows can be addressed in 16-byte pieces too
            Vec<T, V>* out = reinterpret_cast<Vec<T, V>*>(C + (r0 + r) * ldc + s_col_off);
            Vec<T, V> res;
            if (beta == T(0)) {
#pragma unroll
              for (int q = 0; q < V; ++q) res.e[q] = acc[q];
            } else {
              const Vec<T, V> old = *out;
#pragma unroll
              for (int q = 0; q < V; ++q) res.e[q] = old.e[q] * beta + acc[q];
            }
            *out = res;
          } else if (has) {
            T* out = C + (r0 + r) * ldc + s_col_off;
#pragma unroll
            for (int q = 0; q < V; ++q) {
              if (s_col_off + q < n) {
                const T res = beta == T(0) ? acc[q] : nt_load(out + q) * beta + acc[q];
                nt_store(res, out + q);
              }
            }
          }
        }
      } else {
        // the run did not fit the staging areas: straight from global memory, a wave per row
        for (int r = wave; r < r_cnt; r += kSpmmWaves) {
          const int64_t row = r0 + r;
          const int64_t rb = (int64_t)row_ptr[row] - base, re = (int64_t)row_ptr[row + 1] - base;
          T acc = T(0);
          for (int64_t j0 = rb; j0 < re; j0 += kWave) {
            const int64_t j = j0 + lane < re ? j0 + lane : j0;
            const int my_col = col_ind[j] - base;
            const T my_val = alpha * val[j];
            const int c = (int)(re - j0 < kWave ? re - j0 : kWave);
            for (int t = 0; t < c; ++t) {
              const int col = __builtin_amdgcn_readlane(my_col, t);
              const T bv = owns ? B[(int64_t)col * ldb + my_c] : T(0);
              acc = fma_t(readlane_t(my_val, t), bv, acc);
            }
          }
          if (owns) {
            T* out = C + row * ldc + my_c;
            const T res = beta == T(0) ? acc : nt_load(out) * beta + acc;
            nt_store(res, out);
          }
        }
      }
    }
    __syncthreads();  // every wave is done with the tile of run i
    // ---- stage W: the rows of B of run nxt, arrived, into the tile ------------------------------------
    if (has_nxt && nxt_fits) {
      if constexpr (WIDE) {
#pragma unroll
        for (int u = 0; u < L::loads; ++u) {
          const int slot = (u * kSpmmWaves + wave) * L::rpi + sg;
          if (slot < nxt_distinct && s_in) *reinterpret_cast<Raw128*>(tile + (size_t)slot * kWave + sl * V) = b_reg[u];
        }
      } else {
#pragma unroll
        for (int u = 0; u < L::loads_one; ++u) {
          const int slot = u * kSpmmWaves + wave;
          if (slot < nxt_distinct) tile[(size_t)slot * kWave + lane] = b_one[u];
        }
      }
    }
    __syncthreads();
  }
}

// What the probe found, remembered per (row_ptr, col_ind, m, nnz) WITHOUT ever waiting for it: the multiply that
// probes also copies the verdict word to pinned host memory on its stream and records an event; a later multiply
// of the same arrays that finds the event complete launches the one kernel that the verdict names, without probe
// and without gate.  Until then (and inside a stream capture, where nothing is recorded) every multiply probes
// on the device for itself.  A stale entry -- another matrix at the same addresses -- costs speed, never
// correctness: both kernels multiply any matrix.
struct ReuseSeen {
  const int *rp, *ci;
  int m, nnz;
  int state;  // 0: free, 1: verdict on its way, 2: known
  int verdict;
  hipEvent_t ev;
  int* host_word;
};
constexpr int kReuseSeen = 16;
static std::mutex g_reuse_lock;
static ReuseSeen g_reuse[kReuseSeen];
static int g_reuse_next = 0;

// -1: not known (the caller probes; *record is the entry to hand to reuse_record afterwards, or null), else 0 / 1
static int reuse_lookup(hipStream_t s, const int* rp, const int* ci, int m, int nnz, ReuseSeen** record) {
  *record = nullptr;
  std::lock_guard<std::mutex> guard(g_reuse_lock);
  for (ReuseSeen& e : g_reuse) {
    if (e.state == 0 || e.rp != rp || e.ci != ci || e.m != m || e.nnz != nnz) continue;
    if (e.state == 1 && hipEventQuery(e.ev) == hipSuccess) {
      e.verdict = *e.host_word;
      e.state = 2;
    }
    if (e.state == 1) (void)hipGetLastError();  // hipErrorNotReady is not an error
    return e.state == 2 ? e.verdict : -1;
  }
  hipStreamCaptureStatus capturing = hipStreamCaptureStatusNone;
  if (hipStreamIsCapturing(s, &capturing) != hipSuccess || capturing != hipStreamCaptureStatusNone) {
    (void)hipGetLastError();
    return -1;
  }
  // a place for this matrix: the next one in turn whose verdict is not on its way
  for (int tries = 0; tries < kReuseSeen; ++tries) {
    ReuseSeen& e = g_reuse[g_reuse_next];
    g_reuse_next = (g_reuse_next + 1) % kReuseSeen;
    if (e.state == 1) continue;
    if (!e.ev && hipEventCreateWithFlags(&e.ev, hipEventDisableTiming) != hipSuccess) break;
    if (!e.host_word && hipHostMalloc((void**)&e.host_word, sizeof(int), hipHostMallocDefault) != hipSuccess) break;
    e.rp = rp;
    e.ci = ci;
    e.m = m;
    e.nnz = nnz;
    e.state = 0;  // becomes 1 once the copy and the event are on the stream
    *record = &e;
    return -1;
  }
  (void)hipGetLastError();
  return -1;
}

static void reuse_record(hipStream_t s, ReuseSeen* e, const int* d_verdict) {
  std::lock_guard<std::mutex> guard(g_reuse_lock);
  if (hipMemcpyAsync(e->host_word, d_verdict, sizeof(int), hipMemcpyDeviceToHost, s) == hipSuccess &&
      hipEventRecord(e->ev, s) == hipSuccess)
    e->state = 1;
  else
    (void)hipGetLastError();
}

static size_t workspace_bytes(size_t val_size, int n, int k, const asamd_dense_strides* st) {
  if (!st || n <= 0 || k <= 0 || !colmajor_nn(st, n)) return 0;
  return (((size_t)k * (size_t)n * val_size) + 255) & ~(size_t)255;
}

template <typename T>
static int csrmm_impl(hipStream_t s, int m, int n, int k, int nnz, T alpha, const T* val,
                      const int* rp, const int* ci, int base, const T* B, T beta, T* C,
                      const asamd_dense_strides* st, void* ws, size_t ws_bytes) {
  if (!val || !rp || !ci || !B || !C || !st || m <= 0 || n <= 0) return hipErrorInvalidValue;
  if (((uintptr_t)val | (uintptr_t)B | (uintptr_t)C) % alignof(T)) return hipErrorInvalidValue;
  if (n > 1 && st->c_row_stride == 1 && st->c_col_stride != 1) {
    // column-major C: rows of op(B) must be contiguous for the wave-wide loads
    const T* Bt = nullptr;
    int64_t ldbt = 0;
    if (st->b_col_stride == 1) {  // op(B) = B^T of a column-major n x k array: already row-major k x n
      Bt = B;
      ldbt = st->b_row_stride;
    } else if (colmajor_nn(st, n) && ws && k > 0 && ws_bytes >= workspace_bytes(sizeof(T), n, k, st)) {
      const dim3 tgrid((unsigned)(((int64_t)k + kWave - 1) / kWave), (unsigned)((n + kWave - 1) / kWave));
      dense_transpose_kernel<T><<<tgrid, kSpmmBlock, 0, s>>>(k, n, B, st->b_col_stride, (T*)ws, (int64_t)n);
      Bt = (const T*)ws;
      ldbt = n;
    }
    if (Bt && n <= 16 && (n <= 8 || n % 4 == 0)) {
      // few dense columns: the entry-parallel kernel on the row-major B, C written through its strides
      launch_short_n<T>(s, m, n, nnz, alpha, val, rp, ci, base, Bt, ldbt, beta, C, 1, st->c_col_stride);
      return hipGetLastError();
    }
    if (Bt) {
      const dim3 grid((unsigned)(((int64_t)m + kWave - 1) / kWave), (unsigned)((n + kWave - 1) / kWave));
      spmm_colmajor_kernel<T><<<grid, kSpmmBlock, 0, s>>>(m, n, alpha, val, rp, ci, base, Bt, ldbt, beta, C,
                                                          st->c_col_stride);
      return hipGetLastError();
    }
  }
  // a single dense column has unit stride along its one column whatever the layout says
  const bool unit_cols = (st->b_col_stride == 1 && st->c_col_stride == 1) || n == 1;
  if (unit_cols) {
    const int64_t ldb = st->b_row_stride, ldc = st->c_row_stride;
    if (n <= 16) {  // a wave per row would leave 64 - n lanes idle (0.93 ms whatever n is on the matrix below)
      // 9..16 columns that are not whole groups of four: a lane per column loads less padding
      if (n > 8 && n % 4 != 0) launch_group<T, 16, 1>(s, m, n, alpha, val, rp, ci, base, B, ldb, beta, C, ldc);
      else launch_short_n<T>(s, m, n, nnz, alpha, val, rp, ci, base, B, ldb, beta, C, ldc, 1);
      return hipGetLastError();
    }
    if (n <= 32 && (uintptr_t)B % (2 * sizeof(T)) == 0 && ldb % 2 == 0) {
      // 17..32 columns in rows of B that pairs of elements can be loaded from: 16 lanes x 2 columns per row,
      // four rows of B per wave-wide load (n = 32: 0.95 ms with a wave per row -> 0.68 ms, n = 24: 1.00 -> 0.90).
      // Odd row strides were slower this way (n = 31: 1.23 ms against 1.13 ms), and wider groups or vectors
      // were no faster than a wave per row above 32 columns.
      launch_group<T, 16, 2>(s, m, n, alpha, val, rp, ci, base, B, ldb, beta, C, ldc);
      return hipGetLastError();
    }
    const unsigned gx = (unsigned)(((int64_t)m + kSpmmWaves - 1) / kSpmmWaves);
    // rows of B and C that 128-bit loads can address
    constexpr int E = 16 / (int)sizeof(T);
    const bool aligned16 = n % E == 0 && ldb % E == 0 && ldc % E == 0 && (uintptr_t)B % 16 == 0 && (uintptr_t)C % 16 == 0;
    // ALSPARSE_AMD_SPMM_LDS=1 (read at every call): the kernel that shares rows of B through LDS, whatever the
    // structure.  It is not chosen otherwise: on the 27-point stencil 128 x 128 x 64 with n = 64 it takes 0.62 ms
    // where four rows of B per wave instruction take 0.52 ms.
    const char* lds_env = getenv("ALSPARSE_AMD_SPMM_LDS");
    if (lds_env && atoi(lds_env) == 1) {
      static const bool attr_ok =
          hipFuncSetAttribute((const void*)spmm_rowblock_lds_kernel<T, true>, hipFuncAttributeMaxDynamicSharedMemorySize,
                              (int)LdsSpmm<T>::bytes) == hipSuccess &&
          hipFuncSetAttribute((const void*)spmm_rowblock_lds_kernel<T, false>, hipFuncAttributeMaxDynamicSharedMemorySize,
                              (int)LdsSpmm<T>::bytes) == hipSuccess;
      if (!attr_ok) return hipErrorInvalidValue;
      // persistent workgroups, as many as the compute units hold at once (the tile decides)
      const int runs_total = (int)(((int64_t)m + LdsSpmm<T>::run - 1) / LdsSpmm<T>::run);
      const unsigned gy = (unsigned)((n + kWave - 1) / kWave);
      static const int cus = [] {
        int dev = 0, c = 0;
        if (hipGetDevice(&dev) != hipSuccess ||
            hipDeviceGetAttribute(&c, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || c <= 0)
          c = 256;
        return c;
      }();
      // every workgroup must be resident at once: ask the runtime how many a compute unit holds
      static const int per_cu = [] {
        int nb = 0;
        if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&nb, spmm_rowblock_lds_kernel<T, true>, kSpmmBlock,
                                                         LdsSpmm<T>::bytes) != hipSuccess || nb < 1) {
          (void)hipGetLastError();
          nb = 1;
        }
        return nb;
      }();
      int64_t want = (int64_t)cus * per_cu / gy;
      if (want < 1) want = 1;
      const dim3 lgrid((unsigned)(want < runs_total ? want : runs_total), gy);
      // (C is written element by element where it cannot be addressed in 16-byte pieces; B decides the kernel)
      if (n % E == 0 && ldb % E == 0 && (uintptr_t)B % 16 == 0)
        spmm_rowblock_lds_kernel<T, true><<<lgrid, kSpmmBlock, LdsSpmm<T>::bytes, s>>>(
            m, n, alpha, val, rp, ci, base, B, ldb, beta, C, ldc, runs_total, aligned16);
      else
        spmm_rowblock_lds_kernel<T, false><<<lgrid, kSpmmBlock, LdsSpmm<T>::bytes, s>>>(
            m, n, alpha, val, rp, ci, base, B, ldb, beta, C, ldc, runs_total, false);
      return hipGetLastError();
    }
    // Four rows of B per wave instruction (needs rows that 128-bit loads can address), against one wave-wide load
    // per row of B.  Measured on 2^20 rows x 32 entries with random columns, n = 64: B of 4 / 16 / 32 MiB
    // 0.64 / 0.95 / 1.10 ms against 0.97 / 1.05 / 1.11; 64-256 MiB 1.18-1.23 against 1.17-1.22 (the L2-miss path is
    // the limit either way); 512 MiB 1.22 against 1.38; n = 256 (1 GiB) 4.95 against 5.46.  In between the sizes
    // that decide by themselves the structure does: where neighbouring rows of A share columns (a discretisation,
    // a band) the rows of B are found in L1 and four per instruction win (27-point stencil 128 x 128 x 64, B of
    // 256 MiB: 0.52 ms against 0.88).  A device-side probe looks; ALSPARSE_AMD_SPMM_QUAD = 0 / 1 decides instead.
    static const bool quad_off = getenv("ALSPARSE_AMD_SPMM_QUAD") && atoi(getenv("ALSPARSE_AMD_SPMM_QUAD")) == 0;
    static const bool quad_on = getenv("ALSPARSE_AMD_SPMM_QUAD") && atoi(getenv("ALSPARSE_AMD_SPMM_QUAD")) == 1;
    const size_t b_bytes = (size_t)(k > 0 ? k : 0) * (size_t)n * sizeof(T);
    const bool quad_can = !quad_off && aligned16;
    const bool quad_by_size = quad_on || k <= 0 || b_bytes <= ((size_t)48 << 20) || b_bytes > ((size_t)384 << 20);
    const int* gate = nullptr;  // the probe's verdict while it is not known on the host: both kernels are launched
    int shared = 0;
    if (quad_can && !quad_by_size) {
      ReuseSeen* record = nullptr;
      shared = reuse_lookup(s, rp, ci, m, nnz, &record);
      const bool probe_room = ws && ws_bytes >= sizeof(ProbeWords) && (uintptr_t)ws % alignof(ProbeWords) == 0;
      if (shared < 0 && probe_room) {
        ProbeWords* pw = (ProbeWords*)ws;
        spmm_probe_reset_kernel<<<1, 1, 0, s>>>(pw);
        spmm_reuse_probe_kernel<<<kProbeRows / kProbeRowsPerBlock, kSpmmBlock, 0, s>>>(m, rp, ci, base, pw);
        gate = &pw->verdict;
        if (record) reuse_record(s, record, gate);
      } else if (shared < 0) {
        shared = 0;  // nowhere to put the verdict
      }
    }
    if (quad_can && (quad_by_size || shared == 1 || gate)) {
      // persistent waves: as many workgroups as the chip holds at once (fewer for matrices with fewer rows)
      static const int quad_wgs = [] {
        int dev = 0, cus = 0, per_cu = 0;
        if (hipGetDevice(&dev) != hipSuccess ||
            hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus <= 0)
          cus = 256;
        if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, spmm_rowmajor_quad_kernel<T, true>, kSpmmBlock, 0) !=
                hipSuccess || per_cu < 1) {
          (void)hipGetLastError();
          per_cu = 4;
        }
        return cus * per_cu;
      }();
      const unsigned gyq = (unsigned)((n + 16 * E - 1) / (16 * E));
      unsigned gxq = (unsigned)quad_wgs / gyq;
      if (gxq < 1u) gxq = 1u;
      if (gxq > gx) gxq = gx;
      const dim3 grid(gxq, gyq);
      // B within 2 GiB (its row count known): 32-bit offsets into a buffer resource
      const unsigned __int128 span = (unsigned __int128)(k > 0 ? k : 0) * (unsigned __int128)ldb * sizeof(T);
      if (k > 0 && span < ((unsigned __int128)1 << 31))
        spmm_rowmajor_quad_kernel<T, true><<<grid, kSpmmBlock, 0, s>>>(m, n, alpha, val, rp, ci, base, B, ldb,
                                                                       (unsigned)span, beta, C, ldc, gate, 1);
      else
        spmm_rowmajor_quad_kernel<T, false><<<grid, kSpmmBlock, 0, s>>>(m, n, alpha, val, rp, ci, base, B, ldb, 0u,
                                                                        beta, C, ldc, gate, 1);
      if (!gate) return hipGetLastError();
    }
    // widest per-lane vector that still gives every lane of a wave work
    constexpr int kMaxV = 32 / (int)sizeof(T) >= 4 ? 4 : 32 / (int)sizeof(T);  // at most 32 bytes per lane and load
    int V = 1;
    if (n >= 4 * kWave && kMaxV >= 4) V = 4;
    else if (n >= 2 * kWave && kMaxV >= 2) V = 2;
    // A B too large for the 256 MiB memory-side cache is better taken 64 dense columns at a time
    // (grid.y runs slowest, so one slice of B is live at a time and stays cached): measured on a
    // 2^20 x 2^20 matrix with 32 entries per row, n = 128: 3.10 ms with V = 2, against 2 x 1.23 ms.
    if (k > 0 && (size_t)k * (size_t)n * sizeof(T) > ((size_t)192 << 20)) V = 1;
    const size_t vbytes = (size_t)V * sizeof(T);
    const bool vector_ok = V > 1 && ((uintptr_t)B % vbytes == 0) && ((uintptr_t)C % vbytes == 0) &&
                           (ldb % V == 0) && (ldc % V == 0);
    const unsigned gy = (unsigned)((n + kWave * V - 1) / (kWave * V));
    const dim3 grid(gx, gy);
    if constexpr (kMaxV >= 4) {
      if (V == 4) {
        spmm_rowmajor_kernel<T, 4><<<grid, kSpmmBlock, 0, s>>>(m, n, alpha, val, rp, ci, base, B, ldb,
                                                               beta, C, ldc, vector_ok, gate, 0);
        return hipGetLastError();
      }
    }
    if (V == 2)
      spmm_rowmajor_kernel<T, 2><<<grid, kSpmmBlock, 0, s>>>(m, n, alpha, val, rp, ci, base, B, ldb,
                                                             beta, C, ldc, vector_ok, gate, 0);
    else
      spmm_rowmajor_kernel<T, 1><<<grid, kSpmmBlock, 0, s>>>(m, n, alpha, val, rp, ci, base, B, ldb,
                                                             beta, C, ldc, false, gate, 0);
  } else {
    const dim3 block(kWave, kSpmmBlock / kWave);
    unsigned gy = (unsigned)((n + block.y - 1) / block.y);
    if (gy > 65535u) gy = 65535u;
    const dim3 grid((unsigned)(((int64_t)m + kWave - 1) / kWave), gy);
    spmm_strided_kernel<T><<<grid, block, 0, s>>>(m, n, alpha, val, rp, ci, base, B,
                                                  st->b_row_stride, st->b_col_stride, beta, C,
                                                  st->c_row_stride, st->c_col_stride);
  }
  return hipGetLastError();
}

extern "C" int asamd_s_csrmm(hipStream_t stream, int32_t m, int32_t n, int32_t k, int32_t nnz,
                             float alpha, const float* val, const int32_t* row_ptr,
                             const int32_t* col_ind, int32_t base, const float* B, float beta,
                             float* C, const asamd_dense_strides* strides) {
  return csrmm_impl<float>(stream, m, n, k, nnz, alpha, val, row_ptr, col_ind, base, B, beta, C,
                           strides, nullptr, 0);
}

extern "C" size_t asamd_csrmm_workspace_bytes(int32_t val_size, int32_t m, int32_t n, int32_t k,
                                              const asamd_dense_strides* strides) {
  (void)m;
  return (val_size == 4 || val_size == 8 || val_size == 16) ? workspace_bytes((size_t)val_size, n, k, strides) : 0;
}

extern "C" int asamd_s_csrmm_ws(hipStream_t stream, int32_t m, int32_t n, int32_t k, int32_t nnz, float alpha,
                                const float* val, const int32_t* row_ptr, const int32_t* col_ind, int32_t base,
                                const float* B, float beta, float* C, const asamd_dense_strides* strides,
                                void* workspace, size_t workspace_bytes) {
  return csrmm_impl<float>(stream, m, n, k, nnz, alpha, val, row_ptr, col_ind, base, B, beta, C, strides,
                           workspace, workspace_bytes);
}

extern "C" int asamd_d_csrmm_ws(hipStream_t stream, int32_t m, int32_t n, int32_t k, int32_t nnz, double alpha,
                                const double* val, const int32_t* row_ptr, const int32_t* col_ind, int32_t base,
                                const double* B, double beta, double* C, const asamd_dense_strides* strides,
                                void* workspace, size_t workspace_bytes) {
  return csrmm_impl<double>(stream, m, n, k, nnz, alpha, val, row_ptr, col_ind, base, B, beta, C, strides,
                            workspace, workspace_bytes);
}

extern "C" int asamd_d_csrmm(hipStream_t stream, int32_t m, int32_t n, int32_t k, int32_t nnz,
                             double alpha, const double* val, const int32_t* row_ptr,
                             const int32_t* col_ind, int32_t base, const double* B, double beta,
                             double* C, const asamd_dense_strides* strides) {
  return csrmm_impl<double>(stream, m, n, k, nnz, alpha, val, row_ptr, col_ind, base, B, beta, C,
                            strides, nullptr, 0);
}

// ---- the unanalysed, one-lane-per-element path ("plain"): entries of a row in storage order ---
template <typename T>
static int csrmm_plain_impl(hipStream_t s, int m, int n, T alpha, const T* val, const int* rp, const int* ci,
                            int base, const T* B, T beta, T* C, const asamd_dense_strides* st) {
  if (!val || !rp || !ci || !B || !C || !st || m <= 0 || n <= 0) return hipErrorInvalidValue;
  if (((uintptr_t)val | (uintptr_t)B | (uintptr_t)C) % alignof(T)) return hipErrorInvalidValue;
  const dim3 block(kWave, kSpmmBlock / kWave);
  unsigned gy = (unsigned)((n + block.y - 1) / block.y);
  if (gy > 65535u) gy = 65535u;
  const dim3 grid((unsigned)(((int64_t)m + kWave - 1) / kWave), gy);
  spmm_strided_kernel<T><<<grid, block, 0, s>>>(m, n, alpha, val, rp, ci, base, B, st->b_row_stride,
                                                st->b_col_stride, beta, C, st->c_row_stride, st->c_col_stride);
  return hipGetLastError();
}

extern "C" int asamd_s_csrmm_plain(hipStream_t stream, int32_t m, int32_t n, float alpha, const float* val,
                                   const int32_t* row_ptr, const int32_t* col_ind, int32_t base, const float* B,
                                   float beta, float* C, const asamd_dense_strides* strides) {
  return csrmm_plain_impl<float>(stream, m, n, alpha, val, row_ptr, col_ind, base, B, beta, C, strides);
}

extern "C" int asamd_d_csrmm_plain(hipStream_t stream, int32_t m, int32_t n, double alpha, const double* val,
                                   const int32_t* row_ptr, const int32_t* col_ind, int32_t base, const double* B,
                                   double beta, double* C, const asamd_dense_strides* strides) {
  return csrmm_plain_impl<double>(stream, m, n, alpha, val, row_ptr, col_ind, base, B, beta, C, strides);
}

extern "C" int asamd_c_csrmm_plain(hipStream_t stream, int32_t m, int32_t n, asamd_complex8 alpha,
                                   const asamd_complex8* val, const int32_t* row_ptr, const int32_t* col_ind,
                                   int32_t base, const asamd_complex8* B, asamd_complex8 beta, asamd_complex8* C,
                                   const asamd_dense_strides* strides) {
  using T = Cx<float>;
  return csrmm_plain_impl<T>(stream, m, n, T(alpha.real, alpha.imag), (const T*)val, row_ptr, col_ind, base,
                             (const T*)B, T(beta.real, beta.imag), (T*)C, strides);
}

extern "C" int asamd_z_csrmm_plain(hipStream_t stream, int32_t m, int32_t n, asamd_complex16 alpha,
                                   const asamd_complex16* val, const int32_t* row_ptr, const int32_t* col_ind,
                                   int32_t base, const asamd_complex16* B, asamd_complex16 beta, asamd_complex16* C,
                                   const asamd_dense_strides* strides) {
  using T = Cx<double>;
  return csrmm_plain_impl<T>(stream, m, n, T(alpha.real, alpha.imag), (const T*)val, row_ptr, col_ind, base,
                             (const T*)B, T(beta.real, beta.imag), (T*)C, strides);
}

// ---- complex element types: the same kernels over Cx<float> / Cx<double> -------------------
static_assert(sizeof(asamd_complex8) == sizeof(Cx<float>) && sizeof(asamd_complex16) == sizeof(Cx<double>),
              "complex layouts");

extern "C" int asamd_c_csrmm_ws(hipStream_t stream, int32_t m, int32_t n, int32_t k, int32_t nnz,
                                asamd_complex8 alpha, const asamd_complex8* val, const int32_t* row_ptr,
                                const int32_t* col_ind, int32_t base, const asamd_complex8* B, asamd_complex8 beta,
                                asamd_complex8* C, const asamd_dense_strides* strides, void* workspace,
                                size_t workspace_bytes) {
  using T = Cx<float>;
  return csrmm_impl<T>(stream, m, n, k, nnz, T(alpha.real, alpha.imag), (const T*)val, row_ptr, col_ind, base,
                       (const T*)B, T(beta.real, beta.imag), (T*)C, strides, workspace, workspace_bytes);
}

extern "C" int asamd_z_csrmm_ws(hipStream_t stream, int32_t m, int32_t n, int32_t k, int32_t nnz,
                                asamd_complex16 alpha, const asamd_complex16* val, const int32_t* row_ptr,
                                const int32_t* col_ind, int32_t base, const asamd_complex16* B,
                                asamd_complex16 beta, asamd_complex16* C, const asamd_dense_strides* strides,
                                void* workspace, size_t workspace_bytes) {
  using T = Cx<double>;
  return csrmm_impl<T>(stream, m, n, k, nnz, T(alpha.real, alpha.imag), (const T*)val, row_ptr, col_ind, base,
                       (const T*)B, T(beta.real, beta.imag), (T*)C, strides, workspace, workspace_bytes);
}
