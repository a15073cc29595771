// Device-side helpers shared by the gfx950 kernels: wave64 lane-group
// reductions through DPP, XCD-aware workgroup remapping, fused multiply-add
// wrappers.  Stands in for the reference's wave reductions
// (include/alphasparse/common_dcu.h:33-164), written for CDNA4's 64-lane waves.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace asamd {

constexpr int kWave = 64;
constexpr int kXcds = 8;  // MI355X: 8 accelerator complex dies, one L2 each

// Workgroups are handed to the XCDs round-robin (workgroup i runs on XCD
// i % 8).  Kernels whose neighbouring workgroups share gathered operands want
// neighbours on the SAME XCD so the shared lines sit in one L2: this maps the
// hardware workgroup id to a logical id such that every XCD walks one
// contiguous slab of logical ids.
__device__ __forceinline__ unsigned xcd_contiguous_id(unsigned hw_id, unsigned nblocks) {
  const unsigned per = nblocks / kXcds;
  const unsigned rem = nblocks % kXcds;
  const unsigned xcd = hw_id % kXcds;
  const unsigned local = hw_id / kXcds;
  const unsigned start = xcd * per + (xcd < rem ? xcd : rem);
  return start + local;
}

__device__ __forceinline__ float fma_t(float a, float b, float c) { return __builtin_fmaf(a, b, c); }
__device__ __forceinline__ double fma_t(double a, double b, double c) { return __builtin_fma(a, b, c); }

// single operations that the compiler may not contract into fused multiply-adds
// (the pragma takes the `contract` flag off the operation itself, so it stays
// unfused wherever the function is inlined)
template <typename R>
__device__ __forceinline__ R mul_rn(R a, R b) {
#pragma clang fp contract(off)
  return a * b;
}
template <typename R>
__device__ __forceinline__ R add_rn(R a, R b) {
#pragma clang fp contract(off)
  return a + b;
}

// ---- complex scalars ---------------------------------------------------------
// Cx<float> / Cx<double> have the memory layout of the reference's
// ALPHA_Complex8 / ALPHA_Complex16 ({real, imag}, include/alphasparse/types.h:42-56).
// Device arrays of them are assumed aligned to the element size (the entry
// points check), so one element is one 64- or 128-bit load.
//   a * b      the four-multiplication form, every operation rounded on its own,
//              as the reference's cmp_mul (include/alphasparse/complex_compute.h:76-82)
//   fma_t      c + a*b with the fused chain of the reference's device cmp_madde
//              (complex_compute.h:139-146)
template <typename R>
struct alignas(2 * sizeof(R)) Cx {
  R re, im;
  Cx() = default;
  __host__ __device__ constexpr Cx(R r, R i = R(0)) : re(r), im(i) {}
  __device__ __forceinline__ Cx& operator+=(const Cx& o) {
    re += o.re;
    im += o.im;
    return *this;
  }
};
template <typename R>
__device__ __forceinline__ Cx<R> operator+(Cx<R> a, Cx<R> b) { return Cx<R>(add_rn(a.re, b.re), add_rn(a.im, b.im)); }
template <typename R>
__device__ __forceinline__ Cx<R> operator*(Cx<R> a, Cx<R> b) {
  return Cx<R>(add_rn(mul_rn(a.re, b.re), -mul_rn(a.im, b.im)), add_rn(mul_rn(a.im, b.re), mul_rn(a.re, b.im)));
}
template <typename R>
__host__ __device__ __forceinline__ bool operator==(Cx<R> a, Cx<R> b) { return a.re == b.re && a.im == b.im; }
template <typename R>
__host__ __device__ __forceinline__ bool operator!=(Cx<R> a, Cx<R> b) { return !(a == b); }
template <typename R>
__device__ __forceinline__ Cx<R> fma_t(Cx<R> a, Cx<R> b, Cx<R> c) {
  return Cx<R>(fma_t(-a.im, b.im, fma_t(a.re, b.re, c.re)), fma_t(a.re, b.im, fma_t(a.im, b.re, c.im)));
}
__device__ __forceinline__ float conj_t(float a) { return a; }
__device__ __forceinline__ double conj_t(double a) { return a; }
template <typename R>
__device__ __forceinline__ Cx<R> conj_t(Cx<R> a) { return Cx<R>(a.re, -a.im); }

// ---- wave shuffles, streaming loads / stores and atomic adds for every scalar type
template <typename T>
__device__ __forceinline__ T lane_up(T v, unsigned d) { return __shfl_up(v, d, kWave); }
template <typename T>
__device__ __forceinline__ T lane_down(T v, unsigned d) { return __shfl_down(v, d, kWave); }
template <typename T>
__device__ __forceinline__ T lane_xor(T v, int mask) { return __shfl_xor(v, mask, kWave); }
template <typename T>
__device__ __forceinline__ T lane_get(T v, int src) { return __shfl(v, src, kWave); }
template <typename R>
__device__ __forceinline__ Cx<R> lane_up(Cx<R> v, unsigned d) { return Cx<R>(lane_up(v.re, d), lane_up(v.im, d)); }
template <typename R>
__device__ __forceinline__ Cx<R> lane_down(Cx<R> v, unsigned d) { return Cx<R>(lane_down(v.re, d), lane_down(v.im, d)); }
template <typename R>
__device__ __forceinline__ Cx<R> lane_xor(Cx<R> v, int mask) { return Cx<R>(lane_xor(v.re, mask), lane_xor(v.im, mask)); }
template <typename R>
__device__ __forceinline__ Cx<R> lane_get(Cx<R> v, int src) { return Cx<R>(lane_get(v.re, src), lane_get(v.im, src)); }

template <typename T>
__device__ __forceinline__ T nt_load(const T* p) { return __builtin_nontemporal_load(p); }
template <typename T>
__device__ __forceinline__ void nt_store(T v, T* p) { __builtin_nontemporal_store(v, p); }
template <typename R>
__device__ __forceinline__ Cx<R> nt_load(const Cx<R>* p) {
  typedef R Pair __attribute__((ext_vector_type(2)));
  const Pair v = __builtin_nontemporal_load(reinterpret_cast<const Pair*>(p));
  return Cx<R>(v.x, v.y);
}
template <typename R>
__device__ __forceinline__ void nt_store(Cx<R> v, Cx<R>* p) {
  typedef R Pair __attribute__((ext_vector_type(2)));
  Pair q;
  q.x = v.re;
  q.y = v.im;
  __builtin_nontemporal_store(q, reinterpret_cast<Pair*>(p));
}

template <typename T>
__device__ __forceinline__ void atomic_add(T* p, T v) { atomicAdd(p, v); }
// the two halves of a complex sum are independent additions
template <typename R>
__device__ __forceinline__ void atomic_add(Cx<R>* p, Cx<R> v) {
  atomicAdd(&p->re, v.re);
  atomicAdd(&p->im, v.im);
}

// y <- beta*y + alpha*sum with the reference's rounding points: both products
// are rounded separately and then added, never contracted into an fma
// (src/kernel/dcu/level2/mv/csrmv/dcu_gemv_vector.h:50-54 and
// src/plain/kernel/level2/mv/gemv/gemv_x_csr_plain.c:14,21 agree on this).
// beta == 0 does not read y at all.
__device__ __forceinline__ float axpby_rn(float alpha, float sum, float beta, float yold) {
  return add_rn(mul_rn(yold, beta), mul_rn(alpha, sum));
}
__device__ __forceinline__ double axpby_rn(double alpha, double sum, double beta, double yold) {
  return add_rn(mul_rn(yold, beta), mul_rn(alpha, sum));
}
template <typename R>
__device__ __forceinline__ Cx<R> axpby_rn(Cx<R> alpha, Cx<R> sum, Cx<R> beta, Cx<R> yold) {
  return yold * beta + alpha * sum;  // operator* rounds every operation on its own
}
template <typename T>
__device__ __forceinline__ void store_axpby(T* __restrict__ y, int64_t row, T alpha, T sum, T beta) {
  if (beta == T(0)) {
    y[row] = alpha * sum;
  } else {
    y[row] = axpby_rn(alpha, sum, beta, y[row]);
  }
}

// A non-temporal load of an aligned trivially copyable object of 4, 8, 16 or 32 bytes (the streams are touched
// once: they should not push x out of the caches).
template <typename P>
__device__ __forceinline__ P nt_load_object(const P* p) {
  typedef int V2 __attribute__((ext_vector_type(2)));
  typedef int V4 __attribute__((ext_vector_type(4)));
  static_assert(sizeof(P) == 4 || sizeof(P) == 8 || sizeof(P) == 16 || sizeof(P) == 32, "object size");
  if constexpr (sizeof(P) == 4) {
    return __builtin_bit_cast(P, __builtin_nontemporal_load(reinterpret_cast<const int*>(p)));
  } else if constexpr (sizeof(P) == 8) {
    return __builtin_bit_cast(P, __builtin_nontemporal_load(reinterpret_cast<const V2*>(p)));
  } else if constexpr (sizeof(P) == 16) {
    return __builtin_bit_cast(P, __builtin_nontemporal_load(reinterpret_cast<const V4*>(p)));
  } else {
    struct Two {
      V4 a, b;
    } t;
    t.a = __builtin_nontemporal_load(reinterpret_cast<const V4*>(p));
    t.b = __builtin_nontemporal_load(reinterpret_cast<const V4*>(p) + 1);
    return __builtin_bit_cast(P, t);
  }
}

// The same with non-temporal accesses to y: for kernels whose other streams should keep the caches
template <typename T>
__device__ __forceinline__ void store_axpby_nt(T* __restrict__ y, int64_t row, T alpha, T sum, T beta) {
  if (beta == T(0)) {
    nt_store(alpha * sum, y + row);
  } else {
    nt_store(axpby_rn(alpha, sum, beta, nt_load(y + row)), y + row);
  }
}

// ---- DPP moves ------------------------------------------------------------
// dpp_ctrl encodings (GCN3+/CDNA ISA): quad_perm = 0x00..0xFF, row_shr:n =
// 0x110+n, row_ror:n = 0x120+n, row_mirror = 0x140, row_half_mirror = 0x141.
template <int Ctrl>
__device__ __forceinline__ float dpp_mov(float v) {
  return __builtin_bit_cast(
      float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), Ctrl, 0xF, 0xF, true));
}
template <int Ctrl>
__device__ __forceinline__ double dpp_mov(double v) {
  // a 64-bit value travels as two 32-bit halves
  const uint64_t bits = __builtin_bit_cast(uint64_t, v);
  const int lo = __builtin_amdgcn_update_dpp(0, (int)(uint32_t)bits, Ctrl, 0xF, 0xF, true);
  const int hi = __builtin_amdgcn_update_dpp(0, (int)(uint32_t)(bits >> 32), Ctrl, 0xF, 0xF, true);
  return __builtin_bit_cast(double, ((uint64_t)(uint32_t)hi << 32) | (uint64_t)(uint32_t)lo);
}

// Sum over aligned groups of W consecutive lanes (W a power of two, 1..64).
// Every lane of the group ends up holding the group's total.  Up to 16 lanes
// the exchange is pure DPP (quad permutes, then the half-row and row mirrors:
// after the quad steps all four lanes of a quad hold the quad's total, so a
// mirror hands each lane the total of the opposite half); the 32- and
// 64-lane steps cross DPP rows and use the LDS crossbar (ds_bpermute through
// __shfl_xor), which touches no LDS memory.
template <int Ctrl, typename R>
__device__ __forceinline__ Cx<R> dpp_mov(Cx<R> v) {
  return Cx<R>(dpp_mov<Ctrl>(v.re), dpp_mov<Ctrl>(v.im));
}

// The same move restricted to the 16-lane rows named in RowMask (bit r = row r); lanes of the
// other rows, and lanes whose source does not exist, receive zero.
template <int Ctrl, int RowMask>
__device__ __forceinline__ int dpp_mov_rows(int v) {
  return __builtin_amdgcn_update_dpp(0, v, Ctrl, RowMask, 0xF, true);
}
template <int Ctrl, int RowMask>
__device__ __forceinline__ float dpp_mov_rows(float v) {
  return __builtin_bit_cast(float, dpp_mov_rows<Ctrl, RowMask>(__builtin_bit_cast(int, v)));
}
template <int Ctrl, int RowMask>
__device__ __forceinline__ double dpp_mov_rows(double v) {
  const uint64_t bits = __builtin_bit_cast(uint64_t, v);
  const int lo = dpp_mov_rows<Ctrl, RowMask>((int)(uint32_t)bits);
  const int hi = dpp_mov_rows<Ctrl, RowMask>((int)(uint32_t)(bits >> 32));
  return __builtin_bit_cast(double, ((uint64_t)(uint32_t)hi << 32) | (uint64_t)(uint32_t)lo);
}
template <int Ctrl, int RowMask, typename R>
__device__ __forceinline__ Cx<R> dpp_mov_rows(Cx<R> v) {
  return Cx<R>(dpp_mov_rows<Ctrl, RowMask>(v.re), dpp_mov_rows<Ctrl, RowMask>(v.im));
}

// value of the given lane, the same in every lane (v_readlane: no LDS crossbar)
__device__ __forceinline__ int lane_bcast(int v, int src) { return __builtin_amdgcn_readlane(v, src); }
__device__ __forceinline__ float lane_bcast(float v, int src) {
  return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), src));
}
__device__ __forceinline__ double lane_bcast(double v, int src) {
  const uint64_t b = __builtin_bit_cast(uint64_t, v);
  const uint32_t lo = (uint32_t)__builtin_amdgcn_readlane((int)(uint32_t)b, src);
  const uint32_t hi = (uint32_t)__builtin_amdgcn_readlane((int)(uint32_t)(b >> 32), src);
  return __builtin_bit_cast(double, ((uint64_t)hi << 32) | lo);
}
template <typename R>
__device__ __forceinline__ Cx<R> lane_bcast(Cx<R> v, int src) {
  return Cx<R>(lane_bcast(v.re, src), lane_bcast(v.im, src));
}

// Inclusive segmented sum over the 64 lanes of a wave: on return v holds the sum of the lane's
// segment up to and including the lane; `head` marks the first lane of every segment (lane 0 is
// one).  Pure DPP: shifts by 1, 2, 4, 8 inside the 16-lane rows, then lane 15 of rows 0 / 2
// broadcast into rows 1 / 3 and lane 31 into rows 2 and 3 -- the steps of a wave prefix sum, each
// taken only by lanes that have not yet seen the head of their segment.
template <typename T>
__device__ __forceinline__ T segmented_scan(T v, bool head) {
  int f = head;
#define ASAMD_SCAN_STEP(CTRL, ROWS)                      \
  {                                                      \
    const T vd = dpp_mov_rows<CTRL, ROWS>(v);            \
    const int fd = dpp_mov_rows<CTRL, ROWS>(f);          \
    if (!f) {                                            \
      v += vd;                                           \
      f = fd;                                            \
    }                                                    \
  }
  ASAMD_SCAN_STEP(0x111, 0xF)  // row_shr:1
  ASAMD_SCAN_STEP(0x112, 0xF)  // row_shr:2
  ASAMD_SCAN_STEP(0x114, 0xF)  // row_shr:4
  ASAMD_SCAN_STEP(0x118, 0xF)  // row_shr:8
  ASAMD_SCAN_STEP(0x142, 0xA)  // row_bcast:15 into rows 1 and 3
  ASAMD_SCAN_STEP(0x143, 0xC)  // row_bcast:31 into rows 2 and 3
#undef ASAMD_SCAN_STEP
  return v;
}

// v(l) + v(l ^ HALF) for HALF = 16 or 32, without the LDS crossbar that a shuffle goes through:
// v_permlane16_swap / v_permlane32_swap exchange the odd 16-lane rows (the upper 32 lanes) of one register with
// the even rows (the lower 32 lanes) of another, so two copies of v become "the even partner's" and "the odd
// partner's" value in every lane.  (Two idle states in front: the hardware wants them between a write of the
// registers and the swap, and the compiler does not look into the statement.)
template <int HALF, typename T>
__device__ __forceinline__ T sum_with_lane_xor(T v) {
  static_assert(HALF == 16 || HALF == 32, "rows or halves");
  static_assert(sizeof(T) % 4 == 0, "whole words");
  struct Words { int w[sizeof(T) / 4]; };
  Words a = __builtin_bit_cast(Words, v), b = a;
#pragma unroll
  for (int i = 0; i < (int)(sizeof(T) / 4); ++i) {
    if constexpr (HALF == 16)
      asm("s_nop 1\n\tv_permlane16_swap_b32 %0, %1" : "+v"(a.w[i]), "+v"(b.w[i]));
    else
      asm("s_nop 1\n\tv_permlane32_swap_b32 %0, %1" : "+v"(a.w[i]), "+v"(b.w[i]));
  }
  return __builtin_bit_cast(T, a) + __builtin_bit_cast(T, b);
}

template <int W, typename T>
__device__ __forceinline__ T group_sum(T v) {
  static_assert(W >= 1 && W <= 64 && (W & (W - 1)) == 0, "group width");
  if constexpr (W >= 2) v += dpp_mov<0xB1>(v);   // quad_perm [1,0,3,2]
  if constexpr (W >= 4) v += dpp_mov<0x4E>(v);   // quad_perm [2,3,0,1]
  if constexpr (W >= 8) v += dpp_mov<0x141>(v);  // row_half_mirror: lane l <-> 7-l in each 8
  if constexpr (W >= 16) v += dpp_mov<0x140>(v); // row_mirror: lane l <-> 15-l in each 16
  if constexpr (W >= 32) v = sum_with_lane_xor<16>(v);
  if constexpr (W >= 64) v = sum_with_lane_xor<32>(v);
  return v;
}

// ---- buffer loads with the hardware's range check ------------------------------
// A raw buffer resource over [p, p + bytes): loads at byte offsets >= bytes return zero and touch
// no memory.  0x00020000 is the 32-bit data format word of gfx9 resources.
using BufferRsrc = __amdgpu_buffer_rsrc_t;
__device__ __forceinline__ BufferRsrc make_rsrc(const void* p, int bytes) {
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(p), 0, bytes, 0x00020000);
}
__device__ __forceinline__ int buffer_load_u16(BufferRsrc r, int byte_offset) {
  return (int)(unsigned short)__builtin_amdgcn_raw_buffer_load_b16(r, byte_offset, 0, 0);
}
// AUX: the instruction's cache policy bits (0: default, 2: non-temporal)
template <typename T, int AUX = 0>
__device__ __forceinline__ T buffer_load(BufferRsrc r, int byte_offset) {
  if constexpr (sizeof(T) == 4) {
    return __builtin_bit_cast(T, __builtin_amdgcn_raw_buffer_load_b32(r, byte_offset, 0, AUX));
  } else if constexpr (sizeof(T) == 8) {
    return __builtin_bit_cast(T, __builtin_amdgcn_raw_buffer_load_b64(r, byte_offset, 0, AUX));
  } else {
    static_assert(sizeof(T) == 16, "element size");
    return __builtin_bit_cast(T, __builtin_amdgcn_raw_buffer_load_b128(r, byte_offset, 0, AUX));
  }
}

// ---- 128-bit streaming loads ------------------------------------------------
struct alignas(16) Int4 { int x, y, z, w; };
struct alignas(16) Float4 { float x, y, z, w; };
struct alignas(16) Double2 { double x, y; };

// ---- four values at a time --------------------------------------------------
// Which of a kernel's two matrix streams is loaded non-temporally (a kernel argument, the same for all lanes).
// The 256 MB memory-side cache keeps what is loaded plainly from one multiply to the next: the host marks as
// non-temporal what would push the rest out of it (stream_policy in the plan).
constexpr int kStreamNtValues = 1;
constexpr int kStreamNtIndices = 2;

// four consecutive values: 128-bit pieces for the real types, one load per value otherwise
template <typename T>
struct Quad {
  T e[4];
  __device__ __forceinline__ void load(const T* p) {
#pragma unroll
    for (int i = 0; i < 4; ++i) e[i] = p[i];
  }
  __device__ __forceinline__ void load_nt(const T* p) {
#pragma unroll
    for (int i = 0; i < 4; ++i) e[i] = nt_load(p + i);
  }
  __device__ __forceinline__ T get(int i) const { return e[i]; }
};
template <>
struct Quad<float> {
  Float4 q;
  __device__ __forceinline__ void load(const float* p) { q = *reinterpret_cast<const Float4*>(p); }
  __device__ __forceinline__ void load_nt(const float* p) { q = nt_load_object(reinterpret_cast<const Float4*>(p)); }
  __device__ __forceinline__ float get(int i) const { return i == 0 ? q.x : i == 1 ? q.y : i == 2 ? q.z : q.w; }
};
template <>
struct Quad<double> {
  Double2 a, b;
  __device__ __forceinline__ void load(const double* p) {
    a = *reinterpret_cast<const Double2*>(p);
    b = *reinterpret_cast<const Double2*>(p + 2);
  }
  __device__ __forceinline__ void load_nt(const double* p) {
    a = nt_load_object(reinterpret_cast<const Double2*>(p));
    b = nt_load_object(reinterpret_cast<const Double2*>(p + 2));
  }
  __device__ __forceinline__ double get(int i) const { return i == 0 ? a.x : i == 1 ? a.y : i == 2 ? b.x : b.y; }
};


}  // namespace asamd
