// Plain memory kernels that measure what this GPU sustains, for the roofline statements of the SpMV /
// SpMM kernels: read-only, write-only and copy streams (16 bytes per lane and load, several loads in
// flight), random gathers of whole 256-byte rows (what a wave of the row-major SpMM does per entry of A)
// and random gathers of single 4-byte elements (what a lane of a row SpMV kernel does per entry).
// Diagnostics only; the reference has no counterpart.

#include <hip/hip_runtime.h>

#include "asamd_probes.h"
#include "../csrc/hip/device_utils.hpp"

using namespace asamd;

namespace {

constexpr int kCeilThreads = 256;
constexpr int kCeilUnroll = 8;

typedef int Int4v __attribute__((ext_vector_type(4)));

// Every workgroup streams one contiguous share of the buffer (a grid-stride loop, whose workgroups
// touch 4 KiB here and 4 KiB there, measured 5.8 instead of 6.2 TB/s reading and 4.2 instead of
// 6.3 TB/s writing); NT = non-temporal accesses (the lines are not kept in L2: 7.0 TB/s reading).
template <bool NT>
__global__ __launch_bounds__(kCeilThreads) void ceiling_read_kernel(const Int4v* __restrict__ p, size_t n,
                                                                    size_t per_block, int* __restrict__ sink) {
  const size_t b = (size_t)blockIdx.x * per_block, e = b + per_block < n ? b + per_block : n;
  int acc = 0;
  size_t i = b + threadIdx.x;
  for (; i + (kCeilUnroll - 1) * kCeilThreads < e; i += kCeilUnroll * kCeilThreads) {
    Int4v v[kCeilUnroll];
#pragma unroll
    for (int u = 0; u < kCeilUnroll; ++u)
      v[u] = NT ? __builtin_nontemporal_load(p + i + u * kCeilThreads) : p[i + u * kCeilThreads];
#pragma unroll
    for (int u = 0; u < kCeilUnroll; ++u) acc += v[u].x ^ v[u].y ^ v[u].z ^ v[u].w;
  }
  for (; i < e; i += kCeilThreads) {
    const Int4v v = p[i];
    acc += v.x ^ v.y ^ v.z ^ v.w;
  }
  if (acc == 0x12345678) sink[0] = acc;  // keeps the loads alive; practically never taken
}

__global__ __launch_bounds__(kCeilThreads) void ceiling_write_kernel(Int4v* __restrict__ p, size_t n, size_t per_block) {
  const size_t b = (size_t)blockIdx.x * per_block, e = b + per_block < n ? b + per_block : n;
  Int4v v;
  v.x = 1, v.y = 2, v.z = 3, v.w = 4;
  for (size_t i = b + threadIdx.x; i < e; i += kCeilThreads) p[i] = v;
}

template <bool NT>
__global__ __launch_bounds__(kCeilThreads) void ceiling_copy_kernel(Int4v* __restrict__ d, const Int4v* __restrict__ p,
                                                                    size_t n, size_t per_block) {
  constexpr int kU = 4;
  const size_t b = (size_t)blockIdx.x * per_block, e = b + per_block < n ? b + per_block : n;
  size_t i = b + threadIdx.x;
  for (; i + (kU - 1) * kCeilThreads < e; i += kU * kCeilThreads) {
    Int4v v[kU];
#pragma unroll
    for (int u = 0; u < kU; ++u) v[u] = NT ? __builtin_nontemporal_load(p + i + u * kCeilThreads) : p[i + u * kCeilThreads];
#pragma unroll
    for (int u = 0; u < kU; ++u) {
      if (NT) __builtin_nontemporal_store(v[u], d + i + u * kCeilThreads);
      else d[i + u * kCeilThreads] = v[u];
    }
  }
  for (; i < e; i += kCeilThreads) d[i] = p[i];
}

// a 64-bit mix (splitmix64's finaliser): row choice per (wave, step), the same on every lane of a wave
__device__ __forceinline__ uint64_t mix64(uint64_t z) {
  z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
  z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
  return z ^ (z >> 31);
}

// a position in [0, n) from the upper half of a mixed word (multiply-shift: no division)
__device__ __forceinline__ uint32_t pick(uint64_t z, uint32_t n) { return (uint32_t)(((z >> 32) * (uint64_t)n) >> 32); }

// Every wave reads `per_wave` rows of 64 floats (256 bytes: one float per lane) at uniformly random
// row positions among `rows`, eight rows in flight.
__global__ __launch_bounds__(kCeilThreads) void ceiling_row_gather_kernel(const float* __restrict__ p, uint32_t rows,
                                                                          int per_wave, float* __restrict__ sink) {
  const int lane = threadIdx.x % kWave;
  const uint64_t wave = (uint64_t)blockIdx.x * (kCeilThreads / kWave) + threadIdx.x / kWave;
  float acc = 0.f;
  for (int s = 0; s < per_wave; s += 8) {
    float v[8];
#pragma unroll
    for (int u = 0; u < 8; ++u) {
      const uint32_t r = pick(mix64(wave * 0x9E3779B97F4A7C15ull + (uint64_t)(s + u)), rows);
      v[u] = p[(size_t)r * kWave + lane];
    }
#pragma unroll
    for (int u = 0; u < 8; ++u) acc += v[u];
  }
  if (acc == 1.2345e-30f) sink[0] = acc;
}

// Every lane reads `per_lane` single floats at uniformly random positions among `elems`, eight in flight.
__global__ __launch_bounds__(kCeilThreads) void ceiling_elem_gather_kernel(const float* __restrict__ p, uint32_t elems,
                                                                           int per_lane, float* __restrict__ sink) {
  const uint64_t t = (uint64_t)blockIdx.x * kCeilThreads + threadIdx.x;
  float acc = 0.f;
  for (int s = 0; s < per_lane; s += 8) {
    float v[8];
#pragma unroll
    for (int u = 0; u < 8; ++u) v[u] = p[pick(mix64(t * 0x9E3779B97F4A7C15ull + (uint64_t)(s + u)), elems)];
#pragma unroll
    for (int u = 0; u < 8; ++u) acc += v[u];
  }
  if (acc == 1.2345e-30f) sink[0] = acc;
}

// A copy in runs of R floats (R a multiple of 4, 16 bytes per lane): run r of the one side is run
// (r * mult) mod nruns of the other (mult and nruns coprime), so one side streams and the other jumps
// from run to run.  A workgroup takes 128 consecutive runs at a time.
__global__ __launch_bounds__(1024) void ceiling_run_copy_kernel(const float* __restrict__ in, float* __restrict__ out,
                                                                long nruns, int R, bool scatter, long mult) {
  const long per_wg = 128;
  const int q = R / 4;
  for (long r0 = (long)blockIdx.x * per_wg; r0 < nruns; r0 += (long)gridDim.x * per_wg) {
    for (int i = threadIdx.x; i < per_wg * q; i += 1024) {
      const long r = r0 + i / q;
      if (r >= nruns) break;
      const int o = (i % q) * 4;
      const long pr = (r * mult) % nruns;
      const long src = (scatter ? r : pr) * R + o, dst = (scatter ? pr : r) * R + o;
      *reinterpret_cast<Int4v*>(out + dst) = *reinterpret_cast<const Int4v*>(in + src);
    }
  }
}
}  // namespace

extern "C" int asamd_ceiling_kernel(hipStream_t stream, int32_t kind, void* dst, const void* src, size_t nbytes,
                                    int64_t count, void* sink, int64_t* bytes_moved) {
  if (!sink || !bytes_moved || nbytes < 16 || (nbytes & 15u) || (((uintptr_t)dst | (uintptr_t)src) & 15u))
    return hipErrorInvalidValue;
  const size_t n16 = nbytes / 16;
  const size_t grid = 8192;  // workgroups of the streaming kernels, each with a contiguous share
  const size_t per_block = (n16 + grid - 1) / grid;
  switch (kind) {
    case ASAMD_CEILING_READ:
    case ASAMD_CEILING_READ_NT:
      if (!src) return hipErrorInvalidValue;
      if (kind == ASAMD_CEILING_READ_NT)
        ceiling_read_kernel<true><<<(unsigned)grid, kCeilThreads, 0, stream>>>((const Int4v*)src, n16, per_block, (int*)sink);
      else
        ceiling_read_kernel<false><<<(unsigned)grid, kCeilThreads, 0, stream>>>((const Int4v*)src, n16, per_block, (int*)sink);
      *bytes_moved = (int64_t)nbytes;
      break;
    case ASAMD_CEILING_WRITE:
      if (!dst) return hipErrorInvalidValue;
      ceiling_write_kernel<<<(unsigned)grid, kCeilThreads, 0, stream>>>((Int4v*)dst, n16, per_block);
      *bytes_moved = (int64_t)nbytes;
      break;
    case ASAMD_CEILING_COPY:
    case ASAMD_CEILING_COPY_NT:
      if (!src || !dst) return hipErrorInvalidValue;
      if (kind == ASAMD_CEILING_COPY_NT)
        ceiling_copy_kernel<true><<<(unsigned)grid, kCeilThreads, 0, stream>>>((Int4v*)dst, (const Int4v*)src, n16, per_block);
      else
        ceiling_copy_kernel<false><<<(unsigned)grid, kCeilThreads, 0, stream>>>((Int4v*)dst, (const Int4v*)src, n16, per_block);
      *bytes_moved = 2 * (int64_t)nbytes;
      break;
    case ASAMD_CEILING_ROW_GATHER: {
      // count = rows to fetch in total; the buffer holds nbytes / 256 rows
      const uint64_t rows = nbytes / 256;
      if (!src || rows == 0 || rows > 0xffffffffull || count < 8) return hipErrorInvalidValue;
      const int waves_per_block = kCeilThreads / kWave;
      const int64_t waves = 256 * 32 * waves_per_block;
      int per_wave = (int)((count + waves - 1) / waves);
      per_wave = (per_wave + 7) / 8 * 8;
      ceiling_row_gather_kernel<<<256 * 32, kCeilThreads, 0, stream>>>((const float*)src, (uint32_t)rows, per_wave,
                                                                        (float*)sink);
      *bytes_moved = waves * per_wave * 256;
      break;
    }
    case ASAMD_CEILING_ELEM_GATHER: {
      // count = elements to fetch in total; the buffer holds nbytes / 4 floats
      const uint64_t elems = nbytes / 4;
      if (!src || elems > 0xffffffffull || count < 8) return hipErrorInvalidValue;
      const int64_t lanes = (int64_t)256 * 32 * kCeilThreads;
      int per_lane = (int)((count + lanes - 1) / lanes);
      per_lane = (per_lane + 7) / 8 * 8;
      ceiling_elem_gather_kernel<<<256 * 32, kCeilThreads, 0, stream>>>((const float*)src, (uint32_t)elems, per_lane,
                                                                         (float*)sink);
      *bytes_moved = lanes * per_lane * 4;  // useful bytes; every gather moves a whole cache line behind them
      break;
    }
    case ASAMD_CEILING_RUN_GATHER:
    case ASAMD_CEILING_RUN_SCATTER: {
      if (!src || !dst || count < 4 || count % 4 != 0 || count > (1 << 20)) return hipErrorInvalidValue;
      const long nruns = (long)(nbytes / 4 / (size_t)count);
      if (nruns < 2) return hipErrorInvalidValue;
      long mult = 2654435761L % nruns;  // a multiplier that shares no factor with the number of runs
      if (mult < 2) mult = 1;
      auto gcd = [](long a, long b) { while (b) { const long t = a % b; a = b; b = t; } return a; };
      while (gcd(mult, nruns) != 1) ++mult;
      ceiling_run_copy_kernel<<<512, 1024, 0, stream>>>((const float*)src, (float*)dst, nruns, (int)count,
                                                        kind == ASAMD_CEILING_RUN_SCATTER, mult);
      *bytes_moved = 2 * nruns * count * 4;
      break;
    }
    default:
      return hipErrorInvalidValue;
  }
  return hipGetLastError();
}

// Plain copy of known size, to calibrate hardware byte counters against.
__global__ __launch_bounds__(256) void copy_bytes_kernel(Int4* __restrict__ dst, const Int4* __restrict__ src, size_t n16) {
  for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n16; i += (size_t)gridDim.x * blockDim.x)
    dst[i] = src[i];
}

extern "C" int asamd_copy_bytes(hipStream_t stream, void* dst, const void* src, size_t nbytes) {
  if (!dst || !src || (nbytes & 15u) || (((uintptr_t)dst | (uintptr_t)src) & 15u)) return hipErrorInvalidValue;
  const size_t n16 = nbytes / 16;
  if (n16 == 0) return hipSuccess;
  size_t grid = (n16 + 255) / 256;
  if (grid > 256 * 64) grid = 256 * 64;
  copy_bytes_kernel<<<(unsigned)grid, 256, 0, stream>>>((Int4*)dst, (const Int4*)src, n16);
  return hipGetLastError();
}
