/*
 * asamd_probes.h -- plain memory kernels for the benchmark: they measure what the GPU sustains (the
 * practical ceilings that the kernels' roofline figures are read against) and calibrate the hardware
 * byte counters.  Built into libasamd_probes.so beside the workload generators; not part of
 * libalpha_spblas.so and not needed by any user of the library.  No reference counterpart.
 */
#ifndef ALSPARSE_AMD_PROBES_H
#define ALSPARSE_AMD_PROBES_H

#ifndef __HIP_PLATFORM_AMD__
#define __HIP_PLATFORM_AMD__ 1
#endif
#include <hip/hip_runtime_api.h>
#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* Plain 16-byte-per-lane copy of nbytes (a multiple of 16, both pointers 16-byte
 * aligned).  Exists to calibrate hardware byte counters against a transfer of
 * known size; no reference counterpart. */
int asamd_copy_bytes(hipStream_t stream, void *dst, const void *src, size_t nbytes);

/* Plain memory kernels that measure what the GPU sustains (the practical ceilings that the kernels'
 * roofline figures are read against); no reference counterpart.  kind: READ / WRITE / COPY stream nbytes
 * (a multiple of 16; 16 bytes per lane and access) from src / into dst; ROW_GATHER fetches `count`
 * 256-byte rows at random positions of the nbytes at src, one wave per row (what the row-major SpMM does
 * per entry of A with 64 dense columns); ELEM_GATHER fetches `count` single floats at random positions
 * (what a row SpMV kernel does per entry); RUN_GATHER / RUN_SCATTER copy nbytes in runs of `count` floats
 * (a multiple of 4) whose order differs between source and destination: the runs are contiguous on the
 * write side and scattered on the read side (what the second phase of the tiled SpMV reads), or the other
 * way round.  sink: 4 device bytes that are practically never written.
 * *bytes_moved receives the useful bytes of the launch (copy: read + written). */
enum asamd_ceiling_kind {
  ASAMD_CEILING_READ = 0,
  ASAMD_CEILING_WRITE = 1,
  ASAMD_CEILING_COPY = 2,
  ASAMD_CEILING_ROW_GATHER = 3,
  ASAMD_CEILING_ELEM_GATHER = 4,
  ASAMD_CEILING_READ_NT = 5, /* the same streams with non-temporal accesses */
  ASAMD_CEILING_COPY_NT = 6,
  ASAMD_CEILING_RUN_GATHER = 7,
  ASAMD_CEILING_RUN_SCATTER = 8
};
int asamd_ceiling_kernel(hipStream_t stream, int32_t kind, void *dst, const void *src, size_t nbytes,
                         int64_t count, void *sink, int64_t *bytes_moved);

#ifdef __cplusplus
}
#endif

#endif /* ALSPARSE_AMD_PROBES_H */
