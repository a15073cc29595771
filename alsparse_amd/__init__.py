"""MI355X-native CSR SpMV / SpMM behind AlphaSparse's C API.

The product is ``alsparse_amd/lib/libalpha_spblas.so`` (C host library over
hand-written HIP kernels for gfx950).  This package only holds what tests,
the benchmark and Python users need to drive it:

* :mod:`alsparse_amd.capi`       ctypes bindings of the C API, names as in the reference
* :mod:`alsparse_amd.hiprt`      minimal HIP runtime bindings for device buffers and events
* :mod:`alsparse_amd.workloads`  seeded synthetic matrices (the five benchmark shapes)
* :mod:`alsparse_amd.build`      build recipe (hipcc / gcc)
"""

__all__ = ["capi", "hiprt", "workloads", "build"]
