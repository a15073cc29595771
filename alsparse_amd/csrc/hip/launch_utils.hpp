// Host-side helpers shared by the launcher files: element type tags <-> C++ types, the
// scalars and arrays of an asamd_spmv_args record in their element type.
#pragma once

#include <hip/hip_runtime.h>

#include <cstdint>
#include <initializer_list>
#include <type_traits>

#include "alsparse_amd_kernels.h"
#include "device_utils.hpp"

namespace asamd {

template <typename T> struct DtypeOf;
template <> struct DtypeOf<float> { static constexpr int value = ASAMD_DTYPE_FLOAT; };
template <> struct DtypeOf<double> { static constexpr int value = ASAMD_DTYPE_DOUBLE; };
template <> struct DtypeOf<Cx<float>> { static constexpr int value = ASAMD_DTYPE_FLOAT_COMPLEX; };
template <> struct DtypeOf<Cx<double>> { static constexpr int value = ASAMD_DTYPE_DOUBLE_COMPLEX; };
template <typename T>
constexpr bool kIsReal = std::is_floating_point<T>::value;

static_assert(sizeof(asamd_complex8) == sizeof(Cx<float>) && sizeof(asamd_complex16) == sizeof(Cx<double>),
              "complex layouts");

inline int dtype_size(int dtype) {
  static const int kSize[4] = {4, 8, 8, 16};
  return dtype >= 0 && dtype < 4 ? kSize[dtype] : 0;
}

// calls f with a null pointer of the element type: f's parameter type names T
template <typename F>
inline int by_dtype(int dtype, F&& f) {
  switch (dtype) {
    case ASAMD_DTYPE_FLOAT: return f((float*)nullptr);
    case ASAMD_DTYPE_DOUBLE: return f((double*)nullptr);
    case ASAMD_DTYPE_FLOAT_COMPLEX: return f((Cx<float>*)nullptr);
    case ASAMD_DTYPE_DOUBLE_COMPLEX: return f((Cx<double>*)nullptr);
    default: return (int)hipErrorInvalidValue;
  }
}

// host scalar behind a void pointer (the layouts of Cx<R> and ALPHA_Complex8 / 16 are the same)
template <typename T>
inline T scalar_of(const void* p) { return *reinterpret_cast<const T*>(p); }

// the arguments every launcher checks: pointers present, arrays aligned to the element
template <typename T>
inline bool args_ok(const asamd_spmv_args* a) {
  if (!a || !a->alpha || !a->beta || !a->val || !a->row_ptr || !a->col_ind || !a->x || !a->y) return false;
  if (a->dtype != DtypeOf<T>::value || a->m <= 0) return false;
  return (((uintptr_t)a->val | (uintptr_t)a->x | (uintptr_t)a->y) % alignof(T)) == 0;
}

inline int device_cus() {
  int dev = 0, cus = 0;
  if (hipGetDevice(&dev) != hipSuccess ||
      hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus <= 0)
    cus = 256;
  return cus;
}

inline void free_all(std::initializer_list<void*> ptrs) {
  for (void* d : ptrs)
    if (d) (void)hipFree(d);
}

}  // namespace asamd
