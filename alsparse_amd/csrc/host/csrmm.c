/* Device SpMM entry points (raw device arrays). */
#include "internal.h"

#define ASAMD_T float
#define ASAMD_S s
#define ASAMD_KERNEL_CSRMM asamd_s_csrmm_ws
#include "csrmm.inc"
#undef ASAMD_T
#undef ASAMD_S
#undef ASAMD_KERNEL_CSRMM

#define ASAMD_T double
#define ASAMD_S d
#define ASAMD_KERNEL_CSRMM asamd_d_csrmm_ws
#include "csrmm.inc"
#undef ASAMD_T
#undef ASAMD_S
#undef ASAMD_KERNEL_CSRMM

#define ASAMD_T ALPHA_Complex8
#define ASAMD_S c
#define ASAMD_KERNEL_CSRMM asamd_c_csrmm_ws
#include "csrmm.inc"
#undef ASAMD_T
#undef ASAMD_S
#undef ASAMD_KERNEL_CSRMM

#define ASAMD_T ALPHA_Complex16
#define ASAMD_S z
#define ASAMD_KERNEL_CSRMM asamd_z_csrmm_ws
#include "csrmm.inc"
#undef ASAMD_T
#undef ASAMD_S
#undef ASAMD_KERNEL_CSRMM
