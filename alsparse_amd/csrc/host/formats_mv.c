/* Device SpMV entry points for COO and ELL operands (raw device arrays). */
#include "internal.h"

#define ASAMD_T float
#define ASAMD_S s
#define ASAMD_KERNEL_COOMV asamd_s_coomv
#define ASAMD_KERNEL_ELLMV asamd_s_ellmv
#include "formats_mv.inc"
#undef ASAMD_T
#undef ASAMD_S
#undef ASAMD_KERNEL_COOMV
#undef ASAMD_KERNEL_ELLMV

#define ASAMD_T double
#define ASAMD_S d
#define ASAMD_KERNEL_COOMV asamd_d_coomv
#define ASAMD_KERNEL_ELLMV asamd_d_ellmv
#include "formats_mv.inc"
#undef ASAMD_T
#undef ASAMD_S
#undef ASAMD_KERNEL_COOMV
#undef ASAMD_KERNEL_ELLMV

#define ASAMD_T ALPHA_Complex8
#define ASAMD_S c
#define ASAMD_KERNEL_COOMV asamd_c_coomv
#define ASAMD_KERNEL_ELLMV asamd_c_ellmv
#include "formats_mv.inc"
#undef ASAMD_T
#undef ASAMD_S
#undef ASAMD_KERNEL_COOMV
#undef ASAMD_KERNEL_ELLMV

#define ASAMD_T ALPHA_Complex16
#define ASAMD_S z
#define ASAMD_KERNEL_COOMV asamd_z_coomv
#define ASAMD_KERNEL_ELLMV asamd_z_ellmv
#include "formats_mv.inc"
#undef ASAMD_T
#undef ASAMD_S
#undef ASAMD_KERNEL_COOMV
#undef ASAMD_KERNEL_ELLMV
