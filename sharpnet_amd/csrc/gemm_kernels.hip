// Defines the GEMM kernels of one group of kernel_list.hpp; the build compiles
// this file once per group with -DSNHIP_KERNEL_GROUP=<index>.
#include <hip/hip_runtime.h>

#include "kernel_list.hpp"

#ifndef SNHIP_KERNEL_GROUP
#error "build with -DSNHIP_KERNEL_GROUP=<group index>"
#endif

#define SNHIP_PASTE_(a, b) a##b
#define SNHIP_PASTE(a, b) SNHIP_PASTE_(a, b)

SNHIP_PASTE(SNHIP_KERNEL_GROUP_, SNHIP_KERNEL_GROUP)(SNHIP_DEFINE_KERNELS)
