// The GEMM kernel instantiations of this library, as one list shared by the
// dispatch table (sharpnet_hip.hip, which only declares them) and the
// translation unit that defines them (gemm_kernels.hip, compiled once per group
// so that the groups build in parallel).
//
// X(KIND, TM, TN, WM, WN, BK): KIND S = fp32 kernel (sgemm_mfma.hpp), B =
// bf16-input kernel (bgemm_mfma.hpp) on fp32 storage, H = the same kernel on
// operands stored as bf16; a wavefront owns TM x TN MFMA tiles of
// 32 x 32, a workgroup is WM x WN wavefronts, BK is the k extent of an LDS stage.
#pragma once
#include "bgemm_mfma.hpp"
#include "sgemm_mfma.hpp"

#define SNHIP_KERNEL_GROUP_0(X) X(S, 4, 4, 2, 2, 16)
#define SNHIP_KERNEL_GROUP_1(X) X(S, 2, 4, 2, 2, 16)
#define SNHIP_KERNEL_GROUP_2(X) X(S, 4, 2, 2, 2, 16)
#define SNHIP_KERNEL_GROUP_3(X) X(S, 2, 2, 2, 2, 16) X(S, 2, 2, 2, 2, 32)
#define SNHIP_KERNEL_GROUP_4(X) X(S, 1, 2, 2, 2, 16) X(S, 2, 1, 2, 2, 16) X(S, 2, 1, 2, 2, 32)
#define SNHIP_KERNEL_GROUP_5(X) X(S, 1, 1, 2, 2, 16) X(S, 1, 1, 2, 2, 32)
#define SNHIP_KERNEL_GROUP_6(X) X(B, 4, 4, 2, 2, 32)
#define SNHIP_KERNEL_GROUP_7(X) X(B, 2, 2, 2, 2, 32) X(B, 2, 1, 2, 2, 64) X(B, 1, 1, 2, 2, 64)
#define SNHIP_KERNEL_GROUP_8(X) X(H, 4, 4, 2, 2, 64)
#define SNHIP_KERNEL_GROUP_9(X) X(H, 2, 2, 2, 2, 64) X(H, 1, 1, 2, 2, 128)
#define SNHIP_NUM_KERNEL_GROUPS 10

#define SNHIP_ALL_KERNEL_GROUPS(X)                                                                  \
    SNHIP_KERNEL_GROUP_0(X) SNHIP_KERNEL_GROUP_1(X) SNHIP_KERNEL_GROUP_2(X) SNHIP_KERNEL_GROUP_3(X) \
    SNHIP_KERNEL_GROUP_4(X) SNHIP_KERNEL_GROUP_5(X) SNHIP_KERNEL_GROUP_6(X) SNHIP_KERNEL_GROUP_7(X) \
    SNHIP_KERNEL_GROUP_8(X) SNHIP_KERNEL_GROUP_9(X)

// every variant of one configuration; PREFIX is `extern` for a declaration, empty for the definition
#define SNHIP_VARIANTS_S(PREFIX, TM, TN, WM, WN, BK)                    \
    SNHIP_VARIANTS_S_(PREFIX, TM, TN, WM, WN, BK, false)                \
    SNHIP_VARIANTS_S_(PREFIX, TM, TN, WM, WN, BK, true)
#define SNHIP_VARIANTS_S_(PREFIX, TM, TN, WM, WN, BK, EXT)                                                          \
    PREFIX template __global__ void snhip::sgemm_mfma_kernel<snhip::TileCfg<TM, TN, WM, WN, BK>, false, false, EXT>( \
        const snhip::GemmParams);                                                                                    \
    PREFIX template __global__ void snhip::sgemm_mfma_kernel<snhip::TileCfg<TM, TN, WM, WN, BK>, false, true, EXT>(  \
        const snhip::GemmParams);                                                                                    \
    PREFIX template __global__ void snhip::sgemm_mfma_kernel<snhip::TileCfg<TM, TN, WM, WN, BK>, true, false, EXT>(  \
        const snhip::GemmParams);                                                                                    \
    PREFIX template __global__ void snhip::sgemm_mfma_kernel<snhip::TileCfg<TM, TN, WM, WN, BK>, true, true, EXT>(   \
        const snhip::GemmParams);

#define SNHIP_VARIANTS_B(PREFIX, TM, TN, WM, WN, BK)                                                             \
    PREFIX template __global__ void snhip::bgemm_mfma_kernel<snhip::BTileCfg<TM, TN, WM, WN, BK>, false, false>( \
        const snhip::GemmParams);                                                                                \
    PREFIX template __global__ void snhip::bgemm_mfma_kernel<snhip::BTileCfg<TM, TN, WM, WN, BK>, false, true>(  \
        const snhip::GemmParams);                                                                                \
    PREFIX template __global__ void snhip::bgemm_mfma_kernel<snhip::BTileCfg<TM, TN, WM, WN, BK>, true, false>(  \
        const snhip::GemmParams);                                                                                \
    PREFIX template __global__ void snhip::bgemm_mfma_kernel<snhip::BTileCfg<TM, TN, WM, WN, BK>, true, true>(   \
        const snhip::GemmParams);

#define SNHIP_VARIANTS_H(PREFIX, TM, TN, WM, WN, BK)                                                                     \
    PREFIX template __global__ void snhip::bgemm_mfma_kernel<snhip::BTileCfg<TM, TN, WM, WN, BK>, false, false, __bf16>( \
        const snhip::GemmParams);                                                                                        \
    PREFIX template __global__ void snhip::bgemm_mfma_kernel<snhip::BTileCfg<TM, TN, WM, WN, BK>, false, true, __bf16>(  \
        const snhip::GemmParams);                                                                                        \
    PREFIX template __global__ void snhip::bgemm_mfma_kernel<snhip::BTileCfg<TM, TN, WM, WN, BK>, true, false, __bf16>(  \
        const snhip::GemmParams);                                                                                        \
    PREFIX template __global__ void snhip::bgemm_mfma_kernel<snhip::BTileCfg<TM, TN, WM, WN, BK>, true, true, __bf16>(   \
        const snhip::GemmParams);

#define SNHIP_DECLARE_KERNELS(KIND, TM, TN, WM, WN, BK) SNHIP_VARIANTS_##KIND(extern, TM, TN, WM, WN, BK)
#define SNHIP_DEFINE_KERNELS(KIND, TM, TN, WM, WN, BK) SNHIP_VARIANTS_##KIND(, TM, TN, WM, WN, BK)
