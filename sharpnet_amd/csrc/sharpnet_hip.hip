// C ABI of libsharpnet_hip: argument checking, tile-configuration choice and
// kernel launch for the fp32 GEMM path.  Declarations and the reference entry
// point each function replaces are in include/sharpnet_hip.h.
#include "../../include/sharpnet_hip.h"

#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>

#include <mutex>
#include <new>

#include "attention_mfma.hpp"
#include "kernel_list.hpp"
#include "rowops.hpp"
#include "bgemm_dtl.hpp"
#include "sgemm_ksplit.hpp"
#include "sgemm_stream.hpp"

// The GEMM kernels are compiled in gemm_kernels.hip; here they are only declared.
SNHIP_ALL_KERNEL_GROUPS(SNHIP_DECLARE_KERNELS)

using namespace snhip;

// Split-K partial sums of snhip_dot_noalloc: device memory that exists from the moment the code object is loaded,
// so that entry point never has to allocate.  One copy per GPU, held until the process ends.  In host code this
// name is only a handle for hipGetSymbolAddress; kernels and copies get the address that call returned.
constexpr size_t kStaticScratchBytes = size_t(32) << 20;
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];

namespace {

// Device address of `scratch` on each GPU, looked up once per device (with that device current) by snhip_create.
constexpr int kMaxDevices = 64;
std::mutex g_scratch_mutex;
void* g_scratch_ptr[kMaxDevices] = {};

hipError_t static_scratch_address(int dev, void** out) {
    *out = nullptr;
    if (dev < 0 || dev >= kMaxDevices) return hipErrorInvalidDevice;
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    if (g_scratch_ptr[dev] == nullptr) {
        void* ptr = nullptr;
        const hipError_t e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
        if (e != hipSuccess) return e;
        if (ptr == nullptr) return hipErrorInvalidSymbol;
        g_scratch_ptr[dev] = ptr;
    }
    *out = g_scratch_ptr[dev];
    return hipSuccess;
}

constexpr int kVersion = 100;  // 0.1.0

struct Handle {
    int device = 0;
    hipStream_t stream = nullptr;
    float* ws = nullptr;      // split-K partial sums
    size_t ws_bytes = 0;
    int* counters = nullptr;  // split-K arrival counters, zero whenever no GEMM is in flight
    size_t n_counters = 0;
    int splitk_mode = 0;      // 0: automatic, 1: always reduce in a second kernel, 2: always reduce in the GEMM kernel
    int num_cu = 256;
    int math_mode = 0;  // 0: fp32 MFMA, 1: bf16-input MFMA for every GEMM on this handle
    int force_cfg = -1;
    int force_splitk = 0;
    int last_cfg = -1;
    int last_splitk = 0;
    int rnn_step_mode = 0;  // 0: recurrent forward steps as one launch when the shape allows, 1: always GEMM + cell kernel
    unsigned long long rnn_dropout_seed = 0;   // the reference seeds cuDNN's dropout states with 0 (GPUWrapper.cs:472)
    unsigned long long rnn_dropout_calls = 0;  // training-mode forward calls that drew masks so far
    float* static_scratch = nullptr;  // this device's copy of `scratch` (kStaticScratchBytes), never freed
    char last_error[192] = {0};       // text of the last refusal that has more to say than its status code
};

// Upper bound for the split-K workspace; larger requests fall back to fewer splits.
constexpr size_t kMaxWorkspaceBytes = size_t(1) << 30;
// What snhip_create reserves up front: the partial sums of every split-K product of the benchmark shapes fit (the
// largest, 8192 x 64 x 8192 split 8, needs 16 MiB), so that such calls never stop to grow the buffer.
constexpr size_t kInitialWorkspaceBytes = size_t(64) << 20;

typedef void (*KernelFn)(const GemmParams);

struct ConfigEntry {
    int BM, BN, BK, NT, lds_bytes;
    int mfma_per_k2;    // TM*TN: MFMA instructions one wavefront issues per MFMA k step
    int kind;           // 0: fp32 kernel (k step 2, 64 cycles per MFMA), 1: bf16-input kernel (k step 16, 32 cycles),
                        // 2: K split inside the workgroup, 3: streaming kernel, 4: bf16-input kernel on bf16 storage,
                        // 5 / 6: bf16-input streaming kernel on fp32 / bf16 storage
    KernelFn fn[2][2];  // [transposeA][transposeB]
    KernelFn fn_ext[2][2];  // the same with the extended write-out (addend, ReLU, two-level batch, column sum);
                            // nullptr if not built
    // cost-model inputs, calibrated on MI355X
    int occ;            // workgroups that fit on one CU (registers / LDS)
    double eff_alone;   // fraction of the MFMA issue rate reached with one workgroup per CU
    double eff_shared;  // ... with two or more co-resident workgroups hiding each other's stalls
    double edge_slow;   // slow-down of a tile that needs bounds-checked loads
};

template <class CFG>
constexpr ConfigEntry make_entry(int occ, double eff_alone, double eff_shared, double edge_slow) {
    return ConfigEntry{CFG::BM,
                       CFG::BN,
                       CFG::BK,
                       CFG::NT,
                       CFG::LDS_BYTES,
                       CFG::TM * CFG::TN,
                       0,
                       {{sgemm_mfma_kernel<CFG, false, false>, sgemm_mfma_kernel<CFG, false, true>},
                        {sgemm_mfma_kernel<CFG, true, false>, sgemm_mfma_kernel<CFG, true, true>}},
                       {{sgemm_mfma_kernel<CFG, false, false, true>, sgemm_mfma_kernel<CFG, false, true, true>},
                        {sgemm_mfma_kernel<CFG, true, false, true>, sgemm_mfma_kernel<CFG, true, true, true>}},
                       occ,
                       eff_alone,
                       eff_shared,
                       edge_slow};
}

template <class CFG>
constexpr ConfigEntry make_entry_bf16(int occ, double eff_alone, double eff_shared, double edge_slow) {
    return ConfigEntry{CFG::BM,
                       CFG::BN,
                       CFG::BK,
                       CFG::NT,
                       CFG::LDS_BYTES,
                       CFG::TM * CFG::TN,
                       1,
                       {{bgemm_mfma_kernel<CFG, false, false>, bgemm_mfma_kernel<CFG, false, true>},
                        {bgemm_mfma_kernel<CFG, true, false>, bgemm_mfma_kernel<CFG, true, true>}},
                       {{nullptr, nullptr}, {nullptr, nullptr}},
                       occ,
                       eff_alone,
                       eff_shared,
                       edge_slow};
}

template <class CFG>
constexpr ConfigEntry make_entry_bf16_stored(int occ, double eff_alone, double eff_shared, double edge_slow) {
    return ConfigEntry{CFG::BM,
                       CFG::BN,
                       CFG::BK,
                       CFG::NT,
                       CFG::LDS_BYTES,
                       CFG::TM * CFG::TN,
                       4,
                       {{bgemm_mfma_kernel<CFG, false, false, __bf16>, bgemm_mfma_kernel<CFG, false, true, __bf16>},
                        {bgemm_mfma_kernel<CFG, true, false, __bf16>, bgemm_mfma_kernel<CFG, true, true, __bf16>}},
                       {{nullptr, nullptr}, {nullptr, nullptr}},
                       occ,
                       eff_alone,
                       eff_shared,
                       edge_slow};
}

// Tile configurations, largest first.  <TM,TN,WM,WN,BK>: a wavefront owns
// TM x TN MFMA tiles of 32x32, a workgroup is WM x WN wavefronts.
const ConfigEntry kConfigs[] = {
    //                                      occ  alone shared edge
    make_entry<TileCfg<4, 4, 2, 2, 16>>(1, 0.990, 0.990, 1.25),  // 0: 256 x 256
    make_entry<TileCfg<2, 4, 2, 2, 16>>(1, 0.948, 0.948, 1.2),   // 1: 128 x 256
    make_entry<TileCfg<4, 2, 2, 2, 16>>(1, 0.949, 0.949, 1.2),   // 2: 256 x 128
    make_entry<TileCfg<2, 2, 2, 2, 16>>(2, 0.897, 0.929, 1.05),  // 3: 128 x 128
    make_entry<TileCfg<1, 2, 2, 2, 16>>(3, 0.861, 0.906, 1.05),  // 4: 64 x 128
    make_entry<TileCfg<2, 1, 2, 2, 16>>(3, 0.786, 0.866, 1.05),  // 5: 128 x 64
    make_entry<TileCfg<1, 1, 2, 2, 16>>(5, 0.758, 0.815, 1.05),  // 6: 64 x 64
    make_entry<TileCfg<2, 2, 2, 2, 32>>(1, 0.935, 0.935, 1.05),  // 7: 128 x 128, BK 32
    make_entry<TileCfg<2, 1, 2, 2, 32>>(2, 0.819, 0.878, 1.05),  // 8: 128 x 64, BK 32
    make_entry<TileCfg<1, 1, 2, 2, 32>>(4, 0.757, 0.813, 1.05),  // 9: 64 x 64, BK 32
    // bf16-input kernels (fp32 operands in memory: bound by the L2 -> LDS path long before the MFMA rate)
    make_entry_bf16<BTileCfg<4, 4, 2, 2, 32>>(1, 0.80, 0.80, 4.0),   // 10: 256 x 256, BK 32
    make_entry_bf16<BTileCfg<2, 2, 2, 2, 32>>(2, 0.60, 0.75, 1.3),   // 11: 128 x 128, BK 32
    make_entry_bf16<BTileCfg<2, 1, 2, 2, 64>>(2, 0.45, 0.60, 1.15),  // 12: 128 x 64, BK 64
    make_entry_bf16<BTileCfg<1, 1, 2, 2, 64>>(3, 0.45, 0.60, 1.1),   // 13: 64 x 64, BK 64
    // K split over the wavefronts of a workgroup (sgemm_ksplit.hpp): not part of the cost model's search, see
    // prefer_ksplit()
    ConfigEntry{32, 32, 32, 256, KsplitCfg<1>::LDS_BYTES, 1, 2,
                {{sgemm_ksplit_kernel<false, false>, sgemm_ksplit_kernel<false, true>},
                 {sgemm_ksplit_kernel<true, false>, sgemm_ksplit_kernel<true, true>}},
                // the same kernels serve as the extended form: they always apply the addend and the (leaky) ReLU
                {{sgemm_ksplit_kernel<false, false>, sgemm_ksplit_kernel<false, true>},
                 {sgemm_ksplit_kernel<true, false>, sgemm_ksplit_kernel<true, true>}},
                6, 0.5, 0.5, 1.0},  // 14: 32 x 32, four K slices
    ConfigEntry{32, 64, 32, 256, KsplitCfg<2>::LDS_BYTES, 1, 2,
                {{sgemm_ksplit_kernel<false, false, 2>, sgemm_ksplit_kernel<false, true, 2>},
                 {sgemm_ksplit_kernel<true, false, 2>, sgemm_ksplit_kernel<true, true, 2>}},
                {{sgemm_ksplit_kernel<false, false, 2>, sgemm_ksplit_kernel<false, true, 2>},
                 {sgemm_ksplit_kernel<true, false, 2>, sgemm_ksplit_kernel<true, true, 2>}},
                6, 0.5, 0.5, 1.0},  // 15: 32 x 64 (two column tiles), two K slices
    // persistent streaming kernels for batches of small matrices with a short K (sgemm_stream.hpp): not part of
    // the cost model's search either, see prefer_stream().  Panels of 32 k measured faster than panels of 64 on
    // every attention-shaped product (49.0 against 52.6 us for 512 x (256 x 256 x 64)): a third (fourth) workgroup
    // fits on a compute unit and the first MFMA starts after half the bytes.
    ConfigEntry{128, 128, 32, 256, StreamCfg<4, 32>::LDS_BYTES, 4, 3,
                {{sgemm_stream_kernel<4, false, false, 32>, sgemm_stream_kernel<4, false, true, 32>},
                 {sgemm_stream_kernel<4, true, false, 32>, sgemm_stream_kernel<4, true, true, 32>}},
                {{sgemm_stream_kernel<4, false, false, 32, true>, sgemm_stream_kernel<4, false, true, 32, true>},
                 {sgemm_stream_kernel<4, true, false, 32, true>, sgemm_stream_kernel<4, true, true, 32, true>}},
                3, 0.8, 0.9, 1.1},  // 16: 128 x 128, k panels of 32, three workgroups per compute unit
    ConfigEntry{128, 64, 32, 256, StreamCfg<2, 32>::LDS_BYTES, 2, 3,
                {{sgemm_stream_kernel<2, false, false, 32>, sgemm_stream_kernel<2, false, true, 32>},
                 {sgemm_stream_kernel<2, true, false, 32>, sgemm_stream_kernel<2, true, true, 32>}},
                {{sgemm_stream_kernel<2, false, false, 32, true>, sgemm_stream_kernel<2, false, true, 32, true>},
                 {sgemm_stream_kernel<2, true, false, 32, true>, sgemm_stream_kernel<2, true, true, 32, true>}},
                4, 0.7, 0.85, 1.1},  // 17: 128 x 64, k panels of 32, four workgroups per compute unit
    // bf16-input kernels on operands stored as bf16 (SNHIP_MATH_BF16_STORED)
    make_entry_bf16_stored<BTileCfg<4, 4, 2, 2, 64>>(1, 0.85, 0.85, 3.0),   // 18: 256 x 256, BK 64
    make_entry_bf16_stored<BTileCfg<2, 2, 2, 2, 64>>(2, 0.65, 0.80, 1.3),   // 19: 128 x 128, BK 64
    make_entry_bf16_stored<BTileCfg<1, 1, 2, 2, 128>>(2, 0.45, 0.60, 1.1),  // 20: 64 x 64, BK 128
    // K split eight ways over a workgroup of eight wavefronts.  No product takes it by default (configuration 26,
    // 16 x 16 tiles, superseded it); it runs only when forced with snhip_set_tuning(21, 1)
    ConfigEntry{32, 32, 32, 512, KsplitCfg<1, 8>::LDS_BYTES, 1, 2,
                {{sgemm_ksplit_kernel<false, false, 1, 8>, sgemm_ksplit_kernel<false, true, 1, 8>},
                 {sgemm_ksplit_kernel<true, false, 1, 8>, sgemm_ksplit_kernel<true, true, 1, 8>}},
                {{sgemm_ksplit_kernel<false, false, 1, 8>, sgemm_ksplit_kernel<false, true, 1, 8>},
                 {sgemm_ksplit_kernel<true, false, 1, 8>, sgemm_ksplit_kernel<true, true, 1, 8>}},
                1, 0.5, 0.5, 1.0},  // 21: 32 x 32, eight K slices
    // persistent streaming kernels in bf16-input arithmetic (sgemm_stream.hpp), fp32 storage (kind 5) ...
    ConfigEntry{128, 128, 64, 256, BStreamCfg<4>::LDS_BYTES, 4, 5,
                {{bgemm_stream_kernel<4, false, false, float>, bgemm_stream_kernel<4, false, true, float>},
                 {bgemm_stream_kernel<4, true, false, float>, bgemm_stream_kernel<4, true, true, float>}},
                {{bgemm_stream_kernel<4, false, false, float, true>, bgemm_stream_kernel<4, false, true, float, true>},
                 {bgemm_stream_kernel<4, true, false, float, true>, bgemm_stream_kernel<4, true, true, float, true>}},
                2, 0.8, 0.9, 1.1},  // 22: 128 x 128, k panels of 64
    ConfigEntry{128, 64, 128, 256, BStreamCfg<2>::LDS_BYTES, 2, 5,
                {{bgemm_stream_kernel<2, false, false, float>, bgemm_stream_kernel<2, false, true, float>},
                 {bgemm_stream_kernel<2, true, false, float>, bgemm_stream_kernel<2, true, true, float>}},
                {{bgemm_stream_kernel<2, false, false, float, true>, bgemm_stream_kernel<2, false, true, float, true>},
                 {bgemm_stream_kernel<2, true, false, float, true>, bgemm_stream_kernel<2, true, true, float, true>}},
                2, 0.7, 0.85, 1.1},  // 23: 128 x 64, k panels of 128
    // ... and bf16 storage (kind 6)
    ConfigEntry{128, 128, 64, 256, BStreamCfg<4>::LDS_BYTES, 4, 6,
                {{bgemm_stream_kernel<4, false, false, __bf16>, bgemm_stream_kernel<4, false, true, __bf16>},
                 {bgemm_stream_kernel<4, true, false, __bf16>, bgemm_stream_kernel<4, true, true, __bf16>}},
                {{bgemm_stream_kernel<4, false, false, __bf16, true>, bgemm_stream_kernel<4, false, true, __bf16, true>},
                 {bgemm_stream_kernel<4, true, false, __bf16, true>, bgemm_stream_kernel<4, true, true, __bf16, true>}},
                3, 0.8, 0.9, 1.1},  // 24: 128 x 128, k panels of 64
    ConfigEntry{128, 64, 128, 256, BStreamCfg<2>::LDS_BYTES, 2, 6,
                {{bgemm_stream_kernel<2, false, false, __bf16>, bgemm_stream_kernel<2, false, true, __bf16>},
                 {bgemm_stream_kernel<2, true, false, __bf16>, bgemm_stream_kernel<2, true, true, __bf16>}},
                {{bgemm_stream_kernel<2, false, false, __bf16, true>, bgemm_stream_kernel<2, false, true, __bf16, true>},
                 {bgemm_stream_kernel<2, true, false, __bf16, true>, bgemm_stream_kernel<2, true, true, __bf16, true>}},
                3, 0.7, 0.85, 1.1},  // 25: 128 x 64, k panels of 128
    // 16 x 16 tiles (v_mfma_f32_16x16x4_f32), K split over eight wavefronts: see prefer_ksplit()
    ConfigEntry{16, 16, 32, 512, Ksplit16Cfg::LDS_BYTES, 1, 2,
                {{sgemm_ksplit16_kernel<false, false>, sgemm_ksplit16_kernel<false, true>},
                 {sgemm_ksplit16_kernel<true, false>, sgemm_ksplit16_kernel<true, true>}},
                {{sgemm_ksplit16_kernel<false, false>, sgemm_ksplit16_kernel<false, true>},
                 {sgemm_ksplit16_kernel<true, false>, sgemm_ksplit16_kernel<true, true>}},
                4, 0.5, 0.5, 1.0},  // 26: 16 x 16, eight K slices
    // bf16 storage, both operands k-contiguous, tiles through global -> LDS direct loads (bgemm_dtl.hpp): one form
    // only (A plain, B transposed), shapes that are whole tiles; see prefer_dtl()
    ConfigEntry{BDtlCfg::BM, BDtlCfg::BN, BDtlCfg::BK, BDtlCfg::NT, BDtlCfg::LDS_BYTES, 16, 7,
                {{nullptr, bgemm_nt_dtl_kernel<4>}, {nullptr, nullptr}},
                {{nullptr, nullptr}, {nullptr, nullptr}},
                1, 0.9, 0.9, 1.0},  // 27: 256 x 256, k panels of 32, four LDS stages
    ConfigEntry{BDtlCfgT<2>::BM, BDtlCfgT<2>::BN, BDtlCfgT<2>::BK, BDtlCfgT<2>::NT, BDtlCfgT<2>::LDS_BYTES, 4, 7,
                {{nullptr, bgemm_nt_dtl_kernel<2>}, {nullptr, nullptr}},
                {{nullptr, nullptr}, {nullptr, nullptr}},
                2, 0.7, 0.8, 1.0},  // 28: 128 x 128, the same kernel with 64 x 64 per wavefront
};
constexpr int kNumConfigs = sizeof(kConfigs) / sizeof(kConfigs[0]);
constexpr int kKsplit16Config = 26;
constexpr int kBDtlConfig = 27;       // and kBDtlConfig + 1 (128 x 128 tiles)
constexpr int kKsplitConfig = 14;   // and kKsplitConfig + 1
constexpr int kStreamConfig = 16;   // and kStreamConfig + 1
constexpr int kKsplit8Config = 21;
constexpr int kBStreamConfig = 22;        // bf16-input streaming, fp32 storage: 22, 23
constexpr int kBStreamStoredConfig = 24;  // ... bf16 storage: 24, 25

// Fused attention forward kernels (attention_mfma.hpp)
struct AttnEntry {
    int keys, hd, lds_bytes;
    void (*fn)(const AttnParams);
};
template <int NT, int HD>
constexpr AttnEntry attn_entry() {
    return AttnEntry{AttnCfg<NT, HD>::KEYS, HD, AttnCfg<NT, HD>::LDS_BYTES, attention_fwd_kernel<NT, HD>};
}
// smallest first: the first entry that holds the problem is used
const AttnEntry kAttn[] = {attn_entry<2, 32>(), attn_entry<4, 32>(), attn_entry<8, 32>(),
                           attn_entry<2, 64>(), attn_entry<4, 64>(), attn_entry<8, 64>(),
                           attn_entry<2, 128>(), attn_entry<4, 128>()};
template <int NT, int HD>
constexpr AttnEntry attn_bwd_entry() {
    return AttnEntry{AttnCfg<NT, HD>::KEYS, HD, AttnCfg<NT, HD>::LDS_BYTES, attention_fwd_kernel<NT, HD, true>};
}
// (head dimension 128 is left to the five-launch sequence: measured 0.300 ms against 0.287 ms at 1024 x (128 x 128))
const AttnEntry kAttnBwd[] = {attn_bwd_entry<2, 32>(), attn_bwd_entry<4, 32>(), attn_bwd_entry<8, 32>(),
                              attn_bwd_entry<2, 64>(), attn_bwd_entry<4, 64>(), attn_bwd_entry<8, 64>()};

// The same for head dimension exactly 32 or 64 and 65 to 256 keys: attention_fwd16_kernel (two wavefronts per SIMD)
struct Attn16Entry {
    int keys, hd, lds_bytes;
    void (*fn)(const AttnParams);
    int wgs_per_cu;  // resident workgroups per compute unit (registers, LDS): the persistent grid is that many times the CUs
};
template <int KEYS, int HD, bool BWD>
constexpr Attn16Entry attn16_entry() {
    // 128 keys x 32 forward: 104 registers and 35 KB of LDS, two workgroups fit; every other size: one
    return Attn16Entry{KEYS, HD, Attn16Cfg<KEYS, HD>::LDS_BYTES, attention_fwd16_kernel<KEYS, BWD, HD>,
                       (KEYS == 128 && HD == 32 && !BWD) ? 2 : 1};
}
const Attn16Entry kAttn16[] = {attn16_entry<128, 32, false>(), attn16_entry<256, 32, false>(),
                               attn16_entry<128, 64, false>(), attn16_entry<256, 64, false>()};
const Attn16Entry kAttn16Bwd[] = {attn16_entry<128, 32, true>(), attn16_entry<256, 32, true>(),
                                  attn16_entry<128, 64, true>(), attn16_entry<256, 64, true>()};
template <int N>
const Attn16Entry* find_attn16(const Attn16Entry (&table)[N], int keys, int hd) {
    for (const Attn16Entry& c : table)
        if (c.keys == keys && c.hd == hd) return &c;
    return nullptr;
}

int hip_to_status(hipError_t e) {
    switch (e) {
        case hipSuccess:
            return SNHIP_STATUS_SUCCESS;
        case hipErrorOutOfMemory:
            return SNHIP_STATUS_ALLOC_FAILED;
        case hipErrorInvalidValue:
        case hipErrorInvalidDevicePointer:
            return SNHIP_STATUS_INVALID_VALUE;
        case hipErrorNotInitialized:
        case hipErrorNoDevice:
            return SNHIP_STATUS_NOT_INITIALIZED;
        default:
            return SNHIP_STATUS_EXECUTION_FAILED;
    }
}

inline int ceil_div(int a, int b) { return (a + b - 1) / b; }

hipError_t rnn_prepare_kernels();  // rnn_layers.hpp: LDS opt-in of the recurrent step kernels

struct Choice {
    int cfg;
    int splitk;
};

// Estimated run time in engine cycles.  The launch is bound by the slowest of
//  - the MFMA pipes: every CU works off ceil(blocks / num_cu) workgroups, one wavefront per SIMD each;
//  - the per-tile critical path of a workgroup that has the CU to itself (LDS round trip + barrier);
//  - HBM (unique operand bytes + C, plus the split-K partial sums);
//  - the L2 -> LDS path (every workgroup re-reads its A and B panels), chip-wide and per CU.
// Split-K adds a second launch that re-reads the partial sums.  The constants (and the efficiencies in kConfigs) are a fit
// to a sweep on MI355X: every fp32 tile configuration with K split 1, 2 and 4 ways on thirty shapes between 640^3 and
// 4096^3 (squares, ragged ones, short and long K, tall ones); what the model picks there is within 1.7 % of the fastest
// measured candidate (0.2 % on average; 9.7 % and 1.6 % with the hand-set constants before).
double estimate_cycles(const ConfigEntry& c, int M, int N, int K, int batch, int splitk, int num_cu) {
    constexpr double kTileLatency = 700.0;     // cycles per k tile when nothing hides the LDS/barrier latency
    constexpr double kFixed = 2290.0;          // prologue + epilogue of one workgroup
    constexpr double kStoreBytesPerCycle = 40; // C write-out rate of one CU
    constexpr double kChipStoreBytesPerCycle = 1875;  // ... of all of them together (~4.5 TB/s)
    constexpr double kHbmBytesPerCycle = 2000; // ~4.8 TB/s streaming at 2.4 GHz (what a plain copy reaches)
    constexpr double kL2BytesPerCycle = 7000;  // ~17 TB/s aggregate L2 -> CU
    constexpr double kCuBytesPerCycle = 40;    // what one CU can pull from L2 into LDS
    constexpr double kLaunch = 1620.0;
    constexpr double kSplitFixed = 8650.0;     // second launch + dependency gap
    constexpr double kSplitPerPart = 500.0;    // what every further part costs beyond its bytes (384 x 384 x 3000: 16 parts
                                               // 22.4 us, 4 parts 19.3 us)
    const long long tiles_mn = (long long)ceil_div(M, c.BM) * ceil_div(N, c.BN);
    const long long blocks = tiles_mn * batch * splitk;
    const long long per_cu = (blocks + num_cu - 1) / num_cu;
    const int kchunk = ceil_div(ceil_div(K, splitk), c.BK) * c.BK;
    const int nk = ((kchunk / c.BK + 1) / 2) * 2;  // the k loop runs pairs of tiles
    const double mfma_per_tile = c.kind == 0 ? (c.BK / 2) * 64.0 * c.mfma_per_k2 : (c.BK / 16) * 32.0 * c.mfma_per_k2;
    const double elem = c.kind == 4 ? 2.0 : 4.0;  // bytes per operand element in memory
    const long long resident = per_cu < c.occ ? per_cu : c.occ;
    const double eff = resident >= 2 ? c.eff_shared : c.eff_alone;
    const bool has_edge = (M % c.BM != 0) || (N % c.BN != 0);
    const double edge = !has_edge ? 1.0 : (per_cu <= 2 ? c.edge_slow : 1.0 + (c.edge_slow - 1.0) * 0.15);
    // A configuration that never shares a compute unit writes every tile out with the matrix pipes idle, and when all
    // units do so at once they share the chip's write rate: 256 x 256 tiles on 32768 x 2048 x 256 spend 17 of their
    // 72 us per tile there (286 us; the 128 x 128 tiles, two workgroups per unit, 272 us).  (The write-out of the last
    // tile of a unit is a cost every configuration has; it stays in kFixed.)
    const long long writers = blocks < num_cu ? blocks : (long long)num_cu;
    double store_rate = kChipStoreBytesPerCycle / (double)writers;
    if (store_rate > kStoreBytesPerCycle) store_rate = kStoreBytesPerCycle;
    const double t_store = c.occ == 1 ? per_cu * ((double)c.BM * c.BN * 4.0 / store_rate) : 0.0;
    // (the last tile of a unit goes out with nothing left to hide it behind, whatever the configuration)
    const double t_mfma =
        per_cu * nk * mfma_per_tile / eff * edge + t_store + kFixed + (double)c.BM * c.BN * 4.0 / kStoreBytesPerCycle;
    const double tile_alone = mfma_per_tile / c.eff_alone > kTileLatency ? mfma_per_tile / c.eff_alone : kTileLatency;
    const double t_lat = (double)((per_cu + c.occ - 1) / c.occ) *
                         (nk * tile_alone + kFixed + (double)c.BM * c.BN * 4.0 / kStoreBytesPerCycle);
    const double bytes_hbm = (double)batch * (elem * ((double)M * K + (double)K * N) + 4.0 * M * N) +
                             (splitk > 1 ? (double)batch * M * N * 4.0 * splitk : 0.0);
    const double t_mem = bytes_hbm / kHbmBytesPerCycle;
    const double t_l2 = (double)blocks * (c.BM + c.BN) * (double)kchunk * elem / kL2BytesPerCycle;
    const double t_cu = (double)per_cu * (c.BM + c.BN) * (double)kchunk * elem / kCuBytesPerCycle + kFixed;
    double t = t_mfma;
    if (t_cu > t) t = t_cu;
    if (t_lat > t) t = t_lat;
    if (t_mem > t) t = t_mem;
    if (t_l2 > t) t = t_l2;
    // tiles that are mostly padding spend their time in bounds-checked loads of rows that do not exist
    const double padded = (double)ceil_div(M, c.BM) * c.BM * (double)ceil_div(N, c.BN) * c.BN / ((double)M * N);
    if (padded > 1.25) t *= padded / 1.25;
    t += kLaunch;
    if (splitk > 1)
        t += kSplitFixed + kSplitPerPart * splitk + (double)batch * M * N * (2.0 * splitk + 2.0) * 4.0 / kHbmBytesPerCycle;
    return t;
}

// kind of kernel that serves a math mode: 0 fp32, 1 bf16-input on fp32 storage, 4 bf16-input on bf16 storage
inline int kind_of_math(int math) { return math == SNHIP_MATH_BF16_STORED ? 4 : math; }

// tA / tB: the form of the product.  The efficiencies in kConfigs were measured in the NN form; a product with both operands
// transposed is the NN product of the transposed result, so an oblong tile then behaves like its mirror image
// (1280^3 TT: 128 x 64 tiles 41.4 us, 64 x 128 tiles 45.6 us; NN: 44.6 and 41.3 us).  The mixed forms sit in between.
Choice choose(const Handle* h, int M, int N, int K, int batch, int kind, bool tA = false, bool tB = false) {
    Choice best{kind == 0 ? 6 : (kind == 1 ? 13 : 20), 1};
    double best_cost = 1e300;
    const bool forced = h->force_cfg >= 0 && kConfigs[h->force_cfg].kind == kind;
    // A tall operand against a narrow one (N <= 64) with a long K streams op(A) from memory once: measured on
    // 8192 x 64 x 8192, all transposes, 128 x 64 tiles with 32-wide k panels (whole 128-byte lines of a k-contiguous
    // operand per row and tile) and one workgroup per compute unit (split 4) take 78-85 us, against 84-92 us for what the
    // cost model picks (16-wide panels, split 8).  The bf16 kinds likewise: the model sees the memory time of op(A) either
    // way and does not split, but half a chip of workgroups does not pull it at that rate (bf16-input, 64 x 64 x 64
    // tiles: 75.9 us unsplit, 51.7 us split in two).
    // (When 64 x 64 tiles fill the chip without a split the cost model decides: 16384 x 64 x 4096 takes 74.5 us on them,
    // 79.6 us on 128 x 64 tiles split in two.)
    if (!forced && h->force_splitk <= 0 && batch == 1 && N <= 64 && K >= 2048 && (long long)M * K >= (1LL << 24) &&
        (kind != 0 || (long long)ceil_div(M, 64) * ceil_div(N, 64) < h->num_cu)) {
        const int cfg = kind == 0 ? 8 : (kind == 1 ? 13 : (kind == 4 ? 20 : -1));
        if (cfg >= 0) {
            const ConfigEntry& e = kConfigs[cfg];
            const long long tiles = (long long)ceil_div(M, e.BM) * ceil_div(N, e.BN);
            int s = 1;
            while (tiles * s < h->num_cu && s < 32 && K / (2 * s) >= 8 * e.BK) s *= 2;
            const int kchunk = ceil_div(ceil_div(K, s), e.BK) * e.BK;
            if ((long long)kchunk * (s - 1) < K && (size_t)M * N * s * sizeof(float) <= kMaxWorkspaceBytes) return Choice{cfg, s};
        }
    }
    for (int c = 0; c < kNumConfigs; ++c) {
        const ConfigEntry& e = kConfigs[c];
        if (e.kind != kind) continue;
        if (forced && c != h->force_cfg) continue;
        for (int s = 1; s <= 32; s *= 2) {
            if (h->force_splitk > 0 && s != h->force_splitk) continue;
            if (s > 1) {
                if (h->force_splitk <= 0 && K / s < 4 * e.BK) break;
                if ((size_t)M * N * batch * s * sizeof(float) > kMaxWorkspaceBytes) break;
                const int kchunk = ceil_div(ceil_div(K, s), e.BK) * e.BK;
                if ((long long)kchunk * (s - 1) >= K) continue;  // would leave an empty split
            }
            double cost;
            const int mirror = (c == 1 || c == 4) ? c + 1 : ((c == 2 || c == 5) ? c - 1 : c);
            if (tA && tB && mirror != c) {
                ConfigEntry m = e;
                m.eff_alone = kConfigs[mirror].eff_alone;
                m.eff_shared = kConfigs[mirror].eff_shared;
                cost = estimate_cycles(m, M, N, K, batch, s, h->num_cu);
            } else if (tA != tB && mirror != c) {
                // one operand transposed: half way (2048^3 TN: 64 x 128 tiles 128 us, 128 x 64 tiles 129 us, 128 x 128 tiles 124 us)
                ConfigEntry m = e;
                m.eff_alone = 0.5 * (e.eff_alone + kConfigs[mirror].eff_alone);
                m.eff_shared = 0.5 * (e.eff_shared + kConfigs[mirror].eff_shared);
                cost = estimate_cycles(m, M, N, K, batch, s, h->num_cu);
            } else {
                cost = estimate_cycles(e, M, N, K, batch, s, h->num_cu);
            }
            if (cost < best_cost) {
                best_cost = cost;
                best = Choice{c, s};
            }
        }
    }
    // 64 x 64 tiles with at most one workgroup per compute unit: when K is a whole number of 32-wide k panels, the
    // configuration with those panels is 3-5 % ahead of the one with 16-wide panels (1024^3 in all four forms 19.2-19.7
    // against 20.2-20.3 us, 1024 x 1024 x 256 ... 2048, 512 x 512 x 2048); with a ragged K (1000, 1040, 700) it is not.
    // (With both operands transposed also for a ragged K whose 16-wide panels are an odd number - the loop then multiplies
    // a panel of zeros to complete its last pair - while its 32-wide panels are an even number: 1000^3 TT 22.2 against
    // 23.2 us, 960 x 1024 x 1000 20.5 against 20.9; not K = 1040, 700, 1100, 500.)
    const bool odd_pairs_tt = tA && tB && best.splitk == 1 && ceil_div(K, 16) % 2 == 1 && ceil_div(K, 32) % 2 == 0;
    if (kind == 0 && !forced && best.cfg == 6 && (K % 32 == 0 || odd_pairs_tt) && K / best.splitk >= 256 &&
        (long long)ceil_div(M, 64) * ceil_div(N, 64) * batch * best.splitk <= h->num_cu) {
        const int kchunk = ceil_div(ceil_div(K, best.splitk), 32) * 32;
        if ((long long)kchunk * (best.splitk - 1) < K) best.cfg = 9;
    }
    return best;
}

// what transpose_to_bf16_kernel asks of its operands (elem_bytes: 4 for an fp32 source, 2 for a bf16 one)
bool wide_transpose_ok(const void* src, int rows, int cols, long long ld_src, int elem_bytes, const void* dst,
                       long long ld_dst) {
    const int cw = 16 / elem_bytes;
    return rows % 64 == 0 && cols % (8 * cw) == 0 && rows / 64 <= 65535 && (uintptr_t)src % 16 == 0 &&
           (uintptr_t)dst % 16 == 0 && (ld_src * elem_bytes) % 16 == 0 && (ld_dst * 2) % 16 == 0;
}

// dst[c][r] = src[r][c], both bf16 (the caller has checked wide_transpose_ok)
int transpose_bf16(Handle* h, const void* src, int rows, int cols, long long ld_src, void* dst, long long ld_dst) {
    hipLaunchKernelGGL(transpose_to_bf16_kernel<true>, dim3((unsigned)ceil_div(cols, 256), (unsigned)(rows / 64)), dim3(256),
                       0, h->stream, src, ld_src, rows, cols, static_cast<__bf16*>(dst), ld_dst);
    return hip_to_status(hipGetLastError());
}

int ensure_workspace(Handle* h, size_t bytes) {
    if (bytes <= h->ws_bytes) return SNHIP_STATUS_SUCCESS;
    if (h->ws != nullptr) {
        // kernels still in flight may be using the old buffer
        hipError_t e = hipStreamSynchronize(h->stream);
        if (e != hipSuccess) return hip_to_status(e);
        (void)hipFree(h->ws);
        h->ws = nullptr;
        h->ws_bytes = 0;
    }
    void* p = nullptr;
    hipError_t e = hipMalloc(&p, bytes);
    if (e != hipSuccess) {
        (void)hipGetLastError();
        return SNHIP_STATUS_ALLOC_FAILED;
    }
    h->ws = static_cast<float*>(p);
    h->ws_bytes = bytes;
    return SNHIP_STATUS_SUCCESS;
}

// out[z][c] = sum_r x[z][r][c] for nz matrices of rows x cols (row pitch ld, `stride` floats apart).  A matrix too
// tall for cols / 64 workgroups to fill the chip is summed in row chunks through the handle's workspace.
int launch_column_sum(Handle* h, const float* x, float* out, int rows, int cols, long long ld, long long stride, int nz) {
    const int col_blocks = (cols + 63) / 64;
    const long long base = (long long)col_blocks * nz;
    int chunks = 1;
    if (rows >= 512 && base < 2LL * h->num_cu) {
        chunks = (int)((4LL * h->num_cu + base - 1) / base);
        if (chunks > rows / 128) chunks = rows / 128;  // at least 128 rows per chunk
        if (chunks > 4096) chunks = 4096;
    }
    const int rows_per_chunk = chunks > 1 ? ceil_div(rows, chunks) : (rows > 0 ? rows : 1);
    chunks = rows > 0 ? ceil_div(rows, rows_per_chunk) : 1;
    float* dst = out;
    if (chunks > 1) {
        const int st = ensure_workspace(h, (size_t)chunks * nz * cols * sizeof(float));
        if (st != SNHIP_STATUS_SUCCESS) return st;
        dst = h->ws;
    }
    hipLaunchKernelGGL(column_sum_kernel, dim3(col_blocks, nz, chunks), dim3(256), 0, h->stream, x, dst, rows, cols, ld,
                       stride, rows_per_chunk);
    if (chunks > 1) {
        const long long total = (long long)nz * cols;
        hipLaunchKernelGGL(column_sum_finish_kernel, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, h->stream,
                           (const float*)h->ws, out, chunks, cols, nz);
    }
    return hip_to_status(hipGetLastError());
}

// The last-arriving workgroup can add the split-K partial sums itself (splitk_mode 2), which saves the
// second launch.  Measured on MI355X it is slower than the second kernel for every shape tried
// (8192x64x8192 split 4: 171 us against 87 us; 128x256x784 split 4: 21.7 us against 12.9 us): each
// workgroup's device-scope release fence writes back its XCD's L2 and the acquire invalidates it, because
// the eight L2s are not coherent with one another.  Automatic mode therefore always uses the second kernel.
int ensure_counters(Handle* h, size_t n) {
    if (n <= h->n_counters) return SNHIP_STATUS_SUCCESS;
    hipError_t e = hipStreamSynchronize(h->stream);
    if (e != hipSuccess) return hip_to_status(e);
    if (h->counters != nullptr) (void)hipFree(h->counters);
    h->counters = nullptr;
    h->n_counters = 0;
    size_t cap = 4096;
    while (cap < n) cap *= 2;
    void* p = nullptr;
    e = hipMalloc(&p, cap * sizeof(int));
    if (e != hipSuccess) {
        (void)hipGetLastError();
        return SNHIP_STATUS_ALLOC_FAILED;
    }
    e = hipMemset(p, 0, cap * sizeof(int));
    if (e != hipSuccess) {
        (void)hipFree(p);
        return hip_to_status(e);
    }
    h->counters = static_cast<int*>(p);
    h->n_counters = cap;
    return SNHIP_STATUS_SUCCESS;
}

// Everything one GEMM launch can be asked to do (row-major):
//   C[z] = act(alpha * op(A[z]) . op(B[z]) + bias + beta * C[z] + gamma * D[z]),  z = 0 .. batch-1,
//   optionally colsum[z][m] = sum_k op(A[z])[m][k].
// Matrix z of a two-level batch sits at base + (z / batch_inner) * stride2 + (z % batch_inner) * stride.
struct GemmArgs {
    bool tA = false, tB = false;
    int M = 0, N = 0, K = 0;
    float alpha = 1.0f, beta = 0.0f;
    const float* A = nullptr;
    const float* B = nullptr;
    float* C = nullptr;
    int lda = 0, ldb = 0, ldc = 0;
    int batch = 1, batch_inner = 0;  // batch_inner 0: single-level batch
    long long sA = 0, sB = 0, sC = 0, sA2 = 0, sB2 = 0, sC2 = 0;
    const float* bias = nullptr;
    const float* D = nullptr;
    int ldd = 0;
    long long sD = 0, sD2 = 0;
    float gamma = 0.0f;
    int act = ACT_NONE;
    float act_param = 0.0f;
    float* colsum = nullptr;
    int math = -1;  // -1: the handle's math mode
    bool no_alloc = false;  // split-K partial sums go to the static scratch array; nothing is allocated or freed
    bool k_from_m = false;  // hint: op(A)[m][k] == 0 for k < m (see GEMM_FLAG_K_FROM_M); kernels without it multiply the zeros
};

// Whether the product goes to sgemm_ksplit_kernel (32 x 32 tiles, K split inside the workgroup) instead of the
// configuration the cost model chose.  It needs 16-byte pieces along each operand's contiguous direction, and it
// pays when the tiled kernels cannot fill the chip: few 32 x 32 tiles and a K of at least a few groups of 32.
int prefer_ksplit(const Handle* h, const GemmArgs& g, int math, bool two_level) {
    if (math != SNHIP_MATH_FP32 || two_level || g.K < 32 || g.K % 4 != 0) return -1;
    const bool forced = h->force_cfg == kKsplitConfig || h->force_cfg == kKsplitConfig + 1 ||
                        h->force_cfg == kKsplit8Config || h->force_cfg == kKsplit16Config;
    if (h->force_cfg >= 0 && !forced) return -1;
    const bool multi = g.batch > 1;
    auto aligned = [&](const float* ptr, int ld, long long stride, bool rows_contiguous, int rows) {
        return (uintptr_t)ptr % 16 == 0 && ld % 4 == 0 && (!multi || stride % 4 == 0) && (!rows_contiguous || rows % 4 == 0);
    };
    if (!aligned(g.A, g.lda, g.sA, g.tA, g.M) || !aligned(g.B, g.ldb, g.sB, !g.tB, g.N)) return -1;
    if (forced) return h->force_cfg;
    // A tall operand against one of 32 columns or fewer with a long K: 64-wide tiles would be half padding or more and
    // need a second launch for their K splits; here the K slices meet inside the workgroup.  Measured: 16384 x 32 x 4096
    // 61.4 us on 32 x 32 tiles against 75.2 (128 x 64 tiles, split 2), 8192 x 32 x 2048 18.4 against 26.1; on 16 x 16
    // tiles 8192 x 16 x 8192 45.4 against 74.4, 8192 x 8 x 8192 46.2 against 73.6, 4096 x 32 x 4096 (too few 32 x 32 tiles
    // for the chip) 22.9 against 26.6.
    if (h->force_splitk <= 0 && g.batch == 1 && g.N <= 32 && g.K >= 2048 && (long long)g.M * g.K >= (1LL << 24))
        return (g.N > 16 && ceil_div(g.M, 32) >= h->num_cu) ? kKsplitConfig : kKsplit16Config;
    // The mirror image, a wide operand under one of 32 rows or fewer: 32 x 32 tiles when they fill the chip (32 x 16384 x 4096
    // 60.6 us against 76.3 on 64 x 128 tiles split in four, 16 x 8192 x 8192 57.0 against 77.9, 32 x 8192 x 2048 18.1
    // against 25.1; the 16 x 16 tiles gain nothing on this side).
    if (h->force_splitk <= 0 && g.batch == 1 && g.M <= 32 && g.K >= 2048 && (long long)g.N * g.K >= (1LL << 24) &&
        ceil_div(g.N, 32) >= h->num_cu)
        return kKsplitConfig;
    if (h->force_splitk > 0 || g.K > 1024) return -1;
    // Measured on MI355X: 128 x 256 x 784 8.8 us against 12.8 (64 x 64 tiles, split-K 4 + reduction), 128 x 784 x 256
    // 5.5 against 10.5, 512^3 6.8 against 12.9; a loss when a wavefront's share of K gets long (256 x 256 x 4096:
    // 30.5 against 17.2 with split-K 16).  Up to one 32 x 32 tile per compute unit: four K slices.
    const long long rows32 = (long long)ceil_div(g.M, 32) * g.batch;
    // 32 x 32 tiles for a quarter of the compute units or fewer, and a K that gives eight wavefronts a few groups of 32
    // each: 16 x 16 tiles, four times the workgroups (128 x 256 x 784: 5.4 us against 8.7 with eight wavefronts on
    // 32 x 32 tiles, 64 x 128 x 1024: 5.4 against 9.1, 128 x 128 x 512: 5.4 against 6.0)
    // (and up to half of them with a K of 256 or more: 256 x 512 x 1024 8.0 against 10.5 us, 512 x 256 x 768 6.7 against 8.9,
    // 320 x 320 x 512 5.1 against 7.2, 300^3 4.9 against 6.2, 512 x 256 x 256 4.9 against 5.2)
    if (rows32 * ceil_div(g.N, 32) <= (long long)h->num_cu / 4 && g.K >= 512) return kKsplit16Config;
    if (rows32 * ceil_div(g.N, 32) <= (long long)h->num_cu / 2 && g.K >= 256 && !multi) return kKsplit16Config;
    // Between half a chip and a whole chip of 32 x 32 tiles, with a K of 384 or more: eight K slices (two wavefronts per
    // SIMD) instead of four - 512 x 384 x 512 6.1 against 7.2 us, 384 x 384 x 768 7.7 against 8.9, 512 x 512 x 768 8.0
    // against 9.1, 400 x 400 x 640 7.7 against 8.1.
    // (batches of small matrices likewise: 16 x (128 x 128 x 512) 6.2 against 7.3 us, 64 x (64 x 64 x 512) 7.9 against 9.3;
    // with half a chip of tiles or fewer a batch stays on four slices - 32 x (64 x 64 x 1024) 10.8 us, 11.9 on eight slices,
    // 12.7 on 16 x 16 tiles)
    if (rows32 * ceil_div(g.N, 32) <= (long long)h->num_cu && g.K >= 384 &&
        (!multi || rows32 * ceil_div(g.N, 32) > (long long)h->num_cu / 2))
        return kKsplit8Config;
    if (rows32 * ceil_div(g.N, 32) <= (long long)h->num_cu) return kKsplitConfig;
    // (Up to one 32 x 64 tile per compute unit - two K slices, configuration 15 - used to go here too; since the tail of
    // the tiled kernels' k loop was shortened the 64 x 64 tiles are ahead on all of those: 512 x 1024 x 256 7.0 against
    // 8.2 us, 32 x (128 x 128 x 1024) 16.3 against 20.6 us, 256 x 2048 x 512 11.0 against 11.6 us.  The configuration
    // stays reachable through snhip_set_tuning.)
    return -1;
}

// Whether the product goes to sgemm_stream_kernel (configuration 16 or 17) instead of what the cost model chose:
// strided batches of small matrices whose K fits a few 64-wide panels, where the tiled kernels' pipeline never
// fills and every workgroup is prologue and write-out.
int prefer_stream(const Handle* h, const GemmArgs& g, int math, bool two_level, bool wants_ext) {
    (void)two_level;  // the streaming kernels have a variant that walks a two-level batch (their fn_ext entries)
    if (wants_ext) return -1;
    const int first = math == SNHIP_MATH_FP32 ? kStreamConfig
                                              : (math == SNHIP_MATH_BF16_INPUT ? kBStreamConfig : kBStreamStoredConfig);
    const bool forced = h->force_cfg == first || h->force_cfg == first + 1;
    if (h->force_cfg >= 0 && !forced) return -1;
    if (h->force_splitk > 1) return -1;
    if (forced) return h->force_cfg;
    // (fp32: K up to 128 - with 192 and 256 the tiled kernels are level or ahead: 128 x (384 x 384 x 256) 81 against 91 us,
    // 64 x (512 x 512 x 192) 57 against 60 us, 512 x (256 x 256 x 256) 154 against 151 us.  The bf16 kinds, whose MFMA
    // time is an eighth, stay streaming up to 256: the probabilities-times-values product of an attention layer.)
    if (g.batch < 8 || g.K > (math == SNHIP_MATH_FP32 ? 128 : 256) || g.M < 64) return -1;
    const int cfg = g.N <= 64 ? first + 1 : first;
    const long long tiles = (long long)ceil_div(g.M, 128) * ceil_div(g.N, kConfigs[cfg].BN) * g.batch;
    if (tiles < 2LL * h->num_cu) return -1;
    // fp32, where the tiled kernels are close: only the shapes a sweep has it ahead on - matrices of whole 256-row
    // blocks (512 x (256 x 256 x 64) 48.8 against 50.6 us, 64 x (512 x 512 x 128) 42.3 against 43.1) and four tiles per
    // compute unit or more; 8 x (1000 x 1000 x 64) 16.1 us tiled against 19.1, 64 x (384 x 384 x 96) 22.5 against 26.6,
    // 512 x (64 x 64 x 64) 5.9 against 8.8
    if (math == SNHIP_MATH_FP32 &&
        (g.M % 256 != 0 || (g.N % 256 != 0 && g.N > 64) || g.N < 64 || tiles < 4LL * h->num_cu))
        return -1;
    // mostly-empty tiles waste the streaming they are meant to save
    if ((long long)ceil_div(g.M, 128) * 128 * ceil_div(g.N, kConfigs[cfg].BN) * kConfigs[cfg].BN > 2LL * g.M * g.N) return -1;
    return cfg;
}

// Whether a product on operands stored as bf16 goes to bgemm_nt_dtl_kernel (configuration 27) instead of what the
// cost model chose: both operands k-contiguous (A plain, B transposed), M and N whole 256-wide tiles, K whole 32-wide
// panels, rows and matrices on 16-byte boundaries, a plain epilogue (alpha, beta, bias), and enough tiles that the
// 256 x 256 tile is what the cost model would have picked anyway (at least one per compute unit).  Measured on
// MI355X, 8192^3, U(-1, 1) operands: 1.19-1.21 PFLOP/s against 1.12-1.15 for the register-staged 256 x 256 kernel.
int prefer_dtl(const Handle* h, const GemmArgs& g, int math, bool wants_ext) {
    if (math != SNHIP_MATH_BF16_STORED || g.tA || !g.tB || wants_ext) return -1;
    if (h->force_cfg >= 0 && h->force_cfg != kBDtlConfig && h->force_cfg != kBDtlConfig + 1) return -1;
    if (h->force_splitk > 1) return -1;
    if ((uintptr_t)g.A % 16 != 0 || (uintptr_t)g.B % 16 != 0 || g.lda % 8 != 0 || g.ldb % 8 != 0) return -1;
    if (g.batch > 1 && (g.sA % 8 != 0 || g.sB % 8 != 0)) return -1;
    // the 128 x 128 form of the kernel: whole 128-wide tiles
    const bool small_ok = g.M % BDtlCfgT<2>::BM == 0 && g.N % BDtlCfgT<2>::BN == 0 && g.K % BDtlCfgT<2>::BK == 0 &&
                          g.K >= BDtlCfgT<2>::BK;
    if (h->force_cfg == kBDtlConfig + 1) return small_ok ? kBDtlConfig + 1 : -1;
    const bool big_ok = g.M % BDtlCfg::BM == 0 && g.N % BDtlCfg::BN == 0 && g.K % BDtlCfg::BK == 0 && g.K >= BDtlCfg::BK;
    if (h->force_cfg == kBDtlConfig) return big_ok ? kBDtlConfig : -1;
    if (g.K < 8 * BDtlCfg::BK) return -1;
    // 256 x 256 tiles from a little over half a chip of them: 3072^3 (144 tiles) 59.5 us against 75.0 on the
    // register-staged 128 x 128 tiles; level at 128 tiles (4096 x 2048 x 2048: 43.7 against 42.9), behind at 100.
    if (big_ok && 2LL * (g.M / BDtlCfg::BM) * (g.N / BDtlCfg::BN) * g.batch > h->num_cu) return kBDtlConfig;
    // 128 x 128 tiles when they number between a quarter of a chip and a chip and K is not long: 2048^3 24.7 us against
    // 27.6, 1536^3 17.1 against 20.9, 2048 x 1024 x 1024 10.9 against 15.2, 1024^3 10.0 against 12.1 (64 x 64 x 128 tiles);
    // with more tiles the register-staged kernel shares the compute unit better (2560^3 45.5 against 50.8), with a long K
    // and few tiles the 64 x 64 tiles win (1024 x 1024 x 4096: 21.9 against 36.0).
    if (small_ok && g.K <= 2048) {
        const long long t128 = (long long)(g.M / BDtlCfgT<2>::BM) * (g.N / BDtlCfgT<2>::BN) * g.batch;
        if (4 * t128 >= h->num_cu && t128 <= h->num_cu) return kBDtlConfig + 1;
    }
    return -1;
}

// Operand pointers travel as const float* whatever the storage; A and B of SNHIP_MATH_BF16_STORED hold 2-byte
// elements and their strides count those, so host-side offsets are applied in bytes.
inline const float* advance_operand(const float* base, long long elements, int math) {
    if (base == nullptr) return nullptr;
    const long long elem_bytes = snhip_operand_element_bytes(math);
    return reinterpret_cast<const float*>(reinterpret_cast<const char*>(base) + elements * elem_bytes);
}

int gemm_core(Handle* h, const GemmArgs& g) {
    if (h == nullptr) return SNHIP_STATUS_NOT_INITIALIZED;
    const int math = (g.math < 0) ? h->math_mode : g.math;
    h->last_error[0] = 0;  // the text belongs to the call that set it
    {
        // The handle belongs to one device (GPUWrapper.AssociateCurrentThreadWithDevice, GPUWrapper.cs:782-788);
        // a caller thread whose current device differs is switched to it, as cudaSetDevice would have been.
        int cur = -1;
        if (hipGetDevice(&cur) != hipSuccess) return SNHIP_STATUS_NOT_INITIALIZED;
        if (cur != h->device && hipSetDevice(h->device) != hipSuccess) return SNHIP_STATUS_NOT_INITIALIZED;
    }
    const int M = g.M, N = g.N, K = g.K, batch = g.batch;
    if (M < 0 || N < 0 || K < 0 || batch < 0 || g.batch_inner < 0) return SNHIP_STATUS_INVALID_VALUE;
    if (math != SNHIP_MATH_FP32 && math != SNHIP_MATH_BF16_INPUT && math != SNHIP_MATH_BF16_STORED)
        return SNHIP_STATUS_INVALID_VALUE;
    if (g.act < ACT_NONE || g.act > ACT_TANH) return SNHIP_STATUS_NOT_SUPPORTED;
    if (g.colsum != nullptr && !g.tA) return SNHIP_STATUS_NOT_SUPPORTED;  // only sums along the k of a transposed A
    if (g.colsum != nullptr && math == SNHIP_MATH_BF16_STORED) return SNHIP_STATUS_NOT_SUPPORTED;  // sums read fp32
    if (M == 0 || N == 0 || batch == 0) return SNHIP_STATUS_SUCCESS;
    if (g.C == nullptr || g.ldc < N) return SNHIP_STATUS_INVALID_VALUE;
    if (g.D != nullptr && g.ldd < N) return SNHIP_STATUS_INVALID_VALUE;
    const int inner = (g.batch_inner > 0) ? g.batch_inner : batch;
    if (batch % inner != 0) return SNHIP_STATUS_INVALID_VALUE;
    if (inner < batch) {
        // A two-level batch that is really one level - a single matrix per outer step, or outer strides that continue
        // the inner ones - is run as one: every kernel walks a single-level batch, only the extended fp32 ones a
        // two-level one (the others would be launched once per outer step).
        const bool has_d = g.D != nullptr && g.gamma != 0.0f;
        GemmArgs one = g;
        one.batch_inner = 0;
        if (inner == 1) {
            one.sA = g.sA2, one.sB = g.sB2, one.sC = g.sC2, one.sD = g.sD2;
            return gemm_core(h, one);
        }
        if (g.sA2 == inner * g.sA && g.sB2 == inner * g.sB && g.sC2 == inner * g.sC && (!has_d || g.sD2 == inner * g.sD))
            return gemm_core(h, one);
    }
    if (batch > 65535) {
        // grid.y carries batch * splitk: a longer single-level batch goes out in slices (cuBLAS takes any batchCount)
        if (inner < batch) return SNHIP_STATUS_NOT_SUPPORTED;
        GemmArgs part = g;
        part.batch_inner = 0;
        for (int z0 = 0; z0 < batch; z0 += 65535) {
            part.batch = (batch - z0 < 65535) ? (batch - z0) : 65535;
            part.A = advance_operand(g.A, (long long)z0 * g.sA, math);
            part.B = advance_operand(g.B, (long long)z0 * g.sB, math);
            part.C = g.C + (long long)z0 * g.sC;
            part.D = (g.D != nullptr) ? g.D + (long long)z0 * g.sD : nullptr;
            part.colsum = (g.colsum != nullptr) ? g.colsum + (long long)z0 * M : nullptr;
            const int st = gemm_core(h, part);
            if (st != SNHIP_STATUS_SUCCESS) return st;
        }
        return SNHIP_STATUS_SUCCESS;
    }
    const bool multi = batch > 1;
    const bool two_level = multi && inner < batch;

    // everything that can follow alpha * A.B + bias + beta * C
    Epilogue ep;
    ep.bias = g.bias;
    ep.addend = (g.gamma != 0.0f) ? g.D : nullptr;
    ep.ldd = g.ldd;
    ep.strideD = g.sD;
    ep.strideD2 = g.sD2;
    ep.gamma = g.gamma;
    ep.act = g.act;
    ep.act_param = (g.act == ACT_RELU) ? 0.0f : g.act_param;

    hipError_t e;
    // C = act(1 * C + gamma * D) as a pass of its own: used for what the chosen GEMM kernel does not apply itself
    auto after_pass = [&](const float* addend, int act) -> int {
        Epilogue ea = ep;
        ea.bias = nullptr;
        ea.addend = addend;
        ea.act = act;
        const long long total = (long long)M * N * batch;
        const int blocks = (int)((total + 255) / 256 < 65536 ? (total + 255) / 256 : 65536);
        hipLaunchKernelGGL(scale_c_kernel, dim3(blocks), dim3(256), 0, h->stream, g.C, ea, M, N, g.ldc, g.sC, g.sC2, inner,
                           batch, 1.0f);
        return hip_to_status(hipGetLastError());
    };
    // op(A) = A^T: A[z] is K x M with row pitch lda, so the sum over k is a plain column sum (zeros when K == 0)
    auto standalone_colsum = [&]() -> int {
        if (K > 0 && g.A == nullptr) return SNHIP_STATUS_INVALID_VALUE;
        for (int zo = 0; zo < batch / inner; ++zo) {
            const int st = launch_column_sum(h, g.A + (long long)zo * g.sA2, g.colsum + (long long)zo * inner * M, K, M,
                                             (long long)g.lda, g.sA, inner);
            if (st != SNHIP_STATUS_SUCCESS) return st;
        }
        return SNHIP_STATUS_SUCCESS;
    };
    if (K == 0 || g.alpha == 0.0f) {
        // BLAS semantics: A and B are not referenced by the product, C = beta * C (then the rest of the epilogue).
        if (g.colsum != nullptr) {
            const int st = standalone_colsum();
            if (st != SNHIP_STATUS_SUCCESS) return st;
        }
        if (g.beta == 1.0f && ep.bias == nullptr && ep.addend == nullptr && ep.act == ACT_NONE)
            return SNHIP_STATUS_SUCCESS;
        const long long total = (long long)M * N * batch;
        const int blocks = (int)((total + 255) / 256 < 65536 ? (total + 255) / 256 : 65536);
        hipLaunchKernelGGL(scale_c_kernel, dim3(blocks), dim3(256), 0, h->stream, g.C, ep, M, N, g.ldc, g.sC, g.sC2, inner,
                           batch, g.beta);
        return hip_to_status(hipGetLastError());
    }
    if (g.A == nullptr || g.B == nullptr) return SNHIP_STATUS_INVALID_VALUE;
    if (g.lda < (g.tA ? M : K) || g.ldb < (g.tB ? K : N)) return SNHIP_STATUS_INVALID_VALUE;

    if (math == SNHIP_MATH_BF16_STORED) {
        // bf16 storage is read in 16-byte vectors of eight elements from 4-byte-aligned addresses: rows and
        // matrices must start on even element offsets
        if ((uintptr_t)g.A % 4 != 0 || (uintptr_t)g.B % 4 != 0 || g.lda % 2 != 0 || g.ldb % 2 != 0 ||
            (multi && (g.sA % 2 != 0 || g.sB % 2 != 0)) || (two_level && (g.sA2 % 2 != 0 || g.sB2 % 2 != 0)))
            return SNHIP_STATUS_NOT_SUPPORTED;
    }
    // bf16-input arithmetic on a large product of whole tiles: round both operands to bf16 once, into the workspace and
    // into the k-contiguous form (A plain, B transposed), and multiply them with the bf16-storage kernel fed by direct
    // loads.  Each fp32 element is then read once by a streaming pass instead of once per tile that needs it, which is
    // what bounds the fp32-storage kernels (8192^3 on MI355X: NN 1.59 -> 1.00 ms, NT 1.43 -> 0.99 ms, TN 1.18 -> 1.01 ms,
    // the conversion included; a transposing pass over an 8192^2 operand takes 0.085 ms, a plain one 0.07 ms).  Same
    // rounding, same products; the sums may be grouped differently.
    if (math == SNHIP_MATH_BF16_INPUT && !g.no_alloc && batch == 1 && h->force_cfg < 0 && h->force_splitk <= 0 &&
        ep.addend == nullptr && ep.act == ACT_NONE && g.colsum == nullptr &&
        M % BDtlCfg::BM == 0 && N % BDtlCfg::BN == 0 && K % BDtlCfg::BK == 0 && K >= 8 * BDtlCfg::BK &&
        (long long)(M / BDtlCfg::BM) * (N / BDtlCfg::BN) >= h->num_cu &&
        2 * ((size_t)M + N) * K <= kMaxWorkspaceBytes) {
        const size_t a_elems = (size_t)M * K, b_elems = (size_t)N * K;
        GemmArgs s = g;
        s.math = SNHIP_MATH_BF16_STORED;
        s.tA = false, s.tB = true;
        // (the kernel's conditions are checked on a 256-byte aligned stand-in for the workspace, which is not grown
        // before the route is known to be taken)
        s.A = s.B = reinterpret_cast<const float*>(uintptr_t(256));
        s.lda = s.ldb = K;
        if (prefer_dtl(h, s, SNHIP_MATH_BF16_STORED, false) == kBDtlConfig) {
            int st = ensure_workspace(h, 2 * (a_elems + b_elems));
            if (st != SNHIP_STATUS_SUCCESS) return st;
            __bf16* wa = reinterpret_cast<__bf16*>(h->ws);
            __bf16* wb = wa + a_elems;
            s.A = reinterpret_cast<const float*>(wa);
            s.B = reinterpret_cast<const float*>(wb);
            // (an operand that is already k-contiguous without padding takes the one-dimensional pass: 16-byte pieces)
            if (g.tA)
                st = snhip_convert_f32_to_bf16_2d(h, g.A, K, M, g.lda, 1, wa, K);
            else if (g.lda == K)
                st = snhip_convert_f32_to_bf16(h, g.A, wa, (long long)a_elems);
            else
                st = snhip_convert_f32_to_bf16_2d(h, g.A, M, K, g.lda, 0, wa, K);
            if (st != SNHIP_STATUS_SUCCESS) return st;
            if (!g.tB)
                st = snhip_convert_f32_to_bf16_2d(h, g.B, K, N, g.ldb, 1, wb, K);
            else if (g.ldb == K)
                st = snhip_convert_f32_to_bf16(h, g.B, wb, (long long)b_elems);
            else
                st = snhip_convert_f32_to_bf16_2d(h, g.B, N, K, g.ldb, 0, wb, K);
            if (st != SNHIP_STATUS_SUCCESS) return st;
            return gemm_core(h, s);
        }
    }
    // Operands stored as bf16, a large product of whole tiles, but not in the k-contiguous form: the operand(s) lying the
    // other way are transposed once into the workspace (2 bytes read and written per element) and the product runs in
    // the direct-load kernel.  The register-transposing kernels lose more than the pass costs (8192^3: NN 1.13 ms, TN
    // 1.41 ms against 0.95 ms in the k-contiguous form).  Same values multiplied; the sums may be grouped differently.
    if (math == SNHIP_MATH_BF16_STORED && !g.no_alloc && batch == 1 && h->force_cfg < 0 && h->force_splitk <= 0 &&
        (g.tA || !g.tB) && ep.addend == nullptr && ep.act == ACT_NONE && g.colsum == nullptr && M % BDtlCfg::BM == 0 &&
        N % BDtlCfg::BN == 0 && K % BDtlCfg::BK == 0 && K >= 8 * BDtlCfg::BK &&
        (long long)(M / BDtlCfg::BM) * (N / BDtlCfg::BN) >= h->num_cu && 2 * ((size_t)M + N) * K <= kMaxWorkspaceBytes) {
        const size_t a_elems = g.tA ? (size_t)M * K : 0, b_elems = !g.tB ? (size_t)N * K : 0;
        // (checked against the caller's pointers and a 256-byte aligned stand-in for the workspace, which may not
        // exist yet)
        const void* const aligned = reinterpret_cast<const void*>(uintptr_t(256));
        const bool ok_a = !g.tA || wide_transpose_ok(g.A, K, M, g.lda, 2, aligned, K);
        const bool ok_b = g.tB || wide_transpose_ok(g.B, K, N, g.ldb, 2, aligned, K);
        GemmArgs s = g;
        s.math = SNHIP_MATH_BF16_STORED;
        s.tA = false, s.tB = true;
        if (g.tA) s.A = reinterpret_cast<const float*>(uintptr_t(256)), s.lda = K;
        if (!g.tB) s.B = reinterpret_cast<const float*>(uintptr_t(256)), s.ldb = K;
        if (ok_a && ok_b && prefer_dtl(h, s, SNHIP_MATH_BF16_STORED, false) == kBDtlConfig) {
            int st = ensure_workspace(h, 2 * (a_elems + b_elems));
            if (st != SNHIP_STATUS_SUCCESS) return st;
            __bf16* wa = reinterpret_cast<__bf16*>(h->ws);
            __bf16* wb = wa + a_elems;
            if (g.tA) {
                st = transpose_bf16(h, g.A, K, M, g.lda, wa, K);
                if (st != SNHIP_STATUS_SUCCESS) return st;
                s.A = reinterpret_cast<const float*>(wa);
            }
            if (!g.tB) {
                st = transpose_bf16(h, g.B, K, N, g.ldb, wb, K);
                if (st != SNHIP_STATUS_SUCCESS) return st;
                s.B = reinterpret_cast<const float*>(wb);
            }
            return gemm_core(h, s);
        }
    }
    Choice ch = choose(h, M, N, K, batch, kind_of_math(math), g.tA, g.tB);
    const int ks_cfg = prefer_ksplit(h, g, math, two_level);
    if (ks_cfg >= 0) ch = Choice{ks_cfg, 1};
    {
        const bool relu = (ep.act == ACT_RELU || ep.act == ACT_LEAKY_RELU);
        const int st_cfg = prefer_stream(h, g, math, two_level, ep.addend != nullptr || relu || g.colsum != nullptr);
        if (st_cfg >= 0 && ks_cfg < 0) ch = Choice{st_cfg, 1};
    }
    {
        const bool relu = (ep.act == ACT_RELU || ep.act == ACT_LEAKY_RELU);
        const int dtl_cfg = prefer_dtl(h, g, math, ep.addend != nullptr || relu || g.colsum != nullptr || two_level);
        if (dtl_cfg >= 0 && ch.cfg != kBStreamStoredConfig && ch.cfg != kBStreamStoredConfig + 1) ch = Choice{dtl_cfg, 1};
    }
    const ConfigEntry& cfg = kConfigs[ch.cfg];
    if ((long long)batch * ch.splitk > 65535) ch.splitk = 1;
    if (g.no_alloc && h->force_splitk <= 0) {
        // an automatically chosen split is halved until its partial sums fit the static scratch (a forced one is refused
        // below if it does not): the product then runs with fewer K slices than the allocating entry point would use
        while (ch.splitk > 1 && (size_t)M * N * batch * ch.splitk * sizeof(float) > kStaticScratchBytes) ch.splitk /= 2;
    }

    // The extended kernels apply gamma * D and the (leaky) ReLU while writing C, walk a two-level batch, and -
    // transposed A, plain B, no split-K - add up the column sum on the side.  They are used only when one of
    // those is asked for; a configuration without them (the bf16-input kernels) gets the same results from the
    // plain kernel plus passes over C / A, and one launch per outer batch step.
    const KernelFn fn_ext = cfg.fn_ext[g.tA ? 1 : 0][g.tB ? 1 : 0];
    const bool relu_family = (ep.act == ACT_RELU || ep.act == ACT_LEAKY_RELU);
    // (the k-range hint is worth an extended kernel only for a K long enough to have whole tiles to skip)
    const bool want_ext = ep.addend != nullptr || relu_family || two_level || g.colsum != nullptr ||
                          (g.k_from_m && g.tA && K >= 4 * cfg.BK && cfg.kind == 0);
    const bool use_ext = want_ext && fn_ext != nullptr;
    if (two_level && !use_ext) {
        GemmArgs part = g;
        part.batch = inner;
        part.batch_inner = 0;
        for (int zo = 0; zo < batch / inner; ++zo) {
            part.A = advance_operand(g.A, (long long)zo * g.sA2, math);
            part.B = advance_operand(g.B, (long long)zo * g.sB2, math);
            part.C = g.C + (long long)zo * g.sC2;
            part.D = (g.D != nullptr) ? g.D + (long long)zo * g.sD2 : nullptr;
            part.colsum = (g.colsum != nullptr) ? g.colsum + (long long)zo * inner * M : nullptr;
            const int st = gemm_core(h, part);
            if (st != SNHIP_STATUS_SUCCESS) return st;
        }
        return SNHIP_STATUS_SUCCESS;
    }
    const bool fuse_colsum = use_ext && g.colsum != nullptr && ch.splitk == 1 && g.tA && !g.tB && kConfigs[ch.cfg].kind != 2;
    // what is left for a pass over C afterwards: sigmoid / tanh always, and addend / ReLU when the kernel is plain
    const float* addend_after = use_ext ? nullptr : ep.addend;
    const int act_after = (use_ext && relu_family) ? ACT_NONE : ep.act;
    Epilogue ep_kernel = ep;
    if (!use_ext) ep_kernel.addend = nullptr;
    ep_kernel.act = (use_ext && relu_family) ? ep.act : ACT_NONE;

    GemmParams p;
    p.A = g.A;
    p.B = g.B;
    p.C = g.C;
    p.ep = ep_kernel;
    p.colsum = fuse_colsum ? g.colsum : nullptr;
    p.ws = nullptr;
    p.M = M;
    p.N = N;
    p.K = K;
    p.lda = g.lda;
    p.ldb = g.ldb;
    p.ldc = g.ldc;
    p.strideA = g.sA;
    p.strideB = g.sB;
    p.strideC = g.sC;
    p.strideA2 = g.sA2;
    p.strideB2 = g.sB2;
    p.strideC2 = g.sC2;
    p.batch_inner = inner;
    p.tiles_m = ceil_div(M, cfg.BM);
    p.tiles_n = ceil_div(N, cfg.BN);
    p.splitk = ch.splitk;
    p.kchunk = ceil_div(ceil_div(K, ch.splitk), cfg.BK) * cfg.BK;
    p.alpha = g.alpha;
    p.beta = g.beta;
    p.group_m = 8;
    p.flags = 0;
    p.counters = nullptr;
    const long long ntiles = (long long)p.tiles_m * p.tiles_n;
    if (ntiles * batch * ch.splitk > 0x7fffffffLL) return SNHIP_STATUS_NOT_SUPPORTED;  // one-dimensional grid
    p.nz = batch * ch.splitk;
    const bool c_vec = ((uintptr_t)g.C % 16 == 0) && (g.ldc % 4 == 0) && (!multi || g.sC % 4 == 0) &&
                       (!two_level || g.sC2 % 4 == 0) && (g.bias == nullptr || (uintptr_t)g.bias % 16 == 0) &&
                       (ep_kernel.addend == nullptr ||
                        ((uintptr_t)ep_kernel.addend % 16 == 0 && g.ldd % 4 == 0 && (!multi || g.sD % 4 == 0) &&
                         (!two_level || g.sD2 % 4 == 0)));
    if (c_vec) p.flags |= GEMM_FLAG_C_VEC;
    if (g.k_from_m && g.tA && use_ext && cfg.kind == 0) {
        p.flags |= GEMM_FLAG_K_FROM_M;
        // tiles then do unequal work: deal them out longest first when the grid has the regular shape that order is
        // written for (one tile column, no split, whole matrices per XCD)
        if (p.tiles_n == 1 && ch.splitk == 1 && batch % 8 == 0 && h->num_cu % 8 == 0 && p.tiles_m > 1) {
            p.flags |= GEMM_FLAG_LONGEST_FIRST;
            p.group_m = h->num_cu / 8;
        }
    }
    if (cfg.kind == 2 && M <= N) p.flags |= GEMM_FLAG_TILE_N_FASTEST;  // the K-split kernel keeps B's column blocks per XCD
    bool fused_reduce = false;
    if (ch.splitk > 1) {
        const size_t need = (size_t)M * N * batch * ch.splitk * sizeof(float);
        int st = SNHIP_STATUS_SUCCESS;
        if (g.no_alloc) {
            if (need > kStaticScratchBytes || h->static_scratch == nullptr) {
                snprintf(h->last_error, sizeof(h->last_error),
                         "snhip_dot_noalloc: %d x %d x %d with split-K %d needs %zu bytes of partial sums, the static "
                         "scratch holds %zu", M, N, K, ch.splitk, need, kStaticScratchBytes);
                return SNHIP_STATUS_NOT_SUPPORTED;
            }
            p.ws = h->static_scratch;
        } else {
            st = ensure_workspace(h, need);
            if (st != SNHIP_STATUS_SUCCESS) return st;
            p.ws = h->ws;
        }
        if (N % 4 == 0) p.flags |= GEMM_FLAG_WS_VEC;
        fused_reduce = (h->splitk_mode == 2) && !g.no_alloc;  // the arrival counters would have to be allocated
        if (fused_reduce) {
            st = ensure_counters(h, (size_t)(ntiles * batch));
            if (st != SNHIP_STATUS_SUCCESS) return st;
            p.counters = h->counters;
        }
    }
    h->last_cfg = ch.cfg;
    h->last_splitk = ch.splitk;

    const KernelFn fn = use_ext ? fn_ext : cfg.fn[g.tA ? 1 : 0][g.tB ? 1 : 0];
    if (cfg.kind == 2) {  // the K-split kernel reads tile and matrix from a two-dimensional grid
        hipLaunchKernelGGL(fn, dim3((unsigned)ntiles, (unsigned)batch), dim3(cfg.NT), cfg.lds_bytes, h->stream, p);
    } else if (cfg.kind == 3 || cfg.kind == 5 || cfg.kind == 6) {
        // persistent workgroups: as many as fit on the chip at once, the same number on every XCD
        long long wgs = (long long)cfg.occ * h->num_cu;
        if (wgs > ntiles * p.nz) wgs = ntiles * p.nz;
        if (wgs >= 8) wgs -= wgs % 8;
        hipLaunchKernelGGL(fn, dim3((unsigned)wgs), dim3(cfg.NT), cfg.lds_bytes, h->stream, p);
    } else
        hipLaunchKernelGGL(fn, dim3((unsigned)(ntiles * p.nz)), dim3(cfg.NT), cfg.lds_bytes, h->stream, p);
    e = hipGetLastError();
    if (e != hipSuccess) return hip_to_status(e);

    if (ch.splitk > 1 && !fused_reduce) {
        // the reduction kernel applies the whole epilogue itself, whatever kind of GEMM kernel produced the partials
        Epilogue er = ep;
        er.addend = use_ext ? ep.addend : nullptr;
        er.act = ep_kernel.act;
        const long long total = (long long)M * N * batch;
        const int blocks = (int)((total + 255) / 256 < 4096 ? (total + 255) / 256 : 4096);
        hipLaunchKernelGGL(splitk_reduce_kernel, dim3(blocks), dim3(256), 0, h->stream, (const float*)p.ws, g.C, er, M, N,
                           g.ldc, g.sC, g.sC2, inner, ch.splitk, batch, g.alpha, g.beta);
        e = hipGetLastError();
        if (e != hipSuccess) return hip_to_status(e);
    }
    if (addend_after != nullptr || act_after != ACT_NONE) {
        const int st = after_pass(addend_after, act_after);
        if (st != SNHIP_STATUS_SUCCESS) return st;
    }
    if (g.colsum != nullptr && !fuse_colsum) return standalone_colsum();
    return SNHIP_STATUS_SUCCESS;
}

// Plain strided-batched product with an optional bias: the shape every entry point that predates the
// descriptor call reduces to.
int gemm_rm(Handle* h, bool tA, bool tB, int M, int N, int K, float alpha, const float* A, int lda, long long sA,
            const float* B, int ldb, long long sB, float beta, float* C, int ldc, long long sC, int batch,
            const float* bias, int math = -1) {
    GemmArgs g;
    g.tA = tA, g.tB = tB, g.M = M, g.N = N, g.K = K, g.alpha = alpha, g.beta = beta;
    g.A = A, g.lda = lda, g.sA = sA, g.B = B, g.ldb = ldb, g.sB = sB, g.C = C, g.ldc = ldc, g.sC = sC;
    g.batch = batch, g.bias = bias, g.math = math;
    return gemm_core(h, g);
}

inline bool op_is_trans(int op, bool* ok) {
    *ok = (op == SNHIP_OP_N || op == SNHIP_OP_T || op == SNHIP_OP_C);
    return op != SNHIP_OP_N;
}

// Kernels whose LDS stage exceeds the 64 KiB default need an explicit opt-in; it is a property of the function on a
// device, so it is set once per device (every handle created later on that device finds it done).
hipError_t prepare_kernels_once(int dev) {
    static std::mutex mu;
    static bool done[kMaxDevices] = {};
    if (dev < 0 || dev >= kMaxDevices) return hipErrorInvalidDevice;
    std::lock_guard<std::mutex> lock(mu);
    if (done[dev]) return hipSuccess;
    hipError_t e = hipSuccess;
    for (int c = 0; c < kNumConfigs; ++c) {
        for (int ta = 0; ta < 2; ++ta)
            for (int tb = 0; tb < 2; ++tb) {
                if (kConfigs[c].fn[ta][tb] == nullptr) continue;
                e = hipFuncSetAttribute(reinterpret_cast<const void*>(kConfigs[c].fn[ta][tb]),
                                        hipFuncAttributeMaxDynamicSharedMemorySize, kConfigs[c].lds_bytes);
                if (e != hipSuccess) return e;
            }
        for (int ta = 0; ta < 2; ++ta)
            for (int tb = 0; tb < 2; ++tb) {
                if (kConfigs[c].fn_ext[ta][tb] == nullptr) continue;
                e = hipFuncSetAttribute(reinterpret_cast<const void*>(kConfigs[c].fn_ext[ta][tb]),
                                        hipFuncAttributeMaxDynamicSharedMemorySize, kConfigs[c].lds_bytes);
                if (e != hipSuccess) return e;
            }
    }
    for (const AttnEntry& c : kAttn) {
        e = hipFuncSetAttribute(reinterpret_cast<const void*>(c.fn), hipFuncAttributeMaxDynamicSharedMemorySize,
                                c.lds_bytes);
        if (e != hipSuccess) return e;
    }
    for (const AttnEntry& c : kAttnBwd) {
        e = hipFuncSetAttribute(reinterpret_cast<const void*>(c.fn), hipFuncAttributeMaxDynamicSharedMemorySize,
                                c.lds_bytes);
        if (e != hipSuccess) return e;
    }
    for (const Attn16Entry& c : kAttn16) {
        e = hipFuncSetAttribute(reinterpret_cast<const void*>(c.fn), hipFuncAttributeMaxDynamicSharedMemorySize,
                                c.lds_bytes);
        if (e != hipSuccess) return e;
    }
    for (const Attn16Entry& c : kAttn16Bwd) {
        e = hipFuncSetAttribute(reinterpret_cast<const void*>(c.fn), hipFuncAttributeMaxDynamicSharedMemorySize,
                                c.lds_bytes);
        if (e != hipSuccess) return e;
    }
    e = hipFuncSetAttribute(reinterpret_cast<const void*>(attention_fwd16_bf16_kernel<256>),
                            hipFuncAttributeMaxDynamicSharedMemorySize, Attn16BCfg<256>::LDS_BYTES);
    if (e != hipSuccess) return e;
    e = hipFuncSetAttribute(reinterpret_cast<const void*>(attention_fwd16_bf16_kernel<128>),
                            hipFuncAttributeMaxDynamicSharedMemorySize, Attn16BCfg<128>::LDS_BYTES);
    if (e != hipSuccess) return e;
    e = hipFuncSetAttribute(reinterpret_cast<const void*>(attention_fwd16_bf16_kernel<256, true>),
                            hipFuncAttributeMaxDynamicSharedMemorySize, Attn16BCfg<256>::LDS_BYTES);
    if (e != hipSuccess) return e;
    e = hipFuncSetAttribute(reinterpret_cast<const void*>(attention_fwd16_bf16_kernel<128, true>),
                            hipFuncAttributeMaxDynamicSharedMemorySize, Attn16BCfg<128>::LDS_BYTES);
    if (e != hipSuccess) return e;
    e = hipFuncSetAttribute(reinterpret_cast<const void*>(attention_fwd16_long_kernel<false>),
                            hipFuncAttributeMaxDynamicSharedMemorySize, Attn16Cfg<256>::LDS_BYTES);
    if (e != hipSuccess) return e;
    e = hipFuncSetAttribute(reinterpret_cast<const void*>(attention_fwd16_long_kernel<true>),
                            hipFuncAttributeMaxDynamicSharedMemorySize, Attn16Cfg<256>::LDS_BYTES);
    if (e != hipSuccess) return e;
    e = hipFuncSetAttribute(reinterpret_cast<const void*>(attention_fwd16_long_kernel<false, false, true>),
                            hipFuncAttributeMaxDynamicSharedMemorySize, Attn16Cfg<256>::LDS_BYTES);
    if (e != hipSuccess) return e;
    e = hipFuncSetAttribute(reinterpret_cast<const void*>(attention_fwd16_long_kernel<false, false, false, 32>),
                            hipFuncAttributeMaxDynamicSharedMemorySize, Attn16Cfg<256, 32>::LDS_BYTES);
    if (e != hipSuccess) return e;
    e = hipFuncSetAttribute(reinterpret_cast<const void*>(attention_fwd16_long_kernel<true, false, false, 32>),
                            hipFuncAttributeMaxDynamicSharedMemorySize, Attn16Cfg<256, 32>::LDS_BYTES);
    if (e != hipSuccess) return e;
    e = hipFuncSetAttribute(reinterpret_cast<const void*>(attention_fwd16_long_kernel<false, false, true, 32>),
                            hipFuncAttributeMaxDynamicSharedMemorySize, Attn16Cfg<256, 32>::LDS_BYTES);
    if (e != hipSuccess) return e;
    e = hipFuncSetAttribute(reinterpret_cast<const void*>(attention_fwd16_long_kernel<false, true>),
                            hipFuncAttributeMaxDynamicSharedMemorySize, Attn16BCfg<256>::LDS_BYTES);
    if (e != hipSuccess) return e;
    e = hipFuncSetAttribute(reinterpret_cast<const void*>(attention_fwd16_long_kernel<true, true>),
                            hipFuncAttributeMaxDynamicSharedMemorySize, Attn16BCfg<256>::LDS_BYTES);
    if (e != hipSuccess) return e;
    e = hipFuncSetAttribute(reinterpret_cast<const void*>(attention_fwd_long_kernel<32>),
                            hipFuncAttributeMaxDynamicSharedMemorySize, AttnCfg<8, 32>::LDS_BYTES);
    if (e != hipSuccess) return e;
    e = hipFuncSetAttribute(reinterpret_cast<const void*>(attention_fwd_long_kernel<64>),
                            hipFuncAttributeMaxDynamicSharedMemorySize, AttnCfg<8, 64>::LDS_BYTES);
    if (e != hipSuccess) return e;
    e = rnn_prepare_kernels();
    if (e != hipSuccess) return e;
    done[dev] = true;
    return hipSuccess;
}

}  // namespace

// Dense-layer backward on a small batch: when dW and dx are each a product that prefer_ksplit() would give 32 x 32
// tiles with K split over four wavefronts, the two products and the bias gradient go out as ONE launch
// (dense_backward_small_kernel).  Returns kNotTaken when the layer does not qualify (the caller then issues the
// products one by one), else the status of the launch.
constexpr int kNotTaken = -1;
int dense_backward_small(Handle* h, float* dx, float* dW, float* db, const float* x, const float* dy, const float* W,
                         int rows, int in_features, int out_features, float multiplier, float weight_decay_alpha,
                         const float* bias, float bias_decay_alpha) {
    if (h->math_mode != SNHIP_MATH_FP32 || h->force_cfg >= 0 || h->force_splitk > 0) return kNotTaken;
    if (rows <= 0 || in_features <= 0 || out_features <= 0 || x == nullptr || dy == nullptr || W == nullptr) return kNotTaken;
    if (multiplier == 0.0f) return kNotTaken;  // alpha == 0: A and B are not referenced, another path
    GemmArgs gw;  // dW = multiplier * dy^T . x + weight_decay_alpha * W
    gw.tA = true;
    gw.M = out_features, gw.N = in_features, gw.K = rows;
    gw.alpha = multiplier;
    gw.A = dy, gw.lda = out_features, gw.B = x, gw.ldb = in_features, gw.C = dW, gw.ldc = in_features;
    gw.D = W, gw.ldd = in_features, gw.gamma = weight_decay_alpha;
    GemmArgs gx;  // dx = dy . W
    gx.M = rows, gx.N = in_features, gx.K = out_features;
    gx.A = dy, gx.lda = out_features, gx.B = W, gx.ldb = in_features, gx.C = dx, gx.ldc = in_features;
    // each product: one the K-split kernels take (alignment, K), with at most one 32 x 32 tile per compute unit and not so
    // few of them that a long K is better cut eight ways on 16 x 16 tiles
    auto qualifies = [&](const GemmArgs& g) {
        const int c = prefer_ksplit(h, g, SNHIP_MATH_FP32, false);
        if (c != kKsplitConfig && c != kKsplit8Config && c != kKsplit16Config) return false;
        const long long tiles = (long long)ceil_div(g.M, 32) * ceil_div(g.N, 32);
        if (g.K > 1024 || tiles > h->num_cu) return false;
        return !(tiles <= h->num_cu / 4 && g.K >= 512);
    };
    if (!qualifies(gw) || !qualifies(gx)) return kNotTaken;
    {
        int cur = -1;
        if (hipGetDevice(&cur) != hipSuccess) return SNHIP_STATUS_NOT_INITIALIZED;
        if (cur != h->device && hipSetDevice(h->device) != hipSuccess) return SNHIP_STATUS_NOT_INITIALIZED;
    }
    h->last_error[0] = 0;
    auto fill = [](const GemmArgs& g, GemmParams& p) {
        p = GemmParams{};
        p.A = g.A, p.B = g.B, p.C = g.C;
        p.ep.bias = nullptr;
        p.ep.addend = (g.gamma != 0.0f) ? g.D : nullptr;
        p.ep.ldd = g.ldd;
        p.ep.strideD = 0, p.ep.strideD2 = 0;
        p.ep.gamma = g.gamma;
        p.ep.act = ACT_NONE;
        p.ep.act_param = 0.0f;
        p.M = g.M, p.N = g.N, p.K = g.K;
        p.lda = g.lda, p.ldb = g.ldb, p.ldc = g.ldc;
        p.batch_inner = 1;
        p.tiles_m = ceil_div(g.M, 32);
        p.tiles_n = ceil_div(g.N, 32);
        p.splitk = 1;
        p.kchunk = g.K;
        p.alpha = g.alpha, p.beta = 0.0f;
        p.group_m = 8;
        p.nz = 1;
        p.flags = (g.M <= g.N) ? GEMM_FLAG_TILE_N_FASTEST : 0;
    };
    DenseBackwardSmallParams q;
    fill(gw, q.pw);
    fill(gx, q.px);
    // One workgroup per compute unit is resident (the kernel uses more than half of the register file), so a grid
    // beyond the number of compute units runs in two rounds: give the product with more tiles 32 x 64 tiles (two K
    // slices instead of four), then the other one, while that brings the grid under one round.
    q.nt_w = q.nt_x = 1;
    const int blocks_b = (db != nullptr) ? ceil_div(out_features, 64) : 0;
    auto blocks = [&](const GemmParams& p, int nt) { return p.tiles_m * ceil_div(p.N, 32 * nt); };
    if (blocks(q.pw, 1) + blocks(q.px, 1) + blocks_b > h->num_cu) {
        (blocks(q.pw, 1) >= blocks(q.px, 1) ? q.nt_w : q.nt_x) = 2;
        if (blocks(q.pw, q.nt_w) + blocks(q.px, q.nt_x) + blocks_b > h->num_cu) q.nt_w = q.nt_x = 2;
    }
    q.pw.tiles_n = ceil_div(q.pw.N, 32 * q.nt_w);
    q.px.tiles_n = ceil_div(q.px.N, 32 * q.nt_x);
    q.blocks_w = q.pw.tiles_m * q.pw.tiles_n;
    q.blocks_x = q.px.tiles_m * q.px.tiles_n;
    q.dy = dy, q.db = db, q.rows = rows, q.cols = out_features, q.ld = out_features;
    q.bias = (bias_decay_alpha != 0.0f) ? bias : nullptr;
    q.bias_alpha = bias_decay_alpha;
    constexpr int kLdsBytes = KsplitCfg<1, 4>::LDS_BYTES;
    static_assert(KsplitCfg<2, 4>::LDS_BYTES == kLdsBytes, "both tile forms share one LDS size");
    hipLaunchKernelGGL(dense_backward_small_kernel, dim3((unsigned)(q.blocks_w + q.blocks_x + blocks_b)), dim3(256),
                       kLdsBytes, h->stream, q);
    h->last_cfg = kKsplitConfig;
    h->last_splitk = 1;
    return hip_to_status(hipGetLastError());
}

extern "C" {

int snhip_create(void** handle) {
    if (handle == nullptr) return SNHIP_STATUS_INVALID_VALUE;
    *handle = nullptr;
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return SNHIP_STATUS_NOT_INITIALIZED;
    hipDeviceProp_t prop;
    e = hipGetDeviceProperties(&prop, dev);
    if (e != hipSuccess) return SNHIP_STATUS_NOT_INITIALIZED;
    // The code objects in this library exist for gfx950 only.
    if (prop.gcnArchName[0] == '\0' || __builtin_strncmp(prop.gcnArchName, "gfx950", 6) != 0)
        return SNHIP_STATUS_ARCH_MISMATCH;
    e = prepare_kernels_once(dev);
    if (e != hipSuccess) return hip_to_status(e);
    void* scratch_ptr = nullptr;
    e = static_scratch_address(dev, &scratch_ptr);
    if (e != hipSuccess) return hip_to_status(e);
    Handle* h = new (std::nothrow) Handle();
    if (h == nullptr) return SNHIP_STATUS_ALLOC_FAILED;
    h->static_scratch = static_cast<float*>(scratch_ptr);
    h->device = dev;
    h->num_cu = prop.multiProcessorCount > 0 ? prop.multiProcessorCount : 256;
    // (a device too full for it now keeps the lazy growth: the first call that needs workspace tries again)
    (void)ensure_workspace(h, kInitialWorkspaceBytes);
    *handle = h;
    return SNHIP_STATUS_SUCCESS;
}

int snhip_destroy(void* handle) {
    if (handle == nullptr) return SNHIP_STATUS_NOT_INITIALIZED;
    Handle* h = static_cast<Handle*>(handle);
    if (h->ws != nullptr || h->counters != nullptr) {
        (void)hipStreamSynchronize(h->stream);
        if (h->ws != nullptr) (void)hipFree(h->ws);
        if (h->counters != nullptr) (void)hipFree(h->counters);
    }
    delete h;
    return SNHIP_STATUS_SUCCESS;
}

int snhip_reserve_workspace(void* handle, size_t bytes) {
    if (handle == nullptr) return SNHIP_STATUS_NOT_INITIALIZED;
    if (bytes > kMaxWorkspaceBytes) return SNHIP_STATUS_INVALID_VALUE;
    Handle* h = static_cast<Handle*>(handle);
    int cur = -1;
    if (hipGetDevice(&cur) != hipSuccess) return SNHIP_STATUS_NOT_INITIALIZED;
    if (cur != h->device && hipSetDevice(h->device) != hipSuccess) return SNHIP_STATUS_NOT_INITIALIZED;
    return ensure_workspace(h, bytes);
}

int snhip_get_workspace_size(void* handle, size_t* bytes) {
    if (handle == nullptr) return SNHIP_STATUS_NOT_INITIALIZED;
    if (bytes == nullptr) return SNHIP_STATUS_INVALID_VALUE;
    *bytes = static_cast<Handle*>(handle)->ws_bytes;
    return SNHIP_STATUS_SUCCESS;
}

int snhip_set_stream(void* handle, void* stream) {
    if (handle == nullptr) return SNHIP_STATUS_NOT_INITIALIZED;
    static_cast<Handle*>(handle)->stream = static_cast<hipStream_t>(stream);
    return SNHIP_STATUS_SUCCESS;
}

int snhip_get_version(void* handle, int* version) {
    (void)handle;
    if (version == nullptr) return SNHIP_STATUS_INVALID_VALUE;
    *version = kVersion;
    return SNHIP_STATUS_SUCCESS;
}

int snhip_sgemm_strided_batched(void* handle, int transa, int transb, int m, int n, int k, const float* alpha,
                                const void* A, int lda, long long strideA, const void* B, int ldb, long long strideB,
                                const float* beta, void* C, int ldc, long long strideC, int batchCount) {
    if (handle == nullptr) return SNHIP_STATUS_NOT_INITIALIZED;
    if (alpha == nullptr || beta == nullptr) return SNHIP_STATUS_INVALID_VALUE;
    bool oka, okb;
    const bool ta = op_is_trans(transa, &oka), tb = op_is_trans(transb, &okb);
    if (!oka || !okb) return SNHIP_STATUS_INVALID_VALUE;
    if (m < 0 || n < 0 || k < 0 || batchCount < 0) return SNHIP_STATUS_INVALID_VALUE;
    // cuBLAS leading-dimension rules for column-major storage
    const int rows_a = ta ? k : m, rows_b = tb ? n : k;
    if (lda < (rows_a > 1 ? rows_a : 1) || ldb < (rows_b > 1 ? rows_b : 1) || ldc < (m > 1 ? m : 1))
        return SNHIP_STATUS_INVALID_VALUE;
    // A column-major matrix with leading dimension ld is the row-major transpose
    // with row pitch ld.  C^T (n x m) = op(B)^T * op(A)^T, so in row-major terms the
    // left operand is B (transposed iff transb) and the right operand is A.
    return gemm_rm(static_cast<Handle*>(handle), tb, ta, n, m, k, *alpha, static_cast<const float*>(B), ldb, strideB,
                   static_cast<const float*>(A), lda, strideA, *beta, static_cast<float*>(C), ldc, strideC, batchCount,
                   nullptr);
}

int snhip_sgemm(void* handle, int transa, int transb, int m, int n, int k, const float* alpha, const void* A, int lda,
                const void* B, int ldb, const float* beta, void* C, int ldc) {
    return snhip_sgemm_strided_batched(handle, transa, transb, m, n, k, alpha, A, lda, 0, B, ldb, 0, beta, C, ldc, 0, 1);
}

int snhip_gemm_rm(void* handle, int transposeA, int transposeB, int M, int N, int K, float alpha, const float* A,
                  int lda, long long strideA, const float* B, int ldb, long long strideB, float beta, float* C,
                  int ldc, long long strideC, int batch, const float* bias) {
    return gemm_rm(static_cast<Handle*>(handle), transposeA != 0, transposeB != 0, M, N, K, alpha, A, lda, strideA, B,
                   ldb, strideB, beta, C, ldc, strideC, batch, bias);
}

int snhip_sizeof_attention_desc(void) { return (int)sizeof(snhip_attention_desc); }


int snhip_attention_forward(void* handle, const snhip_attention_desc* d) {
    Handle* h = static_cast<Handle*>(handle);
    if (d == nullptr || d->struct_size != (int)sizeof(snhip_attention_desc)) return SNHIP_STATUS_INVALID_VALUE;
    if (h == nullptr) return SNHIP_STATUS_NOT_INITIALIZED;
    {
        int cur = -1;
        if (hipGetDevice(&cur) != hipSuccess) return SNHIP_STATUS_NOT_INITIALIZED;
        if (cur != h->device && hipSetDevice(h->device) != hipSuccess) return SNHIP_STATUS_NOT_INITIALIZED;
    }
    if (d->batch < 0 || d->batch_inner < 0 || d->Tq < 0 || d->Tk < 0 || d->dk < 0 || d->dv < 0)
        return SNHIP_STATUS_INVALID_VALUE;
    if (d->batch == 0 || d->Tq == 0 || d->dv == 0) return SNHIP_STATUS_SUCCESS;
    if (d->Tk == 0 || d->dk == 0) return SNHIP_STATUS_NOT_SUPPORTED;  // a softmax over no keys is not defined
    if (d->Q == nullptr || d->K == nullptr || d->V == nullptr || d->O == nullptr) return SNHIP_STATUS_INVALID_VALUE;
    if (d->ldq < d->dk || d->ldk < d->dk || d->ldv < d->dv || d->ldo < d->dv) return SNHIP_STATUS_INVALID_VALUE;
    const int inner = d->batch_inner > 0 ? d->batch_inner : d->batch;
    if (d->batch % inner != 0) return SNHIP_STATUS_INVALID_VALUE;
    if (d->batch > 65535) return SNHIP_STATUS_NOT_SUPPORTED;
    const int hd = d->dk > d->dv ? d->dk : d->dv;
    const AttnEntry* e = nullptr;
    for (const AttnEntry& c : kAttn)
        if (d->Tk <= c.keys && hd <= c.hd) {
            e = &c;
            break;
        }
    // more keys than one block holds: the two-pass kernel that walks the keys in blocks of 256 (head dimensions that
    // are multiples of 4, up to 64)
    const bool long_keys = (e == nullptr) && hd <= 64 && d->dk % 4 == 0 && d->dv % 4 == 0;
    if (e == nullptr && !long_keys) return SNHIP_STATUS_NOT_SUPPORTED;

    AttnParams p;
    p.Q = d->Q, p.K = d->K, p.V = d->V, p.O = d->O, p.P = d->weights;
    p.Tq = d->Tq, p.Tk = d->Tk, p.dk = d->dk, p.dv = d->dv;
    p.ldq = d->ldq, p.ldk = d->ldk, p.ldv = d->ldv, p.ldo = d->ldo;
    p.sQ = d->strideQ, p.sK = d->strideK, p.sV = d->strideV, p.sO = d->strideO;
    p.sQ2 = d->strideQ_outer, p.sK2 = d->strideK_outer, p.sV2 = d->strideV_outer, p.sO2 = d->strideO_outer;
    p.batch_inner = inner;
    p.batch = d->batch;
    p.scale = d->scale;
    p.causal = d->causal != 0;
    p.flags = 0;
    const bool multi = d->batch > 1, two_level = multi && inner < d->batch;
    if ((uintptr_t)d->O % 16 == 0 && d->ldo % 4 == 0 && (!multi || d->strideO % 4 == 0) &&
        (!two_level || d->strideO_outer % 4 == 0))
        p.flags |= 1;
    if (d->weights != nullptr && (uintptr_t)d->weights % 16 == 0 && d->Tk % 4 == 0) p.flags |= 2;
    const int tiles = ceil_div(d->Tq, AT_BQ);
    if (long_keys) {
        if (tiles > 65535) return SNHIP_STATUS_NOT_SUPPORTED;
        p.q_tiles = 1;
        constexpr int lds32 = AttnCfg<8, 32>::LDS_BYTES, lds64 = AttnCfg<8, 64>::LDS_BYTES;
        // head dimension exactly 32 or 64 and outputs that take 16-byte stores: the form with two wavefronts per SIMD
        if (d->dk == 32 && d->dv == 32 && d->Tk % 4 == 0 && (p.flags & 1) && (d->weights == nullptr || (p.flags & 2))) {
            void (*fn)(const AttnParams) = d->weights == nullptr ? attention_fwd16_long_kernel<true, false, false, 32>
                                                                 : attention_fwd16_long_kernel<false, false, false, 32>;
            hipLaunchKernelGGL(fn, dim3((unsigned)d->batch, (unsigned)tiles), dim3(512), (Attn16Cfg<256, 32>::LDS_BYTES),
                               h->stream, p);
        } else if (d->dk == 64 && d->dv == 64 && d->Tk % 4 == 0 && (p.flags & 1) &&
                   (d->weights == nullptr || (p.flags & 2))) {
            const bool bf16 = h->math_mode == SNHIP_MATH_BF16_INPUT;  // bf16 MFMAs, as this handle's GEMMs
            void (*fn)(const AttnParams);
            if (d->weights == nullptr)
                fn = bf16 ? attention_fwd16_long_kernel<true, true> : attention_fwd16_long_kernel<true, false>;
            else
                fn = bf16 ? attention_fwd16_long_kernel<false, true> : attention_fwd16_long_kernel<false, false>;
            hipLaunchKernelGGL(fn, dim3((unsigned)d->batch, (unsigned)tiles), dim3(512),
                               bf16 ? Attn16BCfg<256>::LDS_BYTES : Attn16Cfg<256>::LDS_BYTES, h->stream, p);
        } else if (hd <= 32)
            hipLaunchKernelGGL(attention_fwd_long_kernel<32>, dim3((unsigned)d->batch, (unsigned)tiles), dim3(256), lds32,
                               h->stream, p);
        else
            hipLaunchKernelGGL(attention_fwd_long_kernel<64>, dim3((unsigned)d->batch, (unsigned)tiles), dim3(256), lds64,
                               h->stream, p);
        return hip_to_status(hipGetLastError());
    }
    // K and V are staged once per workgroup: let one workgroup walk through all query tiles of its matrix unless
    // that would leave compute units without work
    int groups = 1;
    while (groups < tiles && (long long)d->batch * groups < 2LL * h->num_cu) ++groups;
    p.q_tiles = ceil_div(tiles, groups);
    // the full-size case (head dimension exactly 64 on both sides, 129 to 256 keys, outputs that take 16-byte
    // stores) has a form of its own with two wavefronts per SIMD
    const Attn16Entry* e16 = find_attn16(kAttn16, e->keys, e->hd);
    if (e16 != nullptr && d->dk == e->hd && d->dv == e->hd && d->Tk % 4 == 0 && (p.flags & 1) &&
        (d->weights == nullptr || (p.flags & 2))) {
        // one workgroup per compute unit, each walking through its share of the matrices
        const int gx = ceil_div(tiles, p.q_tiles);
        const bool bf16 = h->math_mode == SNHIP_MATH_BF16_INPUT && e->hd == 64;
        const int per_cu = bf16 ? 1 : e16->wgs_per_cu;  // (a second resident workgroup measured no gain in bf16)
        int gy = per_cu * h->num_cu / gx;
        gy = gy < 1 ? 1 : (gy > d->batch ? d->batch : gy);
        // a handle in the bf16-input math mode multiplies in bf16 here as it does in its GEMMs (head dimension 64)
        if (h->math_mode == SNHIP_MATH_BF16_INPUT && e->hd == 64 && e->keys == 256)
            hipLaunchKernelGGL(attention_fwd16_bf16_kernel<256>, dim3((unsigned)gx, (unsigned)gy), dim3(512),
                               Attn16BCfg<256>::LDS_BYTES, h->stream, p);
        else if (h->math_mode == SNHIP_MATH_BF16_INPUT && e->hd == 64 && e->keys == 128)
            hipLaunchKernelGGL(attention_fwd16_bf16_kernel<128>, dim3((unsigned)gx, (unsigned)gy), dim3(512),
                               Attn16BCfg<128>::LDS_BYTES, h->stream, p);
        else
            hipLaunchKernelGGL(e16->fn, dim3((unsigned)gx, (unsigned)gy), dim3(512), e16->lds_bytes, h->stream, p);
    } else
        hipLaunchKernelGGL(e->fn, dim3((unsigned)ceil_div(tiles, p.q_tiles), (unsigned)d->batch), dim3(256),
                           e->lds_bytes, h->stream, p);
    return hip_to_status(hipGetLastError());
}

int snhip_sizeof_attention_bwd_desc(void) { return (int)sizeof(snhip_attention_bwd_desc); }

int snhip_attention_backward(void* handle, const snhip_attention_bwd_desc* d) {
    Handle* h = static_cast<Handle*>(handle);
    // the descriptor grew by one field (causal); a caller built against the shorter one says so through struct_size
    constexpr int kSizeWithoutCausal = (int)offsetof(snhip_attention_bwd_desc, causal);
    if (d == nullptr || (d->struct_size != (int)sizeof(snhip_attention_bwd_desc) && d->struct_size != kSizeWithoutCausal))
        return SNHIP_STATUS_INVALID_VALUE;
    const bool causal = d->struct_size == (int)sizeof(snhip_attention_bwd_desc) && d->causal != 0;
    if (h == nullptr) return SNHIP_STATUS_NOT_INITIALIZED;
    if (d->batch < 0 || d->batch_inner < 0 || d->Tq < 0 || d->Tk < 0 || d->dk < 0 || d->dv < 0)
        return SNHIP_STATUS_INVALID_VALUE;
    if (d->batch == 0 || d->Tq == 0 || d->Tk == 0) return SNHIP_STATUS_SUCCESS;
    if (d->Q == nullptr || d->K == nullptr || d->V == nullptr || d->dO == nullptr || d->weights == nullptr ||
        d->scores_gradients == nullptr || d->dQ == nullptr || d->dK == nullptr || d->dV == nullptr)
        return SNHIP_STATUS_INVALID_VALUE;
    if (d->ldq < d->dk || d->ldk < d->dk || d->ldv < d->dv || d->ldo < d->dv) return SNHIP_STATUS_INVALID_VALUE;
    const int inner = d->batch_inner > 0 ? d->batch_inner : d->batch;
    if (d->batch % inner != 0) return SNHIP_STATUS_INVALID_VALUE;
    if (d->batch > 65535) return SNHIP_STATUS_NOT_SUPPORTED;
    const long long tt = (long long)d->Tq * d->Tk;  // P and dS are contiguous stacks

    // dV = P^T . dO                                                         (ScaledDotProductAttentionLayer.cs:117)
    GemmArgs g;
    g.tA = true;
    g.M = d->Tk, g.N = d->dv, g.K = d->Tq;
    g.A = d->weights, g.lda = d->Tk, g.sA = tt, g.sA2 = tt * inner;
    g.B = d->dO, g.ldb = d->ldo, g.sB = d->strideO, g.sB2 = d->strideO_outer;
    g.C = d->dV, g.ldc = d->ldv, g.sC = d->strideV, g.sC2 = d->strideV_outer;
    g.batch = d->batch, g.batch_inner = d->batch_inner;
    g.k_from_m = causal;  // P[query][key] == 0 for key > query: a tile of keys starts its sum at its first query
    int st = gemm_core(h, g);
    if (st != SNHIP_STATUS_SUCCESS) return st;

    // dS and dQ: one kernel when it fits, else dS = scale * dO . V^T, softmax gradient, dQ = dS . K   (:123-127)
    const int hd = d->dk > d->dv ? d->dk : d->dv;
    const AttnEntry* e = nullptr;
    for (const AttnEntry& c : kAttnBwd)
        if (d->Tk <= c.keys && hd <= c.hd) {
            e = &c;
            break;
        }
    bool fused = false;
    if (d->dk > 0 && d->dv > 0 && (e != nullptr || (d->dk == d->dv && (d->dk == 64 || d->dk == 32)))) {
        AttnParams p;
        p.Q = d->dO, p.K = d->V, p.V = d->K, p.O = d->dQ, p.P = d->scores_gradients, p.Pin = d->weights;
        p.Tq = d->Tq, p.Tk = d->Tk, p.dk = d->dv, p.dv = d->dk;  // first product contracts over dv, second produces dk
        p.ldq = d->ldo, p.ldk = d->ldv, p.ldv = d->ldk, p.ldo = d->ldq;
        p.sQ = d->strideO, p.sK = d->strideV, p.sV = d->strideK, p.sO = d->strideQ;
        p.sQ2 = d->strideO_outer, p.sK2 = d->strideV_outer, p.sV2 = d->strideK_outer, p.sO2 = d->strideQ_outer;
        p.batch_inner = inner;
        p.batch = d->batch;
        p.scale = d->scale;
        p.causal = 0;  // (set below for the kernel that walks key blocks: the others see one block of keys)
        p.flags = 0;
        const bool multi = d->batch > 1, two_level = multi && inner < d->batch;
        if ((uintptr_t)d->dQ % 16 == 0 && d->ldq % 4 == 0 && (!multi || d->strideQ % 4 == 0) &&
            (!two_level || d->strideQ_outer % 4 == 0))
            p.flags |= 1;
        if ((uintptr_t)d->scores_gradients % 16 == 0 && d->Tk % 4 == 0) p.flags |= 2;
        if ((uintptr_t)d->weights % 16 == 0 && d->Tk % 4 == 0) p.flags |= 4;
        const int tiles = ceil_div(d->Tq, AT_BQ);
        int groups = 1;
        while (groups < tiles && (long long)d->batch * groups < 2LL * h->num_cu) ++groups;
        p.q_tiles = ceil_div(tiles, groups);
        const Attn16Entry* e16 = e != nullptr ? find_attn16(kAttn16Bwd, e->keys, e->hd) : nullptr;
        if (e == nullptr) {
            // more than 256 keys, head dimension exactly 32 or 64: the two-pass kernel over key blocks (fp32 in every
            // math mode); anything else takes the three calls below
            if ((p.flags & 7) == 7 && tiles <= 65535) {
                p.q_tiles = 1;
                p.causal = causal ? 1 : 0;  // key blocks wholly above the diagonal are skipped, their dS zero-filled
                if (d->dk == 64)
                    hipLaunchKernelGGL((attention_fwd16_long_kernel<false, false, true, 64>),
                                       dim3((unsigned)d->batch, (unsigned)tiles), dim3(512),
                                       (Attn16Cfg<256, 64>::LDS_BYTES), h->stream, p);
                else
                    hipLaunchKernelGGL((attention_fwd16_long_kernel<false, false, true, 32>),
                                       dim3((unsigned)d->batch, (unsigned)tiles), dim3(512),
                                       (Attn16Cfg<256, 32>::LDS_BYTES), h->stream, p);
                fused = true;
            }
        } else if (e16 != nullptr && d->dk == e->hd && d->dv == e->hd && (p.flags & 7) == 7) {
            fused = true;
            // head dimension exactly 32 or 64, as in the forward call: two wavefronts per SIMD, one workgroup per
            // compute unit
            const int gx = ceil_div(tiles, p.q_tiles);
            int gy = h->num_cu / gx;
            gy = gy < 1 ? 1 : (gy > d->batch ? d->batch : gy);
            if (h->math_mode == SNHIP_MATH_BF16_INPUT && e->hd == 64 && e->keys == 256)  // as this handle's GEMMs
                hipLaunchKernelGGL((attention_fwd16_bf16_kernel<256, true>), dim3((unsigned)gx, (unsigned)gy), dim3(512),
                                   Attn16BCfg<256>::LDS_BYTES, h->stream, p);
            else if (h->math_mode == SNHIP_MATH_BF16_INPUT && e->hd == 64 && e->keys == 128)
                hipLaunchKernelGGL((attention_fwd16_bf16_kernel<128, true>), dim3((unsigned)gx, (unsigned)gy), dim3(512),
                                   Attn16BCfg<128>::LDS_BYTES, h->stream, p);
            else
                hipLaunchKernelGGL(e16->fn, dim3((unsigned)gx, (unsigned)gy), dim3(512), e16->lds_bytes, h->stream, p);
        } else {
            fused = true;
            hipLaunchKernelGGL(e->fn, dim3((unsigned)ceil_div(tiles, p.q_tiles), (unsigned)d->batch), dim3(256),
                               e->lds_bytes, h->stream, p);
        }
        if (fused) {
            st = hip_to_status(hipGetLastError());
            if (st != SNHIP_STATUS_SUCCESS) return st;
        }
    }
    if (!fused) {
        GemmArgs s1;
        s1.tB = true;
        s1.M = d->Tq, s1.N = d->Tk, s1.K = d->dv, s1.alpha = d->scale;
        s1.A = d->dO, s1.lda = d->ldo, s1.sA = d->strideO, s1.sA2 = d->strideO_outer;
        s1.B = d->V, s1.ldb = d->ldv, s1.sB = d->strideV, s1.sB2 = d->strideV_outer;
        s1.C = d->scores_gradients, s1.ldc = d->Tk, s1.sC = tt, s1.sC2 = tt * inner;
        s1.batch = d->batch, s1.batch_inner = d->batch_inner;
        st = gemm_core(h, s1);
        if (st != SNHIP_STATUS_SUCCESS) return st;
        st = snhip_softmax_last_dim_backward(handle, d->weights, d->scores_gradients, d->scores_gradients,
                                             (long long)d->batch * d->Tq, d->Tk);
        if (st != SNHIP_STATUS_SUCCESS) return st;
        GemmArgs s2;
        s2.M = d->Tq, s2.N = d->dk, s2.K = d->Tk;
        s2.A = d->scores_gradients, s2.lda = d->Tk, s2.sA = tt, s2.sA2 = tt * inner;
        s2.B = d->K, s2.ldb = d->ldk, s2.sB = d->strideK, s2.sB2 = d->strideK_outer;
        s2.C = d->dQ, s2.ldc = d->ldq, s2.sC = d->strideQ, s2.sC2 = d->strideQ_outer;
        s2.batch = d->batch, s2.batch_inner = d->batch_inner;
        st = gemm_core(h, s2);
        if (st != SNHIP_STATUS_SUCCESS) return st;
    }

    // dK = dS^T . Q                                                                                    (:128)
    GemmArgs k;
    k.tA = true;
    k.M = d->Tk, k.N = d->dk, k.K = d->Tq;
    k.A = d->scores_gradients, k.lda = d->Tk, k.sA = tt, k.sA2 = tt * inner;
    k.B = d->Q, k.ldb = d->ldq, k.sB = d->strideQ, k.sB2 = d->strideQ_outer;
    k.C = d->dK, k.ldc = d->ldk, k.sC = d->strideK, k.sC2 = d->strideK_outer;
    k.batch = d->batch, k.batch_inner = d->batch_inner;
    k.k_from_m = causal;  // dS[query][key] == 0 for key > query, like the weights it was formed from
    return gemm_core(h, k);
}

int snhip_sizeof_gemm_desc(void) { return (int)sizeof(snhip_gemm_desc); }
int snhip_operand_element_bytes(int math_mode) {
    if (math_mode == SNHIP_MATH_BF16_STORED) return 2;
    return (math_mode == SNHIP_MATH_FP32 || math_mode == SNHIP_MATH_BF16_INPUT) ? 4 : 0;
}

int snhip_gemm_ex(void* handle, const snhip_gemm_desc* d) {
    if (d == nullptr || d->struct_size != (int)sizeof(snhip_gemm_desc)) return SNHIP_STATUS_INVALID_VALUE;
    GemmArgs g;
    g.tA = d->transA != 0, g.tB = d->transB != 0;
    g.M = d->M, g.N = d->N, g.K = d->K;
    g.alpha = d->alpha, g.beta = d->beta;
    g.A = d->A, g.lda = d->lda, g.sA = d->strideA, g.sA2 = d->strideA_outer;
    g.B = d->B, g.ldb = d->ldb, g.sB = d->strideB, g.sB2 = d->strideB_outer;
    g.C = d->C, g.ldc = d->ldc, g.sC = d->strideC, g.sC2 = d->strideC_outer;
    g.batch = d->batch, g.batch_inner = d->batch_inner;
    g.bias = d->bias;
    g.D = d->D, g.ldd = d->ldd, g.sD = d->strideD, g.sD2 = d->strideD_outer, g.gamma = d->gamma;
    g.act = d->activation, g.act_param = d->activation_param;
    g.colsum = d->colsum;
    g.math = d->math;
    return gemm_core(static_cast<Handle*>(handle), g);
}

int snhip_dense_forward(void* handle, float* y, const float* x, const float* weights, const float* bias, int rows,
                        int in_features, int out_features, int activation, float activation_param) {
    GemmArgs g;
    g.tB = true;  // y = x . W^T, W stored (out, in)
    g.M = rows, g.N = out_features, g.K = in_features;
    g.A = x, g.lda = in_features, g.B = weights, g.ldb = in_features, g.C = y, g.ldc = out_features;
    g.bias = bias, g.act = activation, g.act_param = activation_param;
    return gemm_core(static_cast<Handle*>(handle), g);
}

int snhip_dense_backward_ex(void* handle, float* dx, float* weight_gradients, float* bias_gradients, const float* x,
                            const float* dy, const float* weights, int rows, int in_features, int out_features,
                            float multiplier, float weight_decay_alpha, const float* bias, float bias_decay_alpha) {
    Handle* h = static_cast<Handle*>(handle);
    if (bias_decay_alpha != 0.0f && bias_gradients != nullptr && bias == nullptr) return SNHIP_STATUS_INVALID_VALUE;
    if (h != nullptr && dx != nullptr && weight_gradients != nullptr) {
        const int st = dense_backward_small(h, dx, weight_gradients, bias_gradients, x, dy, weights, rows, in_features,
                                            out_features, multiplier, weight_decay_alpha, bias, bias_decay_alpha);
        if (st != kNotTaken) return st;
    }
    if (weight_gradients != nullptr || bias_gradients != nullptr) {
        if (weight_gradients == nullptr) {
            const int st = snhip_bias_gradient(handle, dy, rows, out_features, bias_gradients);
            if (st != SNHIP_STATUS_SUCCESS) return st;
        } else {
            GemmArgs g;  // dW = multiplier * dy^T . x (+ weight_decay_alpha * W), db = column sums of dy
            g.tA = true;
            g.M = out_features, g.N = in_features, g.K = rows;
            g.alpha = multiplier;
            g.A = dy, g.lda = out_features, g.B = x, g.ldb = in_features, g.C = weight_gradients, g.ldc = in_features;
            g.D = weights, g.ldd = in_features, g.gamma = weight_decay_alpha;
            g.colsum = bias_gradients;
            const int st = gemm_core(h, g);
            if (st != SNHIP_STATUS_SUCCESS) return st;
        }
        if (bias_gradients != nullptr && bias_decay_alpha != 0.0f) {  // Linear.cs:178-181
            const int st = snhip_axpy(handle, out_features, bias_decay_alpha, bias, bias_gradients);
            if (st != SNHIP_STATUS_SUCCESS) return st;
        }
    }
    if (dx == nullptr) return SNHIP_STATUS_SUCCESS;
    GemmArgs g;  // dx = dy . W
    g.M = rows, g.N = in_features, g.K = out_features;
    g.A = dy, g.lda = out_features, g.B = weights, g.ldb = in_features, g.C = dx, g.ldc = in_features;
    return gemm_core(h, g);
}

int snhip_dense_backward(void* handle, float* dx, float* weight_gradients, float* bias_gradients, const float* x,
                         const float* dy, const float* weights, int rows, int in_features, int out_features,
                         float multiplier, float weight_decay_alpha) {
    return snhip_dense_backward_ex(handle, dx, weight_gradients, bias_gradients, x, dy, weights, rows, in_features,
                                   out_features, multiplier, weight_decay_alpha, nullptr, 0.0f);
}

int snhip_dot_bias(void* handle, const float* A, int aH, int aW, int transposeA, const float* B, int bH, int bW,
                   int transposeB, float* C, float alpha, float beta, const float* bias) {
    if (aH < 0 || aW < 0 || bH < 0 || bW < 0) return SNHIP_STATUS_INVALID_VALUE;
    // BlasServices.DotMkl, Prod/Data/BlasServices.cs:14-19
    const int M = transposeA ? aW : aH;
    const int N = transposeB ? bH : bW;
    const int K = transposeA ? aH : aW;
    const int Kb = transposeB ? bW : bH;
    if (K != Kb) return SNHIP_STATUS_INVALID_VALUE;
    return gemm_rm(static_cast<Handle*>(handle), transposeA != 0, transposeB != 0, M, N, K, alpha, A, aW, 0, B, bW, 0,
                   beta, C, N, 0, 1, bias);
}

int snhip_dot(void* handle, const float* A, int aH, int aW, int transposeA, const float* B, int bH, int bW,
              int transposeB, float* C, float alpha, float beta) {
    return snhip_dot_bias(handle, A, aH, aW, transposeA, B, bH, bW, transposeB, C, alpha, beta, nullptr);
}

int snhip_dot_noalloc(void* handle, const float* A, int aH, int aW, int transposeA, const float* B, int bH, int bW,
                      int transposeB, float* C, float alpha, float beta) {
    if (handle == nullptr) return SNHIP_STATUS_NOT_INITIALIZED;
    if (aH < 0 || aW < 0 || bH < 0 || bW < 0) return SNHIP_STATUS_INVALID_VALUE;
    GemmArgs g;  // BlasServices.DotMkl's derivation, as in snhip_dot
    g.tA = transposeA != 0, g.tB = transposeB != 0;
    g.M = transposeA ? aW : aH, g.N = transposeB ? bH : bW, g.K = transposeA ? aH : aW;
    if (g.K != (transposeB ? bW : bH)) return SNHIP_STATUS_INVALID_VALUE;
    g.alpha = alpha, g.beta = beta;
    g.A = A, g.lda = aW, g.B = B, g.ldb = bW, g.C = C, g.ldc = g.N;
    g.no_alloc = true;
    return gemm_core(static_cast<Handle*>(handle), g);
}

int snhip_static_scratch_bytes(void) { return (int)kStaticScratchBytes; }

int snhip_get_last_error_message(void* handle, char* buffer, int capacity) {
    if (handle == nullptr) return SNHIP_STATUS_NOT_INITIALIZED;
    if (buffer == nullptr || capacity <= 0) return SNHIP_STATUS_INVALID_VALUE;
    snprintf(buffer, (size_t)capacity, "%s", static_cast<Handle*>(handle)->last_error);
    return SNHIP_STATUS_SUCCESS;
}

int snhip_bmm(void* handle, const float* A, int aH, int aW, int transposeA, long long strideA, const float* B, int bH,
              int bW, int transposeB, long long strideB, float* C, long long strideC, int batch, float alpha,
              float beta) {
    if (aH < 0 || aW < 0 || bH < 0 || bW < 0) return SNHIP_STATUS_INVALID_VALUE;
    const int M = transposeA ? aW : aH;
    const int N = transposeB ? bH : bW;
    const int K = transposeA ? aH : aW;
    const int Kb = transposeB ? bW : bH;
    if (K != Kb) return SNHIP_STATUS_INVALID_VALUE;
    return gemm_rm(static_cast<Handle*>(handle), transposeA != 0, transposeB != 0, M, N, K, alpha, A, aW, strideA, B,
                   bW, strideB, beta, C, N, strideC, batch, nullptr);
}

int snhip_set_math_mode(void* handle, int mode) {
    if (handle == nullptr) return SNHIP_STATUS_NOT_INITIALIZED;
    if (mode != SNHIP_MATH_FP32 && mode != SNHIP_MATH_BF16_INPUT) return SNHIP_STATUS_INVALID_VALUE;
    static_cast<Handle*>(handle)->math_mode = mode;
    return SNHIP_STATUS_SUCCESS;
}

int snhip_dot_bf16(void* handle, const float* A, int aH, int aW, int transposeA, const float* B, int bH, int bW,
                   int transposeB, float* C, float alpha, float beta, const float* bias) {
    if (aH < 0 || aW < 0 || bH < 0 || bW < 0) return SNHIP_STATUS_INVALID_VALUE;
    const int M = transposeA ? aW : aH;
    const int N = transposeB ? bH : bW;
    const int K = transposeA ? aH : aW;
    const int Kb = transposeB ? bW : bH;
    if (K != Kb) return SNHIP_STATUS_INVALID_VALUE;
    return gemm_rm(static_cast<Handle*>(handle), transposeA != 0, transposeB != 0, M, N, K, alpha, A, aW, 0, B, bW, 0,
                   beta, C, N, 0, 1, bias, SNHIP_MATH_BF16_INPUT);
}

int snhip_bmm_bf16(void* handle, const float* A, int aH, int aW, int transposeA, long long strideA, const float* B,
                   int bH, int bW, int transposeB, long long strideB, float* C, long long strideC, int batch,
                   float alpha, float beta) {
    if (aH < 0 || aW < 0 || bH < 0 || bW < 0) return SNHIP_STATUS_INVALID_VALUE;
    const int M = transposeA ? aW : aH;
    const int N = transposeB ? bH : bW;
    const int K = transposeA ? aH : aW;
    const int Kb = transposeB ? bW : bH;
    if (K != Kb) return SNHIP_STATUS_INVALID_VALUE;
    return gemm_rm(static_cast<Handle*>(handle), transposeA != 0, transposeB != 0, M, N, K, alpha, A, aW, strideA, B,
                   bW, strideB, beta, C, N, strideC, batch, nullptr, SNHIP_MATH_BF16_INPUT);
}

int snhip_convert_f32_to_bf16(void* handle, const float* src, void* dst, long long count) {
    if (handle == nullptr) return SNHIP_STATUS_NOT_INITIALIZED;
    if (count < 0) return SNHIP_STATUS_INVALID_VALUE;
    if (count == 0) return SNHIP_STATUS_SUCCESS;
    if (src == nullptr || dst == nullptr || (uintptr_t)dst % 2 != 0) return SNHIP_STATUS_INVALID_VALUE;
    const int vec = ((uintptr_t)src % 16 == 0 && (uintptr_t)dst % 8 == 0) ? 1 : 0;
    const long long work = vec ? (count + 7) / 8 : count;
    const int blocks = (int)((work + 255) / 256 < 16384 ? (work + 255) / 256 : 16384);
    hipLaunchKernelGGL(convert_f32_to_bf16_kernel, dim3(blocks), dim3(256), 0, static_cast<Handle*>(handle)->stream, src,
                       static_cast<__bf16*>(dst), count, vec);
    return hip_to_status(hipGetLastError());
}

int snhip_convert_f32_to_bf16_2d(void* handle, const float* src, int rows, int cols, long long ld_src, int transpose,
                                 void* dst, long long ld_dst) {
    if (handle == nullptr) return SNHIP_STATUS_NOT_INITIALIZED;
    if (rows < 0 || cols < 0) return SNHIP_STATUS_INVALID_VALUE;
    if (rows == 0 || cols == 0) return SNHIP_STATUS_SUCCESS;
    if (src == nullptr || dst == nullptr || (uintptr_t)dst % 2 != 0 || ld_src < cols || ld_dst < (transpose ? rows : cols))
        return SNHIP_STATUS_INVALID_VALUE;
    if (transpose != 0 && wide_transpose_ok(src, rows, cols, ld_src, 4, dst, ld_dst)) {
        hipLaunchKernelGGL(transpose_to_bf16_kernel<false>, dim3((unsigned)ceil_div(cols, 128), (unsigned)(rows / 64)),
                           dim3(256), 0, static_cast<Handle*>(handle)->stream, static_cast<const void*>(src), ld_src, rows,
                           cols, static_cast<__bf16*>(dst), ld_dst);
        return hip_to_status(hipGetLastError());
    }
    if (transpose == 0 && cols % 8 == 0 && (uintptr_t)src % 16 == 0 && (uintptr_t)dst % 16 == 0 && ld_src % 4 == 0 &&
        ld_dst % 8 == 0) {
        const long long blocks = ((long long)rows * (cols / 8) + 255) / 256;
        hipLaunchKernelGGL(convert_rows_to_bf16_kernel, dim3((unsigned)(blocks < 16384 ? blocks : 16384)), dim3(256), 0,
                           static_cast<Handle*>(handle)->stream, src, ld_src, rows, cols, static_cast<__bf16*>(dst), ld_dst);
        return hip_to_status(hipGetLastError());
    }
    if (ceil_div(rows, 32) > 65535) return SNHIP_STATUS_NOT_SUPPORTED;
    hipLaunchKernelGGL(convert_f32_to_bf16_2d_kernel, dim3((unsigned)ceil_div(cols, 32), (unsigned)ceil_div(rows, 32)),
                       dim3(256), 0, static_cast<Handle*>(handle)->stream, src, ld_src, rows, cols, transpose != 0,
                       static_cast<__bf16*>(dst), ld_dst);
    return hip_to_status(hipGetLastError());
}

int snhip_bmm_bf16_stored(void* handle, const void* A, int aH, int aW, int transposeA, long long strideA, const void* B,
                          int bH, int bW, int transposeB, long long strideB, float* C, long long strideC, int batch,
                          float alpha, float beta, const float* bias) {
    if (aH < 0 || aW < 0 || bH < 0 || bW < 0) return SNHIP_STATUS_INVALID_VALUE;
    const int M = transposeA ? aW : aH;
    const int N = transposeB ? bH : bW;
    const int K = transposeA ? aH : aW;
    const int Kb = transposeB ? bW : bH;
    if (K != Kb) return SNHIP_STATUS_INVALID_VALUE;
    // the operand pointers travel as float* through the shared argument block; the bf16-stored kernels read them as bf16
    return gemm_rm(static_cast<Handle*>(handle), transposeA != 0, transposeB != 0, M, N, K, alpha,
                   static_cast<const float*>(A), aW, strideA, static_cast<const float*>(B), bW, strideB, beta, C, N,
                   strideC, batch, bias, SNHIP_MATH_BF16_STORED);
}

int snhip_dot_bf16_stored(void* handle, const void* A, int aH, int aW, int transposeA, const void* B, int bH, int bW,
                          int transposeB, float* C, float alpha, float beta, const float* bias) {
    return snhip_bmm_bf16_stored(handle, A, aH, aW, transposeA, 0, B, bH, bW, transposeB, 0, C, 0, 1, alpha, beta, bias);
}

/* ---- row / column helpers of the Linear and attention layers ---- */

static inline int grid_for(long long total) {
    const long long b = (total + 255) / 256;
    return (int)(b < 1 ? 1 : (b > 16384 ? 16384 : b));
}

int snhip_bias_gradient(void* handle, const float* dy, int rows, int cols, float* bias_gradient) {
    if (handle == nullptr) return SNHIP_STATUS_NOT_INITIALIZED;
    if (rows < 0 || cols < 0) return SNHIP_STATUS_INVALID_VALUE;
    if (cols == 0) return SNHIP_STATUS_SUCCESS;
    if (bias_gradient == nullptr || (rows > 0 && dy == nullptr)) return SNHIP_STATUS_INVALID_VALUE;
    return launch_column_sum(static_cast<Handle*>(handle), dy, bias_gradient, rows, cols, (long long)cols, 0LL, 1);
}

int snhip_activation_forward(void* handle, int activation, float activation_param, const float* x, float* y,
                             long long n) {
    if (handle == nullptr) return SNHIP_STATUS_NOT_INITIALIZED;
    if (n < 0) return SNHIP_STATUS_INVALID_VALUE;
    if (activation < ACT_NONE || activation > ACT_TANH) return SNHIP_STATUS_NOT_SUPPORTED;
    if (n == 0) return SNHIP_STATUS_SUCCESS;
    if (x == nullptr || y == nullptr) return SNHIP_STATUS_INVALID_VALUE;
    hipLaunchKernelGGL(activation_kernel, dim3(grid_for(n)), dim3(256), 0, static_cast<Handle*>(handle)->stream, x, y, n,
                       activation, activation_param);
    return hip_to_status(hipGetLastError());
}

int snhip_activation_backward(void* handle, int activation, float activation_param, const float* y, const float* dy,
                              float* dx, long long n) {
    if (handle == nullptr) return SNHIP_STATUS_NOT_INITIALIZED;
    if (n < 0) return SNHIP_STATUS_INVALID_VALUE;
    if (activation < ACT_NONE || activation > ACT_TANH) return SNHIP_STATUS_NOT_SUPPORTED;
    if (n == 0) return SNHIP_STATUS_SUCCESS;
    if (y == nullptr || dy == nullptr || dx == nullptr) return SNHIP_STATUS_INVALID_VALUE;
    hipLaunchKernelGGL(activation_bwd_kernel, dim3(grid_for(n)), dim3(256), 0, static_cast<Handle*>(handle)->stream, y, dy,
                       dx, n, activation, activation_param);
    return hip_to_status(hipGetLastError());
}

int snhip_transpose_second_and_third_dimension(void* handle, const float* src, float* dst, int d0, int d1, int d2,
                                               int d3) {
    if (handle == nullptr) return SNHIP_STATUS_NOT_INITIALIZED;
    if (d0 < 0 || d1 < 0 || d2 < 0 || d3 < 0) return SNHIP_STATUS_INVALID_VALUE;
    const long long total = (long long)d0 * d1 * d2 * d3;
    if (total == 0) return SNHIP_STATUS_SUCCESS;
    if (src == nullptr || dst == nullptr || src == dst) return SNHIP_STATUS_INVALID_VALUE;
    hipLaunchKernelGGL(transpose_2nd_3rd_kernel, dim3(grid_for(total)), dim3(256), 0, static_cast<Handle*>(handle)->stream,
                       src, dst, d0, d1, d2, d3);
    return hip_to_status(hipGetLastError());
}

int snhip_sgeam(void* handle, int transa, int transb, int m, int n, const float* alpha, const float* A, int lda,
                const float* beta, const float* B, int ldb, float* C, int ldc) {
    if (handle == nullptr) return SNHIP_STATUS_NOT_INITIALIZED;
    bool oka = false, okb = false;
    const bool ta = op_is_trans(transa, &oka), tb = op_is_trans(transb, &okb);
    if (!oka || !okb || m < 0 || n < 0 || alpha == nullptr || beta == nullptr) return SNHIP_STATUS_INVALID_VALUE;
    if (m == 0 || n == 0) return SNHIP_STATUS_SUCCESS;
    const bool use_a = (*alpha != 0.0f), use_b = (*beta != 0.0f);
    if (C == nullptr || ldc < m) return SNHIP_STATUS_INVALID_VALUE;
    if (use_a && (A == nullptr || lda < (ta ? n : m))) return SNHIP_STATUS_INVALID_VALUE;
    if (use_b && (B == nullptr || ldb < (tb ? n : m))) return SNHIP_STATUS_INVALID_VALUE;
    if ((use_a && A == C && ta) || (use_b && B == C && tb)) return SNHIP_STATUS_NOT_SUPPORTED;  // in-place transpose
    if ((long long)ceil_div(n, 32) > 65535) return SNHIP_STATUS_NOT_SUPPORTED;
    // the kernel reads neither A when alpha == 0 nor B when beta == 0 (either may be NULL then)
    hipLaunchKernelGGL(geam_kernel, dim3((unsigned)ceil_div(m, 32), (unsigned)ceil_div(n, 32)), dim3(256), 0,
                       static_cast<Handle*>(handle)->stream, (int)ta, (int)tb, m, n, *alpha, A, (long long)lda, *beta, B,
                       (long long)ldb, C, (long long)ldc);
    return hip_to_status(hipGetLastError());
}

int snhip_sdgmm(void* handle, int mode, int m, int n, const float* A, int lda, const float* x, int incx, float* C,
                int ldc) {
    if (handle == nullptr) return SNHIP_STATUS_NOT_INITIALIZED;
    if ((mode != SNHIP_SIDE_LEFT && mode != SNHIP_SIDE_RIGHT) || m < 0 || n < 0) return SNHIP_STATUS_INVALID_VALUE;
    if (m == 0 || n == 0) return SNHIP_STATUS_SUCCESS;
    if (A == nullptr || x == nullptr || C == nullptr || lda < m || ldc < m || incx == 0) return SNHIP_STATUS_INVALID_VALUE;
    if (incx < 0) return SNHIP_STATUS_NOT_SUPPORTED;
    hipLaunchKernelGGL(dgmm_kernel, dim3(grid_for((long long)m * n)), dim3(256), 0, static_cast<Handle*>(handle)->stream,
                       (int)(mode == SNHIP_SIDE_RIGHT), m, n, A, (long long)lda, x, (long long)incx, C, (long long)ldc);
    return hip_to_status(hipGetLastError());
}

int snhip_broadcast_add_vector(void* handle, const float* vector, float* y, int rows, int cols) {
    if (handle == nullptr) return SNHIP_STATUS_NOT_INITIALIZED;
    if (rows < 0 || cols < 0) return SNHIP_STATUS_INVALID_VALUE;
    if (rows == 0 || cols == 0) return SNHIP_STATUS_SUCCESS;
    if (vector == nullptr || y == nullptr) return SNHIP_STATUS_INVALID_VALUE;
    hipLaunchKernelGGL(broadcast_add_kernel, dim3(grid_for((long long)rows * cols)), dim3(256), 0,
                       static_cast<Handle*>(handle)->stream, y, vector, (long long)rows, cols);
    return hip_to_status(hipGetLastError());
}

int snhip_axpy(void* handle, long long n, float alpha, const float* x, float* y) {
    if (handle == nullptr) return SNHIP_STATUS_NOT_INITIALIZED;
    if (n < 0) return SNHIP_STATUS_INVALID_VALUE;
    if (n == 0) return SNHIP_STATUS_SUCCESS;
    if (x == nullptr || y == nullptr) return SNHIP_STATUS_INVALID_VALUE;
    hipLaunchKernelGGL(axpy_kernel, dim3(grid_for(n)), dim3(256), 0, static_cast<Handle*>(handle)->stream, y, x, alpha, n);
    return hip_to_status(hipGetLastError());
}

int snhip_softmax_last_dim(void* handle, const float* x, float* y, long long rows, int cols) {
    if (handle == nullptr) return SNHIP_STATUS_NOT_INITIALIZED;
    if (rows < 0 || cols < 0 || rows > 0x7fffffffLL * 4) return SNHIP_STATUS_INVALID_VALUE;
    if (rows == 0 || cols == 0) return SNHIP_STATUS_SUCCESS;
    if (x == nullptr || y == nullptr) return SNHIP_STATUS_INVALID_VALUE;
    hipLaunchKernelGGL(softmax_rows_kernel, dim3((unsigned)((rows + 3) / 4)), dim3(256), 0,
                       static_cast<Handle*>(handle)->stream, x, y, rows, cols);
    return hip_to_status(hipGetLastError());
}

int snhip_softmax_last_dim_backward(void* handle, const float* y, const float* dy, float* dx, long long rows, int cols) {
    if (handle == nullptr) return SNHIP_STATUS_NOT_INITIALIZED;
    if (rows < 0 || cols < 0 || rows > 0x7fffffffLL * 4) return SNHIP_STATUS_INVALID_VALUE;
    if (rows == 0 || cols == 0) return SNHIP_STATUS_SUCCESS;
    if (y == nullptr || dy == nullptr || dx == nullptr) return SNHIP_STATUS_INVALID_VALUE;
    hipLaunchKernelGGL(softmax_rows_bwd_kernel, dim3((unsigned)((rows + 3) / 4)), dim3(256), 0,
                       static_cast<Handle*>(handle)->stream, y, dy, dx, rows, cols);
    return hip_to_status(hipGetLastError());
}

int snhip_set_above_main_diagonal(void* handle, float* x, int matrices, int rows, int cols, float value) {
    if (handle == nullptr) return SNHIP_STATUS_NOT_INITIALIZED;
    if (matrices < 0 || rows < 0 || cols < 0) return SNHIP_STATUS_INVALID_VALUE;
    const long long total = (long long)matrices * rows * cols;
    if (total == 0) return SNHIP_STATUS_SUCCESS;
    if (x == nullptr) return SNHIP_STATUS_INVALID_VALUE;
    hipLaunchKernelGGL(set_above_diagonal_kernel, dim3(grid_for(total)), dim3(256), 0,
                       static_cast<Handle*>(handle)->stream, x, (long long)matrices, rows, cols, value);
    return hip_to_status(hipGetLastError());
}

/* ---- memory / stream shims ---- */

int snhip_malloc(void** dptr, size_t bytes) {
    if (dptr == nullptr) return SNHIP_STATUS_INVALID_VALUE;
    *dptr = nullptr;
    if (bytes < 8) bytes = 8;  // GPUTensor never allocates less (GpuTensor.cs:38)
    hipError_t e = hipMalloc(dptr, bytes);
    if (e != hipSuccess) {
        (void)hipGetLastError();
        return SNHIP_STATUS_ALLOC_FAILED;
    }
    return SNHIP_STATUS_SUCCESS;
}

int snhip_free(void* dptr) {
    if (dptr == nullptr) return SNHIP_STATUS_SUCCESS;
    return hip_to_status(hipFree(dptr));
}

int snhip_memset32(void* handle, void* dptr, unsigned int value, size_t count) {
    if (handle == nullptr) return SNHIP_STATUS_NOT_INITIALIZED;
    if (count == 0) return SNHIP_STATUS_SUCCESS;
    if (dptr == nullptr) return SNHIP_STATUS_INVALID_VALUE;
    hipLaunchKernelGGL(fill32_kernel, dim3(grid_for((long long)count)), dim3(256), 0, static_cast<Handle*>(handle)->stream,
                       static_cast<unsigned int*>(dptr), value, (long long)count);
    return hip_to_status(hipGetLastError());
}

int snhip_memcpy_htod_async(void* handle, void* dst, const void* src, size_t bytes) {
    if (handle == nullptr) return SNHIP_STATUS_NOT_INITIALIZED;
    if (bytes == 0) return SNHIP_STATUS_SUCCESS;
    if (dst == nullptr || src == nullptr) return SNHIP_STATUS_INVALID_VALUE;
    return hip_to_status(hipMemcpyAsync(dst, src, bytes, hipMemcpyHostToDevice, static_cast<Handle*>(handle)->stream));
}

int snhip_memcpy_dtoh(void* handle, void* dst, const void* src, size_t bytes) {
    if (handle == nullptr) return SNHIP_STATUS_NOT_INITIALIZED;
    if (bytes == 0) return SNHIP_STATUS_SUCCESS;
    if (dst == nullptr || src == nullptr) return SNHIP_STATUS_INVALID_VALUE;
    hipStream_t s = static_cast<Handle*>(handle)->stream;
    hipError_t e = hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToHost, s);
    if (e != hipSuccess) return hip_to_status(e);
    return hip_to_status(hipStreamSynchronize(s));
}

int snhip_memcpy_dtod_async(void* handle, void* dst, const void* src, size_t bytes) {
    if (handle == nullptr) return SNHIP_STATUS_NOT_INITIALIZED;
    if (bytes == 0) return SNHIP_STATUS_SUCCESS;
    if (dst == nullptr || src == nullptr) return SNHIP_STATUS_INVALID_VALUE;
    return hip_to_status(hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToDevice, static_cast<Handle*>(handle)->stream));
}

int snhip_stream_create(void** stream) {
    if (stream == nullptr) return SNHIP_STATUS_INVALID_VALUE;
    hipStream_t st = nullptr;
    // default priority, blocking with respect to the null stream: the flags-0 stream of StreamWrapper.cs:14
    hipError_t e = hipStreamCreateWithFlags(&st, hipStreamDefault);
    if (e != hipSuccess) return hip_to_status(e);
    *stream = st;
    return SNHIP_STATUS_SUCCESS;
}

int snhip_stream_destroy(void* stream) {
    if (stream == nullptr) return SNHIP_STATUS_SUCCESS;
    return hip_to_status(hipStreamDestroy(static_cast<hipStream_t>(stream)));
}

int snhip_stream_synchronize(void* handle) {
    if (handle == nullptr) return SNHIP_STATUS_NOT_INITIALIZED;
    return hip_to_status(hipStreamSynchronize(static_cast<Handle*>(handle)->stream));
}

/* ---- measurement helpers ---- */

int snhip_event_create(void** event) {
    if (event == nullptr) return SNHIP_STATUS_INVALID_VALUE;
    hipEvent_t ev;
    hipError_t e = hipEventCreate(&ev);
    if (e != hipSuccess) return hip_to_status(e);
    *event = ev;
    return SNHIP_STATUS_SUCCESS;
}

int snhip_event_destroy(void* event) {
    if (event == nullptr) return SNHIP_STATUS_SUCCESS;
    return hip_to_status(hipEventDestroy(static_cast<hipEvent_t>(event)));
}

int snhip_event_record(void* handle, void* event) {
    if (handle == nullptr) return SNHIP_STATUS_NOT_INITIALIZED;
    if (event == nullptr) return SNHIP_STATUS_INVALID_VALUE;
    return hip_to_status(hipEventRecord(static_cast<hipEvent_t>(event), static_cast<Handle*>(handle)->stream));
}

int snhip_event_elapsed_ms(void* start, void* stop, float* ms) {
    if (start == nullptr || stop == nullptr || ms == nullptr) return SNHIP_STATUS_INVALID_VALUE;
    hipError_t e = hipEventSynchronize(static_cast<hipEvent_t>(stop));
    if (e != hipSuccess) return hip_to_status(e);
    return hip_to_status(hipEventElapsedTime(ms, static_cast<hipEvent_t>(start), static_cast<hipEvent_t>(stop)));
}

int snhip_copy_f32(void* handle, void* dst, const void* src, long long count) {
    if (handle == nullptr) return SNHIP_STATUS_NOT_INITIALIZED;
    if (count < 0) return SNHIP_STATUS_INVALID_VALUE;
    if (count == 0) return SNHIP_STATUS_SUCCESS;
    if (dst == nullptr || src == nullptr) return SNHIP_STATUS_INVALID_VALUE;
    Handle* h = static_cast<Handle*>(handle);
    const int vec = ((uintptr_t)dst % 16 == 0 && (uintptr_t)src % 16 == 0) ? 1 : 0;
    const long long work = vec ? (count + 3) / 4 : count;
    const int blocks = (int)((work + 255) / 256 < 16384 ? (work + 255) / 256 : 16384);
    hipLaunchKernelGGL(copy_f32_kernel, dim3(blocks), dim3(256), 0, h->stream, static_cast<const float*>(src),
                       static_cast<float*>(dst), count, vec);
    return hip_to_status(hipGetLastError());
}

int snhip_device_info(void* handle, int info[6]) {
    if (handle == nullptr) return SNHIP_STATUS_NOT_INITIALIZED;
    if (info == nullptr) return SNHIP_STATUS_INVALID_VALUE;
    hipDeviceProp_t prop;
    hipError_t e = hipGetDeviceProperties(&prop, static_cast<Handle*>(handle)->device);
    if (e != hipSuccess) return hip_to_status(e);
    info[0] = prop.multiProcessorCount;
    info[1] = prop.clockRate;
    info[2] = prop.memoryClockRate;
    info[3] = prop.memoryBusWidth;
    info[4] = (int)prop.sharedMemPerBlockOptin;
    int arch = 0;
    for (const char* c = prop.gcnArchName + 3; *c >= '0' && *c <= '9'; ++c) arch = arch * 10 + (*c - '0');
    info[5] = arch;
    return SNHIP_STATUS_SUCCESS;
}

int snhip_set_tuning(void* handle, int config, int splitk) {
    if (handle == nullptr) return SNHIP_STATUS_NOT_INITIALIZED;
    if (config >= kNumConfigs || splitk < 0 || splitk > 64) return SNHIP_STATUS_INVALID_VALUE;
    Handle* h = static_cast<Handle*>(handle);
    h->force_cfg = config < 0 ? -1 : config;
    h->force_splitk = splitk;
    return SNHIP_STATUS_SUCCESS;
}

int snhip_query_tuning(void* handle, int m, int n, int k, int batch, int math_mode, int* config, int* splitk) {
    if (m <= 0 || n <= 0 || k <= 0 || batch <= 0) return SNHIP_STATUS_INVALID_VALUE;
    if (math_mode != SNHIP_MATH_FP32 && math_mode != SNHIP_MATH_BF16_INPUT && math_mode != SNHIP_MATH_BF16_STORED)
        return SNHIP_STATUS_INVALID_VALUE;
    Handle model;  // without a handle: an MI355X with 256 CUs, no overrides
    const Handle* h = handle != nullptr ? static_cast<const Handle*>(handle) : &model;
    Choice ch = choose(h, m, n, k, batch, kind_of_math(math_mode));
    if ((long long)batch * ch.splitk > 65535) ch.splitk = 1;
    if (config != nullptr) *config = ch.cfg;
    if (splitk != nullptr) *splitk = ch.splitk;
    return SNHIP_STATUS_SUCCESS;
}

int snhip_set_splitk_mode(void* handle, int mode) {
    if (handle == nullptr) return SNHIP_STATUS_NOT_INITIALIZED;
    if (mode < 0 || mode > 2) return SNHIP_STATUS_INVALID_VALUE;
    static_cast<Handle*>(handle)->splitk_mode = mode;
    return SNHIP_STATUS_SUCCESS;
}

int snhip_get_last_tuning(void* handle, int* config, int* splitk) {
    if (handle == nullptr) return SNHIP_STATUS_NOT_INITIALIZED;
    Handle* h = static_cast<Handle*>(handle);
    if (config != nullptr) *config = h->last_cfg;
    if (splitk != nullptr) *splitk = h->last_splitk;
    return SNHIP_STATUS_SUCCESS;
}

int snhip_config_count(void) { return kNumConfigs; }

int snhip_config_desc(int config, int desc[6]) {
    if (config < 0 || config >= kNumConfigs || desc == nullptr) return SNHIP_STATUS_INVALID_VALUE;
    desc[0] = kConfigs[config].BM;
    desc[1] = kConfigs[config].BN;
    desc[2] = kConfigs[config].BK;
    desc[3] = kConfigs[config].NT;
    desc[4] = kConfigs[config].lds_bytes;
    desc[5] = kConfigs[config].kind;
    return SNHIP_STATUS_SUCCESS;
}

}  // extern "C"

#include "rnn_layers.hpp"
