// Scaled-dot-product attention forward for gfx950 in one kernel:
//     S = scale * Q . K^T  ->  causal mask (-1e12 above the diagonal)  ->  softmax over keys  ->  O = P . V
// which the reference runs as BatchMatrixMultiplication, SetAllElementsAboveMainDiagonal, softmax over the last
// dimension and a second BatchMatrixMultiplication (Prod/Layers/ScaledDotProductAttentionLayer.cs:46-91), with the
// (batch, Tq, Tk) scores travelling through memory three times.  Here they never leave the registers; the softmax
// output P is written out once if the caller wants it (the reference keeps it for the backward pass, :87-90).
//
// Shape of the work.  A workgroup of four wavefronts owns 128 queries of one (batch, head) matrix; each wavefront owns
// 32 of them and ALL keys (at most 256).  Both products are computed transposed so that the key axis of the scores
// lies along a lane's accumulator registers:
//   S^T[key][query] = K . Q^T   - A operand K from LDS (k-major), B operand Q^T from registers, 8 MFMA tiles of
//                                 32 keys x 32 queries per wavefront, k = head dimension (at most 64);
//   softmax                     - a lane holds 128 of the 256 keys of ITS query (lane l and lane l^32 share a query),
//                                 so max and sum are register reductions plus one cross-lane step;
//   O^T[dv][query] = V^T . P^T  - the B operand of each k step IS the accumulator register pair the score product
//                                 left in place (v_mfma_f32_32x32x2: k = lane / 32), the A operand is a row of V
//                                 from LDS.  P is never rearranged.
// LDS: K as [d][key] (pitch keys + 32) and V as [key][dv] (pitch head dimension + 8), 144 KiB together at the largest
// size; both pitches put the two half-waves of a ds_read_b32 into disjoint banks.  The kernel is instantiated for
// NT = 2, 4, 8 key tiles (up to 64, 128, 256 keys) and a head dimension of up to 32 or 64; keys and dimensions short of
// the instantiated size are zero-filled and masked.  Sizes beyond 256 keys or a head dimension beyond 64 are not
// handled here (the caller runs the four-call sequence instead).
#pragma once
#include <hip/hip_runtime.h>

#include "sgemm_mfma.hpp"

namespace snhip {

constexpr int AT_BQ = 128;  // queries per workgroup

template <int NT, int HD>
struct AttnCfg {
    static_assert(NT % 2 == 0 && NT <= 8 && (HD == 32 || HD == 64), "unsupported attention tile");
    static constexpr int KEYS = NT * 32;   // keys per (batch, head) at most
    static constexpr int KP = KEYS + 32;   // pitch of Ks[d][key]   (== 32 mod 64)
    static constexpr int VP = HD + 8;      // pitch of Vs[key][dv]  (4 * VP == 32 mod 64)
    static constexpr int LDS_BYTES = (HD * KP + KEYS * VP) * 4;
};

struct AttnParams {
    const float* Q;
    const float* K;
    const float* V;
    float* O;
    float* P;  // softmax output [z][Tq][Tk] (contiguous), or nullptr
    int Tq, Tk, dk, dv;
    int ldq, ldk, ldv, ldo;
    long long sQ, sK, sV, sO;      // strides between matrices of the inner batch level, elements
    long long sQ2, sK2, sV2, sO2;  // ... of the outer level
    int batch_inner;
    float scale;
    int causal;
    int flags;  // bit 0: O rows may be written as aligned 16-byte vectors, bit 1: P rows likewise
};

__device__ __forceinline__ f32x4 load4_guarded(const float* p, int nvalid) {
    f32x4 x = {0.0f, 0.0f, 0.0f, 0.0f};
    if (nvalid >= 4) {
        __builtin_memcpy(&x, p, 16);
    } else {
        if (nvalid > 0) x.x = p[0];
        if (nvalid > 1) x.y = p[1];
        if (nvalid > 2) x.z = p[2];
    }
    return x;
}

template <int NT, int HD>
__global__ void __launch_bounds__(256) attention_fwd_kernel(const AttnParams p) {
    using CFG = AttnCfg<NT, HD>;
    constexpr int AT_TK = CFG::KEYS, AT_D = HD, AT_KP = CFG::KP, AT_VP = CFG::VP;
    extern __shared__ __attribute__((aligned(16))) float smem[];
    float* const Ks = smem;                  // [AT_D][AT_KP]
    float* const Vs = smem + AT_D * AT_KP;   // [AT_TK][AT_VP]

    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = tid >> 6;
    const int l32 = lane & 31, lhi = lane >> 5;
    const int z = blockIdx.y;
    const int q0 = blockIdx.x * AT_BQ;
    const BatchIndex bi = split_batch(z, p.batch_inner);
    const float* Qz = p.Q + batch_offset(bi, p.sQ, p.sQ2);
    const float* Kz = p.K + batch_offset(bi, p.sK, p.sK2);
    const float* Vz = p.V + batch_offset(bi, p.sV, p.sV2);
    float* Oz = p.O + batch_offset(bi, p.sO, p.sO2);

    // ---- K -> Ks[d][key]: consecutive threads take consecutive keys, so the transposing LDS stores of one
    //      instruction hit consecutive addresses; a thread walks along d ----
#pragma unroll
    for (int it = 0; it < (AT_TK * AT_D / 4) / 256; ++it) {
        const int idx = it * 256 + tid;
        const int key = idx % AT_TK, v = idx / AT_TK;
        const int nvalid = (key < p.Tk) ? (p.dk - 4 * v) : 0;
        const f32x4 x = load4_guarded(Kz + (long long)key * p.ldk + 4 * v, nvalid);
        Ks[(4 * v + 0) * AT_KP + key] = x.x;
        Ks[(4 * v + 1) * AT_KP + key] = x.y;
        Ks[(4 * v + 2) * AT_KP + key] = x.z;
        Ks[(4 * v + 3) * AT_KP + key] = x.w;
    }
    // ---- V -> Vs[key][dv]: 16 consecutive threads read one 256-byte row ----
#pragma unroll
    for (int it = 0; it < (AT_TK * AT_D / 4) / 256; ++it) {
        const int idx = it * 256 + tid;
        const int key = idx / (AT_D / 4), v = idx % (AT_D / 4);
        const int nvalid = (key < p.Tk) ? (p.dv - 4 * v) : 0;
        const f32x4 x = load4_guarded(Vz + (long long)key * p.ldv + 4 * v, nvalid);
        *reinterpret_cast<f32x4*>(Vs + key * AT_VP + 4 * v) = x;
    }
    // ---- this lane's query row as the B operand of the score product: qf[s] = Q[row][2 s + lane / 32] ----
    const int row = q0 + wave * 32 + l32;
    const bool row_ok = row < p.Tq;
    float qf[AT_D / 2];
    {
        const float* qrow = Qz + (long long)row * p.ldq;
#pragma unroll
        for (int j = 0; j < AT_D / 4; ++j) {
            const f32x4 x = load4_guarded(qrow + 4 * j, row_ok ? (p.dk - 4 * j) : 0);
            qf[2 * j] = lhi ? x.y : x.x;
            qf[2 * j + 1] = lhi ? x.w : x.z;
        }
    }
    __syncthreads();

    // ---- S^T = K . Q^T: 8 tiles of 32 keys x 32 queries ----
    f32x16 sacc[AT_TK / 32];
#pragma unroll
    for (int t = 0; t < AT_TK / 32; ++t)
#pragma unroll
        for (int r = 0; r < 16; ++r) sacc[t][r] = 0.0f;
#pragma unroll
    for (int s = 0; s < AT_D / 2; ++s) {
        const float* kr = Ks + (2 * s + lhi) * AT_KP + l32;
#pragma unroll
        for (int t = 0; t < AT_TK / 32; ++t)
            sacc[t] = __builtin_amdgcn_mfma_f32_32x32x2f32(kr[t * 32], qf[s], sacc[t], 0, 0, 0);
    }

    // ---- scale, mask, softmax over the keys of this lane's query ----
    // sacc[t][r] is key  t*32 + 8*(r/4) + 4*lhi + r%4  of query  l32.
    constexpr float kNegInf = -3.402823466e+38f;
    float m = kNegInf;
#pragma unroll
    for (int t = 0; t < AT_TK / 32; ++t) {
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            const int key = t * 32 + 8 * (r / 4) + 4 * lhi + (r % 4);
            float v = p.scale * sacc[t][r];
            if (p.causal && key > row) v = -1e12f;  // SetAllElementsAboveMainDiagonal(-1e12), :73-76
            if (key >= p.Tk) v = kNegInf;
            sacc[t][r] = v;
            m = fmaxf(m, v);
        }
    }
    m = fmaxf(m, __shfl_xor(m, 32, 64));
    float sum = 0.0f;
#pragma unroll
    for (int t = 0; t < AT_TK / 32; ++t) {
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            const int key = t * 32 + 8 * (r / 4) + 4 * lhi + (r % 4);
            const float e = (key < p.Tk) ? __expf(sacc[t][r] - m) : 0.0f;
            sacc[t][r] = e;
            sum += e;
        }
    }
    sum += __shfl_xor(sum, 32, 64);
    const float inv = 1.0f / sum;
#pragma unroll
    for (int t = 0; t < AT_TK / 32; ++t)
#pragma unroll
        for (int r = 0; r < 16; ++r) sacc[t][r] *= inv;

    // ---- P out (four consecutive keys per register group) ----
    if (p.P != nullptr && row_ok) {
        float* prow = p.P + ((long long)z * p.Tq + row) * p.Tk;
#pragma unroll
        for (int t = 0; t < AT_TK / 32; ++t) {
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                const int key0 = t * 32 + 8 * g + 4 * lhi;
                if (key0 >= p.Tk) continue;
                if ((p.flags & 2) && key0 + 4 <= p.Tk) {
                    *reinterpret_cast<f32x4*>(prow + key0) =
                        f32x4{sacc[t][4 * g], sacc[t][4 * g + 1], sacc[t][4 * g + 2], sacc[t][4 * g + 3]};
                } else {
#pragma unroll
                    for (int j = 0; j < 4; ++j)
                        if (key0 + j < p.Tk) prow[key0 + j] = sacc[t][4 * g + j];
                }
            }
        }
    }

    // ---- O^T = V^T . P^T: the probabilities are already where the B operand wants them ----
    f32x16 oacc[AT_D / 32];
#pragma unroll
    for (int mt = 0; mt < AT_D / 32; ++mt)
#pragma unroll
        for (int r = 0; r < 16; ++r) oacc[mt][r] = 0.0f;
#pragma unroll
    for (int t = 0; t < AT_TK / 32; ++t) {
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            const int key = t * 32 + 8 * (r / 4) + 4 * lhi + (r % 4);
            const float* vr = Vs + key * AT_VP + l32;
#pragma unroll
            for (int mt = 0; mt < AT_D / 32; ++mt)
                oacc[mt] = __builtin_amdgcn_mfma_f32_32x32x2f32(vr[mt * 32], sacc[t][r], oacc[mt], 0, 0, 0);
        }
    }
    // oacc[mt][r] is O[row][mt*32 + 8*(r/4) + 4*lhi + r%4]
    if (row_ok) {
        float* orow = Oz + (long long)row * p.ldo;
#pragma unroll
        for (int mt = 0; mt < AT_D / 32; ++mt) {
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                const int c0 = mt * 32 + 8 * g + 4 * lhi;
                if (c0 >= p.dv) continue;
                if ((p.flags & 1) && c0 + 4 <= p.dv) {
                    *reinterpret_cast<f32x4*>(orow + c0) =
                        f32x4{oacc[mt][4 * g], oacc[mt][4 * g + 1], oacc[mt][4 * g + 2], oacc[mt][4 * g + 3]};
                } else {
#pragma unroll
                    for (int j = 0; j < 4; ++j)
                        if (c0 + j < p.dv) orow[c0 + j] = oacc[mt][4 * g + j];
                }
            }
        }
    }
}

}  // namespace snhip
