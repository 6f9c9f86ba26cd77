// Scaled-dot-product attention forward for gfx950 in one kernel:
//     S = scale * Q . K^T  ->  causal mask (-1e12 above the diagonal)  ->  softmax over keys  ->  O = P . V
// which the reference runs as BatchMatrixMultiplication, SetAllElementsAboveMainDiagonal, softmax over the last
// dimension and a second BatchMatrixMultiplication (Prod/Layers/ScaledDotProductAttentionLayer.cs:46-91), with the
// (batch, Tq, Tk) scores travelling through memory three times.  Here they never leave the registers; the softmax
// output P is written out once if the caller wants it (the reference keeps it for the backward pass, :87-90).
//
// Shape of the work.  A workgroup of four wavefronts stages K and V of one (batch, head) matrix in LDS once and then
// walks through its queries 128 at a time; each wavefront owns 32 of those and ALL keys (at most 256).  Both products are computed transposed so that the key axis of the scores
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
//
// The same kernel, instantiated with BWD, is the first half of the backward pass
// (ScaledDotProductAttentionBackwardPropagation, same file :111-132): with the roles Q <- dO, K <- V, V <- K it
// computes dP^T = V . dO^T in place of the scores, turns it into the score gradient with the stored softmax output
// (dS = scale * P * (dP - sum_k dP * P), the softmax gradient of :125 applied in registers; P is read twice, row sum
// first), writes dS, and its second product is dQ = dS . K.  dV = P^T . dO and dK = dS^T . Q contract over the queries,
// which lie along the lanes here, and stay batched GEMMs.
#pragma once
#include <hip/hip_runtime.h>

#include "sgemm_mfma.hpp"

namespace snhip {

constexpr int AT_BQ = 128;  // queries per workgroup

template <int NT, int HD>
struct AttnCfg {
    static_assert(NT % 2 == 0 && NT <= 8 && (HD == 32 || HD == 64 || HD == 128), "unsupported attention tile");
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
    float* P;  // forward: softmax output [z][Tq][Tk] (contiguous), or nullptr; backward: the score gradient dS (out)
    const float* Pin;  // backward: the stored softmax output [z][Tq][Tk]
    int Tq, Tk, dk, dv;
    int ldq, ldk, ldv, ldo;
    long long sQ, sK, sV, sO;      // strides between matrices of the inner batch level, elements
    long long sQ2, sK2, sV2, sO2;  // ... of the outer level
    int batch_inner;
    int q_tiles;  // 128-query tiles one workgroup walks through (K and V stay in LDS across them)
    int batch;    // number of (batch, head) matrices
    float scale;
    int causal;
    int flags;  // bit 0: O rows may be written as aligned 16-byte vectors, bit 1: P rows likewise
};

// Branch-free variant for dimensions that are multiples of 4: the address is clamped into the matrix by the caller,
// the load is unconditional (so the compiler can keep many of them in flight) and an invalid vector is zeroed
// afterwards.
__device__ __forceinline__ f32x4 load4_select(const float* p, bool valid) {
    f32x4 x;
    __builtin_memcpy(&x, p, 16);
    if (!valid) x = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
    return x;
}

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

template <int NT, int HD, bool BWD = false>
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
    const BatchIndex bi = split_batch(z, p.batch_inner);
    const float* Qz = p.Q + batch_offset(bi, p.sQ, p.sQ2);
    const float* Kz = p.K + batch_offset(bi, p.sK, p.sK2);
    const float* Vz = p.V + batch_offset(bi, p.sV, p.sV2);
    float* Oz = p.O + batch_offset(bi, p.sO, p.sO2);

    const bool vec4 = (p.dk % 4 == 0) && (p.dv % 4 == 0);  // uniform: whole 16-byte vectors are inside or outside

    // This lane's query row as the B operand of the score product.  The product sums over d in any order as long as
    // both operands agree on it: k step s of lane half h (= lane / 32) stands for d = h * D/2 + s, so a lane reads
    // D/2 consecutive floats of its row - whole 16-byte loads that land in their registers with nothing to select.
    // qf[s] = Q[row][(lane / 32) * D/2 + s].  Rows past Tq read the last row instead: a query is one column of both
    // products, so what such a lane computes never meets another row and is never stored.
    auto load_q = [&](float (&dst)[AT_D / 2], int qrow_index) {
        const bool ok = qrow_index < p.Tq;
        const int d0 = lhi * (AT_D / 2);
        const float* qrow = Qz + (long long)(ok ? qrow_index : p.Tq - 1) * p.ldq + d0;
        if (vec4 && p.dk == AT_D) {
#pragma unroll
            for (int j = 0; j < AT_D / 8; ++j) {
                f32x4 x;
                __builtin_memcpy(&x, qrow + 4 * j, 16);
                dst[4 * j] = x.x;
                dst[4 * j + 1] = x.y;
                dst[4 * j + 2] = x.z;
                dst[4 * j + 3] = x.w;
            }
        } else if (vec4) {
#pragma unroll
            for (int j = 0; j < AT_D / 8; ++j) {
                const bool in = d0 + 4 * j < p.dk;
                const f32x4 x = load4_select(in ? qrow + 4 * j : Qz, ok && in);
                dst[4 * j] = x.x;
                dst[4 * j + 1] = x.y;
                dst[4 * j + 2] = x.z;
                dst[4 * j + 3] = x.w;
            }
        } else {
            for (int j = 0; j < AT_D / 8; ++j) {
                const f32x4 x = load4_guarded(qrow + 4 * j, ok ? (p.dk - d0 - 4 * j) : 0);
                dst[4 * j] = x.x;
                dst[4 * j + 1] = x.y;
                dst[4 * j + 2] = x.z;
                dst[4 * j + 3] = x.w;
            }
        }
    };
    // the first tile's queries are asked for before K and V: loads return in order, and step 0 needs them
    const int qt0 = blockIdx.x * p.q_tiles;
    float qf[AT_D / 2];
    load_q(qf, qt0 * AT_BQ + wave * 32 + l32);


    // ---- K -> Ks[d][key]: consecutive threads take consecutive keys, so the transposing LDS stores of one
    //      instruction hit consecutive addresses; a thread walks along d.
    //      V -> Vs[key][dv]: 16 consecutive threads read one 256-byte row.
    //      All loads are issued before the first LDS store, so they are in flight together; V is not needed until
    //      the second product, so it stays in registers while the first score product runs. ----
    constexpr int KIT = (AT_TK * AT_D / 4) / 256;
    f32x4 kx[KIT], vx[KIT];  // fast path: K and V on their way to LDS; V stays in registers while the first
                             // score product runs and is stored after it
    if (vec4) {
#pragma unroll
        for (int it = 0; it < KIT; ++it) {
            const int idx = it * 256 + tid;
            const int key = idx % AT_TK, v = idx / AT_TK;
            const bool ok = key < p.Tk && 4 * v < p.dk;
            kx[it] = load4_select(Kz + (long long)(key < p.Tk ? key : p.Tk - 1) * p.ldk + (4 * v < p.dk ? 4 * v : 0), ok);
        }
    } else {
        for (int it = 0; it < KIT; ++it) {
            const int idx = it * 256 + tid;
            const int key = idx % AT_TK, v = idx / AT_TK;
            const f32x4 x = load4_guarded(Kz + (long long)key * p.ldk + 4 * v, (key < p.Tk) ? (p.dk - 4 * v) : 0);
            Ks[(4 * v + 0) * AT_KP + key] = x.x;
            Ks[(4 * v + 1) * AT_KP + key] = x.y;
            Ks[(4 * v + 2) * AT_KP + key] = x.z;
            Ks[(4 * v + 3) * AT_KP + key] = x.w;
        }
        for (int it = 0; it < KIT; ++it) {
            const int idx = it * 256 + tid;
            const int key = idx / (AT_D / 4), v = idx % (AT_D / 4);
            const f32x4 x = load4_guarded(Vz + (long long)key * p.ldv + 4 * v, (key < p.Tk) ? (p.dv - 4 * v) : 0);
            *reinterpret_cast<f32x4*>(Vs + key * AT_VP + 4 * v) = x;
        }
    }
    auto load_v = [&]() {
#pragma unroll
        for (int it = 0; it < KIT; ++it) {
            const int idx = it * 256 + tid;
            const int key = idx / (AT_D / 4), v = idx % (AT_D / 4);
            const bool ok = key < p.Tk && 4 * v < p.dv;
            vx[it] = load4_select(Vz + (long long)(key < p.Tk ? key : p.Tk - 1) * p.ldv + (4 * v < p.dv ? 4 * v : 0), ok);
        }
    };
    if (vec4) {
        load_v();
#pragma unroll
        for (int it = 0; it < KIT; ++it) {
            const int idx = it * 256 + tid;
            const int key = idx % AT_TK, v = idx / AT_TK;
            Ks[(4 * v + 0) * AT_KP + key] = kx[it].x;
            Ks[(4 * v + 1) * AT_KP + key] = kx[it].y;
            Ks[(4 * v + 2) * AT_KP + key] = kx[it].z;
            Ks[(4 * v + 3) * AT_KP + key] = kx[it].w;
        }
    }

    __syncthreads();

    for (int qt = qt0; qt < qt0 + p.q_tiles; ++qt) {
    const int q0 = qt * AT_BQ;
    if (q0 >= p.Tq) break;
    const int row = q0 + wave * 32 + l32;
    const bool row_ok = row < p.Tq;

    // ---- S^T = K . Q^T: 8 tiles of 32 keys x 32 queries ----
    f32x16 sacc[AT_TK / 32];
#pragma unroll
    for (int t = 0; t < AT_TK / 32; ++t)
#pragma unroll
        for (int r = 0; r < 16; ++r) sacc[t][r] = 0.0f;
    // A operands are read from LDS one k step ahead of the MFMAs that use them (the fences keep the scheduler
    // from sinking the reads back next to their use).
    {
        constexpr int NTILE = AT_TK / 32;
        const float* kbase = Ks + (lhi * (AT_D / 2)) * AT_KP + l32;  // row d = lhi * D/2 + s in step s, as in load_q
        float ka[2][NTILE];
#pragma unroll
        for (int t = 0; t < NTILE; ++t) ka[0][t] = kbase[t * 32];
#pragma unroll
        for (int s = 0; s < AT_D / 2; ++s) {
            if (s + 1 < AT_D / 2) {
#pragma unroll
                for (int t = 0; t < NTILE; ++t) ka[(s + 1) & 1][t] = kbase[(s + 1) * AT_KP + t * 32];
            }
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int t = 0; t < NTILE; ++t)
                sacc[t] = __builtin_amdgcn_mfma_f32_32x32x2f32(ka[s & 1][t], qf[s], sacc[t], 0, 0, 0);
            __builtin_amdgcn_sched_barrier(0);
        }
    }
    if (vec4 && qt == qt0) {
        // V reaches LDS now (uniform branch: the barrier is taken by every wavefront)
#pragma unroll
        for (int it = 0; it < KIT; ++it) {
            const int idx = it * 256 + tid;
            const int key = idx / (AT_D / 4), v = idx % (AT_D / 4);
            *reinterpret_cast<f32x4*>(Vs + key * AT_VP + 4 * v) = vx[it];
        }
        __syncthreads();
    }

    if constexpr (BWD) {
        // sacc holds dP^T (key t*32 + 8*(r/4) + r%4 + 4*lhi of query l32).  Score gradient through the softmax:
        // dS = scale * P * (dP - sum_k dP_k P_k).  P comes from memory in the accumulator layout (four consecutive keys
        // per 16-byte load), once for the row sum and once more (from cache) for the product.
        const float* prow = p.Pin + ((long long)z * p.Tq + (row_ok ? row : p.Tq - 1)) * p.Tk + 4 * lhi;
        const bool p_vec = (p.flags & 4) != 0;  // uniform: rows of P are 16-byte aligned
        auto load_p = [&](int t, int g) {
            const int key0 = t * 32 + 8 * g;    // + 4 * lhi, already in prow
            const int nvalid = p.Tk - key0 - 4 * lhi;
            if (p_vec && p.Tk == AT_TK) {
                f32x4 x;
                __builtin_memcpy(&x, prow + key0, 16);
                return x;
            }
            return load4_guarded(prow + key0, nvalid);
        };
        float rs = 0.0f;
#pragma unroll
        for (int t = 0; t < AT_TK / 32; ++t) {
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                const f32x4 pv = load_p(t, g);
                rs += sacc[t][4 * g] * pv.x + sacc[t][4 * g + 1] * pv.y + sacc[t][4 * g + 2] * pv.z + sacc[t][4 * g + 3] * pv.w;
            }
        }
        rs += __shfl_xor(rs, 32, 64);
#pragma unroll
        for (int t = 0; t < AT_TK / 32; ++t) {
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                const f32x4 pv = load_p(t, g);
                sacc[t][4 * g] = p.scale * pv.x * (sacc[t][4 * g] - rs);
                sacc[t][4 * g + 1] = p.scale * pv.y * (sacc[t][4 * g + 1] - rs);
                sacc[t][4 * g + 2] = p.scale * pv.z * (sacc[t][4 * g + 2] - rs);
                sacc[t][4 * g + 3] = p.scale * pv.w * (sacc[t][4 * g + 3] - rs);
            }
        }
    } else {
    // Scores are kept as log2-domain values s * scale * log2(e), so that exp(s - max) is one v_exp_f32.
    // A masked score (above the diagonal: the reference's -1e12, ScaledDotProductAttentionLayer.cs:73-76; or a key
    // past Tk) becomes a value so negative that its exponential is exactly zero.  Key index of register (t, r) is
    // t*32 + 8*(r/4) + r%4 + 4*lhi: "key > limit" is one compare against a per-lane constant.
    constexpr float kLog2e = 1.44269504088896340736f;
    constexpr float kMasked = -1e12f * kLog2e;
    const float sl = p.scale * kLog2e;
    float m = -3.402823466e+38f;
    if (p.causal || p.Tk < AT_TK) {  // uniform
        int lim = p.Tk - 1;
        if (p.causal && row < lim) lim = row;
        lim -= 4 * lhi;
#pragma unroll
        for (int t = 0; t < AT_TK / 32; ++t) {
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                float v = sl * sacc[t][r];
                v = (t * 32 + 8 * (r / 4) + (r % 4) > lim) ? kMasked : v;
                sacc[t][r] = v;
                m = fmaxf(m, v);
            }
        }
    } else {
#pragma unroll
        for (int t = 0; t < AT_TK / 32; ++t) {
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const float v = sl * sacc[t][r];
                sacc[t][r] = v;
                m = fmaxf(m, v);
            }
        }
    }
    m = fmaxf(m, __shfl_xor(m, 32, 64));
    float sum = 0.0f;
#pragma unroll
    for (int t = 0; t < AT_TK / 32; ++t) {
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            const float e = __builtin_amdgcn_exp2f(sacc[t][r] - m);
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

    }

    // ---- P out (four consecutive keys per register group).  With all keys present and aligned rows the stores
    //      are spread over the second product's MFMAs instead (below); this is the general form. ----
    // (uniform; a tile with query rows past Tq takes the general form, so that the spread stores need no predicate
    // and the second product stays one straight run of instructions)
    const bool p_inline = p.P != nullptr && (p.flags & 2) && p.Tk == AT_TK && q0 + AT_BQ <= p.Tq;
    if (p.P != nullptr && !p_inline && row_ok) {
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

    // the next tile's queries travel while this tile's second product runs
    float qf_next[AT_D / 2];
    load_q(qf_next, (qt + 1 < qt0 + p.q_tiles) ? (q0 + AT_BQ + wave * 32 + l32) : p.Tq);

    // ---- O^T = V^T . P^T: the probabilities are already where the B operand wants them.  Even and odd k steps
    //      accumulate separately, so an MFMA never waits for the result of the one issued just before it. ----
    f32x16 oacc[AT_D / 32];
    auto second_product = [&](auto store_tag) {
        constexpr bool STORE_P = decltype(store_tag)::value;
        constexpr int NSTEP = (AT_TK / 32) * 16;  // k steps: one per accumulator register of the score tiles
        constexpr int MT = AT_D / 32;
        constexpr int LOOK = 2;                   // steps of look-ahead for the LDS reads of V
        f32x16 part[2][MT];
#pragma unroll
        for (int h = 0; h < 2; ++h)
#pragma unroll
            for (int mt = 0; mt < MT; ++mt)
#pragma unroll
                for (int r = 0; r < 16; ++r) part[h][mt][r] = 0.0f;
        const float* vbase = Vs + (4 * lhi) * AT_VP + l32;
        float* const prow = STORE_P ? p.P + ((long long)z * p.Tq + row) * p.Tk + 4 * lhi : nullptr;
        float va[4][MT];
        auto v_off = [](int i) { return ((i / 16) * 32 + 8 * ((i % 16) / 4) + (i % 4)) * AT_VP; };
#pragma unroll
        for (int i = 0; i < LOOK; ++i)
#pragma unroll
            for (int mt = 0; mt < MT; ++mt) va[i][mt] = vbase[v_off(i) + mt * 32];
#pragma unroll
        for (int i = 0; i < NSTEP; ++i) {
            if (i + LOOK < NSTEP) {
#pragma unroll
                for (int mt = 0; mt < MT; ++mt) va[(i + LOOK) % 4][mt] = vbase[v_off(i + LOOK) + mt * 32];
            }
            if (STORE_P && i % 4 == 0) {
                // one 16-byte store of P every four k steps: the write-out rides in the MFMAs' shadow
                const int t = i / 16, g = (i % 16) / 4;
                *reinterpret_cast<f32x4*>(prow + t * 32 + 8 * g) =
                    f32x4{sacc[t][4 * g], sacc[t][4 * g + 1], sacc[t][4 * g + 2], sacc[t][4 * g + 3]};
            }
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int mt = 0; mt < MT; ++mt)
                part[i & 1][mt] = __builtin_amdgcn_mfma_f32_32x32x2f32(va[i % 4][mt], sacc[i / 16][i % 16], part[i & 1][mt],
                                                                       0, 0, 0);
            __builtin_amdgcn_sched_barrier(0);
        }
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) oacc[mt] = part[0][mt] + part[1][mt];
    };
    if (p_inline)
        second_product(std::true_type{});
    else
        second_product(std::false_type{});
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
#pragma unroll
    for (int j = 0; j < AT_D / 2; ++j) qf[j] = qf_next[j];
    }  // query tiles
}

// ---------------------------------------------------------------------------------------------------------------
// The forward pass once more for the common sizes (head dimension exactly HD = 32 or 64 on both sides, up to KEYS
// keys, aligned outputs), laid out so that TWO wavefronts share each SIMD: eight wavefronts per workgroup, each owning
// 16 queries of the 128-query tile and working in 16x16x4 MFMAs.  A wavefront then holds KEYS/4 score registers
// instead of KEYS/2 (64 for 256 keys), everything fits in half the register file, and while one wavefront of a SIMD is
// in its softmax (VALU only) the other keeps the matrix pipe busy.  A workgroup takes several matrices in turn and
// has the next one's K and V in flight while it finishes the current one.
// Both MFMA shapes deliver the same flops per cycle; the 16x16 one reads twice the LDS bytes per flop (32 of the
// 128 bytes per clock a compute unit has).
//   S^T = K . Q^T      A[i = key][k] from Ks[d][key], B[k][j = query] from registers.  k step s of lane group
//                      g = lane / 16 stands for d = (HD / 4) g + s, so a lane holds HD / 4 consecutive floats of its
//                      query row.
//                      sacc[t][r] = S[query lane % 16][key 16 t + 4 g + r]: four consecutive keys per register group.
//   O^T = V^T . P^T    step (t, r): B = sacc[t][r] as it lies, A[i = dv][k = g] = Vs[16 t + 4 g + r][16 mt + lane % 16].
//                      oacc[mt][r] = O[query][16 mt + 4 g + r].
// Pitches: (HD / 4) KP == 16 and 4 VP == 16 (mod 64), so the four lane groups of an operand read hit four different
// sixteen-bank groups.
// ---------------------------------------------------------------------------------------------------------------
template <int KEYS, int HD = 64>
struct Attn16Cfg {
    static_assert(KEYS % 32 == 0 && KEYS <= 256 && (HD == 32 || HD == 64), "unsupported attention tile");
    static constexpr int D = HD;
    // pitch of Ks[d][key]: (D / 4) * KP == 16 (mod 64) spreads the four lane groups of an operand read, and the
    // transposing stores of a wavefront (D / 4 vectors of 64 / (D / 4) keys) land in 64 different banks
    static constexpr int KP = KEYS + (HD == 64 ? 1 : 2);
    static constexpr int VP = D + 4;     // pitch of Vs[key][dv]
    static constexpr int LDS_BYTES = (D * KP + KEYS * VP) * 4;
};

// The two products of the 16-query layout, shared by attention_fwd16_kernel and attention_fwd16_long_kernel.
// S^T = K . Q^T for one wavefront: NKT tiles of 16 keys x 16 queries, K from Ks[d][key] (pitch KP), the lane's NQ query
// floats as the B operand; the A operands are read from LDS one k step ahead of the MFMAs that use them (the fences
// keep the scheduler from sinking the reads back next to their use).
template <int NKT, int NQ, int KP>
__device__ __forceinline__ void attn16_score_product(const float* Ks, int g, int l16, const float (&qf)[NQ],
                                                     f32x4 (&sacc)[NKT]) {
#pragma unroll
    for (int t = 0; t < NKT; ++t) sacc[t] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
    const float* kbase = Ks + (NQ * g) * KP + l16;
    float ka[2][NKT];
#pragma unroll
    for (int t = 0; t < NKT; ++t) ka[0][t] = kbase[t * 16];
#pragma unroll
    for (int s = 0; s < NQ; ++s) {
        if (s + 1 < NQ) {
#pragma unroll
            for (int t = 0; t < NKT; ++t) ka[(s + 1) & 1][t] = kbase[(s + 1) * KP + t * 16];
        }
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int t = 0; t < NKT; ++t)
            sacc[t] = __builtin_amdgcn_mfma_f32_16x16x4f32(ka[s & 1][t], qf[s], sacc[t], 0, 0, 0);
        __builtin_amdgcn_sched_barrier(0);
    }
}

// The same product for the key tiles T0 .. T0 + NT_ - 1 only (the other accumulators are left alone).
template <int T0, int NT_, int NKT, int NQ, int KP>
__device__ __forceinline__ void attn16_score_product_part(const float* Ks, int g, int l16, const float (&qf)[NQ],
                                                          f32x4 (&sacc)[NKT]) {
    static_assert(T0 + NT_ <= NKT, "tile range");
#pragma unroll
    for (int t = 0; t < NT_; ++t) sacc[T0 + t] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
    const float* kbase = Ks + (NQ * g) * KP + l16 + T0 * 16;
    float ka[2][NT_];
#pragma unroll
    for (int t = 0; t < NT_; ++t) ka[0][t] = kbase[t * 16];
#pragma unroll
    for (int s = 0; s < NQ; ++s) {
        if (s + 1 < NQ) {
#pragma unroll
            for (int t = 0; t < NT_; ++t) ka[(s + 1) & 1][t] = kbase[(s + 1) * KP + t * 16];
        }
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int t = 0; t < NT_; ++t)
            sacc[T0 + t] = __builtin_amdgcn_mfma_f32_16x16x4f32(ka[s & 1][t], qf[s], sacc[T0 + t], 0, 0, 0);
        __builtin_amdgcn_sched_barrier(0);
    }
}

// O^T += V^T . P^T for one wavefront: k step (t, r) takes the score register sacc[t][r] as the B operand as it lies and
// A[i = dv][k = g] = Vs[16 t + 4 g + r][16 mt + lane % 16] (pitch VP), read LOOK steps ahead.  STORE_P: the lane's
// probabilities go out on the way, one 16-byte store (four consecutive keys, at prow + 16 t) every four k steps.
template <int NKT, int NDT, int VP, bool STORE_P>
__device__ __forceinline__ void attn16_second_product(const float* Vs, int g, int l16, const f32x4 (&sacc)[NKT],
                                                      f32x4 (&oacc)[NDT], float* prow) {
    constexpr int NSTEP = NKT * 4;
    constexpr int LOOK = 3;
    const float* vbase = Vs + (4 * g) * VP + l16;
    float va[4][NDT];
    auto v_off = [](int i) { return ((i / 4) * 16 + (i % 4)) * VP; };
#pragma unroll
    for (int i = 0; i < LOOK; ++i)
#pragma unroll
        for (int mt = 0; mt < NDT; ++mt) va[i][mt] = vbase[v_off(i) + mt * 16];
#pragma unroll
    for (int i = 0; i < NSTEP; ++i) {
        if (i + LOOK < NSTEP) {
#pragma unroll
            for (int mt = 0; mt < NDT; ++mt) va[(i + LOOK) % 4][mt] = vbase[v_off(i + LOOK) + mt * 16];
        }
        if (STORE_P && i % 4 == 0) *reinterpret_cast<f32x4*>(prow + (i / 4) * 16) = sacc[i / 4];
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int mt = 0; mt < NDT; ++mt)
            oacc[mt] = __builtin_amdgcn_mfma_f32_16x16x4f32(va[i % 4][mt], sacc[i / 4][i % 4], oacc[mt], 0, 0, 0);
        __builtin_amdgcn_sched_barrier(0);
    }
}

//
// BWD: the first half of the backward pass, as in attention_fwd_kernel (Q <- dO, K <- V, V <- K, O <- dQ, P <- dS out,
// Pin <- the stored softmax output): the first product leaves dP^T in the accumulators, the softmax stretch becomes
// dS = scale * P * (dP - sum_keys dP * P), the second product is dQ = dS . K.  A lane's 64 values of P are asked for
// before the first product and wait in registers, so P is read once and its latency is hidden.
template <int KEYS, bool BWD = false, int HD = 64>
__global__ void __launch_bounds__(512) attention_fwd16_kernel(const AttnParams p) {
    using CFG = Attn16Cfg<KEYS, HD>;
    constexpr int D = CFG::D, KP = CFG::KP, VP = CFG::VP;
    constexpr int NKT = KEYS / 16;  // key tiles of 16
    constexpr int NDT = D / 16;     // output column tiles of 16
    constexpr int NQ = D / 4;       // k steps of the score product = query floats per lane
    extern __shared__ __attribute__((aligned(16))) float smem[];
    float* const Ks = smem;            // [D][KP]
    float* const Vs = smem + D * KP;   // [KEYS][VP]

    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = tid >> 6;
    const int l16 = lane & 15, g = lane >> 4;
    const int qt0 = blockIdx.x * p.q_tiles;
    const int qt_end = min(qt0 + p.q_tiles, (p.Tq + AT_BQ - 1) / AT_BQ);

    // Rows past Tq read the last row instead: a query is one column of both products, so what such a lane computes
    // never meets another row and is never stored.
    auto load_q = [&](float (&dst)[NQ], int zz, int qrow_index) {
        const float* qrow = p.Q + batch_offset(split_batch(zz, p.batch_inner), p.sQ, p.sQ2) +
                            (long long)(qrow_index < p.Tq ? qrow_index : p.Tq - 1) * p.ldq + NQ * g;
#pragma unroll
        for (int j = 0; j < NQ / 4; ++j) {
            f32x4 x;
            __builtin_memcpy(&x, qrow + 4 * j, 16);
            dst[4 * j] = x.x, dst[4 * j + 1] = x.y, dst[4 * j + 2] = x.z, dst[4 * j + 3] = x.w;
        }
    };
    // K and V of one matrix on their way to LDS: 16 consecutive threads read one 256-byte row.  The transposing
    // stores into Ks[d][key] are conflict-free because KP == 1 (mod 64): the 16 x 4 (vector, key) pairs of a
    // wavefront land in banks 4 v + c + key.  Addresses are clamped and rows past Tk are zeroed only when they are
    // stored, so nothing waits for these loads before then.
    constexpr int KIT = (KEYS * (D / 4)) / 512;
    f32x4 kx[KIT], vx[KIT];
    // (the thread index goes through an empty asm in both helpers: their address arithmetic is then redone at each
    // call instead of being carried in registers across the products, where every register counts)
    auto load_kv = [&](int zz) {
        int tid = threadIdx.x;
        asm volatile("" : "+v"(tid));
        const BatchIndex bz = split_batch(zz, p.batch_inner);
        const float* Kz = p.K + batch_offset(bz, p.sK, p.sK2);
        const float* Vz = p.V + batch_offset(bz, p.sV, p.sV2);
#pragma unroll
        for (int it = 0; it < KIT; ++it) {
            const int idx = it * 512 + tid;
            const int key = idx / (D / 4), v = idx % (D / 4);
            __builtin_memcpy(&kx[it], Kz + (long long)(key < p.Tk ? key : p.Tk - 1) * p.ldk + 4 * v, 16);
        }
#pragma unroll
        for (int it = 0; it < KIT; ++it) {
            const int idx = it * 512 + tid;
            const int key = idx / (D / 4), v = idx % (D / 4);
            __builtin_memcpy(&vx[it], Vz + (long long)(key < p.Tk ? key : p.Tk - 1) * p.ldv + 4 * v, 16);
        }
    };
    auto store_kv = [&]() {
        int tid = threadIdx.x;
        asm volatile("" : "+v"(tid));
        const f32x4 zero = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
        for (int it = 0; it < KIT; ++it) {
            const int idx = it * 512 + tid;
            const int key = idx / (D / 4), v = idx % (D / 4);
            const f32x4 x = key < p.Tk ? kx[it] : zero;
            Ks[(4 * v + 0) * KP + key] = x.x;
            Ks[(4 * v + 1) * KP + key] = x.y;
            Ks[(4 * v + 2) * KP + key] = x.z;
            Ks[(4 * v + 3) * KP + key] = x.w;
        }
#pragma unroll
        for (int it = 0; it < KIT; ++it) {
            const int idx = it * 512 + tid;
            const int key = idx / (D / 4), v = idx % (D / 4);
            *reinterpret_cast<f32x4*>(Vs + key * VP + 4 * v) = key < p.Tk ? vx[it] : zero;
        }
    };

    // A workgroup walks through the matrices z, z + gridDim.y, ...: while it works on the last query tile of one, K
    // and V of the next are already travelling into registers, so only the first matrix pays for the round trip.
    // The two wavefronts of a SIMD (w and w + 4: wavefronts are dealt to the four SIMDs in turn) share its matrix
    // pipe.  Left alone the older one wins most issue slots and finishes a matrix well ahead of the other; a small
    // standing priority for the younger one evens that out (measured: the pair stays half a product apart, which is
    // what lets one's softmax run under the other's MFMAs; pacing the two into lockstep is slower).
    const int mfma_prio = wave >= 4 ? 1 : 0;
    if (mfma_prio) __builtin_amdgcn_s_setprio(1);
    int z = blockIdx.y;
    if (z >= p.batch || qt0 >= qt_end) return;  // uniform
    float qf[NQ];
    load_q(qf, z, qt0 * AT_BQ + wave * 16 + l16);
    load_kv(z);

    for (; z < p.batch; z += gridDim.y) {
    const int z_next = z + (int)gridDim.y;
    const bool has_next = z_next < p.batch;  // uniform
    float* Oz = p.O + batch_offset(split_batch(z, p.batch_inner), p.sO, p.sO2);
    __syncthreads();  // every wavefront is done with the previous matrix in LDS
    store_kv();
    __syncthreads();

    for (int qt = qt0; qt < qt_end; ++qt) {
        const int q0 = qt * AT_BQ;
        const int row = q0 + wave * 16 + l16;
        const bool row_ok = row < p.Tq;
        const bool last_tile = qt + 1 == qt_end;  // uniform

        // ---- S^T = K . Q^T ----
        f32x4 sacc[NKT];
        f32x4 pin[BWD ? NKT : 1];
        // BWD: the product in two halves of NKT / 2 key tiles, the stored weights of a half asked for in front of that
        // half's MFMAs, so that they arrive behind the product instead of being waited for after it (keys past Tk:
        // dP is zero there, zero rows of the staged operand, and the lane's first keys are read in their place: this kernel
        // is given more than 64 keys, so those exist).
        // 256 keys x 64 do not have the registers for that (66 spilled, measured slower): there the weights are
        // asked for behind the whole product.
        constexpr bool SPLIT = BWD && !(KEYS == 256 && HD == 64);
        if constexpr (SPLIT) {
            constexpr int HALF = NKT / 2;
            const float* prow = p.Pin + ((long long)z * p.Tq + (row_ok ? row : p.Tq - 1)) * p.Tk + 4 * g;
#pragma unroll
            for (int t = 0; t < HALF; ++t)
                __builtin_memcpy(&pin[t], prow + (t * 16 + 4 * g < p.Tk ? t * 16 : 0), 16);
            attn16_score_product_part<0, HALF, NKT, NQ, KP>(Ks, g, l16, qf, sacc);
#pragma unroll
            for (int t = HALF; t < NKT; ++t)
                __builtin_memcpy(&pin[t], prow + (t * 16 + 4 * g < p.Tk ? t * 16 : 0), 16);
            attn16_score_product_part<HALF, HALF, NKT, NQ, KP>(Ks, g, l16, qf, sacc);
        } else {
            attn16_score_product<NKT, NQ, KP>(Ks, g, l16, qf, sacc);
        }
        // The next matrix is asked for here, behind the score product: the wait the compiler puts in front of that
        // product's first MFMA (for the queries) covers every load in flight, and these should not be among them.
        if (!BWD && last_tile && has_next) load_kv(z_next);
        __builtin_amdgcn_sched_barrier(0);

        // ---- softmax over the keys of this lane's query (log2 domain: exp(s - max) is one v_exp_f32; a masked score
        //      - above the diagonal, the reference's -1e12, ScaledDotProductAttentionLayer.cs:73-76, or a key past
        //      Tk - becomes so negative that its exponential is exactly zero).  Key of register (t, r): 16 t + 4 g + r.
        //      The VALU stretch runs at raised priority: the SIMD's other wavefront is then usually inside a product,
        //      always has an MFMA ready, and would otherwise keep winning the issue slot for a pipe that is still busy.
        __builtin_amdgcn_s_setprio(3);
        if constexpr (BWD) {
            // keys past Tk: dP is zero there (zero rows of the staged operand) and so is what is taken for P
            if constexpr (!SPLIT) {
                const float* prow = p.Pin + ((long long)z * p.Tq + (row_ok ? row : p.Tq - 1)) * p.Tk + 4 * g;
#pragma unroll
                for (int t = 0; t < NKT; ++t)
                    __builtin_memcpy(&pin[t], prow + (t * 16 + 4 * g < p.Tk ? t * 16 : 0), 16);
            }
            float rs = 0.0f;
#pragma unroll
            for (int t = 0; t < NKT; ++t) {
                if (p.Tk < KEYS && t * 16 + 4 * g >= p.Tk) pin[t] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
                rs += sacc[t].x * pin[t].x + sacc[t].y * pin[t].y + sacc[t].z * pin[t].z + sacc[t].w * pin[t].w;
            }
            rs += __shfl_xor(rs, 16, 64);
            rs += __shfl_xor(rs, 32, 64);
#pragma unroll
            for (int t = 0; t < NKT; ++t)
#pragma unroll
                for (int r = 0; r < 4; ++r) sacc[t][r] = p.scale * pin[t][r] * (sacc[t][r] - rs);
        } else {
        constexpr float kLog2e = 1.44269504088896340736f;
        constexpr float kMasked = -1e12f * kLog2e;
        const float sl = p.scale * kLog2e;
        float m = -3.402823466e+38f;
        if (p.causal || p.Tk < KEYS) {  // uniform
            int lim = p.Tk - 1;
            if (p.causal && row < lim) lim = row;
            lim -= 4 * g;
#pragma unroll
            for (int t = 0; t < NKT; ++t)
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    float v = sl * sacc[t][r];
                    v = (t * 16 + r > lim) ? kMasked : v;
                    sacc[t][r] = v;
                    m = fmaxf(m, v);
                }
        } else {
#pragma unroll
            for (int t = 0; t < NKT; ++t)
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    const float v = sl * sacc[t][r];
                    sacc[t][r] = v;
                    m = fmaxf(m, v);
                }
        }
        m = fmaxf(m, __shfl_xor(m, 16, 64));
        m = fmaxf(m, __shfl_xor(m, 32, 64));
        float sum = 0.0f;
#pragma unroll
        for (int t = 0; t < NKT; ++t)
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const float e = __builtin_amdgcn_exp2f(sacc[t][r] - m);
                sacc[t][r] = e;
                sum += e;
            }
        sum += __shfl_xor(sum, 16, 64);
        sum += __shfl_xor(sum, 32, 64);
        const float inv = 1.0f / sum;
#pragma unroll
        for (int t = 0; t < NKT; ++t)
#pragma unroll
            for (int r = 0; r < 4; ++r) sacc[t][r] *= inv;
        }
        if (mfma_prio) __builtin_amdgcn_s_setprio(1); else __builtin_amdgcn_s_setprio(0);
        if (BWD && last_tile && has_next) load_kv(z_next);  // (behind the stretch that still holds P in registers)
        __builtin_amdgcn_sched_barrier(0);

        // ---- P out: 16 bytes (four consecutive keys) per register group.  In a full tile with all keys present the
        //      stores are spread over the second product instead (uniform choice). ----
        const bool p_inline = p.P != nullptr && p.Tk == KEYS && q0 + AT_BQ <= p.Tq;
        if (p.P != nullptr && !p_inline && row_ok) {
            float* prow = p.P + ((long long)z * p.Tq + row) * p.Tk + 4 * g;
#pragma unroll
            for (int t = 0; t < NKT; ++t)
                if (t * 16 + 4 * g < p.Tk) *reinterpret_cast<f32x4*>(prow + t * 16) = sacc[t];
        }

        // the next tile's queries (the next matrix's first tile after the last one) travel while this tile's second
        // product runs
        float qf_next[NQ];
        if (!last_tile)
            load_q(qf_next, z, q0 + AT_BQ + wave * 16 + l16);
        else
            load_q(qf_next, has_next ? z_next : z, qt0 * AT_BQ + wave * 16 + l16);

        // ---- O^T = V^T . P^T ----
        f32x4 oacc[NDT];
#pragma unroll
        for (int mt = 0; mt < NDT; ++mt) oacc[mt] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
        if (p_inline)
            attn16_second_product<NKT, NDT, VP, true>(Vs, g, l16, sacc, oacc,
                                                      p.P + ((long long)z * p.Tq + row) * p.Tk + 4 * g);
        else
            attn16_second_product<NKT, NDT, VP, false>(Vs, g, l16, sacc, oacc, nullptr);
        if (row_ok) {
            float* orow = Oz + (long long)row * p.ldo + 4 * g;
#pragma unroll
            for (int mt = 0; mt < NDT; ++mt) *reinterpret_cast<f32x4*>(orow + mt * 16) = oacc[mt];
        }
#pragma unroll
        for (int j = 0; j < NQ; ++j) qf[j] = qf_next[j];
    }  // query tiles
    }  // matrices
}

// ---------------------------------------------------------------------------------------------------------------
// The same forward pass for any number of keys: the keys are walked in blocks of 256 in TWO passes.
//   pass 1: scores of every block (K . Q^T as above), running row maximum and row sum of exponentials - nothing
//           else is kept;
//   pass 2: the scores again, now turned into the final probabilities p = exp(s - max) / sum at once (the softmax
//           formula of the reference, Prod/CPU/CpuTensorActivationFunctions.cs:19-46, with its global maximum),
//           written out if the caller keeps them, and multiplied into O += P_block . V_block.
// Recomputing the scores costs half again the MFMA work of the single-block kernel, and buys exact, never rescaled
// probabilities that are written exactly once - which is what a caller that keeps the (Tq, Tk) softmax output for
// its backward pass needs.  With the causal mask, key blocks that lie wholly above the diagonal of a query tile are
// not computed; their part of the stored probabilities is written as zeros.
// A workgroup owns 128 queries (32 per wavefront) of one (batch, head) matrix; the K block (and in pass 2 the V
// block) is staged in LDS exactly as in the kernel above.  Head dimensions: multiples of 4 up to HD.
// ---------------------------------------------------------------------------------------------------------------
template <int HD>
__global__ void __launch_bounds__(256) attention_fwd_long_kernel(const AttnParams p) {
    using CFG = AttnCfg<8, HD>;
    constexpr int AT_TK = CFG::KEYS, AT_D = HD, AT_KP = CFG::KP, AT_VP = CFG::VP;
    constexpr int NTILE = AT_TK / 32, MT = AT_D / 32;
    extern __shared__ __attribute__((aligned(16))) float smem[];
    float* const Ks = smem;                  // [AT_D][AT_KP]
    float* const Vs = smem + AT_D * AT_KP;   // [AT_TK][AT_VP]

    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = tid >> 6;
    const int l32 = lane & 31, lhi = lane >> 5;
    const int z = blockIdx.x;  // matrices run fastest in the grid, query tiles slowest (see q0)
    const BatchIndex bi = split_batch(z, p.batch_inner);
    const float* Qz = p.Q + batch_offset(bi, p.sQ, p.sQ2);
    const float* Kz = p.K + batch_offset(bi, p.sK, p.sK2);
    const float* Vz = p.V + batch_offset(bi, p.sV, p.sV2);
    float* Oz = p.O + batch_offset(bi, p.sO, p.sO2);

    // last query tile first, for all matrices, then the tile before it, ...: with the causal mask the late tiles see
    // the most key blocks, and started first they leave the short ones to fill the end of the launch
    const int q0 = (int)(gridDim.y - 1 - blockIdx.y) * AT_BQ;
    const int row = q0 + wave * 32 + l32;
    const bool row_ok = row < p.Tq;

    // this lane's query row as the B operand of the score product: qf[s] = Q[row][2 s + lane / 32]
    float qf[AT_D / 2];
    {
        const float* qrow = Qz + (long long)(row_ok ? row : p.Tq - 1) * p.ldq;
#pragma unroll
        for (int j = 0; j < AT_D / 4; ++j) {
            const f32x4 x = load4_select(qrow + (4 * j < p.dk ? 4 * j : 0), row_ok && 4 * j < p.dk);
            qf[2 * j] = lhi ? x.y : x.x;
            qf[2 * j + 1] = lhi ? x.w : x.z;
        }
    }

    const int nblocks = (p.Tk + AT_TK - 1) / AT_TK;
    // causal: the last query of the tile sees keys 0 .. q0 + 127
    int nb_needed = nblocks;
    if (p.causal) {
        const int last_row = (q0 + AT_BQ - 1 < p.Tq - 1) ? q0 + AT_BQ - 1 : p.Tq - 1;
        const int nb = last_row / AT_TK + 1;
        nb_needed = nb < nblocks ? nb : nblocks;
    }

    constexpr int KIT = (AT_TK * AT_D / 4) / 256;
    auto stage_k = [&](int kb) {
        f32x4 kx[KIT];
#pragma unroll
        for (int it = 0; it < KIT; ++it) {
            const int idx = it * 256 + tid;
            const int key = kb * AT_TK + idx % AT_TK, v = idx / AT_TK;
            const bool ok = key < p.Tk && 4 * v < p.dk;
            kx[it] = load4_select(Kz + (long long)(key < p.Tk ? key : p.Tk - 1) * p.ldk + (4 * v < p.dk ? 4 * v : 0), ok);
        }
#pragma unroll
        for (int it = 0; it < KIT; ++it) {
            const int idx = it * 256 + tid;
            const int key = idx % AT_TK, v = idx / AT_TK;
            Ks[(4 * v + 0) * AT_KP + key] = kx[it].x;
            Ks[(4 * v + 1) * AT_KP + key] = kx[it].y;
            Ks[(4 * v + 2) * AT_KP + key] = kx[it].z;
            Ks[(4 * v + 3) * AT_KP + key] = kx[it].w;
        }
    };
    auto stage_v = [&](int kb) {
        f32x4 vx[KIT];
#pragma unroll
        for (int it = 0; it < KIT; ++it) {
            const int idx = it * 256 + tid;
            const int key = kb * AT_TK + idx / (AT_D / 4), v = idx % (AT_D / 4);
            const bool ok = key < p.Tk && 4 * v < p.dv;
            vx[it] = load4_select(Vz + (long long)(key < p.Tk ? key : p.Tk - 1) * p.ldv + (4 * v < p.dv ? 4 * v : 0), ok);
        }
#pragma unroll
        for (int it = 0; it < KIT; ++it) {
            const int idx = it * 256 + tid;
            const int key = idx / (AT_D / 4), v = idx % (AT_D / 4);
            *reinterpret_cast<f32x4*>(Vs + key * AT_VP + 4 * v) = vx[it];
        }
    };

    constexpr float kLog2e = 1.44269504088896340736f;
    constexpr float kMasked = -1e12f * kLog2e;
    const float sl = p.scale * kLog2e;

    // scores of key block kb in the log2 domain, masked: sacc[t][r] belongs to key kb*256 + t*32 + 8*(r/4) + r%4 + 4*lhi
    f32x16 sacc[NTILE];
    auto scores = [&](int kb) {
#pragma unroll
        for (int t = 0; t < NTILE; ++t)
#pragma unroll
            for (int r = 0; r < 16; ++r) sacc[t][r] = 0.0f;
        const float* kbase = Ks + lhi * AT_KP + l32;
        float ka[2][NTILE];
#pragma unroll
        for (int t = 0; t < NTILE; ++t) ka[0][t] = kbase[t * 32];
#pragma unroll
        for (int s = 0; s < AT_D / 2; ++s) {
            if (s + 1 < AT_D / 2) {
#pragma unroll
                for (int t = 0; t < NTILE; ++t) ka[(s + 1) & 1][t] = kbase[(2 * (s + 1)) * AT_KP + t * 32];
            }
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int t = 0; t < NTILE; ++t)
                sacc[t] = __builtin_amdgcn_mfma_f32_32x32x2f32(ka[s & 1][t], qf[s], sacc[t], 0, 0, 0);
            __builtin_amdgcn_sched_barrier(0);
        }
        // last key this lane's query may see, relative to the block and to the lane's own offset
        int lim = p.Tk - 1;
        if (p.causal && row < lim) lim = row;
        lim -= kb * AT_TK + 4 * lhi;
#pragma unroll
        for (int t = 0; t < NTILE; ++t) {
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const float v = sl * sacc[t][r];
                sacc[t][r] = (t * 32 + 8 * (r / 4) + (r % 4) > lim) ? kMasked : v;
            }
        }
    };

    // ---- pass 1: row maximum and row sum over all needed blocks ----
    float m = -3.402823466e+38f, l = 0.0f;
    for (int kb = 0; kb < nb_needed; ++kb) {
        stage_k(kb);
        __syncthreads();
        scores(kb);
        float bm = -3.402823466e+38f;
#pragma unroll
        for (int t = 0; t < NTILE; ++t)
#pragma unroll
            for (int r = 0; r < 16; ++r) bm = fmaxf(bm, sacc[t][r]);
        bm = fmaxf(bm, __shfl_xor(bm, 32, 64));
        const float m_new = fmaxf(m, bm);
        float bs = 0.0f;
#pragma unroll
        for (int t = 0; t < NTILE; ++t)
#pragma unroll
            for (int r = 0; r < 16; ++r) bs += __builtin_amdgcn_exp2f(sacc[t][r] - m_new);
        bs += __shfl_xor(bs, 32, 64);
        l = l * __builtin_amdgcn_exp2f(m - m_new) + bs;
        m = m_new;
        __syncthreads();  // the block has been read by every wavefront: its LDS may be overwritten
    }
    const float inv = 1.0f / l;

    // ---- pass 2: probabilities, P out, O += P . V ----
    f32x16 oacc[MT];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
        for (int r = 0; r < 16; ++r) oacc[mt][r] = 0.0f;
    float* const pbase = (p.P != nullptr) ? p.P + ((long long)z * p.Tq + (row_ok ? row : 0)) * p.Tk : nullptr;
    for (int kb = 0; kb < nb_needed; ++kb) {
        stage_k(kb);
        stage_v(kb);
        __syncthreads();
        scores(kb);
#pragma unroll
        for (int t = 0; t < NTILE; ++t)
#pragma unroll
            for (int r = 0; r < 16; ++r) sacc[t][r] = __builtin_amdgcn_exp2f(sacc[t][r] - m) * inv;

        if (pbase != nullptr && row_ok) {
            float* prow = pbase + kb * AT_TK;
            const bool whole = (p.flags & 2) && (kb + 1) * AT_TK <= p.Tk;  // uniform
#pragma unroll
            for (int t = 0; t < NTILE; ++t) {
#pragma unroll
                for (int g = 0; g < 4; ++g) {
                    const int key0 = t * 32 + 8 * g + 4 * lhi;
                    if (whole) {
                        *reinterpret_cast<f32x4*>(prow + key0) =
                            f32x4{sacc[t][4 * g], sacc[t][4 * g + 1], sacc[t][4 * g + 2], sacc[t][4 * g + 3]};
                    } else {
#pragma unroll
                        for (int j = 0; j < 4; ++j)
                            if (kb * AT_TK + key0 + j < p.Tk) prow[key0 + j] = sacc[t][4 * g + j];
                    }
                }
            }
        }

        // O^T += V^T . P^T: even and odd k steps accumulate separately (no MFMA waits for its predecessor)
        {
            constexpr int NSTEP = NTILE * 16;
            constexpr int LOOK = 2;
            f32x16 part[2][MT];
#pragma unroll
            for (int h = 0; h < 2; ++h)
#pragma unroll
                for (int mt = 0; mt < MT; ++mt)
#pragma unroll
                    for (int r = 0; r < 16; ++r) part[h][mt][r] = 0.0f;
            const float* vbase = Vs + (4 * lhi) * AT_VP + l32;
            float va[4][MT];
            auto v_off = [](int i) { return ((i / 16) * 32 + 8 * ((i % 16) / 4) + (i % 4)) * AT_VP; };
#pragma unroll
            for (int i = 0; i < LOOK; ++i)
#pragma unroll
                for (int mt = 0; mt < MT; ++mt) va[i][mt] = vbase[v_off(i) + mt * 32];
#pragma unroll
            for (int i = 0; i < NSTEP; ++i) {
                if (i + LOOK < NSTEP) {
#pragma unroll
                    for (int mt = 0; mt < MT; ++mt) va[(i + LOOK) % 4][mt] = vbase[v_off(i + LOOK) + mt * 32];
                }
                __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                for (int mt = 0; mt < MT; ++mt)
                    part[i & 1][mt] = __builtin_amdgcn_mfma_f32_32x32x2f32(va[i % 4][mt], sacc[i / 16][i % 16],
                                                                           part[i & 1][mt], 0, 0, 0);
                __builtin_amdgcn_sched_barrier(0);
            }
#pragma unroll
            for (int mt = 0; mt < MT; ++mt) oacc[mt] += part[0][mt] + part[1][mt];
        }
        __syncthreads();
    }

    // causal: the blocks that were skipped hold zeros in the stored probabilities
    // (a wavefront clears whole rows, lanes along the keys: consecutive 16-byte stores, full lines)
    if (p.P != nullptr && nb_needed < nblocks) {  // uniform
        const int first = nb_needed * AT_TK, ncol = p.Tk - first;
        for (int r = wave; r < AT_BQ && q0 + r < p.Tq; r += 4) {
            float* prow = p.P + ((long long)z * p.Tq + q0 + r) * p.Tk + first;
            if (p.flags & 2) {  // rows are 16-byte aligned and Tk is a multiple of 4
                for (int c = 4 * lane; c < ncol; c += 256) *reinterpret_cast<f32x4*>(prow + c) = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
            } else {
                for (int c = lane; c < ncol; c += 64) prow[c] = 0.0f;
            }
        }
    }

    // oacc[mt][r] is O[row][mt*32 + 8*(r/4) + 4*lhi + r%4]
    if (row_ok) {
        float* orow = Oz + (long long)row * p.ldo;
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) {
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

// ---------------------------------------------------------------------------------------------------------------
// attention_fwd16_kernel with bf16-input MFMAs, for handles in the bf16-input math mode (forward, head dimension
// exactly 64): Q, K and V are rounded to bf16 (nearest even) on their way in, the probabilities on their way into the
// second product; sums, the softmax and the stored weights stay fp32.  v_mfma_f32_16x16x16_bf16 takes four consecutive
// k per lane, and its accumulator layout is that of the fp32 16x16x4 shape, so one score register group
// sacc[t] (keys 16 t + 4 g .. + 3 of query lane % 16), rounded, IS the B operand of a k = 16 step of the second product.
//   S^T = K . Q^T      A[i = key][k = 4 g ..] = Kb[key][16 s + 4 g ..] (K row-major in LDS, 8-byte reads),
//                      B = the lane's query floats 16 s + 4 g .. + 3.
//   O^T = V^T . P^T    A[i = dv][k = 4 g ..] = Vt[dv][16 t + 4 g ..] (V transposed in LDS: keys contiguous).
// Pitches (in 4-byte words) are 4 (mod 64): the 16 rows x 4 lane groups of an operand read hit 64 different banks.
// The matrix work shrinks to a sixteenth; what is left is the softmax and the traffic to memory.
// ---------------------------------------------------------------------------------------------------------------
typedef short bf16x4_bits __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x4_t __attribute__((ext_vector_type(4)));

__device__ __forceinline__ bf16x4_bits round_to_bf16x4(f32x4 x) {
    const bf16x4_t h = __builtin_convertvector(x, bf16x4_t);
    bf16x4_bits b;
    __builtin_memcpy(&b, &h, 8);
    return b;
}

template <int KEYS>
struct Attn16BCfg {
    static_assert(KEYS % 32 == 0 && KEYS <= 256, "unsupported key count");
    static constexpr int D = 64;
    static constexpr int KP = D + 8;      // pitch of Kb[key][d], bf16 elements (36 words)
    static constexpr int VP = KEYS + 8;   // pitch of Vt[dv][key], bf16 elements
    static constexpr int LDS_BYTES = (KEYS * KP + D * VP) * 2;
};

// The two products in bf16 MFMAs, shared by attention_fwd16_bf16_kernel and the long-key kernel's bf16 form.
// qb[s] holds the lane's query values 16 s + 4 g .. + 3, rounded.
template <int NKT, int NS, int KP>
__device__ __forceinline__ void attn16_score_product_bf16(const __bf16* Kb, int g, int l16, const bf16x4_bits (&qbits)[NS],
                                                          f32x4 (&sacc)[NKT]) {
#pragma unroll
    for (int t = 0; t < NKT; ++t) sacc[t] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
    const __bf16* kbase = Kb + l16 * KP + 4 * g;
#pragma unroll
    for (int s = 0; s < NS; ++s) {
        const bf16x4_bits qb = qbits[s];
        constexpr int H = NKT / 2;  // operands of half the key tiles at a time (registers)
#pragma unroll
        for (int half = 0; half < 2; ++half) {
            bf16x4_bits ka[H];
#pragma unroll
            for (int t = 0; t < H; ++t)
                ka[t] = *reinterpret_cast<const bf16x4_bits*>(kbase + (half * H + t) * 16 * KP + 16 * s);
#pragma unroll
            for (int t = 0; t < H; ++t)
                sacc[half * H + t] = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(ka[t], qb, sacc[half * H + t], 0, 0, 0);
            __builtin_amdgcn_sched_barrier(0);
        }
    }
}

template <int NKT, int NDT, int VP>
__device__ __forceinline__ void attn16_second_product_bf16(const __bf16* Vt, int g, int l16, const f32x4 (&sacc)[NKT],
                                                           f32x4 (&oacc)[NDT]) {
    const __bf16* vbase = Vt + l16 * VP + 4 * g;
#pragma unroll
    for (int t = 0; t < NKT; ++t) {
        const bf16x4_bits pb = round_to_bf16x4(sacc[t]);
#pragma unroll
        for (int mt = 0; mt < NDT; ++mt) {
            const bf16x4_bits va = *reinterpret_cast<const bf16x4_bits*>(vbase + mt * 16 * VP + 16 * t);
            oacc[mt] = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(va, pb, oacc[mt], 0, 0, 0);
        }
        // (keeps the scheduler from pulling every step's operand reads to the front: registers, not MFMA time, are
        // what is short here)
        if (t % 2 == 1) __builtin_amdgcn_sched_barrier(0);
    }
}

// BWD: the backward instantiation, roles exchanged as in attention_fwd16_kernel (dP^T = V . dO^T, dS from the stored P, dQ = dS . K).
template <int KEYS, bool BWD = false>
__global__ void __launch_bounds__(512) attention_fwd16_bf16_kernel(const AttnParams p) {
    using CFG = Attn16BCfg<KEYS>;
    constexpr int D = CFG::D, KP = CFG::KP, VP = CFG::VP;
    constexpr int NKT = KEYS / 16, NDT = D / 16, NS = D / 16;
    extern __shared__ __attribute__((aligned(16))) float smem[];
    __bf16* const Kb = reinterpret_cast<__bf16*>(smem);  // [KEYS][KP]
    __bf16* const Vt = Kb + KEYS * KP;                    // [D][VP]

    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int l16 = lane & 15, g = lane >> 4;
    const int qt0 = blockIdx.x * p.q_tiles;
    const int qt_end = min(qt0 + p.q_tiles, (p.Tq + AT_BQ - 1) / AT_BQ);

    // the lane's share of its query row, rounded: qb[s] = Q[row][16 s + 4 g .. + 3] (rows past Tq read the last row)
    auto load_q = [&](f32x4 (&dst)[NS], int zz, int qrow_index) {
        const float* qrow = p.Q + batch_offset(split_batch(zz, p.batch_inner), p.sQ, p.sQ2) +
                            (long long)(qrow_index < p.Tq ? qrow_index : p.Tq - 1) * p.ldq + 4 * g;
#pragma unroll
        for (int s = 0; s < NS; ++s) __builtin_memcpy(&dst[s], qrow + 16 * s, 16);
    };
    // K: 16 lanes to a 256-byte row.  V: a thread takes the same four columns of two adjacent keys, so that it can
    // write pairs of keys as whole words into the transposed tile.
    constexpr int KIT = (KEYS * (D / 4)) / 512;
    f32x4 kx[KIT], vx[KIT];
    auto load_kv = [&](int zz) {
        int tid = threadIdx.x;
        asm volatile("" : "+v"(tid));
        const BatchIndex bz = split_batch(zz, p.batch_inner);
        const float* Kz = p.K + batch_offset(bz, p.sK, p.sK2);
        const float* Vz = p.V + batch_offset(bz, p.sV, p.sV2);
#pragma unroll
        for (int it = 0; it < KIT; ++it) {
            const int idx = it * 512 + tid;
            const int key = idx / (D / 4), v = idx % (D / 4);
            __builtin_memcpy(&kx[it], Kz + (long long)(key < p.Tk ? key : p.Tk - 1) * p.ldk + 4 * v, 16);
        }
#pragma unroll
        for (int it = 0; it < KIT / 2; ++it) {
            const int idx = it * 512 + tid;
            const int kp = idx % (KEYS / 2), v = idx / (KEYS / 2);
#pragma unroll
            for (int h = 0; h < 2; ++h) {
                const int key = 2 * kp + h;
                __builtin_memcpy(&vx[2 * it + h], Vz + (long long)(key < p.Tk ? key : p.Tk - 1) * p.ldv + 4 * v, 16);
            }
        }
    };
    auto store_kv = [&]() {
        int tid = threadIdx.x;
        asm volatile("" : "+v"(tid));
        const f32x4 zero = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
        for (int it = 0; it < KIT; ++it) {
            const int idx = it * 512 + tid;
            const int key = idx / (D / 4), v = idx % (D / 4);
            const bf16x4_bits h = round_to_bf16x4(key < p.Tk ? kx[it] : zero);
            *reinterpret_cast<bf16x4_bits*>(Kb + key * KP + 4 * v) = h;
        }
#pragma unroll
        for (int it = 0; it < KIT / 2; ++it) {
            const int idx = it * 512 + tid;
            const int kp = idx % (KEYS / 2), v = idx / (KEYS / 2);
            const bf16x4_bits lo = round_to_bf16x4(2 * kp < p.Tk ? vx[2 * it] : zero);
            const bf16x4_bits hi = round_to_bf16x4(2 * kp + 1 < p.Tk ? vx[2 * it + 1] : zero);
#pragma unroll
            for (int c = 0; c < 4; ++c) {
                const unsigned int w = (unsigned int)(unsigned short)lo[c] | ((unsigned int)(unsigned short)hi[c] << 16);
                *reinterpret_cast<unsigned int*>(Vt + (4 * v + c) * VP + 2 * kp) = w;
            }
        }
    };

    int z = blockIdx.y;
    if (z >= p.batch || qt0 >= qt_end) return;  // uniform
    f32x4 qf[NS];
    load_q(qf, z, qt0 * AT_BQ + wave * 16 + l16);
    load_kv(z);

    for (; z < p.batch; z += gridDim.y) {
    const int z_next = z + (int)gridDim.y;
    const bool has_next = z_next < p.batch;  // uniform
    float* Oz = p.O + batch_offset(split_batch(z, p.batch_inner), p.sO, p.sO2);
    __syncthreads();  // every wavefront is done with the previous matrix in LDS
    store_kv();
    __syncthreads();

    for (int qt = qt0; qt < qt_end; ++qt) {
        const int q0 = qt * AT_BQ;
        const int row = q0 + wave * 16 + l16;
        const bool row_ok = row < p.Tq;
        const bool last_tile = qt + 1 == qt_end;  // uniform

        // ---- S^T = K . Q^T ----
        f32x4 sacc[NKT];
        {
            bf16x4_bits qbits[NS];
#pragma unroll
            for (int s = 0; s < NS; ++s) qbits[s] = round_to_bf16x4(qf[s]);
            attn16_score_product_bf16<NKT, NS, KP>(Kb, g, l16, qbits, sacc);
        }
        // (behind the product: the wait in front of it covers every load in flight, see attention_fwd16_kernel)
        if (!BWD && last_tile && has_next) load_kv(z_next);
        __builtin_amdgcn_sched_barrier(0);

        if constexpr (BWD) {
            // dS = scale * P * (dP - sum_keys dP * P), P read once (keys past Tk: dP is zero there, P taken as zero)
            f32x4 pin[NKT];
            {
                const float* prow = p.Pin + ((long long)z * p.Tq + (row_ok ? row : p.Tq - 1)) * p.Tk + 4 * g;
#pragma unroll
                for (int t = 0; t < NKT; ++t)
                    __builtin_memcpy(&pin[t], prow + (t * 16 + 4 * g < p.Tk ? t * 16 : 0), 16);
            }
            float rs = 0.0f;
#pragma unroll
            for (int t = 0; t < NKT; ++t) {
                if (p.Tk < KEYS && t * 16 + 4 * g >= p.Tk) pin[t] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
                rs += sacc[t].x * pin[t].x + sacc[t].y * pin[t].y + sacc[t].z * pin[t].z + sacc[t].w * pin[t].w;
            }
            rs += __shfl_xor(rs, 16, 64);
            rs += __shfl_xor(rs, 32, 64);
#pragma unroll
            for (int t = 0; t < NKT; ++t)
#pragma unroll
                for (int r = 0; r < 4; ++r) sacc[t][r] = p.scale * pin[t][r] * (sacc[t][r] - rs);
        } else {
        // ---- softmax over the keys, as in attention_fwd16_kernel ----
        constexpr float kLog2e = 1.44269504088896340736f;
        constexpr float kMasked = -1e12f * kLog2e;
        const float sl = p.scale * kLog2e;
        float m = -3.402823466e+38f;
        if (p.causal || p.Tk < KEYS) {  // uniform
            int lim = p.Tk - 1;
            if (p.causal && row < lim) lim = row;
            lim -= 4 * g;
#pragma unroll
            for (int t = 0; t < NKT; ++t)
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    float v = sl * sacc[t][r];
                    v = (t * 16 + r > lim) ? kMasked : v;
                    sacc[t][r] = v;
                    m = fmaxf(m, v);
                }
        } else {
#pragma unroll
            for (int t = 0; t < NKT; ++t)
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    const float v = sl * sacc[t][r];
                    sacc[t][r] = v;
                    m = fmaxf(m, v);
                }
        }
        m = fmaxf(m, __shfl_xor(m, 16, 64));
        m = fmaxf(m, __shfl_xor(m, 32, 64));
        float sum = 0.0f;
#pragma unroll
        for (int t = 0; t < NKT; ++t)
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const float e = __builtin_amdgcn_exp2f(sacc[t][r] - m);
                sacc[t][r] = e;
                sum += e;
            }
        sum += __shfl_xor(sum, 16, 64);
        sum += __shfl_xor(sum, 32, 64);
        const float inv = 1.0f / sum;
#pragma unroll
        for (int t = 0; t < NKT; ++t)
#pragma unroll
            for (int r = 0; r < 4; ++r) sacc[t][r] *= inv;
        }
        if (BWD && last_tile && has_next) load_kv(z_next);  // (behind the stretch that holds P in registers)
        __builtin_amdgcn_sched_barrier(0);

        // ---- P out (fp32, as computed) ----
        if (p.P != nullptr && row_ok) {
            float* prow = p.P + ((long long)z * p.Tq + row) * p.Tk + 4 * g;
#pragma unroll
            for (int t = 0; t < NKT; ++t)
                if (p.Tk == KEYS || t * 16 + 4 * g < p.Tk) *reinterpret_cast<f32x4*>(prow + t * 16) = sacc[t];
        }

        // the next tile's queries (the next matrix's first tile after the last one) travel during the second product
        f32x4 qf_next[NS];
        if (!last_tile)
            load_q(qf_next, z, q0 + AT_BQ + wave * 16 + l16);
        else
            load_q(qf_next, has_next ? z_next : z, qt0 * AT_BQ + wave * 16 + l16);

        // ---- O^T = V^T . P^T ----
        f32x4 oacc[NDT];
#pragma unroll
        for (int mt = 0; mt < NDT; ++mt) oacc[mt] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
        attn16_second_product_bf16<NKT, NDT, VP>(Vt, g, l16, sacc, oacc);
        if (row_ok) {
            float* orow = Oz + (long long)row * p.ldo + 4 * g;
#pragma unroll
            for (int mt = 0; mt < NDT; ++mt) *reinterpret_cast<f32x4*>(orow + mt * 16) = oacc[mt];
        }
#pragma unroll
        for (int s = 0; s < NS; ++s) qf[s] = qf_next[s];
    }  // query tiles
    }  // matrices
}

// ---------------------------------------------------------------------------------------------------------------
// The two-pass kernel for any number of keys in the layout of attention_fwd16_kernel (head dimension exactly HD = 32
// or 64 on both sides, a multiple of 4 keys, aligned outputs): eight wavefronts of 16 queries, 16x16x4 MFMAs, two wavefronts per
// SIMD, and the next key block's K (pass 1) or K and V (pass 2) travelling in registers while the current block is
// worked on, so that a block change costs the two barriers and the LDS stores but not the round trip to memory.
// Same passes, same skipping of causal blocks and the same zero-fill of the skipped weights as
// attention_fwd_long_kernel.  ONE_PASS is for callers that do not keep the weights (P == nullptr, inference): a single
// walk over the key blocks with a running maximum and sum (two thirds of the MFMA work).  BF16: both products in bf16
// MFMAs as in attention_fwd16_bf16_kernel (operands rounded on their way into LDS, probabilities on their way into the
// second product), for handles in the bf16-input math mode.
// BWD: the first half of the backward pass with the roles exchanged as in attention_fwd16_kernel (Q <- dO, K <- V,
// V <- K, Pin <- the stored weights, P <- dS out, O <- dQ): pass 1 gathers the row sums rs = sum_k P . dP over all key
// blocks, pass 2 forms dS = scale . P . (dP - rs) block by block, writes it and accumulates dQ += dS . K.
// ---------------------------------------------------------------------------------------------------------------
// f(integral_constant<int, 0>), f(integral_constant<int, 1>), ... in order
template <class F, int... I>
__device__ __forceinline__ void for_each_index(F&& f, std::integer_sequence<int, I...>) {
    (f(std::integral_constant<int, I>{}), ...);
}

template <bool ONE_PASS, bool BF16 = false, bool BWD = false, int HD = 64>
__global__ void __launch_bounds__(512) attention_fwd16_long_kernel(const AttnParams p) {
    static_assert(!BWD || (!ONE_PASS && !BF16), "the backward instantiation is the two-pass fp32 one");
    static_assert(!BF16 || HD == 64, "the bf16 form is written for head dimension 64");
    constexpr int KEYS = 256;
    using CFG = Attn16Cfg<KEYS, HD>;
    using BCFG = Attn16BCfg<KEYS>;
    constexpr int D = CFG::D, KP = CFG::KP, VP = CFG::VP;
    constexpr int NKT = KEYS / 16, NDT = D / 16, NQ = D / 4;
    extern __shared__ __attribute__((aligned(16))) float smem[];
    float* const Ks = smem;            // [D][KP]
    float* const Vs = smem + D * KP;   // [KEYS][VP]
    __bf16* const Kb = reinterpret_cast<__bf16*>(smem);  // BF16: [KEYS][BCFG::KP]
    __bf16* const Vt = Kb + KEYS * BCFG::KP;              // BF16: [D][BCFG::VP]

    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int l16 = lane & 15, g = lane >> 4;
    const int z = blockIdx.x;  // matrices run fastest in the grid, query tiles slowest, last tile first
    const BatchIndex bi = split_batch(z, p.batch_inner);
    const float* Kz = p.K + batch_offset(bi, p.sK, p.sK2);
    const float* Vz = p.V + batch_offset(bi, p.sV, p.sV2);
    const int q0 = (int)(gridDim.y - 1 - blockIdx.y) * AT_BQ;
    const int row = q0 + wave * 16 + l16;
    const bool row_ok = row < p.Tq;

    // qf[s] = Q[row][(HD / 4) (lane / 16) + s]; rows past Tq read the last row (never stored)
    // (BF16: qb[s] = Q[row][16 s + 4 g .. + 3], the k order of the bf16 MFMA)
    float qf[NQ];
    bf16x4_bits qb[NQ / 4];
    {
        const float* qrow = p.Q + batch_offset(bi, p.sQ, p.sQ2) + (long long)(row_ok ? row : p.Tq - 1) * p.ldq;
#pragma unroll
        for (int j = 0; j < NQ / 4; ++j) {
            if constexpr (BF16) {
                f32x4 x;
                __builtin_memcpy(&x, qrow + 16 * j + 4 * g, 16);
                qb[j] = round_to_bf16x4(x);
            } else {
                f32x4 x;
                __builtin_memcpy(&x, qrow + NQ * g + 4 * j, 16);
                qf[4 * j] = x.x, qf[4 * j + 1] = x.y, qf[4 * j + 2] = x.z, qf[4 * j + 3] = x.w;
            }
        }
    }

    const int nblocks = (p.Tk + KEYS - 1) / KEYS;
    int nb_needed = nblocks;  // causal: the last query of the tile sees keys 0 .. q0 + 127
    if (p.causal) {
        const int last_row = (q0 + AT_BQ - 1 < p.Tq - 1) ? q0 + AT_BQ - 1 : p.Tq - 1;
        const int nb = last_row / KEYS + 1;
        nb_needed = nb < nblocks ? nb : nblocks;
    }

    // one key block on its way to LDS (16 lanes to a 256-byte row; clamped addresses, rows past Tk zeroed when stored;
    // the thread index goes through an empty asm so that the address arithmetic is redone at each call instead of
    // being carried in registers across the products)
    constexpr int KIT = (KEYS * (D / 4)) / 512;
    f32x4 kx[KIT], vx[KIT];
    auto load_block = [&](const float* base, int ld, int kb, f32x4 (&dst)[KIT]) {
        int tid = threadIdx.x;
        asm volatile("" : "+v"(tid));
#pragma unroll
        for (int it = 0; it < KIT; ++it) {
            const int idx = it * 512 + tid;
            const int key = kb * KEYS + idx / (D / 4), v = idx % (D / 4);
            __builtin_memcpy(&dst[it], base + (long long)(key < p.Tk ? key : p.Tk - 1) * ld + 4 * v, 16);
        }
    };
    // BF16: V with the same four columns of two adjacent keys per thread (pairs of keys go into the transposed tile
    // as whole words)
    auto load_block_v_pairs = [&](int kb) {
        int tid = threadIdx.x;
        asm volatile("" : "+v"(tid));
#pragma unroll
        for (int it = 0; it < KIT / 2; ++it) {
            const int idx = it * 512 + tid;
            const int kp = idx % (KEYS / 2), v = idx / (KEYS / 2);
#pragma unroll
            for (int h = 0; h < 2; ++h) {
                const int key = kb * KEYS + 2 * kp + h;
                __builtin_memcpy(&vx[2 * it + h], Vz + (long long)(key < p.Tk ? key : p.Tk - 1) * p.ldv + 4 * v, 16);
            }
        }
    };
    auto load_v = [&](int kb) {
        if constexpr (BF16)
            load_block_v_pairs(kb);
        else
            load_block(Vz, p.ldv, kb, vx);
    };
    auto store_k = [&](int kb) {
        int tid = threadIdx.x;
        asm volatile("" : "+v"(tid));
        const f32x4 zero = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
        for (int it = 0; it < KIT; ++it) {
            const int idx = it * 512 + tid;
            const int key = idx / (D / 4), v = idx % (D / 4);
            const f32x4 x = kb * KEYS + key < p.Tk ? kx[it] : zero;
            if constexpr (BF16) {
                *reinterpret_cast<bf16x4_bits*>(Kb + key * BCFG::KP + 4 * v) = round_to_bf16x4(x);
            } else {
                Ks[(4 * v + 0) * KP + key] = x.x;
                Ks[(4 * v + 1) * KP + key] = x.y;
                Ks[(4 * v + 2) * KP + key] = x.z;
                Ks[(4 * v + 3) * KP + key] = x.w;
            }
        }
    };
    auto store_v = [&](int kb) {
        int tid = threadIdx.x;
        asm volatile("" : "+v"(tid));
        const f32x4 zero = {0.0f, 0.0f, 0.0f, 0.0f};
        if constexpr (BF16) {
#pragma unroll
            for (int it = 0; it < KIT / 2; ++it) {
                const int idx = it * 512 + tid;
                const int kp = idx % (KEYS / 2), v = idx / (KEYS / 2);
                const bf16x4_bits lo = round_to_bf16x4(kb * KEYS + 2 * kp < p.Tk ? vx[2 * it] : zero);
                const bf16x4_bits hi = round_to_bf16x4(kb * KEYS + 2 * kp + 1 < p.Tk ? vx[2 * it + 1] : zero);
#pragma unroll
                for (int c = 0; c < 4; ++c) {
                    const unsigned int w2 = (unsigned int)(unsigned short)lo[c] | ((unsigned int)(unsigned short)hi[c] << 16);
                    *reinterpret_cast<unsigned int*>(Vt + (4 * v + c) * BCFG::VP + 2 * kp) = w2;
                }
            }
        } else {
#pragma unroll
            for (int it = 0; it < KIT; ++it) {
                const int idx = it * 512 + tid;
                const int key = idx / (D / 4), v = idx % (D / 4);
                *reinterpret_cast<f32x4*>(Vs + key * VP + 4 * v) = kb * KEYS + key < p.Tk ? vx[it] : zero;
            }
        }
    };

    constexpr float kLog2e = 1.44269504088896340736f;
    constexpr float kMasked = -1e12f * kLog2e;
    const float sl = p.scale * kLog2e;
    const int mfma_prio = wave >= 4 ? 1 : 0;  // see attention_fwd16_kernel
    auto product_priority = [&]() {
        if (mfma_prio)
            __builtin_amdgcn_s_setprio(1);
        else
            __builtin_amdgcn_s_setprio(0);
    };

    // raw scores of the block in LDS: sacc[t][r] belongs to key kb * 256 + 16 t + 4 g + r
    f32x4 sacc[NKT];
    auto score_product = [&]() {
        if constexpr (BF16)
            attn16_score_product_bf16<NKT, NQ / 4, BCFG::KP>(Kb, g, l16, qb, sacc);
        else
            attn16_score_product<NKT, NQ, KP>(Ks, g, l16, qf, sacc);
    };
    // log2-domain scores with the mask (a key past Tk or above the diagonal becomes kMasked: its exponential is 0)
    auto scale_and_mask = [&](int kb) {
        int lim = p.Tk - 1;
        if (p.causal && row < lim) lim = row;
        lim -= kb * KEYS + 4 * g;
#pragma unroll
        for (int t = 0; t < NKT; ++t)
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const float v = sl * sacc[t][r];
                sacc[t][r] = (t * 16 + r > lim) ? kMasked : v;
            }
    };

    // BWD: the stored weights of this lane's keys in block kb (keys past Tk: the lane's keys of block 0 are read
    // instead - they exist, this kernel is given more than 256 keys - and zero is taken)
    // The product runs in PARTS parts of NKT / PARTS key tiles: the weights of a part are asked for LA parts ahead of
    // its MFMAs and used behind them, so their way from memory is covered by the product, and only LA + 1 parts'
    // weights are in registers at a time (all of them across the whole product do not fit beside its operands).  At
    // head dimension 64 a part is a single key tile, asked for four tiles ahead: with halves or quarters of the block
    // (32 registers of weights in flight) the compiler moved half of the output accumulators to scratch and back in
    // every block (48 bytes per lane); single tiles need 252 registers and no scratch, at the same speed.
    constexpr int PARTS = HD == 64 ? 16 : 2;
    constexpr int LA = HD == 64 ? 4 : 1;  // parts asked for ahead
    constexpr int HALF = NKT / PARTS;  // key tiles per part
    f32x4 pin[BWD ? NKT : 1];
    auto load_weights = [&](int kb, int t0) {
        const float* prow = p.Pin + ((long long)z * p.Tq + (row_ok ? row : p.Tq - 1)) * p.Tk + kb * KEYS + 4 * g;
#pragma unroll
        for (int i = 0; i < (BWD ? HALF : 0); ++i) {
            const int t = t0 + i;
            __builtin_memcpy(&pin[t], prow + (kb * KEYS + t * 16 + 4 * g < p.Tk ? t * 16 : -kb * KEYS), 16);
        }
    };
    auto zero_weights_past_end = [&](int kb, int t0) {
        if ((kb + 1) * KEYS > p.Tk) {  // uniform
#pragma unroll
            for (int i = 0; i < (BWD ? HALF : 0); ++i) {
                const int t = t0 + i;
                if (kb * KEYS + t * 16 + 4 * g >= p.Tk) pin[t] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
            }
        }
    };
    auto row_sum_part = [&](int kb, int t0, float& rs) {
        zero_weights_past_end(kb, t0);
#pragma unroll
        for (int i = 0; i < (BWD ? HALF : 0); ++i) {
            const int t = t0 + i;
            rs += sacc[t].x * pin[t].x + sacc[t].y * pin[t].y + sacc[t].z * pin[t].z + sacc[t].w * pin[t].w;
        }
    };
    auto gradient_part = [&](int kb, int t0, float rs) {
        zero_weights_past_end(kb, t0);
#pragma unroll
        for (int i = 0; i < (BWD ? HALF : 0); ++i) {
            const int t = t0 + i;
#pragma unroll
            for (int r = 0; r < 4; ++r) sacc[t][r] = p.scale * pin[t][r] * (sacc[t][r] - rs);
        }
    };

    // one part of the first product of a block and what follows it (behind_part(first key tile of the part))
    auto bwd_part = [&](auto ic, int kb, auto&& behind_part) {
        constexpr int I = decltype(ic)::value;
        attn16_score_product_part<I * HALF, HALF, NKT, NQ, KP>(Ks, g, l16, qf, sacc);
        if constexpr (I + LA < PARTS) load_weights(kb, (I + LA) * HALF);
        __builtin_amdgcn_sched_barrier(0);
        behind_part(I * HALF);
        __builtin_amdgcn_sched_barrier(0);
    };
    auto bwd_parts = [&](int kb, auto&& behind_part) {
#pragma unroll
        for (int i = 0; i < LA; ++i) load_weights(kb, i * HALF);
        for_each_index([&](auto ic) { bwd_part(ic, kb, behind_part); }, std::make_integer_sequence<int, PARTS>{});
    };

    // ---- pass 1: row maximum and row sum over all needed blocks (BWD: the row sums of P . dP) ----
    float m = -3.402823466e+38f, l = 0.0f;
    float rs = 0.0f;
    load_block(Kz, p.ldk, 0, kx);
    if constexpr (ONE_PASS) load_v(0);
    product_priority();
    for (int kb = 0; !ONE_PASS && kb < nb_needed; ++kb) {
        __syncthreads();  // every wavefront is done with the previous block
        store_k(kb);
        __syncthreads();
        if constexpr (BWD) {
            bwd_parts(kb, [&](int t0) { row_sum_part(kb, t0, rs); });
            // (the second operand of pass 2 is asked for behind this loop: asked for in its last round it would be
            // carried around the loop in registers that the rounds before need)
            load_block(Kz, p.ldk, kb + 1 < nb_needed ? kb + 1 : 0, kx);
            continue;
        }
        score_product();
        // the next block is asked for behind the product (the wait in front of a loop body's first MFMA covers every
        // load in flight); after the last block of this pass that is the first block of the next one
        if (kb + 1 < nb_needed) {
            load_block(Kz, p.ldk, kb + 1, kx);
        } else {
            load_block(Kz, p.ldk, 0, kx);
            load_v(0);
        }
        __builtin_amdgcn_sched_barrier(0);
        __builtin_amdgcn_s_setprio(3);
        scale_and_mask(kb);
        float bm = -3.402823466e+38f;
#pragma unroll
        for (int t = 0; t < NKT; ++t)
#pragma unroll
            for (int r = 0; r < 4; ++r) bm = fmaxf(bm, sacc[t][r]);
        bm = fmaxf(bm, __shfl_xor(bm, 16, 64));
        bm = fmaxf(bm, __shfl_xor(bm, 32, 64));
        const float m_new = fmaxf(m, bm);
        float bs = 0.0f;
#pragma unroll
        for (int t = 0; t < NKT; ++t)
#pragma unroll
            for (int r = 0; r < 4; ++r) bs += __builtin_amdgcn_exp2f(sacc[t][r] - m_new);
        bs += __shfl_xor(bs, 16, 64);
        bs += __shfl_xor(bs, 32, 64);
        l = l * __builtin_amdgcn_exp2f(m - m_new) + bs;
        m = m_new;
        product_priority();
    }
    const float inv = (ONE_PASS || BWD) ? 1.0f : 1.0f / l;
    if constexpr (BWD) {
        load_v(0);
        rs += __shfl_xor(rs, 16, 64);
        rs += __shfl_xor(rs, 32, 64);
    }

    // ---- pass 2: probabilities, P out, O += P . V.  ONE_PASS (no weights kept): this is the only pass; maximum and
    //      sum run along with the blocks, the output is rescaled whenever the maximum moves (a multiplication by
    //      exp2(0) = 1 otherwise) and divided by the sum at the end. ----
    f32x4 oacc[NDT];
#pragma unroll
    for (int mt = 0; mt < NDT; ++mt) oacc[mt] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
    float* const pbase = (p.P != nullptr) ? p.P + ((long long)z * p.Tq + (row_ok ? row : 0)) * p.Tk + 4 * g : nullptr;
    for (int kb = 0; kb < nb_needed; ++kb) {
        __syncthreads();
        store_k(kb);
        store_v(kb);
        __syncthreads();
        if constexpr (BWD) {
            bwd_parts(kb, [&](int t0) {
                __builtin_amdgcn_s_setprio(3);
                gradient_part(kb, t0, rs);
                product_priority();
            });
        } else {
            score_product();
        }
        if (!BWD && kb + 1 < nb_needed) {
            load_block(Kz, p.ldk, kb + 1, kx);
            load_v(kb + 1);
        }
        __builtin_amdgcn_sched_barrier(0);
        __builtin_amdgcn_s_setprio(3);
        if constexpr (!BWD) scale_and_mask(kb);
        if constexpr (BWD) {
            // (the gradient is formed part by part behind the product above)
        } else if constexpr (ONE_PASS) {
            float bm = -3.402823466e+38f;
#pragma unroll
            for (int t = 0; t < NKT; ++t)
#pragma unroll
                for (int r = 0; r < 4; ++r) bm = fmaxf(bm, sacc[t][r]);
            bm = fmaxf(bm, __shfl_xor(bm, 16, 64));
            bm = fmaxf(bm, __shfl_xor(bm, 32, 64));
            const float m_new = fmaxf(m, bm);
            const float shrink = __builtin_amdgcn_exp2f(m - m_new);
            float bs = 0.0f;
#pragma unroll
            for (int t = 0; t < NKT; ++t)
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    const float e = __builtin_amdgcn_exp2f(sacc[t][r] - m_new);
                    sacc[t][r] = e;
                    bs += e;
                }
            bs += __shfl_xor(bs, 16, 64);
            bs += __shfl_xor(bs, 32, 64);
            l = l * shrink + bs;
            m = m_new;
            // oacc[mt][r] belongs to query lane % 16 as well (O^T: the query is the column), so the lane's own factor applies
#pragma unroll
            for (int mt = 0; mt < NDT; ++mt) oacc[mt] *= shrink;
        } else {
#pragma unroll
            for (int t = 0; t < NKT; ++t)
#pragma unroll
                for (int r = 0; r < 4; ++r) sacc[t][r] = __builtin_amdgcn_exp2f(sacc[t][r] - m) * inv;
        }
        product_priority();
        if (BWD && kb + 1 < nb_needed) {  // behind the stretch that holds the weights in registers
            load_block(Kz, p.ldk, kb + 1, kx);
            load_v(kb + 1);
        }
        __builtin_amdgcn_sched_barrier(0);

        // P out: inside the second product when the whole block and the whole tile exist (uniform), else here
        const bool p_inline = !BF16 && pbase != nullptr && (kb + 1) * KEYS <= p.Tk && q0 + AT_BQ <= p.Tq;
        if (pbase != nullptr && !p_inline && row_ok) {
            float* prow = pbase + kb * KEYS;
#pragma unroll
            for (int t = 0; t < NKT; ++t)
                if (kb * KEYS + t * 16 + 4 * g < p.Tk) *reinterpret_cast<f32x4*>(prow + t * 16) = sacc[t];
        }
        if constexpr (BF16)
            attn16_second_product_bf16<NKT, NDT, BCFG::VP>(Vt, g, l16, sacc, oacc);
        else if (p_inline)
            attn16_second_product<NKT, NDT, VP, true>(Vs, g, l16, sacc, oacc, pbase + kb * KEYS);
        else
            attn16_second_product<NKT, NDT, VP, false>(Vs, g, l16, sacc, oacc, nullptr);
    }
    __builtin_amdgcn_s_setprio(0);

    // causal: the blocks that were skipped hold zeros in the stored probabilities (a wavefront clears whole rows, lanes
    // along the keys: consecutive 16-byte stores, full lines)
    if (p.P != nullptr && nb_needed < nblocks) {  // uniform
        const int first = nb_needed * KEYS, ncol = p.Tk - first;
        for (int r = wave; r < AT_BQ && q0 + r < p.Tq; r += 8) {
            float* prow = p.P + ((long long)z * p.Tq + q0 + r) * p.Tk + first;
            for (int c = 4 * lane; c < ncol; c += 256) *reinterpret_cast<f32x4*>(prow + c) = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
        }
    }

    if (row_ok) {
        float* orow = p.O + batch_offset(bi, p.sO, p.sO2) + (long long)row * p.ldo + 4 * g;
        const float norm = ONE_PASS ? 1.0f / l : 1.0f;
#pragma unroll
        for (int mt = 0; mt < NDT; ++mt) *reinterpret_cast<f32x4*>(orow + mt * 16) = oacc[mt] * norm;
    }
}

}  // namespace snhip
