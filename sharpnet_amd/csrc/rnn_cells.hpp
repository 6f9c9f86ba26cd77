// Kernels of the recurrent layers' time steps.
//
// The reference gets its recurrent layers from cuDNN (cudnnRNNForward / cudnnRNNBackwardData_v8 /
// cudnnRNNBackwardWeights_v8, Prod/Layers/RecurrentLayer.cs:353-374,456-503).  Here everything that spans all time
// steps is a GEMM (rnn_layers.hpp); a time step itself is
//   forward    gates[:, t] (+)= h[t-1] . R^T, then the cell          rnn_step_fused_kernel (one launch), or
//                                                                    a GEMM + rnn_cell_fwd_kernel
//   backward   dh = d(gates)[:, t+1] . R, then the cell gradient     rnn_step_bwd_fused_kernel (one launch), or
//                                                                    rnn_cell_bwd_kernel + a GEMM
// with cuDNN's cell formulas:
//
//   RELU / TANH   h' = act(W x + bW + R h + bR)
//   LSTM          i, f, o = sigmoid(.), g = tanh(.) of W x + bW + R h + bR;   c' = f c + i g;   h' = o tanh(c')
//   GRU           r, z = sigmoid(W x + bW + R h + bR);   n = tanh(Wn x + bWn + r (Rn h + bRn));   h' = (1 - z) n + z h
//
// Gate blocks follow each other along a row in the order i, f, g, o / r, z, n.  In the element-wise kernels one
// thread owns one (sample, hidden unit) pair: every access is coalesced along the hidden dimension, every buffer is
// read and written once per step.  Must be included by exactly one translation unit.
#pragma once
#include <hip/hip_runtime.h>

#include "sgemm_mfma.hpp"

namespace snhip {

enum : int { RNN_RELU = 0, RNN_TANH = 1, RNN_LSTM = 2, RNN_GRU = 3 };

__device__ __forceinline__ float sigmoidf_(float v) { return 1.0f / (1.0f + expf(-v)); }

// Pointers are already moved to the step's first row; rows (samples) are `ld_*` floats apart.
struct RnnStepFwd {
    float* gates;          // in: W x + bW (+ R h for every cell but the GRU); out: activated gates (LSTM, GRU)
    float* gh;             // GRU: in: R h; out (third block only): Rn h + bRn
    const float* bias_r;   // bR (gates * hidden) or nullptr
    const float* h_prev;   // state entering the step
    const float* c_prev;   // LSTM: cell state entering the step; nullptr = zeros
    float* c_out;          // LSTM: cell state leaving the step
    float* y;              // where h' goes in the layer's output
    float* h_next;         // the next step's h_prev slot, or nullptr after the last step
    float* hy;             // (batch, hidden) contiguous: final states, or nullptr
    float* cy;
    long long ld_gates, ld_gh, ld_hprev, ld_cprev, ld_c, ld_y, ld_hnext;
    int batch, hidden, cell;
};

__global__ void __launch_bounds__(256) rnn_cell_fwd_kernel(const RnnStepFwd s) {
    const int H = s.hidden;
    const long long idx = (long long)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= (long long)s.batch * H) return;
    const int b = (int)(idx / H), j = (int)(idx % H);
    float* g = s.gates + b * s.ld_gates;
    float h;
    if (s.cell == RNN_RELU || s.cell == RNN_TANH) {
        const float pre = g[j] + (s.bias_r ? s.bias_r[j] : 0.0f);
        h = (s.cell == RNN_RELU) ? (pre < 0.0f ? 0.0f : pre) : tanhf(pre);
    } else if (s.cell == RNN_LSTM) {
        float bi = 0.0f, bf = 0.0f, bg = 0.0f, bo = 0.0f;
        if (s.bias_r) bi = s.bias_r[j], bf = s.bias_r[H + j], bg = s.bias_r[2 * H + j], bo = s.bias_r[3 * H + j];
        const float i = sigmoidf_(g[j] + bi), f = sigmoidf_(g[H + j] + bf);
        const float gg = tanhf(g[2 * H + j] + bg), o = sigmoidf_(g[3 * H + j] + bo);
        const float c = f * (s.c_prev ? s.c_prev[b * s.ld_cprev + j] : 0.0f) + i * gg;
        g[j] = i, g[H + j] = f, g[2 * H + j] = gg, g[3 * H + j] = o;
        s.c_out[b * s.ld_c + j] = c;
        if (s.cy) s.cy[(long long)b * H + j] = c;
        h = o * tanhf(c);
    } else {
        float* gh = s.gh + b * s.ld_gh;
        float br = 0.0f, bz = 0.0f, bn = 0.0f;
        if (s.bias_r) br = s.bias_r[j], bz = s.bias_r[H + j], bn = s.bias_r[2 * H + j];
        const float r = sigmoidf_(g[j] + gh[j] + br), z = sigmoidf_(g[H + j] + gh[H + j] + bz);
        const float q = gh[2 * H + j] + bn;
        const float n = tanhf(g[2 * H + j] + r * q);
        g[j] = r, g[H + j] = z, g[2 * H + j] = n;
        gh[2 * H + j] = q;
        h = (1.0f - z) * n + z * s.h_prev[b * s.ld_hprev + j];
    }
    s.y[b * s.ld_y + j] = h;
    if (s.h_next) s.h_next[b * s.ld_hnext + j] = h;
    if (s.hy) s.hy[(long long)b * H + j] = h;
}

// acc[0..3] (to be added up by the caller) = A . B^T for one wavefront: 32 rows of A (lane l fetches from ap[i] the row
// 8 i + l / 8, floats 4 (l % 8) .. + 3 of a group), 32 rows of B (bp[i] likewise), over the groups of 32 k values
// mbeg .. mend - 1.  Whole-line global loads, DEPTH groups in flight in registers; a group passes through the
// wavefront's private LDS patches pa / pb (32 rows x PITCH floats each) to reach MFMA operand layout (row = l % 32,
// sixteen consecutive k per half-wave).  No workgroup barrier inside.
// TAIL: K is not a multiple of 32 (but of 4); a lane whose four k values of a group lie beyond K reads zeros instead.
__device__ __attribute__((aligned(16))) const float rnn_zero_vector[4] = {0.0f, 0.0f, 0.0f, 0.0f};

template <int D, int P, bool TAIL>
__device__ __forceinline__ void wave_product_32x32(const float* const (&ap)[4], const float* const (&bp)[4], int mbeg,
                                                   int mend, int K, float* pa, float* pb, int lane, f32x16 (&acc)[4]) {
    const int l32 = lane & 31, lhi = lane >> 5, lrow = lane >> 3, lcol = (lane & 7) * 4;
    f32x4 ra[D][4], rb[D][4];
#pragma unroll
    for (int e = 0; e < 4; ++e)
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[e][r] = 0.0f;

    auto load = [&](int slot, int m) {
        const bool ok = !TAIL || 32 * m + lcol < K;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            ra[slot][i] = *reinterpret_cast<const f32x4*>(ok ? ap[i] + m * 32 : rnn_zero_vector);
            rb[slot][i] = *reinterpret_cast<const f32x4*>(ok ? bp[i] + m * 32 : rnn_zero_vector);
        }
    };
    // stage(slot, f): a group goes from the registers it was loaded into, through the wavefront's LDS patch, into
    // operand layout in fragment buffer f.  The wavefront's lanes exchange data through the patch: the fences keep
    // the compiler from moving LDS accesses across these points (the hardware runs one wavefront's LDS
    // instructions in order, so a patch can be rewritten as soon as the reads of the previous group are issued).
    f32x4 fa[2][4], fb[2][4];
    auto stage = [&](int slot, int f) {
        __builtin_amdgcn_fence(__ATOMIC_SEQ_CST, "wavefront");
        __builtin_amdgcn_wave_barrier();
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            *reinterpret_cast<f32x4*>(pa + (8 * i + lrow) * P + lcol) = ra[slot][i];
            *reinterpret_cast<f32x4*>(pb + (8 * i + lrow) * P + lcol) = rb[slot][i];
        }
        __builtin_amdgcn_fence(__ATOMIC_SEQ_CST, "wavefront");
        __builtin_amdgcn_wave_barrier();
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            fa[f][j] = *reinterpret_cast<const f32x4*>(pa + l32 * P + 16 * lhi + 4 * j);
            fb[f][j] = *reinterpret_cast<const f32x4*>(pb + l32 * P + 16 * lhi + 4 * j);
        }
    };
    auto multiply = [&](int f) {
        // element e of vector j is k = 32 m + 16 lhi + 4 j + e for both operands; four independent chains
#pragma unroll
        for (int j = 0; j < 4; ++j)
#pragma unroll
            for (int e = 0; e < 4; ++e)
                acc[e] = __builtin_amdgcn_mfma_f32_32x32x2f32(fa[f][j][e], fb[f][j][e], acc[e], 0, 0, 0);
    };

    // Whole blocks of D groups run without a branch between a load and its use, so that the compiler can wait for
    // exactly the group it needs (s_waitcnt vmcnt(N)) while the later ones are still in flight; the LDS round trip
    // of group i + 1 is issued before the MFMAs of group i (D is even: fragment buffer = slot % 2).
    const int cnt = mend > mbeg ? mend - mbeg : 0;
    const int mmain = mbeg + (cnt / D) * D;
    int m = mbeg;
    if (m < mmain) {
#pragma unroll
        for (int d = 0; d < D; ++d) load(d, m + d);
        stage(0, 0);
        for (; m + D < mmain; m += D) {
            load(0, m + D);
#pragma unroll
            for (int d = 0; d < D; ++d) {
                stage((d + 1) % D, (d + 1) % 2);       // d == D - 1: slot 0 already holds group m + D
                if (d + 1 < D) load(d + 1, m + d + 1 + D);
                multiply(d % 2);
            }
        }
#pragma unroll
        for (int d = 0; d < D; ++d) {
            if (d + 1 < D) stage(d + 1, (d + 1) % 2);
            multiply(d % 2);
        }
    }
    // fewer than D groups left: all loads first, then the products
#pragma unroll
    for (int d = 0; d < D - 1; ++d)
        if (mmain + d < mend) load(d, mmain + d);
#pragma unroll
    for (int d = 0; d < D - 1; ++d)
        if (mmain + d < mend) {
            stage(d, 0);
            multiply(0);
        }
}

// One forward time step in one launch: the product h[t-1] . R^T and the cell arithmetic.
//
// The step's GEMM (batch x G*H x H, e.g. 256 x 2048 x 512) is far too small to fill the chip with 64 x 64 tiles -
// it is bound by the length of one wavefront's chain of MFMAs, not by the MFMA rate.  This kernel cuts it so that
// every SIMD of the chip gets one short chain: a workgroup owns 32 samples x U hidden units x all G gates
// (U = 16; 32 for the single-gate cells), i.e. one or two 32 x 32 MFMA tiles whose 32 columns are gathered from
// the gates' row blocks of R, and splits K (the hidden dimension) over its wavefronts: four wavefronts =
// (tiles) x (K slices).  Each wavefront is on its own in the main loop: per group of 32 k values it reads its
// 32 x 32 pieces of h[t-1] and R with whole-line loads (a lane takes 16 bytes, eight lanes one 128-byte row piece),
// DEPTH groups in flight in registers, passes a group through a private LDS patch to turn it into MFMA operand
// layout (row = lane % 32, sixteen consecutive k per half-wave), and multiplies - no workgroup barrier until the
// partial tiles meet in LDS, where each thread picks up all gates of its (sample, unit) pairs, adds W x + bW from
// the gates buffer and finishes the cell exactly as rnn_cell_fwd_kernel does.
// Requires H % 4 == 0, H >= 32 and 16-byte aligned rows; the caller falls back to GEMM + cell kernel otherwise.
template <int G>
struct RnnFusedCfg {
    static constexpr int U = (G == 1) ? 32 : 16;       // hidden units per workgroup
    static constexpr int COLS = G * U;                 // columns of the workgroup's tile: [gate][unit]
    static constexpr int NT = (COLS + 31) / 32;        // 32-column MFMA tiles
    static constexpr int KS = 4 / NT;                  // K slices
    static constexpr int DEPTH = 4;                    // groups of 32 k values in flight per wavefront
    static constexpr int PITCH = 36;                   // floats per row of an LDS patch (32 + 4: conflict-free b128)
};

template <int G, bool TAIL>
__global__ void __launch_bounds__(256) rnn_step_fused_kernel(const RnnStepFwd s, const float* __restrict__ R) {
    using C = RnnFusedCfg<G>;
    constexpr int U = C::U, NT = C::NT, KS = C::KS, D = C::DEPTH, P = C::PITCH;
    __shared__ float part[KS][NT][32][33];
    __shared__ __attribute__((aligned(16))) float patch[4][2][32 * P];   // per wavefront: h rows, R rows
    const int H = s.hidden;
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63, l32 = lane & 31, lhi = lane >> 5;
    const int nt = wave % NT, kg = wave / NT;
    // unit blocks along x: workgroups are dealt to the eight XCDs by their linear index, so the (few) workgroups that
    // share a slice of R land on one XCD and find it in that XCD's L2
    const int row0 = blockIdx.y * 32, u0 = blockIdx.x * U;

    // global side: instruction i of a group fetches rows 8 i + lane / 8, floats 4 (lane % 8) .. + 3
    const int lrow = lane >> 3, lcol = (lane & 7) * 4;
    const float* ap[4];
    const float* bp[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int ar = (row0 + 8 * i + lrow < s.batch) ? row0 + 8 * i + lrow : s.batch - 1;
        ap[i] = s.h_prev + (long long)ar * s.ld_hprev + lcol;
        const int col = nt * 32 + 8 * i + lrow;                 // column of the workgroup's tile -> row of R
        const int gate = col / U, unit = u0 + col % U;
        bp[i] = R + (long long)((col < C::COLS && unit < H) ? gate * H + unit : 0) * H + lcol;
    }
    float* pa = &patch[wave][0][0];
    float* pb = &patch[wave][1][0];

    const int groups = (H + 31) / 32;                            // groups of 32 k values
    const int per = (groups + KS - 1) / KS;
    const int mbeg = kg * per, mend = (mbeg + per < groups) ? mbeg + per : groups;

    // what the cell arithmetic at the end reads from global memory is fetched now, behind the main loop:
    // thread -> pairs p = threadIdx.x + 256 q of the tile's 32 x U (sample, unit) pairs
    constexpr int Q = 32 * U / 256;
    float gxv[Q][G], brv[Q][G], cpv[Q], hpv[Q];
#pragma unroll
    for (int q = 0; q < Q; ++q) {
        const int p = threadIdx.x + 256 * q;
        const int b = row0 + p / U, j = u0 + p % U;
        const bool ok = b < s.batch && j < H;
#pragma unroll
        for (int g = 0; g < G; ++g) {
            gxv[q][g] = ok ? s.gates[b * s.ld_gates + g * H + j] : 0.0f;
            brv[q][g] = (ok && s.bias_r) ? s.bias_r[g * H + j] : 0.0f;
        }
        cpv[q] = (G == 4 && ok && s.c_prev) ? s.c_prev[b * s.ld_cprev + j] : 0.0f;
        hpv[q] = (G == 3 && ok) ? s.h_prev[b * s.ld_hprev + j] : 0.0f;
    }

    f32x16 acc[4];
    wave_product_32x32<D, P, TAIL>(ap, bp, mbeg, mend, H, pa, pb, lane, acc);
    // accumulator register r holds row 8 (r / 4) + 4 lhi + r % 4, column l32 of the 32 x 32 tile
#pragma unroll
    for (int r = 0; r < 16; ++r)
        part[kg][nt][8 * (r / 4) + 4 * lhi + (r % 4)][l32] = (acc[0][r] + acc[1][r]) + (acc[2][r] + acc[3][r]);
    __syncthreads();

#pragma unroll
    for (int q = 0; q < Q; ++q) {
        const int p = threadIdx.x + 256 * q;
        const int lr = p / U, b = row0 + lr, j = u0 + p % U;
        if (b >= s.batch || j >= H) continue;
        float gh[G];
#pragma unroll
        for (int g = 0; g < G; ++g) {
            const int c = g * U + p % U;
            float v = 0.0f;
#pragma unroll
            for (int k = 0; k < KS; ++k) v += part[k][c / 32][lr][c % 32];
            gh[g] = v + brv[q][g];
        }
        float* gx = s.gates + b * s.ld_gates;
        float h;
        if constexpr (G == 1) {
            const float pre = gxv[q][0] + gh[0];
            h = (s.cell == RNN_RELU) ? (pre < 0.0f ? 0.0f : pre) : tanhf(pre);
        } else if constexpr (G == 4) {
            const float i = sigmoidf_(gxv[q][0] + gh[0]), f = sigmoidf_(gxv[q][1] + gh[1]);
            const float gg = tanhf(gxv[q][2] + gh[2]), o = sigmoidf_(gxv[q][3] + gh[3]);
            const float c = f * cpv[q] + i * gg;
            gx[j] = i, gx[H + j] = f, gx[2 * H + j] = gg, gx[3 * H + j] = o;
            s.c_out[b * s.ld_c + j] = c;
            if (s.cy) s.cy[(long long)b * H + j] = c;
            h = o * tanhf(c);
        } else {
            const float r = sigmoidf_(gxv[q][0] + gh[0]), z = sigmoidf_(gxv[q][1] + gh[1]);
            const float qn = gh[2];
            const float n = tanhf(gxv[q][2] + r * qn);
            gx[j] = r, gx[H + j] = z, gx[2 * H + j] = n;
            s.gh[b * s.ld_gh + 2 * H + j] = qn;
            h = (1.0f - z) * n + z * hpv[q];
        }
        s.y[b * s.ld_y + j] = h;
        if (s.h_next) s.h_next[b * s.ld_hnext + j] = h;
        if (s.hy) s.hy[(long long)b * H + j] = h;
    }
}

struct RnnStepBwd {
    float* gates;          // in: what the forward step left; out: d(W x + bW) of the step
    float* gh;             // GRU: in (third block): Rn h + bRn; out: d(R h + bR)
    const float* h_prev;   // GRU: state that entered the step
    const float* y;        // RELU / TANH: h' of the step
    const float* c_prev;   // LSTM; nullptr = zeros
    const float* c;        // LSTM: cell state that left the step
    const float* dy;       // gradient arriving from the layer above for this step
    float* dh;             // (batch, hidden) contiguous; in: gradient from the step after; out (GRU): dh * z, the part
                           // of the previous step's gradient that does not pass through R
    float* dc;             // LSTM (batch, hidden) contiguous, in and out
    long long ld_gates, ld_gh, ld_hprev, ld_y, ld_cprev, ld_c, ld_dy;
    int batch, hidden, cell;
};

__global__ void __launch_bounds__(256) rnn_cell_bwd_kernel(const RnnStepBwd s) {
    const int H = s.hidden;
    const long long idx = (long long)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= (long long)s.batch * H) return;
    const int b = (int)(idx / H), j = (int)(idx % H);
    float* g = s.gates + b * s.ld_gates;
    const float dh = s.dh[idx] + s.dy[b * s.ld_dy + j];
    if (s.cell == RNN_RELU || s.cell == RNN_TANH) {
        const float h = s.y[b * s.ld_y + j];
        g[j] = (s.cell == RNN_RELU) ? (h > 0.0f ? dh : 0.0f) : dh * (1.0f - h * h);
    } else if (s.cell == RNN_LSTM) {
        const float i = g[j], f = g[H + j], gg = g[2 * H + j], o = g[3 * H + j];
        const float tc = tanhf(s.c[b * s.ld_c + j]);
        const float dc = s.dc[idx] + dh * o * (1.0f - tc * tc);
        const float cp = s.c_prev ? s.c_prev[b * s.ld_cprev + j] : 0.0f;
        g[j] = dc * gg * i * (1.0f - i);
        g[H + j] = dc * cp * f * (1.0f - f);
        g[2 * H + j] = dc * i * (1.0f - gg * gg);
        g[3 * H + j] = dh * tc * o * (1.0f - o);
        s.dc[idx] = dc * f;
    } else {
        float* gh = s.gh + b * s.ld_gh;
        const float r = g[j], z = g[H + j], n = g[2 * H + j], q = gh[2 * H + j];
        const float hp = s.h_prev[b * s.ld_hprev + j];
        const float dn = dh * (1.0f - z) * (1.0f - n * n);
        const float dz = dh * (hp - n) * z * (1.0f - z);
        const float dr = dn * q * r * (1.0f - r);
        g[j] = dr, g[H + j] = dz, g[2 * H + j] = dn;
        gh[j] = dr, gh[H + j] = dz, gh[2 * H + j] = dn * r;
        s.dh[idx] = dh * z;
    }
}

// One backward time step in one launch: dh = d(R h + bR)[step after] . R, then the cell gradient of this step.
//
// The product is batch x H x G*H (256 x 512 x 2048): few output elements, a long K.  A workgroup of eight
// wavefronts owns 32 samples x 16 hidden units and gives each wavefront an eighth of K, so that the chip holds 256
// workgroups (one per compute unit, two wavefronts per SIMD).  With 16 columns the tile is built from
// v_mfma_f32_16x16x4_f32: per group of 32 k values a wavefront loads 32 rows of d(gates) and 16 rows of R^T (which
// the caller lays out once per call) with whole-line loads, passes them through its private LDS patches, and issues
// 16 MFMAs (two 16 x 16 tiles x 8 k steps) on four independent accumulators.  The partial tiles meet in LDS; each
// thread then owns one (sample, unit) pair, adds the gradient arriving from the layer above (and, for the GRU,
// dh * z carried over from the step after) and does what rnn_cell_bwd_kernel does, with its inputs fetched before
// the main loop.  `dg_next` is the d(R h + bR) the step after (in time order of this direction) left behind.
struct RnnBwdFusedCfg {
    static constexpr int KS = 8;
    static constexpr int DEPTH = 4;
    static constexpr int PITCH = 36;
    static constexpr int U = 16;                                       // hidden units per workgroup
    static constexpr int PATCH = (32 + U) * PITCH;                     // floats per wavefront: d(gates) rows, R^T rows
    static constexpr int LDS_BYTES = (KS * PATCH + KS * 32 * (U + 1)) * 4;
};

typedef float f32x4_acc __attribute__((ext_vector_type(4)));

template <int G, bool TAIL>
__global__ void __launch_bounds__(512) rnn_step_bwd_fused_kernel(const RnnStepBwd s, const float* __restrict__ dg_next,
                                                                 long long ld_dg, const float* __restrict__ Rt) {
    using C = RnnBwdFusedCfg;
    constexpr int KS = C::KS, D = C::DEPTH, P = C::PITCH, U = C::U;
    extern __shared__ __attribute__((aligned(16))) float lds_bwd[];
    float(*part)[32][U + 1] = reinterpret_cast<float(*)[32][U + 1]>(lds_bwd + KS * C::PATCH);   // [KS][32][U + 1]
    const int H = s.hidden, GH = G * H;
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63, l16 = lane & 15, lq = lane >> 4;
    const int row0 = blockIdx.y * 32, u0 = blockIdx.x * U;
    float* pa = lds_bwd + wave * C::PATCH;      // 32 rows of d(gates)
    float* pb = pa + 32 * P;                    // U rows of R^T

    // global side: instruction i of a group fetches row 8 i + lane / 8, floats 4 (lane % 8) .. + 3
    const int lrow = lane >> 3, lcol = (lane & 7) * 4;
    const float* ap[4];
    const float* bp[2];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int ar = (row0 + 8 * i + lrow < s.batch) ? row0 + 8 * i + lrow : s.batch - 1;
        ap[i] = dg_next + (long long)ar * ld_dg + lcol;
    }
#pragma unroll
    for (int i = 0; i < 2; ++i) {
        const int unit = (u0 + 8 * i + lrow < H) ? u0 + 8 * i + lrow : H - 1;
        bp[i] = Rt + (long long)unit * GH + lcol;
    }
    const int groups = (GH + 31) / 32;
    const int per = (groups + KS - 1) / KS;
    const int mbeg = wave * per, mend = (mbeg + per < groups) ? mbeg + per : groups;

    // inputs of the cell gradient: thread -> pair p = threadIdx.x of the tile's 32 x 16 (sample, unit) pairs
    constexpr int Q = 1;
    float gv[Q][G], dyv[Q], dhv[Q], av[Q], bv[Q], cv[Q];
#pragma unroll
    for (int q = 0; q < Q; ++q) {
        const int p = threadIdx.x + 512 * q;
        const int b = row0 + p / U, j = u0 + p % U;
        const bool ok = b < s.batch && j < H;
        const long long idx = (long long)b * H + j;
#pragma unroll
        for (int g = 0; g < G; ++g) gv[q][g] = ok ? s.gates[b * s.ld_gates + g * H + j] : 0.0f;
        dyv[q] = ok ? s.dy[b * s.ld_dy + j] : 0.0f;
        dhv[q] = (G == 3 && ok) ? s.dh[idx] : 0.0f;                       // GRU: dh * z of the step after
        if constexpr (G == 1) {
            av[q] = ok ? s.y[b * s.ld_y + j] : 0.0f;                     // h'
            bv[q] = cv[q] = 0.0f;
        } else if constexpr (G == 4) {
            av[q] = ok ? s.c[b * s.ld_c + j] : 0.0f;                     // c'
            bv[q] = (ok && s.c_prev) ? s.c_prev[b * s.ld_cprev + j] : 0.0f;
            cv[q] = ok ? s.dc[idx] : 0.0f;
        } else {
            av[q] = ok ? s.gh[b * s.ld_gh + 2 * H + j] : 0.0f;           // Rn h + bRn
            bv[q] = ok ? s.h_prev[b * s.ld_hprev + j] : 0.0f;
            cv[q] = 0.0f;
        }
    }

    // main loop: as wave_product_32x32, with 16 x 16 x 4 MFMAs.  A lane reads from the patches the four consecutive
    // k values 16 j + 4 (lane / 16) .. + 3 of its row; element e of that vector feeds the MFMA whose four k are
    // 16 j + e, + 4, + 8, + 12 (lane / 16 picks one of them) - the same for both operands.
    f32x4 ra[D][4], rb[D][2], fa[2][2][2], fb[2][2];
    f32x4_acc acc[2][2];
#pragma unroll
    for (int hh = 0; hh < 2; ++hh)
#pragma unroll
        for (int c = 0; c < 2; ++c) acc[hh][c] = f32x4_acc{0.0f, 0.0f, 0.0f, 0.0f};
    auto load = [&](int slot, int m) {
        const bool ok = !TAIL || 32 * m + lcol < GH;   // beyond K (not a multiple of 32): zeros
#pragma unroll
        for (int i = 0; i < 4; ++i) ra[slot][i] = *reinterpret_cast<const f32x4*>(ok ? ap[i] + m * 32 : rnn_zero_vector);
#pragma unroll
        for (int i = 0; i < 2; ++i) rb[slot][i] = *reinterpret_cast<const f32x4*>(ok ? bp[i] + m * 32 : rnn_zero_vector);
    };
    auto stage = [&](int slot, int f) {
        __builtin_amdgcn_fence(__ATOMIC_SEQ_CST, "wavefront");
        __builtin_amdgcn_wave_barrier();
#pragma unroll
        for (int i = 0; i < 4; ++i) *reinterpret_cast<f32x4*>(pa + (8 * i + lrow) * P + lcol) = ra[slot][i];
#pragma unroll
        for (int i = 0; i < 2; ++i) *reinterpret_cast<f32x4*>(pb + (8 * i + lrow) * P + lcol) = rb[slot][i];
        __builtin_amdgcn_fence(__ATOMIC_SEQ_CST, "wavefront");
        __builtin_amdgcn_wave_barrier();
#pragma unroll
        for (int j = 0; j < 2; ++j) {
#pragma unroll
            for (int hh = 0; hh < 2; ++hh)
                fa[f][hh][j] = *reinterpret_cast<const f32x4*>(pa + (16 * hh + l16) * P + 16 * j + 4 * lq);
            fb[f][j] = *reinterpret_cast<const f32x4*>(pb + l16 * P + 16 * j + 4 * lq);
        }
    };
    auto multiply = [&](int f) {
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
            for (int e = 0; e < 4; ++e)
#pragma unroll
                for (int hh = 0; hh < 2; ++hh)
                    acc[hh][e & 1] = __builtin_amdgcn_mfma_f32_16x16x4f32(fa[f][hh][j][e], fb[f][j][e], acc[hh][e & 1], 0, 0, 0);
    };
    {
        const int cnt = mend > mbeg ? mend - mbeg : 0;
        const int mmain = mbeg + (cnt / D) * D;
        int m = mbeg;
        if (m < mmain) {
#pragma unroll
            for (int d = 0; d < D; ++d) load(d, m + d);
            stage(0, 0);
            for (; m + D < mmain; m += D) {
                load(0, m + D);
#pragma unroll
                for (int d = 0; d < D; ++d) {
                    stage((d + 1) % D, (d + 1) % 2);
                    if (d + 1 < D) load(d + 1, m + d + 1 + D);
                    multiply(d % 2);
                }
            }
#pragma unroll
            for (int d = 0; d < D; ++d) {
                if (d + 1 < D) stage(d + 1, (d + 1) % 2);
                multiply(d % 2);
            }
        }
#pragma unroll
        for (int d = 0; d < D - 1; ++d)
            if (mmain + d < mend) load(d, mmain + d);
#pragma unroll
        for (int d = 0; d < D - 1; ++d)
            if (mmain + d < mend) {
                stage(d, 0);
                multiply(0);
            }
    }
    // accumulator register r of a 16 x 16 tile holds row 4 (lane / 16) + r, column lane % 16
#pragma unroll
    for (int hh = 0; hh < 2; ++hh)
#pragma unroll
        for (int r = 0; r < 4; ++r) part[wave][16 * hh + 4 * lq + r][l16] = acc[hh][0][r] + acc[hh][1][r];
    __syncthreads();

#pragma unroll
    for (int q = 0; q < Q; ++q) {
        const int p = threadIdx.x + 512 * q;
        const int lr = p / U, b = row0 + lr, j = u0 + p % U;
        if (b >= s.batch || j >= H) continue;
        const long long idx = (long long)b * H + j;
        float rec = 0.0f;
#pragma unroll
        for (int k = 0; k < KS; ++k) rec += part[k][lr][p % U];
        const float dh = rec + dhv[q] + dyv[q];
        float* g = s.gates + b * s.ld_gates;
        if constexpr (G == 1) {
            const float h = av[q];
            g[j] = (s.cell == RNN_RELU) ? (h > 0.0f ? dh : 0.0f) : dh * (1.0f - h * h);
        } else if constexpr (G == 4) {
            const float i = gv[q][0], f = gv[q][1], gg = gv[q][2], o = gv[q][3];
            const float tc = tanhf(av[q]);
            const float dc = cv[q] + dh * o * (1.0f - tc * tc);
            g[j] = dc * gg * i * (1.0f - i);
            g[H + j] = dc * bv[q] * f * (1.0f - f);
            g[2 * H + j] = dc * i * (1.0f - gg * gg);
            g[3 * H + j] = dh * tc * o * (1.0f - o);
            s.dc[idx] = dc * f;
        } else {
            const float r = gv[q][0], z = gv[q][1], n = gv[q][2], qn = av[q], hp = bv[q];
            const float dn = dh * (1.0f - z) * (1.0f - n * n);
            const float dz = dh * (hp - n) * z * (1.0f - z);
            const float dr = dn * qn * r * (1.0f - r);
            float* gh = s.gh + b * s.ld_gh;
            g[j] = dr, g[H + j] = dz, g[2 * H + j] = dn;
            gh[j] = dr, gh[H + j] = dz, gh[2 * H + j] = dn * r;
            s.dh[idx] = dh * z;
        }
    }
}

// dst[r][0..cols) = src[r][0..cols) (src == nullptr: zeros); rows ld_dst / ld_src floats apart.
__global__ void __launch_bounds__(256) set_rows_kernel(float* dst, long long ld_dst, const float* src, long long ld_src,
                                                       int rows, int cols) {
    const long long idx = (long long)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= (long long)rows * cols) return;
    const int r = (int)(idx / cols), c = (int)(idx % cols);
    dst[r * ld_dst + c] = src ? src[r * ld_src + c] : 0.0f;
}

// ---------------------------------------------------------------------------
// Dropout between stacked layers.  The mask is a pure function of (seed, call, boundary, element), so the backward
// pass and a caller's own check can regenerate it instead of storing it:
//   Philox4x32-10 (Salmon et al., "Parallel random numbers: as easy as 1, 2, 3", SC'11) with
//   key = {seed low word, seed high word} and counter = {e / 4 low word, e / 4 high word, boundary, call};
//   element e takes output word e % 4; it is dropped when (word >> 8) * 2^-24 < rate, else multiplied by 1 / (1 - rate).
// e numbers the elements of the (steps, batch, dirs * hidden) activations between layers `boundary` and `boundary + 1`
// in that (step-major) order.
// ---------------------------------------------------------------------------
struct Philox4 {
    unsigned int v[4];
};
__device__ __host__ __forceinline__ Philox4 philox4x32_10(unsigned int c0, unsigned int c1, unsigned int c2, unsigned int c3,
                                                          unsigned int k0, unsigned int k1) {
    constexpr unsigned int M0 = 0xD2511F53u, M1 = 0xCD9E8D57u, W0 = 0x9E3779B9u, W1 = 0xBB67AE85u;
#pragma unroll
    for (int round = 0; round < 10; ++round) {
        const unsigned long long p0 = (unsigned long long)M0 * c0, p1 = (unsigned long long)M1 * c2;
        const unsigned int n0 = (unsigned int)(p1 >> 32) ^ c1 ^ k0, n1 = (unsigned int)p1;
        const unsigned int n2 = (unsigned int)(p0 >> 32) ^ c3 ^ k1, n3 = (unsigned int)p0;
        c0 = n0, c1 = n1, c2 = n2, c3 = n3;
        k0 += W0, k1 += W1;
    }
    return Philox4{{c0, c1, c2, c3}};
}

// {seed low word, seed high word, call} into a forward call's reserve buffer, for its backward calls
__global__ void rnn_dropout_note_kernel(unsigned int* dst, unsigned int seed_lo, unsigned int seed_hi, unsigned int call) {
    if (threadIdx.x == 0 && blockIdx.x == 0) dst[0] = seed_lo, dst[1] = seed_hi, dst[2] = call;
}

struct RnnDropout {
    unsigned long long seed;
    unsigned int call, boundary;
    float rate, scale;  // scale = 1 / (1 - rate)
    // when not null: {seed low word, seed high word, call} as the forward call left them in its reserve buffer; they
    // replace the three values above (the backward pass of a layer may run after other layers have drawn their masks)
    const unsigned int* stored;
};

// dst[e] = src[e] * mask[e] over `count` step-major elements (count % 4 == 0 is not required); src == nullptr writes the
// mask itself.  to_batch_major != 0: dst is laid out (batch, steps, width) and e is translated (the mask as a caller
// sees it beside y).
__global__ void __launch_bounds__(256) rnn_dropout_kernel(float* dst, const float* src, long long count, RnnDropout d,
                                                          int to_batch_major, int batch, int steps, int width) {
    const long long chunks = (count + 3) / 4;
    unsigned int k0 = (unsigned int)d.seed, k1 = (unsigned int)(d.seed >> 32), call = d.call;
    if (d.stored != nullptr) k0 = d.stored[0], k1 = d.stored[1], call = d.stored[2];
    for (long long c = (long long)blockIdx.x * 256 + threadIdx.x; c < chunks; c += (long long)gridDim.x * 256) {
        const Philox4 r = philox4x32_10((unsigned int)c, (unsigned int)(c >> 32), d.boundary, call, k0, k1);
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const long long e = 4 * c + j;
            if (e >= count) break;
            const float u = (float)(r.v[j] >> 8) * (1.0f / 16777216.0f);
            const float m = u < d.rate ? 0.0f : d.scale;
            long long o = e;
            if (to_batch_major) {
                const long long row = e / width;  // step * batch + sample
                const long long t = row / batch, b = row - t * batch;
                o = (b * steps + t) * width + (e - row * width);
            }
            dst[o] = src == nullptr ? m : (m != 0.0f ? src[e] * m : 0.0f);
        }
    }
}

}  // namespace snhip
