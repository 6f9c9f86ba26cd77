// Element-wise halves of the recurrent cells; the matrix halves are the GEMM kernels.
//
// The reference gets its recurrent layers from cuDNN (cudnnRNNForward / cudnnRNNBackwardData_v8 /
// cudnnRNNBackwardWeights_v8, Prod/Layers/RecurrentLayer.cs:353-374,456-503).  Here one time step of one
// direction is a GEMM  gates[:, t] (+)= h[t-1] . R^T  followed by rnn_cell_fwd_kernel, and on the way back
// rnn_cell_bwd_kernel followed by  dh = d(gates)[:, t] . R.  cuDNN's cell formulas:
//
//   RELU / TANH   h' = act(W x + bW + R h + bR)
//   LSTM          i, f, o = sigmoid(.), g = tanh(.) of W x + bW + R h + bR;   c' = f c + i g;   h' = o tanh(c')
//   GRU           r, z = sigmoid(W x + bW + R h + bR);   n = tanh(Wn x + bWn + r (Rn h + bRn));   h' = (1 - z) n + z h
//
// Gate blocks follow each other along a row in the order i, f, g, o / r, z, n.  One thread owns one (sample,
// hidden unit) pair: every access is coalesced along the hidden dimension, every buffer is read and written
// once per step (HBM/L2-bound, a few hundred KB per step).  Must be included by exactly one translation unit.
#pragma once
#include <hip/hip_runtime.h>

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

// dst[r][0..cols) = src[r][0..cols) (src == nullptr: zeros); rows ld_dst / ld_src floats apart.
__global__ void __launch_bounds__(256) set_rows_kernel(float* dst, long long ld_dst, const float* src, long long ld_src,
                                                       int rows, int cols) {
    const long long idx = (long long)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= (long long)rows * cols) return;
    const int r = (int)(idx / cols), c = (int)(idx % cols);
    dst[r * ld_dst + c] = src ? src[r * ld_src + c] : 0.0f;
}

}  // namespace snhip
