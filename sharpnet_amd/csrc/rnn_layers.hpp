// Recurrent layers (RELU / TANH / LSTM / GRU cells, stacked, one or two directions) as sequences of GEMM launches
// and the element-wise kernels of rnn_cells.hpp.  Included at the end of sharpnet_hip.hip and nowhere else: it uses
// that file's Handle, GemmArgs and gemm_core.  Entry points are declared in include/sharpnet_hip.h.
//
// Work of one layer and direction (n = batch * steps rows, G gates, H hidden units, I inputs):
//   forward    gates (n x G*H) = X (n x I) . W^T + bW                                  one GEMM over all steps
//              per step: gates[:, t] += h[t-1] . R^T (batch x G*H x H), cell -> h[t] into y and into the slot the
//                        next step reads: one launch (rnn_step_fused_kernel) when H % 4 == 0, else GEMM + cell kernel
//   backward   per step, last to first: dh = d(gates)[:, t+1] . R (batch x H x G*H), cell gradient -> d(gates)[:, t]:
//                        one launch (rnn_step_bwd_fused_kernel) when H % 4 == 0, else cell kernel + GEMM
//              dX (n x I) = d(gates) . W                                               one GEMM
//   weights    dW += d(gates)^T . X, dR += d(gates_h)^T . Hprev, bias gradients = column sums     two GEMMs
// Hprev (n x H) holds, for every (sample, step), the state that entered the step, so the recurrent weight gradient
// is a single product over all steps.
// Everything the library keeps between the calls is stored step-major ((steps, batch, width)): the rows one time
// step works on are contiguous, whereas in the caller's batch-major tensors they lie steps * width floats apart.
// x is copied into that order once per forward call; y, dy and dx are read and written in place through their
// row pitch.
#pragma once
#include "rnn_cells.hpp"

namespace {

struct RnnDims {
    int cell, G, H, I, K, L, P;      // P = K * L pseudo-layers
    bool bias_w, bias_r;
    int batch, steps;
    long long n;                      // batch * steps
    long long per_p;                  // floats of one pseudo-layer's region
    long long gates_off, hprev_off, cells_off, gh_off;   // inside a pseudo-layer's region
    long long out_off;                // start of the stacked layers' outputs, after all regions
    long long xt_off;                 // step-major copy of x
    bool dropout;                     // units are dropped between the stacked layers in training
    long long drop_off;               // the stacked layers' outputs after dropout (what the next layer reads), if any
    long long rng_off;                // {seed low, seed high, call} of the forward call's masks, as three 32-bit words
    long long total;                  // floats carried from forward to backward
    long long rt_off;                 // inside the backward scratch: the transposed recurrent matrix of direction 0
    long long dir1_off;               // ... dh, dc and the transposed recurrent matrix of direction 1
    long long bwd_ws;                 // floats of scratch the backward calls need
};

int rnn_gates(int cell) { return cell == RNN_LSTM ? 4 : (cell == RNN_GRU ? 3 : 1); }

int rnn_check_desc(const snhip_rnn_desc* d) {
    if (d == nullptr || d->struct_size != (int)sizeof(snhip_rnn_desc)) return SNHIP_STATUS_INVALID_VALUE;
    if (d->cell_mode < SNHIP_RNN_RELU || d->cell_mode > SNHIP_RNN_GRU) return SNHIP_STATUS_INVALID_VALUE;
    if (d->bias_mode < SNHIP_RNN_NO_BIAS || d->bias_mode > SNHIP_RNN_SINGLE_REC_BIAS) return SNHIP_STATUS_INVALID_VALUE;
    if (d->bidirectional != 0 && d->bidirectional != 1) return SNHIP_STATUS_INVALID_VALUE;
    if (d->num_layers < 1 || d->input_size < 1 || d->hidden_size < 1) return SNHIP_STATUS_INVALID_VALUE;
    if (!(d->dropout >= 0.0f && d->dropout < 1.0f)) return SNHIP_STATUS_INVALID_VALUE;  // also refuses NaN
    return SNHIP_STATUS_SUCCESS;
}

// cuDNN drops units of the outputs that feed the next stacked layer (RNNDescriptor.dropoutRate, handed to
// cudnnSetRNNDescriptor_v8 through GPUWrapper.DropoutDesc, Prod/GPU/GPUWrapper.cs:460-474), in training only; a single
// layer has nothing to drop.  The buffers are sized from the descriptor alone, so an inference call with such a
// descriptor reserves the room and does not use it.
bool rnn_has_dropout(const snhip_rnn_desc* d) { return d->dropout > 0.0f && d->num_layers > 1; }

RnnDims rnn_dims(const snhip_rnn_desc* d, int batch, int steps) {
    RnnDims r;
    r.cell = d->cell_mode;
    r.G = rnn_gates(d->cell_mode);
    r.H = d->hidden_size;
    r.I = d->input_size;
    r.K = d->bidirectional ? 2 : 1;
    r.L = d->num_layers;
    r.P = r.K * r.L;
    r.bias_w = d->bias_mode == SNHIP_RNN_DOUBLE_BIAS || d->bias_mode == SNHIP_RNN_SINGLE_INP_BIAS;
    r.bias_r = d->bias_mode == SNHIP_RNN_DOUBLE_BIAS || d->bias_mode == SNHIP_RNN_SINGLE_REC_BIAS;
    r.batch = batch;
    r.steps = steps;
    r.n = (long long)batch * steps;
    r.gates_off = 0;
    r.hprev_off = r.n * r.G * r.H;
    r.cells_off = r.hprev_off + r.n * r.H;
    r.gh_off = r.cells_off + (r.cell == RNN_LSTM ? r.n * r.H : 0);
    r.per_p = r.gh_off + (r.cell == RNN_GRU ? r.n * 3 * r.H : 0);
    r.out_off = r.per_p * r.P;
    r.xt_off = r.out_off + (long long)(r.L - 1) * r.n * r.K * r.H;
    r.dropout = rnn_has_dropout(d);
    r.drop_off = r.xt_off + r.n * r.I;
    r.rng_off = r.drop_off + (r.dropout ? (long long)(r.L - 1) * r.n * r.K * r.H : 0);
    r.total = r.rng_off + (r.dropout ? 4 : 0);
    // dh, dc, one bias gradient, two buffers for the gradients that travel between stacked layers, and R^T
    r.rt_off = 2LL * batch * r.H + (long long)r.G * r.H + (r.L > 1 ? 2 * r.n * r.K * r.H : 0);
    r.dir1_off = r.rt_off + (long long)r.G * r.H * r.H;
    r.bwd_ws = r.dir1_off + (r.K == 2 ? 2LL * batch * r.H + (long long)r.G * r.H * r.H : 0);
    return r;
}

long long rnn_layer_inputs(const RnnDims& r, int layer) { return layer == 0 ? r.I : (long long)r.K * r.H; }
long long rnn_matrix_floats(const RnnDims& r, int p) {
    return (long long)r.G * r.H * (rnn_layer_inputs(r, p / r.K) + r.H);
}
long long rnn_bias_floats(const RnnDims& r) { return (long long)r.G * r.H * ((r.bias_w ? 1 : 0) + (r.bias_r ? 1 : 0)); }
long long rnn_all_matrices(const RnnDims& r) {
    long long s = 0;
    for (int p = 0; p < r.P; ++p) s += rnn_matrix_floats(r, p);
    return s;
}

// Where the stacked matrices and bias vectors of one pseudo-layer sit in a weight space, in floats (-1: absent).
struct RnnOffsets {
    long long W, R, bW, bR;
};
RnnOffsets rnn_offsets(const RnnDims& r, int p) {
    RnnOffsets o;
    o.W = 0;
    for (int q = 0; q < p; ++q) o.W += rnn_matrix_floats(r, q);
    o.R = o.W + (long long)r.G * r.H * rnn_layer_inputs(r, p / r.K);
    const long long b = rnn_all_matrices(r) + (long long)p * rnn_bias_floats(r);
    o.bW = r.bias_w ? b : -1;
    o.bR = r.bias_r ? b + (r.bias_w ? (long long)r.G * r.H : 0) : -1;
    return o;
}
struct RnnWeights {
    float* W;    // (G*H, inputs)
    float* R;    // (G*H, H)
    float* bW;   // (G*H) or nullptr
    float* bR;
};
RnnWeights rnn_weights(const RnnDims& r, float* space, int p) {
    const RnnOffsets o = rnn_offsets(r, p);
    return RnnWeights{space + o.W, space + o.R, o.bW >= 0 ? space + o.bW : nullptr, o.bR >= 0 ? space + o.bR : nullptr};
}

int rnn_set_rows(Handle* h, float* dst, long long ld_dst, const float* src, long long ld_src, int rows, int cols) {
    const long long total = (long long)rows * cols;
    hipLaunchKernelGGL(set_rows_kernel, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, h->stream, dst, ld_dst, src,
                       ld_src, rows, cols);
    return hip_to_status(hipGetLastError());
}

// dst = src * mask (src == nullptr: the mask itself) over the (steps, batch, dirs * hidden) activations behind layer
// `boundary`; see rnn_dropout_kernel for how the mask is drawn.
int rnn_apply_dropout(Handle* h, const RnnDims& r, float rate, float* dst, const float* src, int boundary,
                      unsigned long long seed, unsigned int call, const unsigned int* stored, bool to_batch_major) {
    const long long count = r.n * r.K * r.H;
    RnnDropout d;
    d.seed = seed, d.call = call, d.boundary = (unsigned int)boundary;
    d.rate = rate, d.scale = 1.0f / (1.0f - rate);
    d.stored = stored;
    const long long blocks = ((count + 3) / 4 + 255) / 256;
    hipLaunchKernelGGL(rnn_dropout_kernel, dim3((unsigned)(blocks < 65536 ? blocks : 65536)), dim3(256), 0, h->stream, dst,
                       src, count, d, to_batch_major ? 1 : 0, r.batch, r.steps, r.K * r.H);
    return hip_to_status(hipGetLastError());
}

// The backward step kernel stages more than the 64 KiB of LDS a kernel gets without asking.
hipError_t rnn_prepare_kernels() {
    const void* fns[6] = {reinterpret_cast<const void*>(rnn_step_bwd_fused_kernel<1, false>),
                          reinterpret_cast<const void*>(rnn_step_bwd_fused_kernel<3, false>),
                          reinterpret_cast<const void*>(rnn_step_bwd_fused_kernel<4, false>),
                          reinterpret_cast<const void*>(rnn_step_bwd_fused_kernel<1, true>),
                          reinterpret_cast<const void*>(rnn_step_bwd_fused_kernel<3, true>),
                          reinterpret_cast<const void*>(rnn_step_bwd_fused_kernel<4, true>)};
    for (const void* f : fns) {
        const hipError_t e = hipFuncSetAttribute(f, hipFuncAttributeMaxDynamicSharedMemorySize, RnnBwdFusedCfg::LDS_BYTES);
        if (e != hipSuccess) return e;
    }
    return hipSuccess;
}

int rnn_common_checks(Handle* h, const snhip_rnn_desc* desc, int batch, int steps) {
    const int st = rnn_check_desc(desc);
    if (st != SNHIP_STATUS_SUCCESS) return st;
    if (h == nullptr) return SNHIP_STATUS_NOT_INITIALIZED;
    if (batch < 0 || steps < 0) return SNHIP_STATUS_INVALID_VALUE;
    // row counts and row pitches travel as 32-bit integers through the GEMM arguments
    const long long widest = (long long)rnn_gates(desc->cell_mode) * desc->hidden_size;
    const long long in_max = desc->input_size > 2LL * desc->hidden_size ? desc->input_size : 2LL * desc->hidden_size;
    if ((long long)batch * steps > 0x7fffffffLL || (long long)steps * (widest > in_max ? widest : in_max) > 0x7fffffffLL ||
        (long long)batch * desc->hidden_size > 0x7fffffffLL)
        return SNHIP_STATUS_NOT_SUPPORTED;
    // the handle belongs to one device; a caller thread on another one is switched over, as in the GEMM calls
    int cur = -1;
    if (hipGetDevice(&cur) != hipSuccess) return SNHIP_STATUS_NOT_INITIALIZED;
    if (cur != h->device && hipSetDevice(h->device) != hipSuccess) return SNHIP_STATUS_NOT_INITIALIZED;
    return SNHIP_STATUS_SUCCESS;
}

}  // namespace

extern "C" {

int snhip_sizeof_rnn_desc(void) { return (int)sizeof(snhip_rnn_desc); }

int snhip_rnn_weight_space_size(const snhip_rnn_desc* desc, size_t* bytes) {
    const int st = rnn_check_desc(desc);
    if (st != SNHIP_STATUS_SUCCESS) return st;
    if (bytes == nullptr) return SNHIP_STATUS_INVALID_VALUE;
    const RnnDims r = rnn_dims(desc, 0, 0);
    *bytes = (size_t)(rnn_all_matrices(r) + (long long)r.P * rnn_bias_floats(r)) * sizeof(float);
    return SNHIP_STATUS_SUCCESS;
}

int snhip_rnn_weight_params(const snhip_rnn_desc* desc, int pseudo_layer, int lin_layer_id, long long* matrix_offset,
                            int* rows, int* cols, long long* bias_offset) {
    const int st = rnn_check_desc(desc);
    if (st != SNHIP_STATUS_SUCCESS) return st;
    const RnnDims r = rnn_dims(desc, 0, 0);
    if (pseudo_layer < 0 || pseudo_layer >= r.P || lin_layer_id < 0 || lin_layer_id >= 2 * r.G)
        return SNHIP_STATUS_INVALID_VALUE;
    const bool recurrent = lin_layer_id >= r.G;
    const int gate = recurrent ? lin_layer_id - r.G : lin_layer_id;
    const long long inputs = recurrent ? r.H : rnn_layer_inputs(r, pseudo_layer / r.K);
    const RnnOffsets o = rnn_offsets(r, pseudo_layer);
    const long long b = recurrent ? o.bR : o.bW;
    if (matrix_offset != nullptr) *matrix_offset = (recurrent ? o.R : o.W) + (long long)gate * r.H * inputs;
    if (rows != nullptr) *rows = r.H;
    if (cols != nullptr) *cols = (int)inputs;
    if (bias_offset != nullptr) *bias_offset = b >= 0 ? b + (long long)gate * r.H : -1;
    return SNHIP_STATUS_SUCCESS;
}

int snhip_rnn_temp_space_sizes(const snhip_rnn_desc* desc, int training, int batch, int steps, size_t* workspace_bytes,
                               size_t* reserve_bytes) {
    const int st = rnn_check_desc(desc);
    if (st != SNHIP_STATUS_SUCCESS) return st;
    if (batch < 0 || steps < 0 || workspace_bytes == nullptr || reserve_bytes == nullptr)
        return SNHIP_STATUS_INVALID_VALUE;
    const RnnDims r = rnn_dims(desc, batch, steps);
    // inference keeps the gates in the workspace; training keeps them in reserve and its backward calls use the
    // workspace (the reference sizes it once, in the forward call, and reuses that size: RecurrentLayer.cs:335-345,461)
    const long long ws = training ? r.bwd_ws : (r.total > r.bwd_ws ? r.total : r.bwd_ws);
    *workspace_bytes = (size_t)(ws > 4 ? ws : 4) * sizeof(float);
    *reserve_bytes = training ? (size_t)(r.total > 4 ? r.total : 4) * sizeof(float) : 0;
    return SNHIP_STATUS_SUCCESS;
}

int snhip_rnn_set_step_mode(void* handle, int mode) {
    if (handle == nullptr) return SNHIP_STATUS_NOT_INITIALIZED;
    if (mode < 0 || mode > 1) return SNHIP_STATUS_INVALID_VALUE;
    static_cast<Handle*>(handle)->rnn_step_mode = mode;
    return SNHIP_STATUS_SUCCESS;
}

int snhip_rnn_forward(void* handle, const snhip_rnn_desc* desc, int training, int batch, int steps, const float* x,
                      float* y, const float* hx, float* hy, const float* cx, float* cy, const float* weights,
                      void* workspace, size_t workspace_bytes, void* reserve, size_t reserve_bytes) {
    Handle* h = static_cast<Handle*>(handle);
    int st = rnn_check_desc(desc);
    if (st != SNHIP_STATUS_SUCCESS) return st;
    st = rnn_common_checks(h, desc, batch, steps);
    if (st != SNHIP_STATUS_SUCCESS) return st;
    if (batch == 0 || steps == 0) return SNHIP_STATUS_SUCCESS;
    if (x == nullptr || y == nullptr || weights == nullptr) return SNHIP_STATUS_INVALID_VALUE;
    const RnnDims r = rnn_dims(desc, batch, steps);
    float* keep = static_cast<float*>(training ? reserve : workspace);
    const size_t keep_bytes = training ? reserve_bytes : workspace_bytes;
    if (keep == nullptr || keep_bytes < (size_t)r.total * sizeof(float)) return SNHIP_STATUS_INVALID_VALUE;
    const int B = batch, T = steps, H = r.H, G = r.G, K = r.K;
    const long long GH = (long long)G * H, KH = (long long)K * H;

    // (batch, steps, inputs) -> (steps, batch, inputs)
    st = snhip_transpose_second_and_third_dimension(handle, x, keep + r.xt_off, 1, B, T, r.I);
    if (st != SNHIP_STATUS_SUCCESS) return st;

    // dropout between the stacked layers, training only: this call's masks are numbered by the handle's count of such
    // calls; seed and count go into the reserve buffer for the backward calls
    const bool drop = training != 0 && r.dropout;
    const unsigned long long seed = h->rnn_dropout_seed;
    const unsigned int call = (unsigned int)h->rnn_dropout_calls;
    if (drop) {
        ++h->rnn_dropout_calls;
        hipLaunchKernelGGL(rnn_dropout_note_kernel, dim3(1), dim3(64), 0, h->stream,
                           reinterpret_cast<unsigned int*>(keep + r.rng_off), (unsigned int)seed, (unsigned int)(seed >> 32), call);
        st = hip_to_status(hipGetLastError());
        if (st != SNHIP_STATUS_SUCCESS) return st;
    }

    for (int layer = 0; layer < r.L; ++layer) {
        const float* inp = layer == 0 ? keep + r.xt_off
                                      : keep + (drop ? r.drop_off : r.out_off) + (long long)(layer - 1) * r.n * KH;
        const bool top = layer == r.L - 1;
        float* out = top ? y : keep + r.out_off + (long long)layer * r.n * KH;
        // rows of step t: the caller's y is batch-major, the stacked layers' outputs are step-major
        const long long out_step = top ? KH : (long long)B * KH, out_ld = top ? (long long)T * KH : KH;
        const long long I = rnn_layer_inputs(r, layer);
        // per direction: where its buffers are, the input projections of every step at once, the initial state
        struct Dir {
            RnnWeights w;
            float *gates, *hprev, *cells, *gh;
            const float *hx, *cx;
            int first, step;
        } dirs[2];
        bool fused = H % 4 == 0 && H >= 32 && h->rnn_step_mode == 0;
        for (int d = 0; d < K; ++d) {
            const int p = layer * K + d;
            Dir& D = dirs[d];
            D.w = rnn_weights(r, const_cast<float*>(weights), p);
            float* region = keep + (long long)p * r.per_p;
            D.gates = region + r.gates_off, D.hprev = region + r.hprev_off;
            D.cells = region + r.cells_off, D.gh = region + r.gh_off;
            D.hx = hx ? hx + (long long)p * B * H : nullptr;
            D.cx = cx ? cx + (long long)p * B * H : nullptr;
            D.first = d == 0 ? 0 : T - 1, D.step = d == 0 ? 1 : -1;

            GemmArgs g;
            g.tB = true;
            g.M = (int)r.n, g.N = (int)GH, g.K = (int)I;
            g.A = inp, g.lda = (int)I, g.B = D.w.W, g.ldb = (int)I, g.C = D.gates, g.ldc = (int)GH;
            g.bias = D.w.bW;
            st = gemm_core(h, g);
            if (st != SNHIP_STATUS_SUCCESS) return st;
            st = rnn_set_rows(h, D.hprev + (long long)D.first * B * H, H, D.hx, H, B, H);
            if (st != SNHIP_STATUS_SUCCESS) return st;
            // product and cell in one launch per step when the rows can be read in 16-byte pieces
            fused = fused && (uintptr_t)D.hprev % 16 == 0 && (uintptr_t)D.w.R % 16 == 0;
        }
        // the directions are independent and advance together (one launch per direction and step: a combined grid
        // of both directions was measured and gains nothing, the second direction's workgroups queue behind the first's)
        for (int k = 0; k < T; ++k) {
            const bool last = k == T - 1;
            for (int d = 0; d < K; ++d) {
                const Dir& D = dirs[d];
                const int p = layer * K + d;
                const int t = D.first + D.step * k;
                const bool zero_state = k == 0 && D.hx == nullptr;
                if (!fused && (r.cell == RNN_GRU || !zero_state)) {
                    GemmArgs s;  // h[t-1] . R^T
                    s.tB = true;
                    s.M = B, s.N = (int)GH, s.K = H;
                    s.A = D.hprev + (long long)t * B * H, s.lda = H;
                    s.B = D.w.R, s.ldb = H;
                    if (r.cell == RNN_GRU) {
                        s.C = D.gh + (long long)t * B * 3 * H, s.ldc = 3 * H;
                    } else {
                        s.C = D.gates + (long long)t * B * GH, s.ldc = (int)GH, s.beta = 1.0f;
                    }
                    st = gemm_core(h, s);
                    if (st != SNHIP_STATUS_SUCCESS) return st;
                }
                RnnStepFwd c;
                c.gates = D.gates + (long long)t * B * GH, c.ld_gates = GH;
                c.gh = D.gh + (long long)t * B * 3 * H, c.ld_gh = 3LL * H;
                c.bias_r = D.w.bR;
                c.h_prev = D.hprev + (long long)t * B * H, c.ld_hprev = H;
                c.c_prev = k == 0 ? D.cx : D.cells + (long long)(t - D.step) * B * H, c.ld_cprev = H;
                c.c_out = D.cells + (long long)t * B * H, c.ld_c = H;
                c.y = out + (long long)t * out_step + (long long)d * H, c.ld_y = out_ld;
                c.h_next = last ? nullptr : D.hprev + (long long)(t + D.step) * B * H, c.ld_hnext = H;
                c.hy = (last && hy) ? hy + (long long)p * B * H : nullptr;
                c.cy = (last && cy && r.cell == RNN_LSTM) ? cy + (long long)p * B * H : nullptr;
                c.batch = B, c.hidden = H, c.cell = r.cell;
                if (fused) {
                    const int U = G == 1 ? 32 : 16;
                    const dim3 grid((unsigned)((H + U - 1) / U), (unsigned)((B + 31) / 32));
                    const bool tail = H % 32 != 0;
                    auto fn = G == 4   ? (tail ? rnn_step_fused_kernel<4, true> : rnn_step_fused_kernel<4, false>)
                              : G == 3 ? (tail ? rnn_step_fused_kernel<3, true> : rnn_step_fused_kernel<3, false>)
                                       : (tail ? rnn_step_fused_kernel<1, true> : rnn_step_fused_kernel<1, false>);
                    hipLaunchKernelGGL(fn, grid, dim3(256), 0, h->stream, c, (const float*)D.w.R);
                } else {
                    hipLaunchKernelGGL(rnn_cell_fwd_kernel, dim3((unsigned)(((long long)B * H + 255) / 256)), dim3(256), 0,
                                       h->stream, c);
                }
                st = hip_to_status(hipGetLastError());
                if (st != SNHIP_STATUS_SUCCESS) return st;
            }
        }
        if (drop && !top) {  // what the next layer reads: this layer's outputs with units dropped
            st = rnn_apply_dropout(h, r, desc->dropout, keep + r.drop_off + (long long)layer * r.n * KH, out, layer, seed, call,
                                   nullptr, false);
            if (st != SNHIP_STATUS_SUCCESS) return st;
        }
    }
    return SNHIP_STATUS_SUCCESS;
}

int snhip_rnn_backward_data(void* handle, const snhip_rnn_desc* desc, int batch, int steps, const float* y,
                            const float* dy, float* dx, const float* hx, const float* dhy, float* dhx,
                            const float* cx, const float* dcy, float* dcx, const float* weights, void* workspace,
                            size_t workspace_bytes, void* reserve, size_t reserve_bytes) {
    Handle* h = static_cast<Handle*>(handle);
    int st = rnn_common_checks(h, desc, batch, steps);
    if (st != SNHIP_STATUS_SUCCESS) return st;
    if (batch == 0 || steps == 0) return SNHIP_STATUS_SUCCESS;
    (void)hx;  // the states that entered every step are in reserve
    if (y == nullptr || dy == nullptr || weights == nullptr) return SNHIP_STATUS_INVALID_VALUE;
    const RnnDims r = rnn_dims(desc, batch, steps);
    float* keep = static_cast<float*>(reserve);
    float* ws = static_cast<float*>(workspace);
    if (keep == nullptr || reserve_bytes < (size_t)r.total * sizeof(float)) return SNHIP_STATUS_INVALID_VALUE;
    if (ws == nullptr || workspace_bytes < (size_t)r.bwd_ws * sizeof(float)) return SNHIP_STATUS_INVALID_VALUE;
    const int B = batch, T = steps, H = r.H, G = r.G, K = r.K;
    const long long GH = (long long)G * H, KH = (long long)K * H;
    float* between[2] = {ws + 2LL * B * H + GH, ws + 2LL * B * H + GH + r.n * KH};

    for (int layer = r.L - 1; layer >= 0; --layer) {
        const bool top = layer == r.L - 1;
        const float* out = top ? y : keep + r.out_off + (long long)layer * r.n * KH;
        const float* dout = top ? dy : between[layer & 1];
        const long long out_step = top ? KH : (long long)B * KH, out_ld = top ? (long long)T * KH : KH;
        float* dinp = layer == 0 ? dx : between[(layer - 1) & 1];
        if (r.dropout && !top) {
            // the layer above produced the gradient of what it read, this layer's outputs after dropout: the same
            // mask (regenerated from the seed and call number the forward call left in reserve) takes it to the
            // gradient of the outputs themselves
            st = rnn_apply_dropout(h, r, desc->dropout, between[layer & 1], between[layer & 1], layer, 0, 0,
                                   reinterpret_cast<const unsigned int*>(keep + r.rng_off), false);
            if (st != SNHIP_STATUS_SUCCESS) return st;
        }
        const long long I = rnn_layer_inputs(r, layer);
        struct Dir {
            RnnWeights w;
            float *gates, *hprev, *cells, *gh, *dh, *dc, *Rt;
            const float* cx;
            int first, step;
        } dirs[2];
        // every step but the first one processed runs as one launch (product with R, then the cell gradient) when
        // rows can be read in 16-byte pieces; that kernel wants the rows of R^T
        bool fused = H % 4 == 0 && H >= 32 && T > 1 && h->rnn_step_mode == 0;
        for (int d = 0; d < K; ++d) {
            const int p = layer * K + d;
            Dir& D = dirs[d];
            D.w = rnn_weights(r, const_cast<float*>(weights), p);
            float* region = keep + (long long)p * r.per_p;
            D.gates = region + r.gates_off, D.hprev = region + r.hprev_off;
            D.cells = region + r.cells_off, D.gh = region + r.gh_off;
            D.dh = d == 0 ? ws : ws + r.dir1_off;
            D.dc = D.dh + (long long)B * H;
            D.Rt = d == 0 ? ws + r.rt_off : ws + r.dir1_off + 2LL * B * H;
            D.cx = cx ? cx + (long long)p * B * H : nullptr;
            D.first = d == 0 ? 0 : T - 1, D.step = d == 0 ? 1 : -1;
            st = rnn_set_rows(h, D.dh, H, dhy ? dhy + (long long)p * B * H : nullptr, H, B, H);
            if (st != SNHIP_STATUS_SUCCESS) return st;
            if (r.cell == RNN_LSTM) {
                st = rnn_set_rows(h, D.dc, H, dcy ? dcy + (long long)p * B * H : nullptr, H, B, H);
                if (st != SNHIP_STATUS_SUCCESS) return st;
            }
            fused = fused && (uintptr_t)D.gates % 16 == 0 && (uintptr_t)D.Rt % 16 == 0;
        }
        if (fused)
            for (int d = 0; d < K; ++d) {
                st = snhip_transpose_second_and_third_dimension(handle, dirs[d].w.R, dirs[d].Rt, 1, (int)GH, H, 1);
                if (st != SNHIP_STATUS_SUCCESS) return st;
            }
        for (int k = T - 1; k >= 0; --k) {
            const bool one_launch = fused && k < T - 1;
            for (int d = 0; d < K; ++d) {
                const Dir& D = dirs[d];
                const int t = D.first + D.step * k;
                RnnStepBwd c;
                c.gates = D.gates + (long long)t * B * GH, c.ld_gates = GH;
                c.gh = D.gh + (long long)t * B * 3 * H, c.ld_gh = 3LL * H;
                c.h_prev = D.hprev + (long long)t * B * H, c.ld_hprev = H;
                c.y = out + (long long)t * out_step + (long long)d * H, c.ld_y = out_ld;
                c.c_prev = k == 0 ? D.cx : D.cells + (long long)(t - D.step) * B * H, c.ld_cprev = H;
                c.c = D.cells + (long long)t * B * H, c.ld_c = H;
                c.dy = dout + (long long)t * out_step + (long long)d * H, c.ld_dy = out_ld;
                c.dh = D.dh, c.dc = D.dc;
                c.batch = B, c.hidden = H, c.cell = r.cell;
                if (one_launch) {
                    const float* dg_next = ((r.cell == RNN_GRU) ? D.gh : D.gates) + (long long)(t + D.step) * B * GH;
                    const dim3 grid((unsigned)((H + RnnBwdFusedCfg::U - 1) / RnnBwdFusedCfg::U), (unsigned)((B + 31) / 32));
                    const bool tail = GH % 32 != 0;
                    auto fn = G == 4   ? (tail ? rnn_step_bwd_fused_kernel<4, true> : rnn_step_bwd_fused_kernel<4, false>)
                              : G == 3 ? (tail ? rnn_step_bwd_fused_kernel<3, true> : rnn_step_bwd_fused_kernel<3, false>)
                                       : (tail ? rnn_step_bwd_fused_kernel<1, true> : rnn_step_bwd_fused_kernel<1, false>);
                    hipLaunchKernelGGL(fn, grid, dim3(512), RnnBwdFusedCfg::LDS_BYTES, h->stream, c, dg_next, GH,
                                       (const float*)D.Rt);
                    st = hip_to_status(hipGetLastError());
                    if (st != SNHIP_STATUS_SUCCESS) return st;
                    continue;
                }
                hipLaunchKernelGGL(rnn_cell_bwd_kernel, dim3((unsigned)(((long long)B * H + 255) / 256)), dim3(256), 0,
                                   h->stream, c);
                st = hip_to_status(hipGetLastError());
                if (st != SNHIP_STATUS_SUCCESS) return st;
                // dh = d(R h)[:, t] . R for the step before (GRU: added to dh * z); with the one-launch steps only the
                // gradient of the initial state is left to multiply, and only if somebody asks for it
                if (fused ? (k > 0 || dhx == nullptr) : (k == 0 && dhx == nullptr)) continue;
                GemmArgs s;
                s.M = B, s.N = H, s.K = (int)GH;
                s.A = (r.cell == RNN_GRU) ? D.gh + (long long)t * B * 3 * H : D.gates + (long long)t * B * GH;
                s.lda = (int)GH;
                s.B = D.w.R, s.ldb = H;
                s.C = D.dh, s.ldc = H;
                s.beta = (r.cell == RNN_GRU) ? 1.0f : 0.0f;
                st = gemm_core(h, s);
                if (st != SNHIP_STATUS_SUCCESS) return st;
            }
            if (!one_launch) continue;
            if (k == 0 && dhx != nullptr)
                for (int d = 0; d < K; ++d) {  // the last launch left d(gates) of the first step: one more product for dhx
                    const Dir& D = dirs[d];
                    GemmArgs s;
                    s.M = B, s.N = H, s.K = (int)GH;
                    s.A = (r.cell == RNN_GRU) ? D.gh + (long long)D.first * B * 3 * H : D.gates + (long long)D.first * B * GH;
                    s.lda = (int)GH;
                    s.B = D.w.R, s.ldb = H;
                    s.C = D.dh, s.ldc = H;
                    s.beta = (r.cell == RNN_GRU) ? 1.0f : 0.0f;
                    st = gemm_core(h, s);
                    if (st != SNHIP_STATUS_SUCCESS) return st;
                }
        }
        for (int d = 0; d < K; ++d) {
            const Dir& D = dirs[d];
            const int p = layer * K + d;
            if (dhx != nullptr) {
                st = rnn_set_rows(h, dhx + (long long)p * B * H, H, D.dh, H, B, H);
                if (st != SNHIP_STATUS_SUCCESS) return st;
            }
            if (dcx != nullptr && r.cell == RNN_LSTM) {
                st = rnn_set_rows(h, dcx + (long long)p * B * H, H, D.dc, H, B, H);
                if (st != SNHIP_STATUS_SUCCESS) return st;
            }
            if (dinp == nullptr) continue;
            GemmArgs g;  // gradient of the layer's input: both directions add up
            g.K = (int)GH, g.N = (int)I;
            g.A = D.gates, g.lda = (int)GH, g.B = D.w.W, g.ldb = (int)I, g.C = dinp;
            g.beta = d == 0 ? 0.0f : 1.0f;
            if (layer == 0) {
                // one product per step: step-major rows in, the caller's batch-major dx out
                g.M = B, g.batch = T;
                g.sA = (long long)B * GH, g.sB = 0, g.sC = I, g.ldc = (int)(T * I);
            } else {
                g.M = (int)r.n, g.ldc = (int)I;
            }
            st = gemm_core(h, g);
            if (st != SNHIP_STATUS_SUCCESS) return st;
        }
    }
    return SNHIP_STATUS_SUCCESS;
}

int snhip_rnn_backward_weights(void* handle, const snhip_rnn_desc* desc, int batch, int steps, const float* x,
                               const float* hx, const float* y, float* weight_gradients, void* workspace,
                               size_t workspace_bytes, void* reserve, size_t reserve_bytes) {
    Handle* h = static_cast<Handle*>(handle);
    int st = rnn_common_checks(h, desc, batch, steps);
    if (st != SNHIP_STATUS_SUCCESS) return st;
    if (batch == 0 || steps == 0) return SNHIP_STATUS_SUCCESS;
    (void)hx, (void)y;  // both are in reserve, arranged per step, and so is a step-major copy of x
    if (x == nullptr || weight_gradients == nullptr) return SNHIP_STATUS_INVALID_VALUE;
    const RnnDims r = rnn_dims(desc, batch, steps);
    float* keep = static_cast<float*>(reserve);
    float* ws = static_cast<float*>(workspace);
    if (keep == nullptr || reserve_bytes < (size_t)r.total * sizeof(float)) return SNHIP_STATUS_INVALID_VALUE;
    if (ws == nullptr || workspace_bytes < (size_t)r.bwd_ws * sizeof(float)) return SNHIP_STATUS_INVALID_VALUE;
    const int H = r.H, G = r.G, K = r.K;
    const long long GH = (long long)G * H;
    float* colsum = ws + 2LL * batch * H;

    for (int layer = 0; layer < r.L; ++layer) {
        const float* inp = layer == 0 ? keep + r.xt_off
                                      : keep + (r.dropout ? r.drop_off : r.out_off) + (long long)(layer - 1) * r.n * K * H;
        const long long I = rnn_layer_inputs(r, layer);
        for (int d = 0; d < K; ++d) {
            const int p = layer * K + d;
            const RnnWeights dw = rnn_weights(r, weight_gradients, p);
            float* region = keep + (long long)p * r.per_p;
            const float* dgates = region + r.gates_off;
            const float* hprev = region + r.hprev_off;
            const float* dgh = (r.cell == RNN_GRU) ? region + r.gh_off : dgates;

            GemmArgs g;  // dW += d(gates)^T . X, column sums of d(gates) on the side
            g.tA = true;
            g.M = (int)GH, g.N = (int)I, g.K = (int)r.n;
            g.A = dgates, g.lda = (int)GH, g.B = inp, g.ldb = (int)I, g.C = dw.W, g.ldc = (int)I;
            g.beta = 1.0f;
            g.colsum = (dw.bW != nullptr || (dw.bR != nullptr && r.cell != RNN_GRU)) ? colsum : nullptr;
            st = gemm_core(h, g);
            if (st != SNHIP_STATUS_SUCCESS) return st;
            if (dw.bW != nullptr) {
                st = snhip_axpy(handle, GH, 1.0f, colsum, dw.bW);
                if (st != SNHIP_STATUS_SUCCESS) return st;
            }
            if (dw.bR != nullptr && r.cell != RNN_GRU) {
                st = snhip_axpy(handle, GH, 1.0f, colsum, dw.bR);
                if (st != SNHIP_STATUS_SUCCESS) return st;
            }

            GemmArgs q;  // dR += d(R h + bR)^T . Hprev
            q.tA = true;
            q.M = (int)GH, q.N = H, q.K = (int)r.n;
            q.A = dgh, q.lda = (int)GH, q.B = hprev, q.ldb = H, q.C = dw.R, q.ldc = H;
            q.beta = 1.0f;
            q.colsum = (dw.bR != nullptr && r.cell == RNN_GRU) ? colsum : nullptr;
            st = gemm_core(h, q);
            if (st != SNHIP_STATUS_SUCCESS) return st;
            if (q.colsum != nullptr) {
                st = snhip_axpy(handle, GH, 1.0f, colsum, dw.bR);
                if (st != SNHIP_STATUS_SUCCESS) return st;
            }
        }
    }
    return SNHIP_STATUS_SUCCESS;
}

int snhip_rnn_set_dropout_seed(void* handle, unsigned long long seed) {
    if (handle == nullptr) return SNHIP_STATUS_NOT_INITIALIZED;
    Handle* h = static_cast<Handle*>(handle);
    h->rnn_dropout_seed = seed;
    h->rnn_dropout_calls = 0;
    return SNHIP_STATUS_SUCCESS;
}

int snhip_rnn_get_dropout_calls(void* handle, unsigned long long* calls) {
    if (handle == nullptr) return SNHIP_STATUS_NOT_INITIALIZED;
    if (calls == nullptr) return SNHIP_STATUS_INVALID_VALUE;
    *calls = static_cast<Handle*>(handle)->rnn_dropout_calls;
    return SNHIP_STATUS_SUCCESS;
}

int snhip_rnn_dropout_mask(void* handle, const snhip_rnn_desc* desc, int batch, int steps, unsigned long long call,
                           int boundary, float* mask) {
    Handle* h = static_cast<Handle*>(handle);
    const int st = rnn_common_checks(h, desc, batch, steps);
    if (st != SNHIP_STATUS_SUCCESS) return st;
    if (boundary < 0 || boundary >= desc->num_layers - 1) return SNHIP_STATUS_INVALID_VALUE;
    if (batch == 0 || steps == 0) return SNHIP_STATUS_SUCCESS;
    if (mask == nullptr) return SNHIP_STATUS_INVALID_VALUE;
    const RnnDims r = rnn_dims(desc, batch, steps);
    return rnn_apply_dropout(h, r, desc->dropout, mask, nullptr, boundary, h->rnn_dropout_seed, (unsigned int)call, nullptr,
                             true);
}

}  // extern "C"
