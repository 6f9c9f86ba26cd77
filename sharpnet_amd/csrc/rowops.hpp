// Row / column helpers that sit right next to the GEMMs in the reference's
// Linear and scaled-dot-product-attention layers.  All are HBM-bound: one pass
// over the data, coalesced along the contiguous (last) dimension, deterministic
// (no float atomics).
//
//   column_sum_kernel        Compute_BiasGradient_from_dy       Prod/CPU/CpuTensor.cs:1736-1740 (GPU: GpuTensor.cs:686-701)
//   broadcast_add_kernel     BroadcastAddVectorToOutput         Prod/CPU/CpuTensor.cs:1468-1487 (GPU: GpuTensor.cs:633-644)
//   axpy_kernel              Update_Adding_Alpha_X (saxpy)      Prod/Layers/Linear.cs:178
//   softmax_rows_kernel      softmax over the last dimension    Prod/CPU/CpuTensorActivationFunctions.cs:19-46
//   softmax_rows_bwd_kernel  its gradient as cuDNN computes it  Prod/GPU/GpuTensor.cs ActivationBackward (cudnnSoftmaxBackward)
//   set_above_diagonal_kernel SetAllElementsAboveMainDiagonal   Prod/CPU/CpuTensor.cs:3037-3052
#pragma once
#include <hip/hip_runtime.h>

namespace snhip {

__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v = fmaxf(v, __shfl_xor(v, off, 64));
    return v;
}
__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, 64);
    return v;
}

// out[c] = sum over rows of x[r][c].  A workgroup of 4 wavefronts owns 64
// columns; wavefront w adds rows w, w+4, ... (lanes along columns, 256-byte
// coalesced reads), the four partial sums meet in LDS in a fixed order.
__global__ void __launch_bounds__(256) column_sum_kernel(const float* __restrict__ x, float* __restrict__ out, int rows,
                                                         int cols) {
    __shared__ float part[4][64];
    const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
    const int c = blockIdx.x * 64 + lane;
    float s = 0.0f;
    if (c < cols)
        for (int r = w; r < rows; r += 4) s += x[(long long)r * cols + c];
    part[w][lane] = s;
    __syncthreads();
    if (w == 0 && c < cols) out[c] = (part[0][lane] + part[1][lane]) + (part[2][lane] + part[3][lane]);
}

// y[r][c] += v[c]
__global__ void __launch_bounds__(256) broadcast_add_kernel(float* y, const float* __restrict__ v, long long rows, int cols) {
    const long long total = rows * cols;
    for (long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += (long long)gridDim.x * blockDim.x)
        y[i] += v[i % cols];
}

// y += alpha * x
__global__ void __launch_bounds__(256) axpy_kernel(float* y, const float* __restrict__ x, float alpha, long long n) {
    for (long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (long long)gridDim.x * blockDim.x)
        y[i] += alpha * x[i];
}

// One wavefront per row: y = softmax(x) over `cols` contiguous elements,
// max-subtracted, fp32 throughout (x and y may be the same buffer).
__global__ void __launch_bounds__(256) softmax_rows_kernel(const float* x, float* y, long long rows, int cols) {
    const int lane = threadIdx.x & 63;
    const long long row = (long long)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (row >= rows) return;
    const float* xr = x + row * cols;
    float* yr = y + row * cols;
    float m = -3.402823466e+38f;
    for (int c = lane; c < cols; c += 64) m = fmaxf(m, xr[c]);
    m = wave_max(m);
    float s = 0.0f;
    for (int c = lane; c < cols; c += 64) {
        const float e = expf(xr[c] - m);
        yr[c] = e;
        s += e;
    }
    s = wave_sum(s);
    for (int c = lane; c < cols; c += 64) yr[c] = yr[c] / s;
}

// dx = y * (dy - sum_j dy_j * y_j) per row (dx may alias dy).
__global__ void __launch_bounds__(256) softmax_rows_bwd_kernel(const float* __restrict__ y, const float* dy, float* dx,
                                                               long long rows, int cols) {
    const int lane = threadIdx.x & 63;
    const long long row = (long long)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (row >= rows) return;
    const float* yr = y + row * cols;
    const float* dyr = dy + row * cols;
    float* dxr = dx + row * cols;
    float s = 0.0f;
    for (int c = lane; c < cols; c += 64) s += dyr[c] * yr[c];
    s = wave_sum(s);
    for (int c = lane; c < cols; c += 64) dxr[c] = yr[c] * (dyr[c] - s);
}

// x[b][r][c] = value for c > r
__global__ void __launch_bounds__(256) set_above_diagonal_kernel(float* x, long long matrices, int rows, int cols,
                                                                 float value) {
    const long long total = matrices * rows * cols;
    for (long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x; i < total;
         i += (long long)gridDim.x * blockDim.x) {
        const int c = (int)(i % cols);
        const int r = (int)((i / cols) % rows);
        if (c > r) x[i] = value;
    }
}

}  // namespace snhip
