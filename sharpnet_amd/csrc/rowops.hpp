// Small kernels that belong to exactly one translation unit: the GEMM's split-K reduction and degenerate
// (alpha == 0 / K == 0) forms, the copy used to calibrate traffic counters, and the
// row / column helpers that sit right next to the GEMMs in the reference's
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

#include "sgemm_mfma.hpp"

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

// out[z][k][c] = sum of x[z][r][c] over the rows r of chunk k (row pitch ld, matrix z at x + z * stride;
// blockIdx.y = z, blockIdx.z = k, chunks of rows_per_chunk rows).  A workgroup of 4 wavefronts owns 64 columns of
// one chunk; wavefront w adds rows w, w+4, ... of it (lanes along columns, 256-byte coalesced reads, four rows in
// flight per wavefront), the four partial sums meet in LDS in a fixed order.  With one chunk this is the whole
// column sum; a tall matrix is cut into chunks so that the launch fills the chip, and column_sum_finish_kernel
// adds the chunks in index order (deterministic, no float atomics).
__global__ void __launch_bounds__(256) column_sum_kernel(const float* __restrict__ x, float* __restrict__ out, int rows,
                                                         int cols, long long ld, long long stride, int rows_per_chunk) {
    __shared__ float part[4][64];
    const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
    const int c = blockIdx.x * 64 + lane;
    const float* xz = x + (long long)blockIdx.y * stride;
    const int r0 = blockIdx.z * rows_per_chunk;
    const int r1 = (r0 + rows_per_chunk < rows) ? r0 + rows_per_chunk : rows;
    float s0 = 0.0f, s1 = 0.0f, s2 = 0.0f, s3 = 0.0f;
    if (c < cols) {
        int r = r0 + w;
        for (; r + 12 < r1; r += 16) {
            s0 += xz[(long long)r * ld + c];
            s1 += xz[(long long)(r + 4) * ld + c];
            s2 += xz[(long long)(r + 8) * ld + c];
            s3 += xz[(long long)(r + 12) * ld + c];
        }
        for (; r < r1; r += 4) s0 += xz[(long long)r * ld + c];
    }
    part[w][lane] = (s0 + s1) + (s2 + s3);
    __syncthreads();
    if (w == 0 && c < cols)
        out[((long long)blockIdx.y * gridDim.z + blockIdx.z) * cols + c] =
            (part[0][lane] + part[1][lane]) + (part[2][lane] + part[3][lane]);
}

// out[z][c] = partial[z][0][c] + partial[z][1][c] + ... in index order.
__global__ void __launch_bounds__(256) column_sum_finish_kernel(const float* __restrict__ partial, float* __restrict__ out,
                                                                int chunks, int cols, int nz) {
    const long long idx = (long long)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= (long long)nz * cols) return;
    const int z = (int)(idx / cols), c = (int)(idx % cols);
    float s = 0.0f;
    for (int k = 0; k < chunks; ++k) s += partial[((long long)z * chunks + k) * cols + c];
    out[idx] = s;
}

// dst[i] = value for count 32-bit words (a kernel rather than a memset node, so that a caller may record it into a
// HIP graph like any other launch of this library).
__global__ void __launch_bounds__(256) fill32_kernel(unsigned int* dst, unsigned int value, long long count) {
    for (long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x; i < count; i += (long long)gridDim.x * blockDim.x)
        dst[i] = value;
}

// y = act(x) element-wise (x and y may be the same buffer); `act` as in the GEMM epilogue.
__global__ void __launch_bounds__(256) activation_kernel(const float* x, float* y, long long n, int act, float a) {
    for (long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (long long)gridDim.x * blockDim.x)
        y[i] = activate(x[i], act, a);
}

// dx = dy * act'(x) written in terms of the output y = act(x), as the reference's CPU gradients are
// (Prod/CPU/CpuTensorActivationFunctions.cs:190-244): ReLU y > 0, leaky ReLU y >= 0 ? 1 : a,
// sigmoid y (1 - y), tanh 1 - y^2.  dx may alias dy.
__global__ void __launch_bounds__(256) activation_bwd_kernel(const float* __restrict__ y, const float* dy, float* dx,
                                                             long long n, int act, float a) {
    for (long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (long long)gridDim.x * blockDim.x) {
        const float yy = y[i], g = dy[i];
        float o;
        switch (act) {
            case ACT_RELU:
                o = yy > 0.0f ? g : 0.0f;
                break;
            case ACT_LEAKY_RELU:
                o = yy >= 0.0f ? g : a * g;
                break;
            case ACT_SIGMOID:
                o = g * yy * (1.0f - yy);
                break;
            case ACT_TANH:
                o = g * (1.0f - yy * yy);
                break;
            default:
                o = g;
        }
        dx[i] = o;
    }
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

// dst[a][c][b][d] = src[a][b][c][d]: TransposeSecondAndThirdDimension (Prod/CPU/CpuTensor.cs:301-322, GPU kernel
// SinglePrecision.cu:1285), the head split / merge copy of MultiheadAttention.cs:207-230.  One thread per element
// of dst, so writes are contiguous and reads are contiguous over d.
__global__ void __launch_bounds__(256) transpose_2nd_3rd_kernel(const float* __restrict__ src, float* __restrict__ dst,
                                                                int A, int B, int C, int D) {
    const long long total = (long long)A * B * C * D;
    for (long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x; i < total;
         i += (long long)gridDim.x * blockDim.x) {
        const int d = (int)(i % D);
        long long t = i / D;
        const int b = (int)(t % B);
        t /= B;
        const int c = (int)(t % C);
        const int a = (int)(t / C);
        dst[i] = src[(((long long)a * B + b) * C + c) * D + d];
    }
}

// Column-major C (m x n, ldc) = alpha * op(A) + beta * op(B): cublasSgeam, which the reference uses with
// transa = T, beta = 0 as its matrix transpose (Prod/GPU/GpuTensor.cs:1256-1291).  A workgroup of 32 x 8 threads owns
// a 32 x 32 tile of C; a transposed operand goes through a padded LDS tile so that both its reads and the writes
// of C are contiguous.  An operand whose scalar is zero is never read (BLAS rule: 0 * NaN must not reach C).
__global__ void __launch_bounds__(256) geam_kernel(int ta, int tb, int m, int n, float alpha, const float* __restrict__ A,
                                                   long long lda, float beta, const float* __restrict__ B, long long ldb,
                                                   float* C, long long ldc) {
    __shared__ float tA[32][33], tB[32][33];
    const int tx = threadIdx.x & 31, ty = threadIdx.x >> 5;
    const int i0 = blockIdx.x * 32, j0 = blockIdx.y * 32;
    const bool use_a = (alpha != 0.0f), use_b = (beta != 0.0f);
    ta = ta && use_a;
    if (ta || (tb && use_b)) {
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            const int r = ty + 8 * k;  // index along i inside the tile; tx runs along j: contiguous in a transposed operand
            if (i0 + r < m && j0 + tx < n) {
                if (ta) tA[r][tx] = A[(long long)(i0 + r) * lda + (j0 + tx)];
                if (tb && use_b) tB[r][tx] = B[(long long)(i0 + r) * ldb + (j0 + tx)];
            }
        }
        __syncthreads();
    }
#pragma unroll
    for (int k = 0; k < 4; ++k) {
        const int c = ty + 8 * k;  // index along j inside the tile; tx runs along i: contiguous in C
        const int i = i0 + tx, j = j0 + c;
        if (i < m && j < n) {
            float v = 0.0f;
            if (use_a) v = alpha * (ta ? tA[tx][c] : A[(long long)j * lda + i]);
            if (use_b) v += beta * (tb ? tB[tx][c] : B[(long long)j * ldb + i]);
            C[(long long)j * ldc + i] = v;
        }
    }
}

// Column-major C (m x n, ldc) = A . diag(x) (right, x has n entries) or diag(x) . A (left, m entries): cublasSdgmm,
// the reference's MultiplyTensor (Prod/GPU/GpuTensor.cs:1380-1395).  C may be A.
__global__ void __launch_bounds__(256) dgmm_kernel(int right, int m, int n, const float* A, long long lda,
                                                   const float* __restrict__ x, long long incx, float* C, long long ldc) {
    const long long total = (long long)m * n;
    for (long long idx = (long long)blockIdx.x * blockDim.x + threadIdx.x; idx < total;
         idx += (long long)gridDim.x * blockDim.x) {
        const int i = (int)(idx % m), j = (int)(idx / m);
        const float s = x[(long long)(right ? j : i) * incx];
        C[(long long)j * ldc + i] = A[(long long)j * lda + i] * s;
    }
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

// C = act(alpha * sum_s ws[batch][s] + bias + beta * C + gamma * D), splits summed in index order so the result
// does not depend on scheduling.
__global__ void __launch_bounds__(256) splitk_reduce_kernel(const float* __restrict__ ws, float* C, const Epilogue ep,
                                                            int M, int N, int ldc, long long strideC, long long strideC2,
                                                            int batch_inner, int splitk, int batch, float alpha,
                                                            float beta) {
    const long long mn = (long long)M * N;
    const long long total = mn * batch;
    for (long long idx = (long long)blockIdx.x * blockDim.x + threadIdx.x; idx < total;
         idx += (long long)gridDim.x * blockDim.x) {
        const int b = (int)(idx / mn);
        const long long e = idx - b * mn;
        const int row = (int)(e / N), col = (int)(e - (long long)row * N);
        const float* w = ws + (long long)b * splitk * mn + e;
        float s = 0.0f;
        for (int k = 0; k < splitk; ++k) s += w[(long long)k * mn];
        float o = alpha * s;
        if (ep.bias != nullptr) o += ep.bias[col];
        float* c = C + batch_offset(split_batch(b, batch_inner), strideC, strideC2) + (long long)row * ldc + col;
        if (beta != 0.0f) o += beta * *c;
        if (ep.addend != nullptr)
            o += ep.gamma * ep.addend[batch_offset(split_batch(b, batch_inner), ep.strideD, ep.strideD2) + (long long)row * ep.ldd + col];
        *c = activate(o, ep.act, ep.act_param);
    }
}

// C = act(bias + beta * C + gamma * D): the alpha == 0 or K == 0 degenerate product.
__global__ void __launch_bounds__(256) scale_c_kernel(float* C, const Epilogue ep, int M, int N, int ldc,
                                                      long long strideC, long long strideC2, int batch_inner, int batch,
                                                      float beta) {
    const long long mn = (long long)M * N;
    const long long total = mn * batch;
    for (long long idx = (long long)blockIdx.x * blockDim.x + threadIdx.x; idx < total;
         idx += (long long)gridDim.x * blockDim.x) {
        const int b = (int)(idx / mn);
        const long long e = idx - b * mn;
        const int row = (int)(e / N), col = (int)(e - (long long)row * N);
        float* c = C + batch_offset(split_batch(b, batch_inner), strideC, strideC2) + (long long)row * ldc + col;
        float o = (beta != 0.0f) ? beta * *c : 0.0f;
        if (ep.bias != nullptr) o += ep.bias[col];
        if (ep.addend != nullptr)
            o += ep.gamma * ep.addend[batch_offset(split_batch(b, batch_inner), ep.strideD, ep.strideD2) + (long long)row * ep.ldd + col];
        *c = activate(o, ep.act, ep.act_param);
    }
}

// Plain device-to-device copy of `count` floats (16-byte vectors when both
// pointers allow it).  Exists as the known-size reference launch against which
// hardware traffic counters are scaled; it is not on the GEMM path.
__global__ void __launch_bounds__(256) copy_f32_kernel(const float* __restrict__ src, float* __restrict__ dst,
                                                       long long count, int vec) {
    const long long stride = (long long)gridDim.x * blockDim.x;
    long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x;
    if (vec) {
        const long long n4 = count / 4;
        const f32x4* s4 = reinterpret_cast<const f32x4*>(src);
        f32x4* d4 = reinterpret_cast<f32x4*>(dst);
        for (long long j = i; j < n4; j += stride) d4[j] = s4[j];
        for (long long j = n4 * 4 + i; j < count; j += stride) dst[j] = src[j];
    } else {
        for (; i < count; i += stride) dst[i] = src[i];
    }
}

// dst[i] = bf16(src[i]), round to nearest even (the rounding the bf16-input GEMM applies on its way into LDS):
// the one pass that turns an fp32 operand into the bf16 storage of the bf16-stored GEMM entry points.
// Eight elements per thread and step (two 16-byte loads, one 16-byte store) when the pointers allow it.
__global__ void __launch_bounds__(256) convert_f32_to_bf16_kernel(const float* __restrict__ src, __bf16* __restrict__ dst,
                                                                  long long count, int vec) {
    typedef __bf16 bf16x4_t __attribute__((ext_vector_type(4)));
    const long long stride = (long long)gridDim.x * blockDim.x;
    const long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x;
    long long done = 0;
    if (vec) {
        const long long n8 = count / 8;
        const f32x4* s4 = reinterpret_cast<const f32x4*>(src);
        for (long long j = i; j < n8; j += stride) {
            const f32x4 a = s4[2 * j], b = s4[2 * j + 1];
            const bf16x4_t lo = __builtin_convertvector(a, bf16x4_t), hi = __builtin_convertvector(b, bf16x4_t);
            bf16x4_t* d = reinterpret_cast<bf16x4_t*>(dst + 8 * j);
            d[0] = lo;
            d[1] = hi;
        }
        done = n8 * 8;
    }
    for (long long j = done + i; j < count; j += stride) dst[j] = (__bf16)src[j];
}

// dst (bf16) = src (fp32) or its transpose, both row-major with their own row pitch: brings an operand into bf16
// storage with whichever dimension contiguous the caller wants (the bf16-stored GEMM is fastest when both operands
// are contiguous along k).  32 x 32 tiles through LDS so that reads and writes are both along rows.
__global__ void __launch_bounds__(256) convert_f32_to_bf16_2d_kernel(const float* __restrict__ src, long long ld_src,
                                                                     int rows, int cols, int transpose,
                                                                     __bf16* __restrict__ dst, long long ld_dst) {
    __shared__ float t[32][33];
    const int tx = threadIdx.x & 31, ty = threadIdx.x >> 5;
    const int r0 = blockIdx.y * 32, c0 = blockIdx.x * 32;
#pragma unroll
    for (int k = 0; k < 4; ++k) {
        const int r = r0 + ty + 8 * k, c = c0 + tx;
        if (r < rows && c < cols) t[ty + 8 * k][tx] = src[(long long)r * ld_src + c];
    }
    __syncthreads();
#pragma unroll
    for (int k = 0; k < 4; ++k) {
        if (transpose) {
            const int c = c0 + ty + 8 * k, r = r0 + tx;
            if (r < rows && c < cols) dst[(long long)c * ld_dst + r] = (__bf16)t[tx][ty + 8 * k];
        } else {
            const int r = r0 + ty + 8 * k, c = c0 + tx;
            if (r < rows && c < cols) dst[(long long)r * ld_dst + c] = (__bf16)t[ty + 8 * k][tx];
        }
    }
}

// dst[c][r] (bf16) = src[r][c] for matrices of whole 64-row blocks whose rows start on 16-byte boundaries on both
// sides: no LDS.  A thread owns 8 rows x CW columns (CW = 4 fp32 or 8 bf16 source elements: one 16-byte load per
// row), turns them in registers and writes CW rows of the transpose, 16 bytes (8 bf16) each.  Lanes 0-7 of a
// wavefront run along the rows, lanes / 8 along the columns: a load instruction reads 128 contiguous bytes from each
// of 8 source rows per row step, a store instruction writes 128 contiguous bytes to each of 8 destination rows.
// Requirements (checked by the host): rows % 64 == 0, cols % (8 * CW) == 0, 16-byte aligned bases and row pitches.
typedef unsigned short u16x8 __attribute__((ext_vector_type(8)));
template <bool SRC_BF16>
__global__ void __launch_bounds__(256) transpose_to_bf16_kernel(const void* __restrict__ src, long long ld_src, int rows,
                                                                int cols, __bf16* __restrict__ dst, long long ld_dst) {
    constexpr int CW = SRC_BF16 ? 8 : 4;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const long long r0 = (long long)blockIdx.y * 64 + (lane & 7) * 8;
    const long long cw0 = ((long long)blockIdx.x * 4 + wave) * (8 * CW);  // first column of this wavefront
    if (cw0 >= cols) return;                                              // uniform over the wavefront
    const long long c0 = cw0 + (lane >> 3) * CW;
    u16x8 out[CW];
    if constexpr (SRC_BF16) {
        const unsigned short* s = static_cast<const unsigned short*>(src) + r0 * ld_src + c0;
        u16x8 v[8];
#pragma unroll
        for (int j = 0; j < 8; ++j) v[j] = *reinterpret_cast<const u16x8*>(s + j * ld_src);
#pragma unroll
        for (int i = 0; i < CW; ++i)
#pragma unroll
            for (int j = 0; j < 8; ++j) out[i][j] = v[j][i];
    } else {
        const float* s = static_cast<const float*>(src) + r0 * ld_src + c0;
        f32x4 v[8];
#pragma unroll
        for (int j = 0; j < 8; ++j) v[j] = *reinterpret_cast<const f32x4*>(s + j * ld_src);
#pragma unroll
        for (int i = 0; i < CW; ++i)
#pragma unroll
            for (int j = 0; j < 8; ++j) out[i][j] = __builtin_bit_cast(unsigned short, (__bf16)v[j][i]);
    }
#pragma unroll
    for (int i = 0; i < CW; ++i) *reinterpret_cast<u16x8*>(dst + (c0 + i) * ld_dst + r0) = out[i];
}

// dst[r][c] (bf16) = src[r][c] (fp32) for padded matrices whose rows start on 16-byte boundaries on both sides and
// hold a multiple of 8 columns: a thread rounds 8 consecutive values of a row (two 16-byte loads, one 16-byte store),
// consecutive threads walk along the row and on into the next one.
__global__ void __launch_bounds__(256) convert_rows_to_bf16_kernel(const float* __restrict__ src, long long ld_src, int rows,
                                                                   int cols, __bf16* __restrict__ dst, long long ld_dst) {
    const int chunks = cols / 8;  // per row
    const long long total = (long long)rows * chunks;
    for (long long i = (long long)blockIdx.x * 256 + threadIdx.x; i < total; i += (long long)gridDim.x * 256) {
        const long long r = i / chunks;
        const int c = (int)(i - r * chunks);
        const float* s = src + r * ld_src + 8 * c;
        const f32x4 lo = *reinterpret_cast<const f32x4*>(s);
        const f32x4 hi = *reinterpret_cast<const f32x4*>(s + 4);
        u16x8 o;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            o[j] = __builtin_bit_cast(unsigned short, (__bf16)lo[j]);
            o[4 + j] = __builtin_bit_cast(unsigned short, (__bf16)hi[j]);
        }
        *reinterpret_cast<u16x8*>(dst + r * ld_dst + 8 * c) = o;
    }
}

}  // namespace snhip
