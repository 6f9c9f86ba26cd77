/*
 * libsharpnet_hip - C ABI of the MI355X (gfx950) matrix-multiplication path
 * that stands in for the cuBLAS / nvcuda entry points SharpNet's GPUTensor<float>
 * binds through P/Invoke for Tensor.Dot and Tensor.BatchMatrixMultiplication.
 *
 * Conventions (chosen so the C# side needs no change beyond the DllImport name):
 *   - every function returns an int that uses the cublasStatus_t numbering of
 *     /root/reference/Prod/GPU/CublasWrapper.cs:8-20, so GPUWrapper.CheckStatus
 *     (Prod/GPU/GPUWrapper.cs:662-668) keeps working;
 *   - transpose flags use cublasOperation_t numbering, N=0 T=1 C=2
 *     (CublasWrapper.cs:22-27); C is treated as T (real data);
 *   - all matrix pointers are raw device addresses (hipMalloc, or any offset
 *     into such an allocation: only 4-byte alignment is required);
 *   - alpha / beta are read from HOST memory at call time;
 *   - calls are asynchronous on the handle's stream (the null stream unless
 *     snhip_set_stream was called) and are ordered with earlier work on it;
 *   - a handle belongs to the device that was current when it was created and
 *     must be used by one host thread at a time (GPUWrapper.cs:824-832);
 *   - when beta == 0 the destination is never read.
 */
#ifndef SHARPNET_HIP_H
#define SHARPNET_HIP_H

#include <stddef.h>

#ifdef __cplusplus
extern "C" {
#endif

#define SNHIP_STATUS_SUCCESS 0
#define SNHIP_STATUS_NOT_INITIALIZED 1
#define SNHIP_STATUS_ALLOC_FAILED 3
#define SNHIP_STATUS_INVALID_VALUE 7
#define SNHIP_STATUS_ARCH_MISMATCH 8
#define SNHIP_STATUS_MAPPING_ERROR 11
#define SNHIP_STATUS_EXECUTION_FAILED 13
#define SNHIP_STATUS_INTERNAL_ERROR 14
#define SNHIP_STATUS_NOT_SUPPORTED 15

#define SNHIP_OP_N 0
#define SNHIP_OP_T 1
#define SNHIP_OP_C 2

/* ---- handle lifetime --------------------------------------------------- */

/* Replaces cublasCreate_v2 (CublasWrapper.cs:223, called at GPUWrapper.cs:100). */
int snhip_create(void** handle);
/* Replaces cublasDestroy_v2 (CublasWrapper.cs:225). Frees the split-K workspace. */
int snhip_destroy(void* handle);
/* The handle owns one scratch buffer: split-K partial sums, partial column sums, bf16 copies of operands.
 * snhip_create reserves 64 MiB of it (as cublasCreate_v2 brings its own workspace).  Beyond that it grows on demand, and growing
 * means a stream synchronisation, hipFree and hipMalloc in the middle of a call - not allowed under HIP graph capture
 * and unwelcome in a serving loop.  snhip_reserve_workspace sizes it ahead of time (it never shrinks): after it,
 * no call whose need is at most `bytes` synchronises or allocates.  The largest need of any call is 1 GiB (the cap
 * the split-K choice observes; larger values are refused with status 7); a product of M x N x batch floats split S
 * ways needs 4 * M * N * batch * S bytes (S as reported by snhip_query_tuning).  No reference counterpart (cuBLAS
 * manages its own workspace; cublasSetWorkspace is not bound by the reference). */
int snhip_reserve_workspace(void* handle, size_t bytes);
int snhip_get_workspace_size(void* handle, size_t* bytes);
/* No counterpart is bound by the reference (it never calls cublasSetStream, so
 * GEMMs run on the legacy default stream); offered for callers with their own
 * hipStream_t.  stream == NULL selects the null stream again. */
int snhip_set_stream(void* handle, void* stream);
/* Replaces cublasGetVersion_v2 (CublasWrapper.cs:250): major*10000+minor*100+patch. */
int snhip_get_version(void* handle, int* version);

/* ---- cuBLAS-shaped GEMM (column-major semantics) ------------------------- */

/* Replaces cublasSgemm_v2 (CublasWrapper.cs:229), call site GpuTensor.cs:1218.
 * Column-major: C(m x n, ldc) = alpha * op(A) * op(B) + beta * C. */
int snhip_sgemm(void* handle, int transa, int transb, int m, int n, int k, const float* alpha, const void* A, int lda,
                const void* B, int ldb, const float* beta, void* C, int ldc);

/* Replaces cublasSgemmStridedBatched (CublasWrapper.cs:231-244), call site
 * GpuTensor.cs:1192.  Strides are element counts (C# long). */
int snhip_sgemm_strided_batched(void* handle, int transa, int transb, int m, int n, int k, const float* alpha,
                                const void* A, int lda, long long strideA, const void* B, int ldb, long long strideB,
                                const float* beta, void* C, int ldc, long long strideC, int batchCount);

/* ---- row-major entry points (parameter list of BlasServices.DotMkl) ------ */

/* Same parameters as BlasServices.DotMkl (Prod/Data/BlasServices.cs:10):
 * A is aH x aW, B is bH x bW, both row-major and dense; M,N,K and the leading
 * dimensions are derived exactly as lines 14-19 do; C is M x N with ldc = N.
 * transposeA / transposeB are 0 or 1. */
int snhip_dot(void* handle, const float* A, int aH, int aW, int transposeA, const float* B, int bH, int bW,
              int transposeB, float* C, float alpha, float beta);

/* snhip_dot for callers that cannot allocate device memory: code under HIP graph capture, tight serving loops,
 * harnesses that forbid hipMalloc.  No counterpart in the reference.  Same arguments, same kernels, same choice
 * of tile configuration and split-K factor, bit-identical results; the difference is where split-K partial sums
 * go: into a fixed array of snhip_static_scratch_bytes() (32 MiB) that is part of the library's code object on
 * every GPU, instead of the handle's lazily grown workspace.  The call never allocates, frees or synchronises.
 * A split-K factor the library chose by itself is halved until the partial sums fit the array (down to no split):
 * results are then within the same bound but bit-identical to snhip_dot's only while the factor is unchanged
 * (snhip_get_last_tuning reports it).  A factor forced with snhip_set_tuning whose partial sums need more than the
 * array holds is refused with status 15 (NOT_SUPPORTED) before anything is launched; snhip_get_last_error_message
 * then says how many bytes were needed.  Products that run without split-K use no scratch and are never refused.  All handles of one GPU share that GPU's array: calls that
 * overlap in time on one GPU (two handles on two streams) race on it. */
int snhip_dot_noalloc(void* handle, const float* A, int aH, int aW, int transposeA, const float* B, int bH, int bW,
                      int transposeB, float* C, float alpha, float beta);
/* Size in bytes of the static scratch array (returns the size, not a status). */
int snhip_static_scratch_bytes(void);
/* Copies the detail text of the handle's most recent product call into buffer as a NUL-terminated string of at
 * most capacity bytes: empty unless that call was refused with more to say than its status code (every product call
 * clears the text on entry, so it never describes an older call). */
int snhip_get_last_error_message(void* handle, char* buffer, int capacity);

/* snhip_dot followed by C[m][n] += bias[n], in one kernel.  Replaces the pair
 * Dot + BroadcastAddVectorToOutput of Linear.DenseForwardPropagation
 * (Prod/Layers/Linear.cs:130-131; GPU bias add at GpuTensor.cs:633-644).
 * bias may be NULL. */
int snhip_dot_bias(void* handle, const float* A, int aH, int aW, int transposeA, const float* B, int bH, int bW,
                   int transposeB, float* C, float alpha, float beta, const float* bias);

/* Row-major strided batch: for i in [0,batch): C_i = alpha op(A_i) op(B_i) + beta C_i
 * with X_i = X + i*strideX.  Parameters as CpuTensor.BatchMatrixMultiplication
 * derives them (Prod/CPU/CpuTensor.cs:3004-3025): aH=Shape[1], aW=MultDim1,
 * stride=MultDim0. */
int snhip_bmm(void* handle, const float* A, int aH, int aW, int transposeA, long long strideA, const float* B, int bH,
              int bW, int transposeB, long long strideB, float* C, long long strideC, int batch, float alpha,
              float beta);

/* General row-major form with explicit leading dimensions (views / slices,
 * e.g. attention heads addressed in place).  op(A) is M x K, op(B) is K x N. */
int snhip_gemm_rm(void* handle, int transposeA, int transposeB, int M, int N, int K, float alpha, const float* A,
                  int lda, long long strideA, const float* B, int ldb, long long strideB, float beta, float* C,
                  int ldc, long long strideC, int batch, const float* bias);

/* ---- the other two cuBLAS entry points the reference binds -------------------- */
/* Column-major C (m x n) = alpha * op(A) + beta * op(B): argument for argument cublasSgeam
 * (Prod/GPU/CublasWrapper.cs:250), which the reference calls with transa = T, beta = 0, B = NULL as its 2-D transpose
 * (Prod/GPU/GpuTensor.cs:1256-1291).  An operand whose scalar is zero is not read and may be NULL.  In-place
 * transposition (C == A with transa) is not supported (status 15). */
int snhip_sgeam(void* handle, int transa, int transb, int m, int n, const float* alpha, const float* A, int lda,
                const float* beta, const float* B, int ldb, float* C, int ldc);
/* Column-major C (m x n) = A * diag(x) (mode = SNHIP_SIDE_RIGHT, x has n entries) or diag(x) * A (SNHIP_SIDE_LEFT, m
 * entries): cublasSdgmm (CublasWrapper.cs:246) with cublasSideMode_t's numbering, the reference's Tensor.MultiplyTensor
 * (GpuTensor.cs:1380-1395).  C may be A. */
#define SNHIP_SIDE_LEFT 0
#define SNHIP_SIDE_RIGHT 1
int snhip_sdgmm(void* handle, int mode, int m, int n, const float* A, int lda, const float* x, int incx, float* C,
                int ldc);

/* ---- fused Linear-layer forms ---------------------------------------------- */
/* Element-wise functions the GEMM epilogue can apply; the reference runs them as the ActivationLayer that follows
 * a Linear layer (cudnnActivationMode_t RELU / LEAKY_RELU / SIGMOID / TANH, Prod/GPU/CudnnWrapper.cs:267-281;
 * definitions Prod/CPU/CpuTensorActivationFunctions.cs:184-245). */
#define SNHIP_ACT_NONE 0
#define SNHIP_ACT_RELU 1
#define SNHIP_ACT_LEAKY_RELU 2 /* activation_param = slope for x < 0 */
#define SNHIP_ACT_SIGMOID 3
#define SNHIP_ACT_TANH 4

/* One launch, everything optional beyond the product itself (row-major, strided batch of `batch` matrices):
 *     C[z] = act(alpha * op(A[z]) . op(B[z]) + bias[col] + beta * C[z] + gamma * D[z])
 *     colsum[z][m] = sum_k op(A[z])[m][k]                       (transA = 1 only)
 * Matrix z of operand X sits at X + (z / batch_inner) * strideX_outer + (z % batch_inner) * strideX; batch_inner = 0
 * means a single level (strideX only).  The two levels let the heads of a (batch, time, heads * dim) activation be
 * multiplied in place (lda = heads * dim, strideX = dim, strideX_outer = time * heads * dim), which replaces the
 * reference's TransposeSecondAndThirdDimension copies (Prod/Layers/MultiheadAttention.cs:207-227).
 * gamma * D is the weight-decay term of Prod/Layers/Linear.cs:168-178; colsum is Compute_BiasGradient_from_dy
 * (Linear.cs:160-165) taken from the dy tiles the dW product reads anyway.
 * Zero-initialise the struct, set struct_size = sizeof(snhip_gemm_desc), then fill what is needed. */
typedef struct snhip_gemm_desc {
    int struct_size;
    int transA, transB;
    int M, N, K;
    float alpha, beta;
    const float* A;
    const float* B;
    float* C;
    int lda, ldb, ldc;
    int batch;       /* number of matrices (>= 1) */
    int batch_inner; /* 0, or the number of matrices per outer step (must divide batch) */
    long long strideA, strideB, strideC;                   /* elements */
    long long strideA_outer, strideB_outer, strideC_outer; /* elements; used when 0 < batch_inner < batch */
    const float* bias; /* length N, or NULL */
    const float* D;    /* M x N addend with row pitch ldd, or NULL */
    int ldd;
    long long strideD, strideD_outer;
    float gamma;
    int activation; /* SNHIP_ACT_* */
    float activation_param;
    float* colsum; /* [batch][M], or NULL */
    int math;      /* -1: the handle's math mode, else SNHIP_MATH_* */
} snhip_gemm_desc;
int snhip_gemm_ex(void* handle, const snhip_gemm_desc* desc);
/* sizeof(snhip_gemm_desc) as this library was built: lets a binding check its own struct layout (returns the size,
 * not a status). */
int snhip_sizeof_gemm_desc(void);

/* y[rows x out] = act(x[rows x in] . W^T + bias), W stored (out, in): Linear.DenseForwardPropagation
 * (Prod/Layers/Linear.cs:125-132) with the following ActivationLayer folded in (SNHIP_ACT_NONE for none). */
int snhip_dense_forward(void* handle, float* y, const float* x, const float* weights, const float* bias, int rows,
                        int in_features, int out_features, int activation, float activation_param);

/* Linear.DenseBackwardPropagation (Prod/Layers/Linear.cs:143-191) in at most two launches - one when dW and dx are
 * both a handful of 32 x 32 tiles (a layer on a small batch, e.g. 128 x 784 -> 256: the two products and the bias
 * gradient then share one grid; not while a tile configuration is forced with snhip_set_tuning):
 *   weight_gradients = multiplier * dy^T . x + weight_decay_alpha * weights   (Linear.cs:151-158,168-178)
 *   bias_gradients   = column sums of dy, or NULL to skip                    (Linear.cs:160-165)
 *   dx               = dy . weights, or NULL when the previous layer is the input (Linear.cs:184-190)
 * multiplier is 1/batch or 1 by compatibility mode; weight_decay_alpha = k * batch * weight_decay (0: none). */
int snhip_dense_backward(void* handle, float* dx, float* weight_gradients, float* bias_gradients, const float* x,
                         const float* dy, const float* weights, int rows, int in_features, int out_features,
                         float multiplier, float weight_decay_alpha);
/* The same with the weight decay the reference applies to the bias gradient in its PyTorch compatibility mode
 * (Linear.cs:178-181):  bias_gradients += bias_decay_alpha * bias  (bias of length out_features; ignored when
 * bias_decay_alpha is 0 or bias_gradients is NULL).  In the one-launch form this rides in the column-sum workgroups. */
int snhip_dense_backward_ex(void* handle, float* dx, float* weight_gradients, float* bias_gradients, const float* x,
                            const float* dy, const float* weights, int rows, int in_features, int out_features,
                            float multiplier, float weight_decay_alpha, const float* bias, float bias_decay_alpha);

/* y = act(x) and dx = dy * act'(x) expressed through y, element-wise over n floats (in place allowed):
 * Tensor.ActivationForward / ActivationBackward for the modes above (Prod/GPU/GpuTensor.cs ActivationForward,
 * Prod/CPU/CpuTensorActivationFunctions.cs:184-245). */
int snhip_activation_forward(void* handle, int activation, float activation_param, const float* x, float* y,
                             long long n);
int snhip_activation_backward(void* handle, int activation, float activation_param, const float* y, const float* dy,
                              float* dx, long long n);

/* ---- scaled-dot-product attention forward in one launch ------------------------ */
/* O[z] = softmax(scale * Q[z] . K[z]^T, causal mask -1e12 above the diagonal) . V[z] for z in [0, batch): what
 * ScaledDotProductAttentionLayer.ScaledDotProductAttentionForwardPropagation (Prod/Layers/
 * ScaledDotProductAttentionLayer.cs:46-91) computes with two BatchMatrixMultiplication calls, a mask and a softmax
 * pass, here without the (batch, Tq, Tk) scores ever being stored.  `weights` ([batch][Tq][Tk], contiguous) receives the
 * softmax output the reference keeps for its backward pass (:87-90); NULL skips it (inference).
 * Q is Tq x dk, K is Tk x dk, V is Tk x dv, O is Tq x dv, each with its own row pitch and two-level batch strides as in
 * snhip_gemm_desc, so heads can be read from and written to a (batch, steps, heads * dim) activation in place.
 * Supported: any Tk with dk, dv <= 64 (beyond 256 keys: dk and dv multiples of 4; the keys are then walked in blocks
 * of 256 in two passes, row maximum and sum first, so the stored weights are final when they are written; without
 * `weights` the output may come from a single pass with a running maximum, which rounds differently), or
 * Tk <= 128 with dk, dv <= 128; anything else returns status 15 (NOT_SUPPORTED) and the caller issues the reference's
 * sequence of calls instead.  On a handle in the bf16-input math mode the two products use bf16 MFMAs where a kernel
 * for them exists (head dimension exactly 64; beyond 256 keys: a multiple of 4 keys), fp32 MFMAs otherwise. */
typedef struct snhip_attention_desc {
    int struct_size;
    int batch, batch_inner; /* matrices; batch_inner as in snhip_gemm_desc (0: single level) */
    int Tq, Tk, dk, dv;
    float scale; /* 1/sqrt(dk) with use_scale, else 1 */
    int causal;  /* 0 / 1 */
    const float* Q;
    const float* K;
    const float* V;
    float* O;
    float* weights; /* or NULL */
    int ldq, ldk, ldv, ldo;
    long long strideQ, strideK, strideV, strideO;                             /* elements */
    long long strideQ_outer, strideK_outer, strideV_outer, strideO_outer;     /* used when 0 < batch_inner < batch */
} snhip_attention_desc;
int snhip_attention_forward(void* handle, const snhip_attention_desc* desc);
int snhip_sizeof_attention_desc(void);

/* Backward of the above: ScaledDotProductAttentionLayer.ScaledDotProductAttentionBackwardPropagation
 * (Prod/Layers/ScaledDotProductAttentionLayer.cs:111-132) as one call:
 *     dV = P^T . dO;   dS = softmax-gradient(P, scale * dO . V^T);   dQ = dS . K;   dK = dS^T . Q
 * `weights` is the softmax output the forward pass kept, `scores_gradients` ([batch][Tq][Tk], contiguous) is the buffer
 * the reference takes from its memory pool for dS (:121) and must be supplied.  Q / dQ, K / dK and V / dV share their
 * row pitch and batch strides; dO has its own.  `scale` is the factor the reference applies here (1/sqrt(dV.Shape[2])
 * with use_scale, :113-119).  Three launches when Tk <= 256 and both dimensions <= 64, or up to 128 keys with
 * dimensions up to 128, or any multiple of 4 keys with both dimensions exactly 32 or exactly 64 and 16-byte aligned buffers (dS and
 * dQ come from one kernel); otherwise five, the reference's own sequence. */
typedef struct snhip_attention_bwd_desc {
    int struct_size;
    int batch, batch_inner;
    int Tq, Tk, dk, dv;
    float scale;
    const float* Q;
    const float* K;
    const float* V;
    const float* dO;
    const float* weights;
    float* scores_gradients;
    float* dQ;
    float* dK;
    float* dV;
    int ldq, ldk, ldv, ldo;
    long long strideQ, strideK, strideV, strideO;
    long long strideQ_outer, strideK_outer, strideV_outer, strideO_outer;
    int causal; /* 0 / 1: `weights` come from a causally masked forward call (zero above the diagonal).  A hint that
                 * never changes the result for such weights: key blocks above the diagonal are skipped and the sums
                 * over queries of dV and dK start at the first query that sees the key.  A descriptor without this
                 * field (struct_size = its offset) is accepted and means 0. */
} snhip_attention_bwd_desc;
int snhip_attention_backward(void* handle, const snhip_attention_bwd_desc* desc);
int snhip_sizeof_attention_bwd_desc(void);

/* ---- recurrent layers on the GEMM ------------------------------------------ */
/* Replace the cuDNN calls of Prod/Layers/RecurrentLayer.cs: cudnnGetRNNWeightSpaceSize (:138), cudnnGetRNNWeightParams
 * (:176), cudnnGetRNNTempSpaceSizes (:335), cudnnRNNForward (:353), cudnnRNNBackwardData_v8 (:456) and
 * cudnnRNNBackwardWeights_v8 (:485); bindings at Prod/GPU/CudnnWrapper.cs:1038-1125.  Same cell formulas as cuDNN's
 * CUDNN_RNN_ALGO_STANDARD with linear input, data batch-major and unpacked ((batch, steps, features),
 * Prod/GPU/GPUWrapper.cs:538), every sequence of full length.  x is (batch, steps, input_size), y and dy are
 * (batch, steps, dirs * hidden_size) with the reverse direction in the second half of a row; hx, hy, cx, cy and their
 * gradients are (dirs * num_layers, batch, hidden_size), any of them may be NULL (zeros in, nothing out).
 * Each time step is one GEMM with the recurrent matrix plus one element-wise kernel; the input projections of all
 * steps, dx and both weight gradients are one GEMM each per layer and direction.  Dropout between stacked layers
 * (training only, as in cuDNN) draws its masks from the library's own counter-based generator, see
 * snhip_rnn_set_dropout_seed below: cuDNN's stream cannot be reproduced, the semantics are the same. */
#define SNHIP_RNN_RELU 0 /* cudnnRNNMode_t, Prod/GPU/CudnnWrapper.cs:313-327 */
#define SNHIP_RNN_TANH 1
#define SNHIP_RNN_LSTM 2
#define SNHIP_RNN_GRU 3
#define SNHIP_RNN_NO_BIAS 0 /* cudnnRNNBiasMode_t, :396-410 */
#define SNHIP_RNN_SINGLE_INP_BIAS 1
#define SNHIP_RNN_DOUBLE_BIAS 2
#define SNHIP_RNN_SINGLE_REC_BIAS 3
typedef struct snhip_rnn_desc { /* the fields of Prod/Layers/RNNDescriptor.cs this path uses */
    int struct_size;            /* sizeof(snhip_rnn_desc) */
    int cell_mode, bias_mode;
    int bidirectional;          /* 0 / 1 */
    int num_layers;
    int input_size, hidden_size;
    float dropout;              /* RNNDescriptor.dropoutRate (Prod/Layers/RNNDescriptor.cs:21), in [0, 1): in training the
                                   outputs of every layer but the last are multiplied, on their way into the next layer,
                                   by a mask of zeros (probability dropout) and 1 / (1 - dropout); no effect at inference
                                   or with one layer, as in cuDNN. */
} snhip_rnn_desc;
int snhip_sizeof_rnn_desc(void);
/* Bytes of the weight space.  Layout: all matrices (pseudo-layer by pseudo-layer = layer * dirs + direction: the
 * input matrices of the gates i,f,g,o / r,z,n, then the recurrent ones, each hidden_size x inputs, row-major), then
 * the bias vectors in the same order.  The reference never assumes a layout: it asks for addresses (:176). */
int snhip_rnn_weight_space_size(const snhip_rnn_desc* desc, size_t* bytes);
/* Offsets in floats from the start of the weight space of matrix and bias `lin_layer_id` (0 .. gates-1: input side,
 * gates .. 2*gates-1: recurrent side) of `pseudo_layer`; *bias_offset = -1 when the bias mode has no such vector. */
int snhip_rnn_weight_params(const snhip_rnn_desc* desc, int pseudo_layer, int lin_layer_id, long long* matrix_offset,
                            int* rows, int* cols, long long* bias_offset);
/* Sizes of the two buffers the calls below take.  reserve (training only) carries the forward pass's gates, cell
 * states and layer outputs to the two backward calls; workspace is scratch for one call. */
int snhip_rnn_temp_space_sizes(const snhip_rnn_desc* desc, int training, int batch, int steps,
                               size_t* workspace_bytes, size_t* reserve_bytes);
int snhip_rnn_forward(void* handle, const snhip_rnn_desc* desc, int training, int batch, int steps, const float* x,
                      float* y, const float* hx, float* hy, const float* cx, float* cy, const float* weights,
                      void* workspace, size_t workspace_bytes, void* reserve, size_t reserve_bytes);
/* Dropout masks.  The reference seeds cuDNN's dropout states once with 0 and lets every call advance them
 * (GPUWrapper.DropoutDesc, Prod/GPU/GPUWrapper.cs:460-474); here a handle counts its training-mode forward calls that drop
 * units (from 0; snhip_rnn_set_dropout_seed sets the seed and resets the count) and the mask is a pure function of
 * (seed, call, boundary, element): Philox4x32-10 with key {seed & 0xffffffff, seed >> 32} and counter
 * {e / 4 (low word), e / 4 (high word), boundary, call}; element e - numbered in (step, sample, unit) order over the
 * (steps, batch, dirs * hidden) outputs of layer `boundary` - takes output word e % 4 and is dropped when
 * (word >> 8) / 2^24 < dropout.  The forward call stores seed and call number in its reserve buffer, so the backward calls
 * of a layer use the masks of that layer's own forward call whatever ran in between.
 * snhip_rnn_dropout_mask writes the mask of one boundary (0 .. num_layers - 2) of call number `call` under the handle's
 * current seed, values 0 or 1 / (1 - dropout), laid out like y: (batch, steps, dirs * hidden). */
int snhip_rnn_set_dropout_seed(void* handle, unsigned long long seed);
int snhip_rnn_get_dropout_calls(void* handle, unsigned long long* calls);
int snhip_rnn_dropout_mask(void* handle, const snhip_rnn_desc* desc, int batch, int steps, unsigned long long call,
                           int boundary, float* mask);
/* Tuning hook: 0 (default) runs a time step, forward or backward, as one launch - the product with the recurrent
 * matrix and the cell arithmetic in one kernel - whenever hidden_size is a multiple of 4 and at least 32; 1 always
 * issues the GEMM and the cell kernel separately (what other hidden sizes get).  Same results within rounding
 * (different summation order). */
int snhip_rnn_set_step_mode(void* handle, int mode);
/* dx may be NULL (first layer of a network).  Leaves the gate gradients in reserve for snhip_rnn_backward_weights. */
int snhip_rnn_backward_data(void* handle, const snhip_rnn_desc* desc, int batch, int steps, const float* y,
                            const float* dy, float* dx, const float* hx, const float* dhy, float* dhx,
                            const float* cx, const float* dcy, float* dcx, const float* weights, void* workspace,
                            size_t workspace_bytes, void* reserve, size_t reserve_bytes);
/* Adds to weight_gradients (CUDNN_WGRAD_MODE_ADD, RecurrentLayer.cs:488: the caller zeroes them first), same layout
 * as the weight space.  Must follow snhip_rnn_backward_data on the same reserve buffer. */
int snhip_rnn_backward_weights(void* handle, const snhip_rnn_desc* desc, int batch, int steps, const float* x,
                               const float* hx, const float* y, float* weight_gradients, void* workspace,
                               size_t workspace_bytes, void* reserve, size_t reserve_bytes);

/* ---- bf16-input / fp32-accumulate variant (no reference counterpart) ------ */
/* Operands stay fp32 in device memory; they are rounded to bf16 (nearest even)
 * on their way into LDS and multiplied with v_mfma_f32_32x32x16_bf16, products
 * accumulated in fp32, C is fp32.  Expected deviation from the fp32 result:
 * <= 1e-2 * max|C|.  The reference has only the fp32 SGEMM (GpuTensor.cs:1218). */
#define SNHIP_MATH_FP32 0
#define SNHIP_MATH_BF16_INPUT 1
#define SNHIP_MATH_BF16_STORED 2 /* per call only (snhip_gemm_desc.math, snhip_*_bf16_stored): A and B point at bf16 data */
/* Selects the arithmetic used by every GEMM entry point of this handle
 * (the role cublasSetMathMode plays for cuBLAS handles). Default SNHIP_MATH_FP32. */
int snhip_set_math_mode(void* handle, int mode);
/* Bytes one element of A or B takes in device memory under a math mode: 2 for SNHIP_MATH_BF16_STORED, 4 for the
 * other two, 0 for a value that is no mode (returns that size, not a status).  Strides and pitches of such operands
 * count elements, and this is the factor the library itself applies wherever it offsets an operand on the host. */
int snhip_operand_element_bytes(int math_mode);
/* snhip_dot_bias / snhip_bmm in bf16-input arithmetic regardless of the handle's mode. */
int snhip_dot_bf16(void* handle, const float* A, int aH, int aW, int transposeA, const float* B, int bH, int bW,
                   int transposeB, float* C, float alpha, float beta, const float* bias);
int snhip_bmm_bf16(void* handle, const float* A, int aH, int aW, int transposeA, long long strideA, const float* B,
                   int bH, int bW, int transposeB, long long strideB, float* C, long long strideC, int batch,
                   float alpha, float beta);

/* The same arithmetic on operands that are ALREADY bf16 in device memory (2 bytes per element: half the operand
 * bytes from HBM and, what matters more for large products, half the bytes from L2 into LDS).  A and B point at
 * bf16 data, aW / bW and the strides count bf16 elements, C and bias are fp32.  Results are bit-identical to
 * snhip_dot_bf16 / snhip_bmm_bf16 on the fp32 operands these were converted from (same rounding, same products, same
 * order of summation for a given tile configuration).  A, B must be 4-byte aligned and rows / matrices must start on
 * even element offsets (aW, bW, strides even), else status 15.  snhip_gemm_ex takes the same operands with
 * math = SNHIP_MATH_BF16_STORED (no column sum in that mode). */
int snhip_dot_bf16_stored(void* handle, const void* A, int aH, int aW, int transposeA, const void* B, int bH, int bW,
                          int transposeB, float* C, float alpha, float beta, const float* bias);
int snhip_bmm_bf16_stored(void* handle, const void* A, int aH, int aW, int transposeA, long long strideA, const void* B,
                          int bH, int bW, int transposeB, long long strideB, float* C, long long strideC, int batch,
                          float alpha, float beta, const float* bias);
/* dst[i] = bf16(src[i]) for count elements, round to nearest even: the one pass that produces such operands. */
int snhip_convert_f32_to_bf16(void* handle, const float* src, void* dst, long long count);
/* The same for a rows x cols matrix with row pitches (elements), optionally transposed on the way:
 * dst[r][c] = bf16(src[r][c]) or, with transpose != 0, dst[c][r] = bf16(src[r][c]).  The bf16-stored products run
 * fastest when both operands are contiguous along k (A not transposed, B transposed): an operand that is used many
 * times (weights) can be brought into that form once. */
int snhip_convert_f32_to_bf16_2d(void* handle, const float* src, int rows, int cols, long long ld_src, int transpose,
                                 void* dst, long long ld_dst);

/* ---- row / column helpers next to the GEMMs in Linear and attention ------- */
/* bias_gradient[c] = sum_r dy[r][c].  Replaces Tensor.Compute_BiasGradient_from_dy
 * (Prod/Layers/Linear.cs:164; GPU: cudnnConvolutionBackwardBias, GpuTensor.cs:686-701). */
int snhip_bias_gradient(void* handle, const float* dy, int rows, int cols, float* bias_gradient);
/* y[r][c] += vector[c].  Replaces Tensor.BroadcastAddVectorToOutput (Linear.cs:131; GPU:
 * cudnnAddTensor, GpuTensor.cs:633-644) for callers that do not use snhip_dot_bias. */
int snhip_broadcast_add_vector(void* handle, const float* vector, float* y, int rows, int cols);
/* y += alpha * x.  Replaces Tensor.Update_Adding_Alpha_X (weight decay, Linear.cs:168-181). */
int snhip_axpy(void* handle, long long n, float alpha, const float* x, float* y);
/* y = softmax(x) over the last dimension of a (rows, cols) view, max-subtracted fp32.  Replaces
 * ActivationForward(SOFTMAX_LAST_DIMENSION) between the two attention products
 * (Prod/Layers/ScaledDotProductAttentionLayer.cs:81; CPU: CpuTensorActivationFunctions.cs:19-46).
 * x and y may be the same buffer. */
int snhip_softmax_last_dim(void* handle, const float* x, float* y, long long rows, int cols);
/* dx = y * (dy - sum_j dy_j y_j) per row, the softmax gradient the reference's GPU path gets from
 * cuDNN (ScaledDotProductAttentionLayer.cs:125).  dx may alias dy. */
int snhip_softmax_last_dim_backward(void* handle, const float* y, const float* dy, float* dx, long long rows, int cols);
/* x[b][r][c] = value for c > r.  Replaces Tensor.SetAllElementsAboveMainDiagonal (causal mask,
 * ScaledDotProductAttentionLayer.cs:73-76; CPU: CpuTensor.cs:3037-3052). */
int snhip_set_above_main_diagonal(void* handle, float* x, int matrices, int rows, int cols, float value);

/* dst[a][c][b][d] = src[a][b][c][d] for src of shape (d0, d1, d2, d3): Tensor.TransposeSecondAndThirdDimension
 * (Prod/CPU/CpuTensor.cs:301-322; CUDA kernel Prod/GPU/Kernels/SinglePrecision.cu:1285).  The multi-head attention
 * layer uses it to split and merge heads (Prod/Layers/MultiheadAttention.cs:207-230); with snhip_gemm_ex's two-level
 * batch those copies are not needed, this entry point serves callers that keep the reference's sequence. */
int snhip_transpose_second_and_third_dimension(void* handle, const float* src, float* dst, int d0, int d1, int d2,
                                               int d3);

/* ---- device memory / stream shims --------------------------------------- */
/* Replace the nvcuda calls GPUTensor makes: cuMemAlloc_v2 (GpuTensor.cs:41),
 * cuMemFree_v2 (:1634), cuMemsetD32 (:1583), cuMemcpyHtoDAsync (:77),
 * cuMemcpyDtoH (:1668), cuMemcpyDtoDAsync (:1499), cuStreamSynchronize
 * (Prod/GPU/StreamWrapper.cs:20). */
int snhip_malloc(void** dptr, size_t bytes);
int snhip_free(void* dptr);
int snhip_memset32(void* handle, void* dptr, unsigned int value, size_t count);
int snhip_memcpy_htod_async(void* handle, void* dst, const void* src, size_t bytes);
int snhip_memcpy_dtoh(void* handle, void* dst, const void* src, size_t bytes);
int snhip_memcpy_dtod_async(void* handle, void* dst, const void* src, size_t bytes);
int snhip_stream_synchronize(void* handle);
/* Replace cuStreamCreate(flags 0) / cuStreamDestroy_v2 (Prod/GPU/StreamWrapper.cs:14,45); the stream is
 * created at the default priority and can be given to snhip_set_stream. */
int snhip_stream_create(void** stream);
int snhip_stream_destroy(void* stream);

/* ---- measurement helpers (no reference counterpart) ---------------------- */
/* hipEvent wrappers recording on the handle's stream, for timing launches. */
int snhip_event_create(void** event);
int snhip_event_destroy(void* event);
int snhip_event_record(void* handle, void* event);
int snhip_event_elapsed_ms(void* start, void* stop, float* ms); /* waits for stop */

/* Plain copy kernel of `count` floats on the handle's stream: the known-size
 * launch that rocprof traffic counters (FETCH_SIZE / WRITE_SIZE) are scaled by. */
int snhip_copy_f32(void* handle, void* dst, const void* src, long long count);

/* Device facts: info[0]=compute units, [1]=max engine clock kHz, [2]=memory
 * clock kHz, [3]=memory bus width bits, [4]=LDS bytes per workgroup (opt-in max),
 * [5]=gfx architecture number (950 for MI355X). */
int snhip_device_info(void* handle, int info[6]);

/* Tuning hooks: force the tile configuration / split-K factor used by the next
 * calls on this handle (-1 / 0 = automatic), and read back what the last GEMM
 * call selected.  config ids index the table in sharpnet_hip.hip. */
int snhip_set_tuning(void* handle, int config, int splitk);
int snhip_get_last_tuning(void* handle, int* config, int* splitk);
/* What the automatic choice would be for a row-major M x N x K product of `batch` matrices (no launch, no
 * device access).  handle may be NULL: the model then assumes an MI355X (256 CUs) and no overrides.  The answer is
 * the tiled kernels' cost model; whether the K-split kernel (kind 2) takes a small product over also depends on the
 * operands' alignment, which this call does not see. */
int snhip_query_tuning(void* handle, int m, int n, int k, int batch, int math_mode, int* config, int* splitk);
/* How split-K partial sums are added: 0 = automatic (currently always a second kernel, the faster
 * choice on MI355X), 1 = a second kernel, 2 = in the GEMM kernel by the last workgroup to arrive for
 * its tile.  The order of summation is fixed in both, so results are run-to-run identical either way. */
int snhip_set_splitk_mode(void* handle, int mode);
int snhip_config_count(void);
/* desc[0..5] = BM, BN, BK, threads, dynamic LDS bytes, kind (0 fp32 tiled kernel, 1 bf16-input kernel, 2 fp32 kernel
 * with 32 x 32 tiles and K split over the wavefronts of a workgroup: chosen by itself for products with few output
 * tiles, never part of a split-K launch, used only when the operands can be read in 16-byte pieces; 3 fp32 kernel
 * with persistent workgroups and 32-wide k panels: chosen by itself for strided batches of small matrices with a
 * short K, never part of a split-K launch; 4 tiled kernel for operands stored as bf16 (SNHIP_MATH_BF16_STORED);
 * 5 / 6 the persistent kernel of kind 3 with bf16 arithmetic on fp32-stored / bf16-stored operands; 7 the kernel
 * for bf16-stored operands that are both contiguous along k (A plain, B transposed) and whole 256 x 256 x 32 tiles,
 * fed by global -> LDS direct loads: chosen by itself when the shape allows) */
int snhip_config_desc(int config, int desc[6]);

#ifdef __cplusplus
}
#endif
#endif /* SHARPNET_HIP_H */
