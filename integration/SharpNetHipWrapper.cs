// Prod/GPU/SharpNetHipWrapper.cs
using System;
using System.Runtime.InteropServices;

namespace SharpNet.GPU
{
    public static class SharpNetHipWrapper
    {
        private const string DLL_NAME = "sharpnet_hip";   // libsharpnet_hip.so on Linux

        [DllImport(DLL_NAME)] public static extern cublasStatus_t snhip_create(ref IntPtr handle);
        [DllImport(DLL_NAME)] public static extern cublasStatus_t snhip_destroy(IntPtr handle);
        [DllImport(DLL_NAME)] public static extern cublasStatus_t snhip_set_stream(IntPtr handle, IntPtr stream);
        [DllImport(DLL_NAME)] public static extern cublasStatus_t snhip_get_version(IntPtr handle, out int version);

        [DllImport(DLL_NAME)]
        public static extern cublasStatus_t snhip_sgemm(IntPtr handle, cublasOperation_t transa, cublasOperation_t transb,
            int m, int n, int k, ref float alpha, IntPtr A, int lda, IntPtr B, int ldb, ref float beta, IntPtr C, int ldc);

        [DllImport(DLL_NAME)]
        public static extern cublasStatus_t snhip_sgemm_strided_batched(IntPtr handle, cublasOperation_t transa,
            cublasOperation_t transb, int m, int n, int k, ref float alpha, IntPtr A, int lda, long strideA,
            IntPtr B, int ldb, long strideB, ref float beta, IntPtr C, int ldc, long strideC, int batchCount);

        [DllImport(DLL_NAME)]
        public static extern cublasStatus_t snhip_sgeam(IntPtr handle, cublasOperation_t transa, cublasOperation_t transb,
            int m, int n, ref float alpha, IntPtr A, int lda, ref float beta, IntPtr B, int ldb, IntPtr C, int ldc);
        [DllImport(DLL_NAME)]
        public static extern cublasStatus_t snhip_sdgmm(IntPtr handle, cublasSideMode_t mode, int m, int n, IntPtr A, int lda,
            IntPtr x, int incx, IntPtr C, int ldc);

        // row-major forms (parameter list of BlasServices.DotMkl); transposeA/B: 0 or 1
        [DllImport(DLL_NAME)]
        public static extern cublasStatus_t snhip_dot(IntPtr handle, IntPtr A, int aH, int aW, int transposeA,
            IntPtr B, int bH, int bW, int transposeB, IntPtr C, float alpha, float beta);
        // snhip_dot that never allocates (split-K partial sums in the library's static 32 MiB array); status 15 + message
        // when they would not fit
        [DllImport(DLL_NAME)]
        public static extern cublasStatus_t snhip_dot_noalloc(IntPtr handle, IntPtr A, int aH, int aW, int transposeA,
            IntPtr B, int bH, int bW, int transposeB, IntPtr C, float alpha, float beta);
        [DllImport(DLL_NAME)] public static extern int snhip_static_scratch_bytes();
        [DllImport(DLL_NAME)]
        public static extern cublasStatus_t snhip_get_last_error_message(IntPtr handle, System.Text.StringBuilder buffer, int capacity);
        [DllImport(DLL_NAME)]
        public static extern cublasStatus_t snhip_dot_bias(IntPtr handle, IntPtr A, int aH, int aW, int transposeA,
            IntPtr B, int bH, int bW, int transposeB, IntPtr C, float alpha, float beta, IntPtr bias);
        [DllImport(DLL_NAME)]
        public static extern cublasStatus_t snhip_bmm(IntPtr handle, IntPtr A, int aH, int aW, int transposeA, long strideA,
            IntPtr B, int bH, int bW, int transposeB, long strideB, IntPtr C, long strideC, int batch, float alpha, float beta);

        // split-K workspace sized once at set-up (no allocation inside later calls that fit)
        [DllImport(DLL_NAME)] public static extern cublasStatus_t snhip_reserve_workspace(IntPtr handle, UIntPtr bytes);
        [DllImport(DLL_NAME)] public static extern cublasStatus_t snhip_get_workspace_size(IntPtr handle, out UIntPtr bytes);

        // operands stored as bf16: convert once (dst: 2 bytes per element), then multiply; C, alpha, beta, bias stay fp32
        [DllImport(DLL_NAME)]
        public static extern cublasStatus_t snhip_convert_f32_to_bf16(IntPtr handle, IntPtr src, IntPtr dst, long count);
        [DllImport(DLL_NAME)]
        public static extern cublasStatus_t snhip_convert_f32_to_bf16_2d(IntPtr handle, IntPtr src, int rows, int cols,
            long ldSrc, int transpose, IntPtr dst, long ldDst);
        [DllImport(DLL_NAME)]
        public static extern cublasStatus_t snhip_dot_bf16_stored(IntPtr handle, IntPtr A, int aH, int aW, int transposeA,
            IntPtr B, int bH, int bW, int transposeB, IntPtr C, float alpha, float beta, IntPtr bias);
        [DllImport(DLL_NAME)]
        public static extern cublasStatus_t snhip_bmm_bf16_stored(IntPtr handle, IntPtr A, int aH, int aW, int transposeA,
            long strideA, IntPtr B, int bH, int bW, int transposeB, long strideB, IntPtr C, long strideC, int batch,
            float alpha, float beta, IntPtr bias);

        // bf16-input / fp32-accumulate arithmetic for every GEMM of the handle (0 = fp32, 1 = bf16 inputs)
        [DllImport(DLL_NAME)] public static extern cublasStatus_t snhip_set_math_mode(IntPtr handle, int mode);
        [DllImport(DLL_NAME)] public static extern int snhip_operand_element_bytes(int mathMode);   // 4, 4, 2 for modes 0, 1, 2
        // ... or per call, whatever the handle's mode (operands fp32 in memory)
        [DllImport(DLL_NAME)]
        public static extern cublasStatus_t snhip_dot_bf16(IntPtr handle, IntPtr A, int aH, int aW, int transposeA,
            IntPtr B, int bH, int bW, int transposeB, IntPtr C, float alpha, float beta, IntPtr bias);
        [DllImport(DLL_NAME)]
        public static extern cublasStatus_t snhip_bmm_bf16(IntPtr handle, IntPtr A, int aH, int aW, int transposeA, long strideA,
            IntPtr B, int bH, int bW, int transposeB, long strideB, IntPtr C, long strideC, int batch, float alpha, float beta);
        // which tile configuration and split-K factor the last product of the handle ran with
        [DllImport(DLL_NAME)] public static extern cublasStatus_t snhip_get_last_tuning(IntPtr handle, out int config, out int splitk);

        // helpers next to the GEMMs in Linear / ScaledDotProductAttention
        [DllImport(DLL_NAME)] public static extern cublasStatus_t snhip_bias_gradient(IntPtr handle, IntPtr dy, int rows, int cols, IntPtr biasGradient);
        [DllImport(DLL_NAME)] public static extern cublasStatus_t snhip_broadcast_add_vector(IntPtr handle, IntPtr vector, IntPtr y, int rows, int cols);
        [DllImport(DLL_NAME)] public static extern cublasStatus_t snhip_axpy(IntPtr handle, long n, float alpha, IntPtr x, IntPtr y);
        [DllImport(DLL_NAME)] public static extern cublasStatus_t snhip_softmax_last_dim(IntPtr handle, IntPtr x, IntPtr y, long rows, int cols);
        [DllImport(DLL_NAME)] public static extern cublasStatus_t snhip_softmax_last_dim_backward(IntPtr handle, IntPtr y, IntPtr dy, IntPtr dx, long rows, int cols);
        [DllImport(DLL_NAME)] public static extern cublasStatus_t snhip_set_above_main_diagonal(IntPtr handle, IntPtr x, int matrices, int rows, int cols, float value);

        [DllImport(DLL_NAME)] public static extern cublasStatus_t snhip_transpose_second_and_third_dimension(IntPtr handle, IntPtr src, IntPtr dst, int d0, int d1, int d2, int d3);

        // Linear layer in one / two launches; activation: 0 none, 1 relu, 2 leaky relu (param = slope), 3 sigmoid, 4 tanh
        [DllImport(DLL_NAME)] public static extern cublasStatus_t snhip_dense_forward(IntPtr handle, IntPtr y, IntPtr x, IntPtr weights, IntPtr bias, int rows, int inFeatures, int outFeatures, int activation, float activationParam);
        [DllImport(DLL_NAME)] public static extern cublasStatus_t snhip_dense_backward(IntPtr handle, IntPtr dx, IntPtr weightGradients, IntPtr biasGradients, IntPtr x, IntPtr dy, IntPtr weights, int rows, int inFeatures, int outFeatures, float multiplier, float weightDecayAlpha);
        // ... with the PyTorch-mode weight decay on the bias gradient (Linear.cs:178-181): biasGradients += biasDecayAlpha * bias
        [DllImport(DLL_NAME)] public static extern cublasStatus_t snhip_dense_backward_ex(IntPtr handle, IntPtr dx, IntPtr weightGradients, IntPtr biasGradients, IntPtr x, IntPtr dy, IntPtr weights, int rows, int inFeatures, int outFeatures, float multiplier, float weightDecayAlpha, IntPtr bias, float biasDecayAlpha);
        [DllImport(DLL_NAME)] public static extern cublasStatus_t snhip_activation_forward(IntPtr handle, int activation, float activationParam, IntPtr x, IntPtr y, long n);
        [DllImport(DLL_NAME)] public static extern cublasStatus_t snhip_activation_backward(IntPtr handle, int activation, float activationParam, IntPtr y, IntPtr dy, IntPtr dx, long n);

        // general descriptor form (zero the struct, set struct_size = Marshal.SizeOf<GemmDesc>(), check it once
        // against snhip_sizeof_gemm_desc())
        [StructLayout(LayoutKind.Sequential)]
        public struct GemmDesc
        {
            public int struct_size, transA, transB, M, N, K;
            public float alpha, beta;
            public IntPtr A, B, C;
            public int lda, ldb, ldc, batch, batch_inner;
            public long strideA, strideB, strideC, strideA_outer, strideB_outer, strideC_outer;
            public IntPtr bias, D;
            public int ldd;
            public long strideD, strideD_outer;
            public float gamma;
            public int activation;
            public float activation_param;
            public IntPtr colsum;
            public int math;     // -1: the handle's math mode
        }
        [StructLayout(LayoutKind.Sequential)]
        public struct AttentionDesc
        {
            public int struct_size, batch, batch_inner, Tq, Tk, dk, dv;
            public float scale;
            public int causal;
            public IntPtr Q, K, V, O, weights;
            public int ldq, ldk, ldv, ldo;
            public long strideQ, strideK, strideV, strideO, strideQ_outer, strideK_outer, strideV_outer, strideO_outer;
        }
        [DllImport(DLL_NAME)] public static extern cublasStatus_t snhip_attention_forward(IntPtr handle, ref AttentionDesc desc);
        [DllImport(DLL_NAME)] public static extern int snhip_sizeof_attention_desc();
        [StructLayout(LayoutKind.Sequential)]
        public struct AttentionBwdDesc
        {
            public int struct_size, batch, batch_inner, Tq, Tk, dk, dv;
            public float scale;
            public IntPtr Q, K, V, dO, weights, scores_gradients, dQ, dK, dV;
            public int ldq, ldk, ldv, ldo;   // dQ, dK, dV use the pitch and strides of Q, K, V
            public long strideQ, strideK, strideV, strideO, strideQ_outer, strideK_outer, strideV_outer, strideO_outer;
            public int causal;               // weights come from a causally masked forward call: lets the library skip the zeros
        }
        [DllImport(DLL_NAME)] public static extern cublasStatus_t snhip_attention_backward(IntPtr handle, ref AttentionBwdDesc desc);
        [DllImport(DLL_NAME)] public static extern int snhip_sizeof_attention_bwd_desc();
        [StructLayout(LayoutKind.Sequential)]
        public struct RnnDesc   // RNNDescriptor.cs: cellMode, biasMode, dirMode, numLayers, inputSize, hiddenSize
        {
            public int struct_size, cell_mode, bias_mode, bidirectional, num_layers, input_size, hidden_size;
            public float dropout;   // RNNDescriptor.dropoutRate: between stacked layers, in training
        }
        [DllImport(DLL_NAME)] public static extern int snhip_sizeof_rnn_desc();
        [DllImport(DLL_NAME)] public static extern cublasStatus_t snhip_rnn_weight_space_size(ref RnnDesc desc, out size_t bytes);   // size_t: the reference's own struct (Prod/GPU/size_t.cs)
        [DllImport(DLL_NAME)] public static extern cublasStatus_t snhip_rnn_weight_params(ref RnnDesc desc, int pseudoLayer, int linLayerID,
            out long matrixOffset, out int rows, out int cols, out long biasOffset);   // offsets in floats, bias -1 if absent
        [DllImport(DLL_NAME)] public static extern cublasStatus_t snhip_rnn_temp_space_sizes(ref RnnDesc desc, int training, int batch, int steps,
            out size_t workspaceBytes, out size_t reserveBytes);
        [DllImport(DLL_NAME)] public static extern cublasStatus_t snhip_rnn_forward(IntPtr handle, ref RnnDesc desc, int training, int batch, int steps,
            IntPtr x, IntPtr y, IntPtr hx, IntPtr hy, IntPtr cx, IntPtr cy, IntPtr weights, IntPtr workspace, size_t workspaceBytes,
            IntPtr reserve, size_t reserveBytes);
        [DllImport(DLL_NAME)] public static extern cublasStatus_t snhip_rnn_backward_data(IntPtr handle, ref RnnDesc desc, int batch, int steps,
            IntPtr y, IntPtr dy, IntPtr dx, IntPtr hx, IntPtr dhy, IntPtr dhx, IntPtr cx, IntPtr dcy, IntPtr dcx, IntPtr weights,
            IntPtr workspace, size_t workspaceBytes, IntPtr reserve, size_t reserveBytes);
        [DllImport(DLL_NAME)] public static extern cublasStatus_t snhip_rnn_backward_weights(IntPtr handle, ref RnnDesc desc, int batch, int steps,
            IntPtr x, IntPtr hx, IntPtr y, IntPtr weightGradients, IntPtr workspace, size_t workspaceBytes, IntPtr reserve, size_t reserveBytes);
        // dropout masks come from the library's own generator (the reference seeds cuDNN's with 0, GPUWrapper.cs:472)
        [DllImport(DLL_NAME)] public static extern cublasStatus_t snhip_rnn_set_dropout_seed(IntPtr handle, ulong seed);
        [DllImport(DLL_NAME)] public static extern cublasStatus_t snhip_rnn_get_dropout_calls(IntPtr handle, out ulong calls);
        [DllImport(DLL_NAME)] public static extern cublasStatus_t snhip_rnn_dropout_mask(IntPtr handle, ref RnnDesc desc, int batch, int steps,
            ulong call, int boundary, IntPtr mask);
        [DllImport(DLL_NAME)] public static extern cublasStatus_t snhip_gemm_ex(IntPtr handle, ref GemmDesc desc);
        [DllImport(DLL_NAME)] public static extern int snhip_sizeof_gemm_desc();

        // device memory / stream (replace the nvcuda P/Invokes used by GPUTensor)
        [DllImport(DLL_NAME)] public static extern cublasStatus_t snhip_malloc(out IntPtr dptr, UIntPtr bytes);
        [DllImport(DLL_NAME)] public static extern cublasStatus_t snhip_free(IntPtr dptr);
        [DllImport(DLL_NAME)] public static extern cublasStatus_t snhip_memset32(IntPtr handle, IntPtr dptr, uint value, UIntPtr count);
        [DllImport(DLL_NAME)] public static extern cublasStatus_t snhip_memcpy_htod_async(IntPtr handle, IntPtr dst, IntPtr src, UIntPtr bytes);
        [DllImport(DLL_NAME)] public static extern cublasStatus_t snhip_memcpy_dtoh(IntPtr handle, IntPtr dst, IntPtr src, UIntPtr bytes);
        [DllImport(DLL_NAME)] public static extern cublasStatus_t snhip_memcpy_dtod_async(IntPtr handle, IntPtr dst, IntPtr src, UIntPtr bytes);
        [DllImport(DLL_NAME)] public static extern cublasStatus_t snhip_stream_synchronize(IntPtr handle);
        [DllImport(DLL_NAME)] public static extern cublasStatus_t snhip_stream_create(out IntPtr stream);
        [DllImport(DLL_NAME)] public static extern cublasStatus_t snhip_stream_destroy(IntPtr stream);
    }
}
