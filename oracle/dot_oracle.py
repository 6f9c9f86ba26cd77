"""TEST INFRASTRUCTURE - not part of the product.

Only tests/, ``__graft_entry__.smoke()`` and bench.py's ``cpu_baseline`` leg may
import this module.  Nothing under sharpnet_amd/ does.

CPU restatement of the reference path behind ``Tensor.Dot`` /
``Tensor.BatchMatrixMultiplication`` and of the layer code that calls it.
The GEMM arithmetic of the reference lives in a third-party binary that is not
part of the reference tree: Intel MKL ``cblas_sgemm`` bound as ``mkl_rt.dll``
with no pinned version (Prod/Data/BlasServices.cs:44-45; README.md:22).  The
functions below restate the reference's own code around that call:

======================================  ==========================================  =======
function                                follows                                      pinned by
======================================  ==========================================  =======
dot_shapes / dot / dot_f64              Prod/Data/BlasServices.cs:10-21,             TestGpuTensor.cs:53-109 known answers, QR
                                        Prod/CPU/CpuTensor.cs:2991-3002              identity (TestCpuTensor.cs:826-863), brute force
bmm                                     Prod/CPU/CpuTensor.cs:3004-3025              looped 2-D oracle == its definition; attention
                                                                                     fixture ParallelRunWithPyTorch.cs:963-1010
sgemm_colmajor                          cuBLAS SGEMM as called at                    transposition identity against dot_f64
                                        Prod/GPU/GpuTensor.cs:1192,1218
dense_forward / dense_backward          Prod/Layers/Linear.cs:125-191                loss fixture ParallelRunWithPyTorch.cs:102-138,
                                                                                     TestNetworkPropagation.cs:36-105
activation_forward /                    Prod/CPU/CpuTensorActivationFunctions.cs     relu + its gradient: the loss fixture above (the
activation_backward                     :184-245 (tanh, relu, leaky relu, sigmoid)   ReLU sits between its two Linear layers); sigmoid:
                                                                                     stored predictions TestNetworkPropagation.cs:36-105;
                                                                                     tanh / leaky: identities tanh x = 2 s(2x) - 1,
                                                                                     leaky(x,a) = relu(x) - a relu(-x); every gradient:
                                                                                     central finite differences of the forward
dense_backward(weight_decay_alpha)      Prod/Layers/Linear.cs:168-178                linearity: dW(alpha) - dW(0) == alpha * W exactly
softmax_last_dim                        Prod/CPU/CpuTensorActivationFunctions.cs     attention loss fixture (same file :963-1010)
                                        :19-46
sdpa_forward                            Prod/Layers/ScaledDotProductAttention        same
                                        Layer.cs:46-91
softmax_last_dim_backward /             ScaledDotProductAttentionLayer.cs:111-132    central finite differences of sdpa_forward
sdpa_backward                           (softmax gradient: cuDNN definition)         (tests/test_oracle.py)
mha_forward / mha_backward              Prod/Layers/MultiheadAttention.cs:178-292    stored losses before / after 10 epochs of
                                        (head split / merge as explicit transposes)  ParallelRunWithPyTorch.cs:1013-1131, 4 cases
sgeam_colmajor / sdgmm_colmajor /       cuBLAS Sgeam / Sdgmm as called at            reference's known transposes TestCpuTensor.cs:82-100,
transpose / multiply_tensor             Prod/GPU/GpuTensor.cs:1256-1291,1380-1395;   closed form of TestCpuTensor.cs:216-241
                                        Prod/CPU/CpuTensor.cs:1060-1094              (expected[i] = a[i] * x[i / 49])
round_to_bf16                           IEEE-754 round-to-nearest-even to a          closed-form ties/neighbours and torch's CPU
                                        bfloat16 (what v_cvt_pk_bf16_f32 does);      bfloat16 cast (independent implementation)
                                        no reference counterpart (variant is new)
mkl_dot (baseline only)                 the same cblas_sgemm call the reference      compared with dot_f64 within the fp32 bound
                                        makes, through this image's own MKL
======================================  ==========================================  =======

Every function is pinned (tests/test_oracle.py); none is "parity unpinned".
"""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB = None
_f32p = ctypes.POINTER(ctypes.c_float)


def build(force=False):
    """Compile dot_oracle.c with gcc (see Makefile)."""
    so = os.path.join(_HERE, "liboracle.so")
    src = os.path.join(_HERE, "dot_oracle.c")
    if force or not os.path.exists(so) or os.path.getmtime(so) < os.path.getmtime(src):
        if force and os.path.exists(so):
            os.remove(so)
        subprocess.run(["make", "-C", _HERE, "liboracle.so"], check=True, stdout=subprocess.PIPE,
                       stderr=subprocess.STDOUT)
    return so


def _lib():
    global _LIB
    if _LIB is None:
        so = os.path.join(_HERE, "liboracle.so")
        if not os.path.exists(so):
            build()
        lib = ctypes.CDLL(so)
        i, f = ctypes.c_int, ctypes.c_float
        lib.oracle_dot.argtypes = [_f32p, i, i, i, _f32p, i, i, i, _f32p, f, f]
        lib.oracle_dot.restype = None
        lib.oracle_bmm.argtypes = [_f32p, i, i, i, _f32p, i, i, i, _f32p, i, f, f]
        lib.oracle_bmm.restype = None
        lib.oracle_sgemm_colmajor.argtypes = [i, i, i, i, i, f, _f32p, i, _f32p, i, f, _f32p, i]
        lib.oracle_sgemm_colmajor.restype = None
        _LIB = lib
    return _LIB


def _p(a):
    return a.ctypes.data_as(_f32p)


def _as2d(x):
    """Operands with >= 2 dims are read as (Shape[0], MultDim0) (CpuTensor.cs:2998, Tensor.cs:1521-1526)."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    assert x.ndim >= 2
    return x.reshape(x.shape[0], -1)


def dot_shapes(aH, aW, transposeA, bH, bW, transposeB):
    """M, N, K, lda, ldb, ldc as BlasServices.DotMkl derives them (BlasServices.cs:14-19)."""
    M = aW if transposeA else aH
    N = bH if transposeB else bW
    K = aH if transposeA else aW
    return M, N, K, aW, bW, N


def dot(a, transposeA, b, transposeB, alpha=1.0, beta=0.0, c=None):
    """C restatement (double accumulator, one rounding).  Returns a new (M, N) float32 array."""
    a2, b2 = _as2d(a), _as2d(b)
    M, N, K, _, _, _ = dot_shapes(a2.shape[0], a2.shape[1], transposeA, b2.shape[0], b2.shape[1], transposeB)
    Kb = b2.shape[1] if transposeB else b2.shape[0]
    assert K == Kb, "inner dimensions differ: %d vs %d" % (K, Kb)
    if c is None:
        assert beta == 0.0
        out = np.empty((M, N), dtype=np.float32)
    else:
        out = np.array(c, dtype=np.float32, copy=True).reshape(M, N)
    _lib().oracle_dot(_p(a2), a2.shape[0], a2.shape[1], int(transposeA), _p(b2), b2.shape[0], b2.shape[1],
                      int(transposeB), _p(out), float(alpha), float(beta))
    return out


def dot_f64(a, transposeA, b, transposeB, alpha=1.0, beta=0.0, c=None):
    """The same contract in numpy float64 (not rounded): the closed form the C code is checked against."""
    a2 = _as2d(a).astype(np.float64)
    b2 = _as2d(b).astype(np.float64)
    opa = a2.T if transposeA else a2
    opb = b2.T if transposeB else b2
    r = float(np.float32(alpha)) * (opa @ opb)
    if beta != 0.0:
        r = r + float(np.float32(beta)) * np.asarray(c, dtype=np.float64).reshape(r.shape)
    return r


def bmm(a3, transposeA, b3, transposeB, alpha=1.0, beta=0.0, c3=None):
    """CpuTensor.BatchMatrixMultiplication (CpuTensor.cs:3004-3025): serial loop of Dot over Shape[0]."""
    a3 = np.ascontiguousarray(a3, dtype=np.float32)
    b3 = np.ascontiguousarray(b3, dtype=np.float32)
    assert a3.ndim == 3 and b3.ndim == 3 and a3.shape[0] == b3.shape[0]
    batch, aH, aW = a3.shape
    _, bH, bW = b3.shape
    M, N, _, _, _, _ = dot_shapes(aH, aW, transposeA, bH, bW, transposeB)
    if c3 is None:
        assert beta == 0.0
        out = np.empty((batch, M, N), dtype=np.float32)
    else:
        out = np.array(c3, dtype=np.float32, copy=True).reshape(batch, M, N)
    _lib().oracle_bmm(_p(a3), aH, aW, int(transposeA), _p(b3), bH, bW, int(transposeB), _p(out), batch,
                      float(alpha), float(beta))
    return out


def sgemm_colmajor(transa, transb, m, n, k, alpha, A, lda, B, ldb, beta, C, ldc):
    """Column-major SGEMM on flat float32 buffers; returns the updated copy of C."""
    A = np.ascontiguousarray(A, dtype=np.float32).reshape(-1)
    B = np.ascontiguousarray(B, dtype=np.float32).reshape(-1)
    out = np.array(C, dtype=np.float32, copy=True).reshape(-1)
    _lib().oracle_sgemm_colmajor(int(transa), int(transb), m, n, k, float(alpha), _p(A), lda, _p(B), ldb, float(beta),
                                 _p(out), ldc)
    return out


def sgeam_colmajor(transa, transb, m, n, alpha, A, lda, beta, B, ldb, C, ldc):
    """Column-major C (m x n) = alpha * op(A) + beta * op(B) on flat float32 buffers (cublasSgeam); returns the
    updated copy of C.  An operand whose scalar is zero is not read."""
    out = np.array(C, dtype=np.float32).copy()

    def op(buf, ld, trans):
        buf = np.asarray(buf, dtype=np.float32)
        if trans:       # stored n x m column-major: element (i, j) of op at j + i * ld
            return np.array([[buf[j + i * ld] for j in range(n)] for i in range(m)], dtype=np.float64).reshape(m, n)
        return np.array([[buf[i + j * ld] for j in range(n)] for i in range(m)], dtype=np.float64).reshape(m, n)
    acc = np.zeros((m, n), dtype=np.float64)
    if alpha != 0:
        acc += np.float32(alpha) * op(A, lda, transa)
    if beta != 0:
        acc += np.float32(beta) * op(B, ldb, transb)
    for j in range(n):
        for i in range(m):
            out[i + j * ldc] = np.float32(acc[i, j])
    return out


def sdgmm_colmajor(right, m, n, A, lda, x, incx, C, ldc):
    """Column-major C (m x n) = A . diag(x) (right) or diag(x) . A (left) (cublasSdgmm); returns the updated copy of C."""
    A = np.asarray(A, dtype=np.float32)
    x = np.asarray(x, dtype=np.float32)
    out = np.array(C, dtype=np.float32).copy()
    for j in range(n):
        for i in range(m):
            out[i + j * ldc] = np.float32(A[i + j * lda] * x[(j if right else i) * incx])
    return out


def transpose(a2d):
    """Tensor.Transpose as the GPU path performs it (GpuTensor.cs:1256-1291): Sgeam(T, N, M, N, 1, this, lda = N, 0, -,
    ldb = M, transposed, ldc = M) on the row-major buffers."""
    a2d = np.asarray(a2d, dtype=np.float32)
    M, N = a2d.shape
    out = sgeam_colmajor(True, False, M, N, 1.0, a2d.reshape(-1), N, 0.0, None, M, np.zeros(M * N, np.float32), M)
    return out.reshape(N, M)


def multiply_tensor(a, diagonal):
    """Tensor.MultiplyTensor as the GPU path performs it (GpuTensor.cs:1380-1395): Sdgmm(RIGHT, m = Count / n,
    n = diagonal.Count, a, lda = m, diagonal, 1, c, ldc = m)."""
    a = np.asarray(a, dtype=np.float32)
    d = np.asarray(diagonal, dtype=np.float32).reshape(-1)
    n = d.size
    m = a.size // n
    return sdgmm_colmajor(True, m, n, a.reshape(-1), m, d, 1, np.zeros(a.size, np.float32), m).reshape(a.shape)


def round_to_bf16(x):
    """float32 -> nearest bfloat16 (ties to even), returned as float32.  NaN stays NaN."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    u = x.view(np.uint32).astype(np.uint64)
    rounded = ((u + 0x7FFF + ((u >> 16) & 1)) & 0xFFFF0000).astype(np.uint32)
    out = rounded.view(np.float32).reshape(x.shape).copy()
    nan = np.isnan(x)
    out[nan] = x[nan]
    return out


def tolerance(K, a, b):
    """fp32 parity bound: 1e-4 * sqrt(K) * max|a| * max|b| (at least one ulp-scale floor for empty K)."""
    amax = float(np.max(np.abs(a))) if np.size(a) else 0.0
    bmax = float(np.max(np.abs(b))) if np.size(b) else 0.0
    return 1e-4 * np.sqrt(max(K, 1)) * amax * bmax


# ---------------------------------------------------------------------------
# Layer-level restatements (callers of Dot)
# ---------------------------------------------------------------------------

def dense_forward(x, weights, bias=None, flatten_last=False):
    """Linear.DenseForwardPropagation (Linear.cs:125-132): y2D = x2D . W^T, then y2D[n,:] += bias."""
    x = np.asarray(x, dtype=np.float32)
    x2 = x.reshape(-1, x.shape[-1]) if flatten_last else x.reshape(x.shape[0], -1)
    y = dot(x2, False, weights, True, 1.0, 0.0)
    if bias is not None:
        y = (y + np.asarray(bias, dtype=np.float32).reshape(1, -1)).astype(np.float32)  # CpuTensor.cs:1468-1487
    return y


def activation_forward(x, mode, alpha=0.0):
    """Tensor.ActivationForward for 'relu' (max(0,x)), 'leaky_relu' (x >= 0 ? x : alpha x), 'sigmoid', 'tanh'
    (CpuTensorActivationFunctions.cs:184-245), float32 in and out."""
    x = np.asarray(x, dtype=np.float32)
    if mode in (None, "identity"):
        return x.copy()
    if mode == "relu":
        return np.maximum(x, np.float32(0))
    if mode == "leaky_relu":
        return np.where(x >= 0, x, np.float32(alpha) * x).astype(np.float32)
    if mode == "sigmoid":
        return (1.0 / (1.0 + np.exp(-x.astype(np.float64)))).astype(np.float32)
    if mode == "tanh":
        return np.tanh(x.astype(np.float64)).astype(np.float32)
    raise ValueError(mode)


def activation_backward(y, dy, mode, alpha=0.0):
    """dx from the OUTPUT y of the activation and dy, as the reference's CPU gradients are written
    (ReluGradient :202-206 y > 0, LeakyReluGradient :214-219 y >= 0 ? dy : alpha dy, SigmoidGradient :240-244
    dy y (1 - y), TanhGradient :190-194 dy (1 - y^2))."""
    y = np.asarray(y, dtype=np.float32)
    dy = np.asarray(dy, dtype=np.float32)
    if mode in (None, "identity"):
        return dy.copy()
    if mode == "relu":
        return np.where(y > 0, dy, np.float32(0)).astype(np.float32)
    if mode == "leaky_relu":
        return np.where(y >= 0, dy, np.float32(alpha) * dy).astype(np.float32)
    if mode == "sigmoid":
        return (dy * y * (np.float32(1) - y)).astype(np.float32)
    if mode == "tanh":
        return (dy * (np.float32(1) - y * y)).astype(np.float32)
    raise ValueError(mode)


def dense_backward(x, dy, weights, multiplier=1.0, prev_is_input=False, flatten_last=False, weight_decay_alpha=0.0):
    """Linear.DenseBackwardPropagation (Linear.cs:142-191).

    Returns (dW, db, dx): dW = multiplier * dy^T . x (:158) + weight_decay_alpha * W (:168-178, alpha as computed
    there: k * batch * weight_decay), db = column sums of dy (:164), dx = dy . W (:190) or None when the previous
    layer is the input layer (:184-187).
    """
    x = np.asarray(x, dtype=np.float32)
    dy = np.asarray(dy, dtype=np.float32)
    x2 = x.reshape(-1, x.shape[-1]) if flatten_last else x.reshape(x.shape[0], -1)
    dy2 = dy.reshape(-1, dy.shape[-1]) if flatten_last else dy.reshape(dy.shape[0], -1)
    dW = dot(dy2, True, x2, False, multiplier, 0.0)
    if weight_decay_alpha:
        dW = (dW + np.float32(weight_decay_alpha) * np.asarray(weights, dtype=np.float32)).astype(np.float32)
    db = dy2.astype(np.float64).sum(axis=0).astype(np.float32)
    dx = None if prev_is_input else dot(dy2, False, weights, False, 1.0, 0.0)
    return dW, db, dx


def softmax_last_dim(x):
    """Max-subtracted softmax over the last dimension in float32 (CpuTensorActivationFunctions.cs:19-46)."""
    x = np.asarray(x, dtype=np.float32)
    m = x.max(axis=-1, keepdims=True)
    e = np.exp((x - m).astype(np.float32)).astype(np.float32)
    return (e / e.sum(axis=-1, keepdims=True, dtype=np.float32)).astype(np.float32)


def sdpa_forward(Q, K, V, use_scale=True, is_causal=False):
    """ScaledDotProductAttentionForwardPropagation (ScaledDotProductAttentionLayer.cs:46-91).

    Q, K, V: (batch, T, d).  scores = scaling * Q.K^T (:71), entries above the main diagonal set to
    -1e12 when causal (:73-76), weights = softmax over the last dim (:81), y = weights . V (:85).
    Returns (y, weights).
    """
    d = Q.shape[-1]
    scaling = 1.0 / np.sqrt(np.float32(d)) if use_scale else 1.0
    scores = bmm(Q, False, K, True, float(scaling), 0.0)
    if is_causal:
        T1, T2 = scores.shape[1], scores.shape[2]
        mask = np.triu(np.ones((T1, T2), dtype=bool), k=1)
        scores[:, mask] = np.float32(-1e12)
    weights = softmax_last_dim(scores)
    y = bmm(weights, False, V, False, 1.0, 0.0)
    return y, weights


def softmax_last_dim_backward(y, dy):
    """Softmax gradient over the last dimension as the reference's GPU path obtains it from cuDNN
    (ActivationBackward(SOFTMAX_LAST_DIMENSION), ScaledDotProductAttentionLayer.cs:125):
    dx = y * (dy - sum_j dy_j y_j).  (The reference's CPU helper, CpuTensorActivationFunctions.cs:109-121,
    is a loss-specific shortcut and is not the Jacobian; this function is pinned by finite differences.)"""
    y = np.asarray(y, dtype=np.float64)
    dy = np.asarray(dy, dtype=np.float64)
    s = np.sum(dy * y, axis=-1, keepdims=True)
    return (y * (dy - s)).astype(np.float32)


def sdpa_backward(Q, K, V, dy, weights, use_scale=True):
    """ScaledDotProductAttentionBackwardPropagation (ScaledDotProductAttentionLayer.cs:111-132).
    Returns (dQ, dK, dV)."""
    d = V.shape[-1]
    scaling = 1.0 / np.sqrt(np.float32(d)) if use_scale else 1.0
    dV = bmm(weights, True, dy, False, 1.0, 0.0)                       # :117
    dW = bmm(dy, False, V, True, float(scaling), 0.0)                  # :123
    dS = softmax_last_dim_backward(weights, dW)                        # :125
    dQ = bmm(dS, False, K, False, 1.0, 0.0)                            # :127
    dK = bmm(dS, True, Q, False, 1.0, 0.0)                             # :128
    return dQ, dK, dV


def _split_heads(x2d, batch, steps, heads, dim):
    """(batch*steps, heads*dim) -> (batch*heads, steps, dim): Reshape + TransposeSecondAndThirdDimension
    (MultiheadAttention.cs:207-211)."""
    return np.ascontiguousarray(x2d.reshape(batch, steps, heads, dim).transpose(0, 2, 1, 3)).reshape(batch * heads, steps, dim)


def _merge_heads(x3d, batch, steps, heads, dim):
    """(batch*heads, steps, dim) -> (batch, steps, heads*dim) (MultiheadAttention.cs:228-230)."""
    return np.ascontiguousarray(x3d.reshape(batch, heads, steps, dim).transpose(0, 2, 1, 3)).reshape(batch, steps, heads * dim)


def mha_forward(Q, K, V, w_Q, w_K, w_V, w_O, num_heads, key_dim, value_dim, b_Q=None, b_K=None, b_V=None, b_O=None,
                is_causal=False, use_scale=True):
    """MultiheadAttention.ForwardPropagation (MultiheadAttention.cs:178-240).  Q, K, V: (batch, steps, embed);
    weights (out, in).  Returns (y, cache) with cache holding what BackwardPropagation reads."""
    Q, K, V = (np.asarray(t, dtype=np.float32) for t in (Q, K, V))
    batch, tq, tkv = K.shape[0], Q.shape[1], V.shape[1]
    Qh = _split_heads(dense_forward(Q, w_Q, b_Q, flatten_last=True), batch, tq, num_heads, key_dim)
    Kh = _split_heads(dense_forward(K, w_K, b_K, flatten_last=True), batch, tkv, num_heads, key_dim)
    Vh = _split_heads(dense_forward(V, w_V, b_V, flatten_last=True), batch, tkv, num_heads, value_dim)
    heads, weights = sdpa_forward(Qh, Kh, Vh, use_scale=use_scale, is_causal=is_causal)
    merged = _merge_heads(heads, batch, tkv, num_heads, value_dim)
    y = dense_forward(merged, w_O, b_O, flatten_last=True).reshape(batch, tkv, -1)
    return y, dict(Q=Q, K=K, V=V, Qh=Qh, Kh=Kh, Vh=Vh, weights=weights, merged=merged, w=(w_Q, w_K, w_V, w_O),
                   dims=(batch, tq, tkv, num_heads, key_dim, value_dim), use_scale=use_scale)


def mha_backward(dy, cache):
    """MultiheadAttention.BackwardPropagation (MultiheadAttention.cs:243-292), multiplier 1 (PyTorch / TensorFlow mode).
    Returns dict with dQ, dK, dV and (dW, db) for each of the four projections."""
    batch, tq, tkv, H, dk, dv = cache["dims"]
    w_Q, w_K, w_V, w_O = cache["w"]
    dWo, dbo, dmerged = dense_backward(cache["merged"], dy, w_O, flatten_last=True)
    d_heads = _split_heads(dmerged.reshape(batch * tkv, H * dv), batch, tkv, H, dv)
    dQh, dKh, dVh = sdpa_backward(cache["Qh"], cache["Kh"], cache["Vh"], d_heads, cache["weights"], use_scale=cache["use_scale"])
    out = {}
    for name, dh, x, w, steps, dim in (("Q", dQh, cache["Q"], w_Q, tq, dk), ("K", dKh, cache["K"], w_K, tkv, dk),
                                      ("V", dVh, cache["V"], w_V, tkv, dv)):
        dpacked = _merge_heads(dh, batch, steps, H, dim)
        dW, db, dx = dense_backward(x, dpacked, w, flatten_last=True)
        out["d" + name] = dx.reshape(x.shape)
        out["dw_" + name], out["db_" + name] = dW, db
    out["dw_O"], out["db_O"] = dWo, dbo
    return out


# ---------------------------------------------------------------------------
# CPU baseline: the reference's own CPU route, MKL cblas_sgemm RowMajor
# ---------------------------------------------------------------------------
_MKL = None


def _find_mkl():
    global _MKL
    if _MKL is not None:
        return _MKL or None
    _MKL = False
    cands = [os.environ.get("MKL_RT_PATH"), "/opt/conda/lib/libmkl_rt.so", "/opt/conda/lib/libmkl_rt.so.2",
             "/opt/conda/lib/libmkl_rt.so.1", "/usr/lib/x86_64-linux-gnu/libmkl_rt.so", "libmkl_rt.so"]
    for c in cands:
        if not c:
            continue
        try:
            lib = ctypes.CDLL(c)
            fn = lib.cblas_sgemm
            i, f = ctypes.c_int, ctypes.c_float
            fn.argtypes = [i, i, i, i, i, i, f, _f32p, i, _f32p, i, f, _f32p, i]
            fn.restype = None
            _MKL = lib
            break
        except (OSError, AttributeError):
            continue
    return _MKL or None


def mkl_available():
    return _find_mkl() is not None


def mkl_dot(a2, transposeA, b2, transposeB, out, alpha=1.0, beta=0.0):
    """The call BlasServices.DotMkl makes (BlasServices.cs:20): cblas_sgemm(RowMajor=101, 111|112, ...).

    Uses libmkl_rt from this image when it is installed, else torch's CPU matmul (MKL-backed build).
    a2, b2, out must be C-contiguous float32 2-D arrays; out is updated in place.
    """
    aH, aW = a2.shape
    bH, bW = b2.shape
    M, N, K, lda, ldb, ldc = dot_shapes(aH, aW, transposeA, bH, bW, transposeB)
    lib = _find_mkl()
    if lib is not None:
        lib.cblas_sgemm(101, 112 if transposeA else 111, 112 if transposeB else 111, M, N, K, float(alpha), _p(a2),
                        lda, _p(b2), ldb, float(beta), _p(out), ldc)
        return "libmkl_rt cblas_sgemm"
    import torch
    ta, tb, to = torch.from_numpy(a2), torch.from_numpy(b2), torch.from_numpy(out)
    opa = ta.t() if transposeA else ta
    opb = tb.t() if transposeB else tb
    with torch.backends.mkldnn.flags(enabled=False):
        if beta == 0.0:
            torch.mm(opa, opb, out=to)
            if alpha != 1.0:
                to.mul_(alpha)
        else:
            torch.addmm(to, opa, opb, beta=beta, alpha=alpha, out=to)
    return "torch.mm (MKL build)"


def mkl_bmm_serial(a3, transposeA, b3, transposeB, out3, alpha=1.0, beta=0.0):
    """CpuTensor.BatchMatrixMultiplication as the reference runs it (CpuTensor.cs:3018-3024): a serial loop over the
    matrices of the batch, one cblas_sgemm (BlasServices.cs:20) each.  a3, b3, out3: C-contiguous float32 3-D arrays."""
    n = a3.shape[0]
    assert b3.shape[0] == n and out3.shape[0] == n
    lib = _find_mkl()
    if lib is None:
        for i in range(n):
            mkl_dot(a3[i], transposeA, b3[i], transposeB, out3[i], alpha, beta)
        return "torch.mm (MKL build), serial loop"
    aH, aW = a3.shape[1:]
    bH, bW = b3.shape[1:]
    M, N, K, lda, ldb, ldc = dot_shapes(aH, aW, transposeA, bH, bW, transposeB)
    ta, tb = (112 if transposeA else 111), (112 if transposeB else 111)
    pa, pb, pc = a3.ctypes.data, b3.ctypes.data, out3.ctypes.data
    sa, sb, sc = a3.strides[0], b3.strides[0], out3.strides[0]
    fn, cast, al, be = lib.cblas_sgemm, ctypes.cast, float(alpha), float(beta)
    for i in range(n):
        fn(101, ta, tb, M, N, K, al, cast(pa + i * sa, _f32p), lda, cast(pb + i * sb, _f32p), ldb, be,
           cast(pc + i * sc, _f32p), ldc)
    return "libmkl_rt cblas_sgemm, serial loop"


def mkl_threads():
    lib = _find_mkl()
    if lib is not None:
        try:
            lib.mkl_get_max_threads.restype = ctypes.c_int
            return int(lib.mkl_get_max_threads())
        except AttributeError:
            pass
    import torch
    return torch.get_num_threads()
