"""Host mirror of ScaledDotProductAttention forward / backward
(Prod/Layers/ScaledDotProductAttentionLayer.cs:46-91, 111-132) on GPUTensor.

Q, K, V, y are (batch, time, dim) tensors; the (batch, Tq, Tv) score and weight
buffers are materialised exactly as the reference does.  Forward returns the
weights buffer (kept for backward when training).
"""
import ctypes
import math

from . import hiplib
from .gpu_tensor import GPUTensor
from .hiplib import CublasStatus, check_status

# limits of snhip_attention_forward's single-block kernels: (keys, head dimension) pairs
FUSED_ATTENTION_LIMITS = ((256, 64), (128, 128))


def fused_attention_supported(tkv, dk, dv):
    """Whether snhip_attention_forward has a kernel for the sizes (it says the same with status 15): one key block, or
    any number of keys with head dimensions that are multiples of 4 and at most 64."""
    if any(tkv <= keys and max(dk, dv) <= dim for keys, dim in FUSED_ATTENTION_LIMITS):
        return True
    return max(dk, dv) <= 64 and dk % 4 == 0 and dv % 4 == 0


def fused_attention_forward(Q, K, V, O, weights, *, batch, heads, tq, tkv, dk, dv, scale, is_causal, packed):
    """snhip_attention_forward.  packed=True: Q, K, V, O are (batch, steps, heads*dim) activations whose heads are
    addressed in place; False: contiguous (batch*heads, steps, dim) stacks.  Returns False (nothing launched) when
    the sizes are outside what the kernel handles."""
    if not fused_attention_supported(tkv, dk, dv):
        return False

    def strides(steps, dim):
        if packed:
            return heads * dim, dim, steps * heads * dim
        return dim, steps * dim, heads * steps * dim
    ldq, sq, sq2 = strides(tq, dk)
    ldk, sk, sk2 = strides(tkv, dk)
    ldv, sv, sv2 = strides(tkv, dv)
    ldo, so, so2 = strides(tq, dv)
    d = hiplib.AttentionDesc(batch=batch * heads, batch_inner=heads, Tq=tq, Tk=tkv, dk=dk, dv=dv, scale=scale,
                             causal=int(bool(is_causal)), Q=Q.Pointer, K=K.Pointer, V=V.Pointer, O=O.Pointer,
                             weights=weights.Pointer if weights is not None else None, ldq=ldq, ldk=ldk, ldv=ldv, ldo=ldo,
                             strideQ=sq, strideK=sk, strideV=sv, strideO=so, strideQ_outer=sq2, strideK_outer=sk2,
                             strideV_outer=sv2, strideO_outer=so2)
    st = Q._lib.snhip_attention_forward(Q.Wrapper.handle, ctypes.byref(d))
    if st == CublasStatus.CUBLAS_STATUS_NOT_SUPPORTED:
        return False
    check_status(st, "snhip_attention_forward")
    return True


def attention_backward(dQ, dK, dV, Q, K, V, dO, weights, scores_gradients, *, batch, heads, tq, tkv, dk, dv, scale, packed,
                       is_causal=False):
    """snhip_attention_backward: dV, dS (into scores_gradients), dQ, dK in three launches (five beyond the one-kernel
    limits).  Layout conventions as in fused_attention_forward; weights and scores_gradients are contiguous
    (batch*heads, tq, tkv) stacks.  is_causal: the weights come from a causally masked forward call (the layer's own
    flag, ScaledDotProductAttentionLayer.cs:25): the library then skips what the mask zeroed."""
    def strides(steps, dim):
        if packed:
            return heads * dim, dim, steps * heads * dim
        return dim, steps * dim, heads * steps * dim
    ldq, sq, sq2 = strides(tq, dk)
    ldk, sk, sk2 = strides(tkv, dk)
    ldv, sv, sv2 = strides(tkv, dv)
    ldo, so, so2 = strides(tq, dv)
    d = hiplib.AttentionBwdDesc(batch=batch * heads, batch_inner=heads, Tq=tq, Tk=tkv, dk=dk, dv=dv, scale=scale,
                                Q=Q.Pointer, K=K.Pointer, V=V.Pointer, dO=dO.Pointer, weights=weights.Pointer,
                                scores_gradients=scores_gradients.Pointer, dQ=dQ.Pointer, dK=dK.Pointer, dV=dV.Pointer,
                                ldq=ldq, ldk=ldk, ldv=ldv, ldo=ldo, strideQ=sq, strideK=sk, strideV=sv, strideO=so,
                                strideQ_outer=sq2, strideK_outer=sk2, strideV_outer=sv2, strideO_outer=so2,
                                causal=int(bool(is_causal)))
    check_status(Q._lib.snhip_attention_backward(Q.Wrapper.handle, ctypes.byref(d)), "snhip_attention_backward")


def ScaledDotProductAttentionForwardPropagation(Q, K, V, y, isTraining, use_scale, is_causal, fused=True):
    """fused=True runs the whole chain as one launch when the sizes allow it (any number of keys with a head dimension
    of at most 64 - beyond 256 keys a multiple of 4 -, or up to 128 keys with a head dimension of up to 128);
    otherwise, or with fused=False, the reference's four calls."""
    if V.Shape != K.Shape:
        raise ValueError("V.Shape and K.Shape must be equal, but are %s and %s" % (V.Shape, K.Shape))
    if V.Shape != y.Shape:
        raise ValueError("V.Shape and y.Shape must be equal, but are %s and %s" % (V.Shape, y.Shape))
    if Q.Shape[2] != V.Shape[2]:
        raise ValueError("queries.Shape[2] and values.Shape[2] must be equal (same embedding dim)")
    batch_size, query_time_steps, value_time_steps, embedding_dim = K.Shape[0], Q.Shape[1], V.Shape[1], K.Shape[2]
    if fused:
        weights_buffer = GPUTensor([batch_size, query_time_steps, value_time_steps], None, Q.Wrapper) if isTraining else None
        if fused_attention_forward(Q, K, V, y, weights_buffer, batch=batch_size, heads=1, tq=query_time_steps,
                                   tkv=value_time_steps, dk=embedding_dim, dv=V.Shape[2],
                                   scale=1.0 / math.sqrt(embedding_dim) if use_scale else 1.0, is_causal=is_causal,
                                   packed=False):
            return weights_buffer
        if weights_buffer is not None:
            weights_buffer.Dispose()
    scores_buffer = GPUTensor([batch_size, query_time_steps, value_time_steps], None, Q.Wrapper)
    scaling = 1.0 / math.sqrt(embedding_dim) if use_scale else 1.0
    scores_buffer.BatchMatrixMultiplication(Q, False, K, True, scaling, 0.0)              # :71
    if is_causal:
        scores_buffer.SetAllElementsAboveMainDiagonal(-1e12)                               # :73-76
    weights_buffer = GPUTensor(scores_buffer.Shape, None, Q.Wrapper)
    scores_buffer.SoftmaxLastDimension(weights_buffer)                                     # :81
    y.BatchMatrixMultiplication(weights_buffer, False, V, False, 1.0, 0.0)                 # :85
    scores_buffer.Dispose()
    if not isTraining:
        weights_buffer.Dispose()
        return None
    return weights_buffer


def ScaledDotProductAttentionBackwardPropagation(dQ, dK, dV, Q, K, V, dy, weights_buffer, use_scale, fused=True,
                                                 is_causal=False):
    """fused=True: one library call (the score gradient and dQ come out of one kernel when the sizes allow it);
    False: the reference's five calls one by one.  is_causal (the layer's flag; the reference's static method does not
    take it) only lets the fused call skip what the mask zeroed."""
    embedding_dim = dV.Shape[2]
    if fused:
        scaling = 1.0 / math.sqrt(embedding_dim) if use_scale else 1.0
        scores_gradients_buffer = GPUTensor(weights_buffer.Shape, None, Q.Wrapper)
        attention_backward(dQ, dK, dV, Q, K, V, dy, weights_buffer, scores_gradients_buffer, batch=K.Shape[0], heads=1,
                           tq=Q.Shape[1], tkv=V.Shape[1], dk=K.Shape[2], dv=V.Shape[2], scale=scaling, packed=False,
                           is_causal=is_causal)
        scores_gradients_buffer.Dispose()
        weights_buffer.Dispose()
        return
    dV.BatchMatrixMultiplication(weights_buffer, True, dy, False, 1.0, 0.0)                # :117
    scaling = 1.0 / math.sqrt(embedding_dim) if use_scale else 1.0
    scores_gradients_buffer = GPUTensor(weights_buffer.Shape, None, Q.Wrapper)
    scores_gradients_buffer.BatchMatrixMultiplication(dy, False, V, True, scaling, 0.0)    # :123
    weights_buffer.SoftmaxLastDimensionBackward(scores_gradients_buffer, scores_gradients_buffer)   # :125
    dQ.BatchMatrixMultiplication(scores_gradients_buffer, False, K, False, 1.0, 0.0)      # :127
    dK.BatchMatrixMultiplication(scores_gradients_buffer, True, Q, False, 1.0, 0.0)       # :128
    scores_gradients_buffer.Dispose()
    weights_buffer.Dispose()


# ---------------------------------------------------------------------------------------------------------------
# Multi-head attention (Prod/Layers/MultiheadAttention.cs:178-292)
# ---------------------------------------------------------------------------------------------------------------
class MultiheadAttentionState:
    """What ForwardPropagation keeps for BackwardPropagation (MultiheadAttention.cs:53-57)."""

    def __init__(self):
        self.weights_buffer = None      # (batch*heads, Tq, Tkv) softmax output
        self.Q_heads = self.K_heads = self.V_heads = None   # projections; packed (batch*T, heads*dim) when heads stay in
        self.attention_heads_T = None   # place, (batch*heads, T, dim) copies in the reference's sequence
        self.dims = None
        self.heads_in_place = True
        self.is_causal = False          # the layer's mask flag: backward may skip what it zeroed


def _heads_gemm(c, a, b, *, transA, transB, M, N, K, alpha, batch, heads, a_packed, b_packed, c_packed,
                a_steps, b_steps, c_steps, a_dim, b_dim, c_dim):
    """One product per (batch, head).  A packed operand is a (batch, steps, heads*dim) activation whose head h is the
    column block [h*dim, (h+1)*dim): leading dimension heads*dim, head stride dim, batch stride steps*heads*dim.
    An unpacked one is a contiguous (batch*heads, rows, cols) stack."""
    def strides(packed, steps, dim, rows, cols):
        if packed:
            return heads * dim, dim, steps * heads * dim
        return cols, rows * cols, heads * rows * cols
    a_rows, a_cols = (K, M) if transA else (M, K)
    b_rows, b_cols = (N, K) if transB else (K, N)
    lda, sA, sA2 = strides(a_packed, a_steps, a_dim, a_rows, a_cols)
    ldb, sB, sB2 = strides(b_packed, b_steps, b_dim, b_rows, b_cols)
    ldc, sC, sC2 = strides(c_packed, c_steps, c_dim, M, N)
    c.GemmEx(transA=int(transA), transB=int(transB), M=M, N=N, K=K, alpha=alpha, beta=0.0, A=a, lda=lda, strideA=sA,
             strideA_outer=sA2, B=b, ldb=ldb, strideB=sB, strideB_outer=sB2, ldc=ldc, strideC=sC, strideC_outer=sC2,
             batch=batch * heads, batch_inner=heads)


def MultiheadAttentionForwardPropagation(Q, K, V, y, w_Q, w_K, w_V, out_proj_weight, num_heads, key_dim, value_dim,
                                         w_Q_bias=None, w_K_bias=None, w_V_bias=None, out_proj_bias=None,
                                         isTraining=True, use_scale=True, is_causal=False, heads_in_place=True,
                                         fused_attention=True):
    """MultiheadAttention.ForwardPropagation.  heads_in_place=True multiplies the heads where the projections left
    them (two-level strided batch, no TransposeSecondAndThirdDimension copies, the attention output lands directly
    in the (batch, steps, heads*value_dim) layout the output projection reads); False issues the reference's
    sequence call by call.  Returns the state BackwardPropagation needs."""
    from . import linear
    if V.Shape != K.Shape:
        raise ValueError("V.Shape and K.Shape must be equal, but are %s and %s" % (V.Shape, K.Shape))
    if V.Shape != y.Shape:
        raise ValueError("V.Shape and y.Shape must be equal, but are %s and %s" % (V.Shape, y.Shape))
    if Q.Shape[2] != V.Shape[2]:
        raise ValueError("queries.Shape[2] and values.Shape[2] must be equal (same embedding dim)")
    if Q.Shape[1] != V.Shape[1]:
        # y has V's shape (checked above) but receives one row per query: with more queries than keys the products
        # would write past y and the attention buffers (the reference fails its BatchMatrixMultiplication shape
        # assertion at this point instead)
        raise ValueError("queries.Shape[1] and values.Shape[1] must be equal, but are %d and %d" % (Q.Shape[1], V.Shape[1]))
    w = Q.Wrapper
    batch_size, tq, tkv = K.Shape[0], Q.Shape[1], V.Shape[1]
    H, dk, dv = num_heads, key_dim, value_dim
    st = MultiheadAttentionState()
    st.dims = (batch_size, tq, tkv, H, dk, dv)
    st.heads_in_place = heads_in_place
    st.is_causal = bool(is_causal)
    Q_heads = GPUTensor([batch_size * tq, H * dk], None, w)
    K_heads = GPUTensor([batch_size * tkv, H * dk], None, w)
    V_heads = GPUTensor([batch_size * tkv, H * dv], None, w)
    linear.DenseForwardPropagation(Q_heads, Q, w_Q, w_Q_bias, True)                          # :201-202
    linear.DenseForwardPropagation(K_heads, K, w_K, w_K_bias, True)                          # :207-208
    linear.DenseForwardPropagation(V_heads, V, w_V, w_V_bias, True)                          # :213-214
    scaling = 1.0 / math.sqrt(dk) if use_scale else 1.0
    fused_done = False
    if heads_in_place and fused_attention:
        weights = GPUTensor([batch_size * H, tq, tkv], None, w)
        attention_heads_T = GPUTensor([batch_size, tkv, H * dv], None, w)
        fused_done = fused_attention_forward(Q_heads, K_heads, V_heads, attention_heads_T, weights, batch=batch_size,
                                             heads=H, tq=tq, tkv=tkv, dk=dk, dv=dv, scale=scaling, is_causal=is_causal,
                                             packed=True)
        if fused_done:
            st.Q_heads, st.K_heads, st.V_heads = Q_heads, K_heads, V_heads
        else:
            weights.Dispose()
            attention_heads_T.Dispose()
    if fused_done:
        pass
    elif heads_in_place:
        scores = GPUTensor([batch_size * H, tq, tkv], None, w)
        _heads_gemm(scores, Q_heads, K_heads, transA=False, transB=True, M=tq, N=tkv, K=dk, alpha=scaling,
                    batch=batch_size, heads=H, a_packed=True, b_packed=True, c_packed=False, a_steps=tq, b_steps=tkv,
                    c_steps=0, a_dim=dk, b_dim=dk, c_dim=0)
        if is_causal:
            scores.SetAllElementsAboveMainDiagonal(-1e12)
        weights = GPUTensor(scores.Shape, None, w)
        scores.SoftmaxLastDimension(weights)
        scores.Dispose()
        attention_heads_T = GPUTensor([batch_size, tkv, H * dv], None, w)
        _heads_gemm(attention_heads_T, weights, V_heads, transA=False, transB=False, M=tq, N=dv, K=tkv, alpha=1.0,
                    batch=batch_size, heads=H, a_packed=False, b_packed=True, c_packed=True, a_steps=0, b_steps=tkv,
                    c_steps=tkv, a_dim=0, b_dim=dv, c_dim=dv)
        st.Q_heads, st.K_heads, st.V_heads = Q_heads, K_heads, V_heads
    else:
        def split(packed, steps, dim):                                                      # :203-205
            t = GPUTensor([batch_size, H, steps, dim], None, w)
            packed.Reshape(batch_size, steps, H, dim).TransposeSecondAndThirdDimension(t)
            packed.Dispose()
            return t.Reshape(batch_size * H, steps, dim)
        Q_heads_T, K_heads_T, V_heads_T = split(Q_heads, tq, dk), split(K_heads, tkv, dk), split(V_heads, tkv, dv)
        attention_heads = GPUTensor(V_heads_T.Shape, None, w)
        weights = ScaledDotProductAttentionForwardPropagation(Q_heads_T, K_heads_T, V_heads_T, attention_heads, True,
                                                              use_scale, is_causal, fused=False)   # :221
        attention_heads_T = GPUTensor([batch_size, tkv, H, dv], None, w)
        attention_heads.Reshape(batch_size, H, tkv, dv).TransposeSecondAndThirdDimension(attention_heads_T)   # :224
        attention_heads_T = attention_heads_T.Reshape(batch_size, tkv, H * dv)
        st.Q_heads, st.K_heads, st.V_heads = Q_heads_T, K_heads_T, V_heads_T
    linear.DenseForwardPropagation(y, attention_heads_T, out_proj_weight, out_proj_bias, True)   # :226
    st.weights_buffer, st.attention_heads_T = weights, attention_heads_T
    return st if isTraining else None


def MultiheadAttentionBackwardPropagation(dQ, dK, dV, Q, K, V, dy, st, w_Q, w_K, w_V, out_proj_weight, grads,
                                          use_scale=True, compatibility_mode="PyTorch", fused_attention=True):
    """MultiheadAttention.BackwardPropagation (:243-292).  ``grads`` maps 'w_Q', 'w_K', 'w_V', 'out_proj_weight' to
    (weightGradients, biasGradientsOrNone) tensors that are filled in; dQ, dK, dV receive the input gradients."""
    from . import linear
    w = Q.Wrapper
    batch_size, tq, tkv, H, dk, dv = st.dims
    d_attention_heads_T = GPUTensor(st.attention_heads_T.Shape, None, w)
    gw, gb = grads["out_proj_weight"]
    linear.DenseBackwardPropagation(d_attention_heads_T, gw, gb, st.attention_heads_T, dy, out_proj_weight,
                                    compatibility_mode=compatibility_mode, flattenInputTensorOnLastDimension=True)   # :258
    # The reference's backward takes the scale from the value dimension (embedding_dim = dV.Shape[2],
    # ScaledDotProductAttentionLayer.cs:113-121) while its forward uses the key dimension (:60); the two agree
    # whenever key_dim == value_dim, which is all the reference ever tests.  Mirrored as is.
    scaling = 1.0 / math.sqrt(dv) if use_scale else 1.0
    P = st.weights_buffer
    if st.heads_in_place:
        dQ_p = GPUTensor([batch_size * tq, H * dk], None, w)
        dK_p = GPUTensor([batch_size * tkv, H * dk], None, w)
        dV_p = GPUTensor([batch_size * tkv, H * dv], None, w)
        dS = GPUTensor(P.Shape, None, w)
        if fused_attention:
            attention_backward(dQ_p, dK_p, dV_p, st.Q_heads, st.K_heads, st.V_heads, d_attention_heads_T, P, dS,
                               batch=batch_size, heads=H, tq=tq, tkv=tkv, dk=dk, dv=dv, scale=scaling, packed=True,
                               is_causal=st.is_causal)
        else:
            common = dict(batch=batch_size, heads=H)
            # dV = P^T . dO                                                          (ScaledDotProductAttentionLayer.cs:117)
            _heads_gemm(dV_p, P, d_attention_heads_T, transA=True, transB=False, M=tkv, N=dv, K=tq, alpha=1.0,
                        a_packed=False, b_packed=True, c_packed=True, a_steps=0, b_steps=tq, c_steps=tkv, a_dim=0, b_dim=dv,
                        c_dim=dv, **common)
            # dS = scale * dO . V^T, then through the softmax                         (:123-125)
            _heads_gemm(dS, d_attention_heads_T, st.V_heads, transA=False, transB=True, M=tq, N=tkv, K=dv, alpha=scaling,
                        a_packed=True, b_packed=True, c_packed=False, a_steps=tq, b_steps=tkv, c_steps=0, a_dim=dv,
                        b_dim=dv, c_dim=0, **common)
            P.SoftmaxLastDimensionBackward(dS, dS)
            # dQ = dS . K, dK = dS^T . Q                                             (:127-128)
            _heads_gemm(dQ_p, dS, st.K_heads, transA=False, transB=False, M=tq, N=dk, K=tkv, alpha=1.0, a_packed=False,
                        b_packed=True, c_packed=True, a_steps=0, b_steps=tkv, c_steps=tq, a_dim=0, b_dim=dk, c_dim=dk,
                        **common)
            _heads_gemm(dK_p, dS, st.Q_heads, transA=True, transB=False, M=tkv, N=dk, K=tq, alpha=1.0, a_packed=False,
                        b_packed=True, c_packed=True, a_steps=0, b_steps=tq, c_steps=tkv, a_dim=0, b_dim=dk, c_dim=dk,
                        **common)
        dS.Dispose()
    else:
        d_attention_heads = GPUTensor([batch_size, H, tkv, dv], None, w)
        d_attention_heads_T.Reshape(batch_size, tkv, H, dv).TransposeSecondAndThirdDimension(d_attention_heads)     # :263
        d_attention_heads = d_attention_heads.Reshape(batch_size * H, tkv, dv)
        dQ_h, dK_h, dV_h = (GPUTensor(t.Shape, None, w) for t in (st.Q_heads, st.K_heads, st.V_heads))
        ScaledDotProductAttentionBackwardPropagation(dQ_h, dK_h, dV_h, st.Q_heads, st.K_heads, st.V_heads,
                                                     d_attention_heads, P, use_scale, fused=False)                  # :270
        def merge(t, steps, dim):                                                                                   # :276,279,282
            out = GPUTensor([batch_size, steps, H, dim], None, w)
            t.Reshape(batch_size, H, steps, dim).TransposeSecondAndThirdDimension(out)
            t.Dispose()
            return out.Reshape(batch_size * steps, H * dim)
        dQ_p, dK_p, dV_p = merge(dQ_h, tq, dk), merge(dK_h, tkv, dk), merge(dV_h, tkv, dv)
    for dx, x, dpacked, wt, key in ((dQ, Q, dQ_p, w_Q, "w_Q"), (dK, K, dK_p, w_K, "w_K"), (dV, V, dV_p, w_V, "w_V")):
        gw, gb = grads[key]
        linear.DenseBackwardPropagation(dx, gw, gb, x, dpacked, wt, compatibility_mode=compatibility_mode,
                                        flattenInputTensorOnLastDimension=True)                                      # :277-283
        dpacked.Dispose()
    d_attention_heads_T.Dispose()
