"""Host mirror of ScaledDotProductAttention forward / backward
(Prod/Layers/ScaledDotProductAttentionLayer.cs:46-91, 111-132) on GPUTensor.

Q, K, V, y are (batch, time, dim) tensors; the (batch, Tq, Tv) score and weight
buffers are materialised exactly as the reference does.  Forward returns the
weights buffer (kept for backward when training).
"""
import math

from .gpu_tensor import GPUTensor


def ScaledDotProductAttentionForwardPropagation(Q, K, V, y, isTraining, use_scale, is_causal):
    if V.Shape != K.Shape:
        raise ValueError("V.Shape and K.Shape must be equal, but are %s and %s" % (V.Shape, K.Shape))
    if V.Shape != y.Shape:
        raise ValueError("V.Shape and y.Shape must be equal, but are %s and %s" % (V.Shape, y.Shape))
    if Q.Shape[2] != V.Shape[2]:
        raise ValueError("queries.Shape[2] and values.Shape[2] must be equal (same embedding dim)")
    batch_size, query_time_steps, value_time_steps, embedding_dim = K.Shape[0], Q.Shape[1], V.Shape[1], K.Shape[2]
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


def ScaledDotProductAttentionBackwardPropagation(dQ, dK, dV, Q, K, V, dy, weights_buffer, use_scale):
    embedding_dim = dV.Shape[2]
    dV.BatchMatrixMultiplication(weights_buffer, True, dy, False, 1.0, 0.0)                # :117
    scaling = 1.0 / math.sqrt(embedding_dim) if use_scale else 1.0
    scores_gradients_buffer = GPUTensor(weights_buffer.Shape, None, Q.Wrapper)
    scores_gradients_buffer.BatchMatrixMultiplication(dy, False, V, True, scaling, 0.0)    # :123
    weights_buffer.SoftmaxLastDimensionBackward(scores_gradients_buffer, scores_gradients_buffer)   # :125
    dQ.BatchMatrixMultiplication(scores_gradients_buffer, False, K, False, 1.0, 0.0)      # :127
    dK.BatchMatrixMultiplication(scores_gradients_buffer, True, Q, False, 1.0, 0.0)       # :128
    scores_gradients_buffer.Dispose()
    weights_buffer.Dispose()
