"""Host mirror of the reference's Linear layer math (Prod/Layers/Linear.cs:125-191) on GPUTensor.

Same static entry points, argument order and semantics as the C#:
``DenseForwardPropagation(y, x, weights, bias, flatten)`` and
``DenseBackwardPropagation(dx, weightGradients, biasGradients, x, dy, weights, ...)``.
Weights are stored (out_features, in_features) (Linear.cs:22).  Every product
runs in libsharpnet_hip.so.

``fused=True`` (default) uses the library's Linear-layer entry points: forward is
one launch (bias add and, optionally, the activation of the ActivationLayer that
follows, folded into the GEMM's write-out), backward is two (dW with the bias
gradient and the weight-decay term riding along, then dx).  ``fused=False``
issues the reference's own sequence of calls one by one.
"""
from .hiplib import activation_code, check_status


def DenseForwardPropagation(y, x, weights, biasIfAny_1D, flattenInputTensorOnLastDimension, fused=True,
                            activation=None, activation_parameter=0.0):
    xAs2DMatrix = x.As2DTensor(flattenInputTensorOnLastDimension)
    yAs2DMatrix = y.As2DTensor(flattenInputTensorOnLastDimension)
    act = activation_code(activation)
    if fused:
        rows, in_features = xAs2DMatrix.Shape
        out_features = weights.Shape[0]
        assert weights.Shape[1] == in_features and yAs2DMatrix.Shape == [rows, out_features]
        check_status(y._lib.snhip_dense_forward(y.Wrapper.handle, yAs2DMatrix.Pointer, xAs2DMatrix.Pointer,
                                                weights.Pointer, biasIfAny_1D.Pointer if biasIfAny_1D is not None else None,
                                                rows, in_features, out_features, act, float(activation_parameter)),
                     "snhip_dense_forward")
        return
    # y = x * Weights^T + B   (Linear.cs:129-131), then the activation layer
    yAs2DMatrix.Dot(xAs2DMatrix, False, weights, True, 1.0, 0.0)
    if biasIfAny_1D is not None:
        biasIfAny_1D.BroadcastAddVectorToOutput(yAs2DMatrix)
    if act:
        yAs2DMatrix.ActivationForward(act, activation_parameter, yAs2DMatrix)


def DenseBackwardPropagation(dx, weightGradients, biasGradients_1D, x, dy, weights, bias_1D=None,
                             compatibility_mode="SharpNet", use_weight_decay_in_backpropagation=False, weight_decay=0.0,
                             prevLayerIsInputLayer=False, flattenInputTensorOnLastDimension=False, fused=True):
    xAs2DMatrix = x.As2DTensor(flattenInputTensorOnLastDimension)
    dyAs2DMatrix = dy.As2DTensor(flattenInputTensorOnLastDimension)
    batchSize = x.Shape[0]
    # dW = multiplier * dy^T * x   (Linear.cs:151-158)
    multiplier = 1.0 / batchSize
    if compatibility_mode in ("TensorFlow", "PyTorch"):
        multiplier = 1.0
    alpha = 0.0
    if use_weight_decay_in_backpropagation and weight_decay > 0:            # Linear.cs:168-181
        weight_decay_multiplier = 1 if compatibility_mode == "PyTorch" else 2
        alpha = weight_decay_multiplier * batchSize * float(weight_decay)
    if fused:
        rows, in_features = xAs2DMatrix.Shape
        out_features = weights.Shape[0]
        assert dyAs2DMatrix.Shape == [rows, out_features] and weightGradients.Shape == [out_features, in_features]
        # weight decay on the bias gradient as well in the PyTorch mode (Linear.cs:178-181)
        bias_alpha = alpha if (alpha and compatibility_mode == "PyTorch" and biasGradients_1D is not None) else 0.0
        check_status(dy._lib.snhip_dense_backward_ex(
            dy.Wrapper.handle, None if prevLayerIsInputLayer else dx.As2DTensor(flattenInputTensorOnLastDimension).Pointer,
            weightGradients.Pointer, biasGradients_1D.Pointer if biasGradients_1D is not None else None,
            xAs2DMatrix.Pointer, dyAs2DMatrix.Pointer, weights.Pointer, rows, in_features, out_features, multiplier, alpha,
            bias_1D.Pointer if bias_alpha else None, bias_alpha), "snhip_dense_backward_ex")
        return
    weightGradients.Dot(dyAs2DMatrix, True, xAs2DMatrix, False, multiplier, 0.0)
    if biasGradients_1D is not None:
        dyAs2DMatrix.Compute_BiasGradient_from_dy(biasGradients_1D)          # Linear.cs:160-165
    if alpha:
        weightGradients.Update_Adding_Alpha_X(alpha, weights)
        if compatibility_mode == "PyTorch" and biasGradients_1D is not None:
            biasGradients_1D.Update_Adding_Alpha_X(alpha, bias_1D)
    if prevLayerIsInputLayer:                                               # Linear.cs:184-187
        return
    dx.Dot(dyAs2DMatrix, False, weights, False, 1.0, 0.0)                   # dx = dy * Weights (Linear.cs:190)
