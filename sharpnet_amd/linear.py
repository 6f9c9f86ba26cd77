"""Host mirror of the reference's Linear layer math (Prod/Layers/Linear.cs:125-191) on GPUTensor.

Same static entry points, argument order and semantics as the C#:
``DenseForwardPropagation(y, x, weights, bias, flatten)`` and
``DenseBackwardPropagation(dx, weightGradients, biasGradients, x, dy, weights, ...)``.
Weights are stored (out_features, in_features) (Linear.cs:22).  Every product
runs in libsharpnet_hip.so; ``fuse_bias=True`` (default) folds the bias add into
the forward GEMM's epilogue, ``False`` issues the reference's two calls.
"""


def DenseForwardPropagation(y, x, weights, biasIfAny_1D, flattenInputTensorOnLastDimension, fuse_bias=True):
    xAs2DMatrix = x.As2DTensor(flattenInputTensorOnLastDimension)
    yAs2DMatrix = y.As2DTensor(flattenInputTensorOnLastDimension)
    # y = x * Weights^T + B   (Linear.cs:129-131)
    if fuse_bias and biasIfAny_1D is not None:
        yAs2DMatrix.DotRowMajor(xAs2DMatrix, False, weights, True, 1.0, 0.0, bias=biasIfAny_1D)
    else:
        yAs2DMatrix.Dot(xAs2DMatrix, False, weights, True, 1.0, 0.0)
        if biasIfAny_1D is not None:
            biasIfAny_1D.BroadcastAddVectorToOutput(yAs2DMatrix)


def DenseBackwardPropagation(dx, weightGradients, biasGradients_1D, x, dy, weights, bias_1D=None,
                             compatibility_mode="SharpNet", use_weight_decay_in_backpropagation=False, weight_decay=0.0,
                             prevLayerIsInputLayer=False, flattenInputTensorOnLastDimension=False):
    xAs2DMatrix = x.As2DTensor(flattenInputTensorOnLastDimension)
    dyAs2DMatrix = dy.As2DTensor(flattenInputTensorOnLastDimension)
    batchSize = x.Shape[0]
    # dW = multiplier * dy^T * x   (Linear.cs:151-158)
    multiplier = 1.0 / batchSize
    if compatibility_mode in ("TensorFlow", "PyTorch"):
        multiplier = 1.0
    weightGradients.Dot(dyAs2DMatrix, True, xAs2DMatrix, False, multiplier, 0.0)
    if biasGradients_1D is not None:
        dyAs2DMatrix.Compute_BiasGradient_from_dy(biasGradients_1D)          # Linear.cs:160-165
    if use_weight_decay_in_backpropagation and weight_decay > 0:            # Linear.cs:168-181
        weight_decay_multiplier = 1 if compatibility_mode == "PyTorch" else 2
        alpha = weight_decay_multiplier * batchSize * float(weight_decay)
        weightGradients.Update_Adding_Alpha_X(alpha, weights)
        if compatibility_mode == "PyTorch" and biasGradients_1D is not None:
            biasGradients_1D.Update_Adding_Alpha_X(alpha, bias_1D)
    if prevLayerIsInputLayer:                                               # Linear.cs:184-187
        return
    dx.Dot(dyAs2DMatrix, False, weights, False, 1.0, 0.0)                   # dx = dy * Weights (Linear.cs:190)
