"""The reference's stacked-SimpleRNN training run, shared by the oracle test and the GPU test."""
import numpy as np

from oracle import rnn_oracle as ro
from tests.helpers import numpy_array_for_tests, y_numpy_array_for_tests


def simple_rnn_chain(fx, forward=None, backward=None):
    """The network of Tests/NonReg/ParallelRunWithPyTorch.cs:896-953: SimpleRNN(2, sequences, bidirectional, 2 layers)
    -> SimpleRNN(2, last step), MSE, SGD(0.01, momentum 0.9), batch 2, 10 epochs.  Returns (loss before, loss after)."""
    forward = forward or ro.layer_forward
    backward = backward or ro.layer_backward
    X = numpy_array_for_tests(*fx["x_shape"])
    Y = y_numpy_array_for_tests(*fx["y_shape"])
    d1 = ro.RnnDesc(ro.TANH, 1, 2, num_layers=2, bidirectional=True, bias_mode=ro.DOUBLE_BIAS)
    d2 = ro.RnnDesc(ro.TANH, 4, 2, num_layers=1, bidirectional=False, bias_mode=ro.DOUBLE_BIAS)
    P = [np.zeros(ro.weight_space_size(d1), np.float32), np.zeros(ro.weight_space_size(d2), np.float32)]
    for desc, w, ih, hh in ((d1, P[0], fx["layer1_weight_ih"], fx["layer1_weight_hh"]),
                            (d2, P[1], fx["layer2_weight_ih"], fx["layer2_weight_hh"])):
        for p in range(desc.pseudo_layers):
            for lin, src in ((0, ih[p]), (1, hh[p])):
                off, (r, c), _ = ro.weight_params(desc, p, lin)
                w[off:off + r * c] = np.array(src, np.float32).reshape(r, c).ravel()
    vel = [np.zeros_like(p) for p in P]

    def predict(x):
        s, c1 = forward(d1, x, P[0], True)
        y, c2 = forward(d2, s, P[1], False)
        return y, (c1, c2)

    def loss():
        return float(np.mean((predict(X)[0].astype(np.float64) - Y) ** 2))

    before = loss()
    bs = fx["batch_size"]
    for _ in range(fx["epochs"]):
        for i in range(0, X.shape[0], bs):
            x, y = X[i:i + bs], Y[i:i + bs]
            pred, (c1, c2) = predict(x)
            dpred = (2.0 * (pred - y) / y.shape[1]).astype(np.float32)        # MSE gradient; 1/batch sits in the update
            ds, g2 = backward(d2, dpred, c2)
            _, g1 = backward(d1, ds, c1)
            for k, g in enumerate((g1, g2)):
                vel[k] = (np.float32(fx["momentum"]) * vel[k] - g * np.float32(fx["lr"] / bs)).astype(np.float32)
                P[k] = (P[k] + vel[k]).astype(np.float32)
    return before, loss()
