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


CELLS = {"relu": ro.RELU, "tanh": ro.TANH, "lstm": ro.LSTM, "gru": ro.GRU}


def zero_weight_chain(fx, case, forward=None, backward=None):
    """The networks of Tests/NonReg/TestNetworkPropagation.cs:1193-1330: a recurrent layer whose weights start at zero
    feeding Linear(1), Huber loss, SGD with momentum on the whole batch.  Returns (prediction before, after)."""
    from oracle import dot_oracle as do
    forward = forward or ro.layer_forward
    backward = backward or ro.layer_backward
    cell = CELLS[case["cell"]]
    bias_mode = ro.DOUBLE_BIAS if cell == ro.GRU else ro.SINGLE_INP_BIAS          # Prod/Networks/Network.cs:188-205
    desc = ro.RnnDesc(cell, 1, case["hidden"], 1, case["bidirectional"], bias_mode)
    rs = case["return_sequences"]
    X = np.array(fx["x"], np.float32)
    Y = np.array(fx["y_sequences"] if rs else fx["y_last"], np.float32)
    P = [np.zeros(ro.weight_space_size(desc), np.float32),
         np.array(case["dense_weight"], np.float32).reshape(1, desc.dirs * case["hidden"]), np.zeros(1, np.float32)]
    V = [np.zeros_like(p) for p in P]
    batch = X.shape[0]

    def predict():
        y, cache = forward(desc, X, P[0], rs)
        return do.dense_forward(y, P[1], P[2], flatten_last=True), (y, cache)

    before = predict()[0]
    for _ in range(fx["epochs"]):
        out, (y, cache) = predict()
        err = out.reshape(batch, -1) - Y.reshape(batch, -1)
        # Huber gradient: the clipped error over the elements of a sample (Prod/CPU/CpuTensor.cs:2427-2437)
        g = (np.clip(err, -fx["huber_delta"], fx["huber_delta"]) / err.shape[1]).reshape(out.shape).astype(np.float32)
        dW, db, dy = do.dense_backward(y, g, P[1], flatten_last=True)
        _, dw_rnn = backward(desc, dy.reshape(y.shape), cache)
        for i, grad in enumerate((dw_rnn, dW, db)):          # CpuTensor.cs:470-489 with lr / batchSize (Optimizer.cs:26-29)
            V[i] = (np.float32(fx["momentum"]) * V[i] - grad * np.float32(fx["lr"] / batch)).astype(np.float32)
            P[i] = (P[i] + V[i]).astype(np.float32)
    return before, predict()[0]
