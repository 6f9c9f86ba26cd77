"""Pins of oracle/rnn_oracle.py: torch's CPU RNN / LSTM / GRU modules (a library routine with the same parameter
convention as cuDNN) for values and gradients, and the reference's stored SimpleRNN losses."""
import numpy as np
import pytest
import torch

from oracle import rnn_oracle as ro
from tests.rnn_chain import simple_rnn_chain, zero_weight_chain

CELLS = {ro.RELU: ("RNN", "relu"), ro.TANH: ("RNN", "tanh"), ro.LSTM: ("LSTM", None), ro.GRU: ("GRU", None)}


def torch_module(desc):
    kind, nonlin = CELLS[desc.cell]
    kw = dict(input_size=desc.input_size, hidden_size=desc.hidden_size, num_layers=desc.num_layers, batch_first=True,
              bidirectional=desc.bidirectional, bias=desc.bias_mode != ro.NO_BIAS)
    if nonlin:
        kw["nonlinearity"] = nonlin
    return getattr(torch.nn, kind)(**kw).double()


def weights_from_torch(desc, module, rng):
    """Fills a weight space gate by gate through weight_params from the module's stacked parameters."""
    w = np.zeros(ro.weight_space_size(desc), np.float32)
    G, H = desc.gates, desc.hidden_size
    with torch.no_grad():
        for p in range(desc.pseudo_layers):
            sfx = "_l%d%s" % (p // desc.dirs, "_reverse" if p % desc.dirs else "")
            for lin in range(2 * G):
                side, gate = ("hh", lin - G) if lin >= G else ("ih", lin)
                off, (rows, cols), boff = ro.weight_params(desc, p, lin)
                block = rng.uniform(-0.6, 0.6, (rows, cols)).astype(np.float32)
                w[off:off + rows * cols] = block.ravel()
                getattr(module, "weight_" + side + sfx)[gate * H:(gate + 1) * H] = torch.from_numpy(block.astype(np.float64))
                if desc.bias_mode == ro.NO_BIAS:
                    continue
                tb = getattr(module, "bias_" + side + sfx)
                if boff is None:
                    tb[gate * H:(gate + 1) * H] = 0.0
                else:
                    b = rng.uniform(-0.5, 0.5, H).astype(np.float32)
                    w[boff:boff + H] = b
                    tb[gate * H:(gate + 1) * H] = torch.from_numpy(b.astype(np.float64))
    return w


def grads_from_torch(desc, module):
    g = np.zeros(ro.weight_space_size(desc), np.float64)
    G, H = desc.gates, desc.hidden_size
    for p in range(desc.pseudo_layers):
        sfx = "_l%d%s" % (p // desc.dirs, "_reverse" if p % desc.dirs else "")
        for lin in range(2 * G):
            side, gate = ("hh", lin - G) if lin >= G else ("ih", lin)
            off, (rows, cols), boff = ro.weight_params(desc, p, lin)
            g[off:off + rows * cols] = getattr(module, "weight_" + side + sfx).grad[gate * H:(gate + 1) * H].numpy().ravel()
            if boff is not None:
                g[boff:boff + H] = getattr(module, "bias_" + side + sfx).grad[gate * H:(gate + 1) * H].numpy()
    return g


def test_weight_space_is_a_partition():
    for cell in CELLS:
        for mode in (ro.NO_BIAS, ro.SINGLE_INP_BIAS, ro.DOUBLE_BIAS, ro.SINGLE_REC_BIAS):
            d = ro.RnnDesc(cell, 5, 3, num_layers=2, bidirectional=True, bias_mode=mode)
            seen = np.zeros(ro.weight_space_size(d), np.int32)
            for p in range(d.pseudo_layers):
                for lin in range(d.lin_layer_ids):
                    off, (r, c), boff = ro.weight_params(d, p, lin)
                    seen[off:off + r * c] += 1
                    if boff is not None:
                        seen[boff:boff + r] += 1
            assert np.all(seen == 1), (cell, mode)


@pytest.mark.parametrize("cell", list(CELLS))
@pytest.mark.parametrize("bidirectional,layers", [(False, 1), (True, 1), (False, 2), (True, 2)])
@pytest.mark.parametrize("bias_mode", [ro.DOUBLE_BIAS, ro.SINGLE_INP_BIAS, ro.SINGLE_REC_BIAS, ro.NO_BIAS])
def test_against_torch_modules(cell, bidirectional, layers, bias_mode):
    rng = np.random.default_rng(cell * 100 + layers * 10 + int(bidirectional) + bias_mode)
    desc = ro.RnnDesc(cell, input_size=4, hidden_size=3, num_layers=layers, bidirectional=bidirectional, bias_mode=bias_mode)
    m = torch_module(desc)
    w = weights_from_torch(desc, m, rng)
    B, T = 5, 6
    x = rng.uniform(-1, 1, (B, T, 4)).astype(np.float32)
    hx = rng.uniform(-1, 1, (desc.pseudo_layers, B, 3)).astype(np.float32)
    cx = rng.uniform(-1, 1, (desc.pseudo_layers, B, 3)).astype(np.float32)
    dy = rng.uniform(-1, 1, (B, T, desc.dirs * 3)).astype(np.float32)
    dhy = rng.uniform(-1, 1, hx.shape).astype(np.float32)
    dcy = rng.uniform(-1, 1, hx.shape).astype(np.float32)
    for with_state in (False, True):
        xt = torch.from_numpy(x.astype(np.float64)).requires_grad_(True)
        ht = torch.from_numpy(hx.astype(np.float64)).requires_grad_(True)
        ct = torch.from_numpy(cx.astype(np.float64)).requires_grad_(True)
        m.zero_grad()
        if cell == ro.LSTM:
            yt, (hyt, cyt) = m(xt, (ht, ct)) if with_state else m(xt)
        else:
            yt, hyt = m(xt, ht) if with_state else m(xt)
            cyt = None
        y, hy, cy, cache = ro.rnn_forward(desc, x, w, hx if with_state else None, cx if with_state else None)
        assert np.max(np.abs(y - yt.detach().numpy())) < 2e-6
        assert np.max(np.abs(hy - hyt.detach().numpy())) < 2e-6
        if cyt is not None:
            assert np.max(np.abs(cy - cyt.detach().numpy())) < 2e-6
        loss = (yt * torch.from_numpy(dy.astype(np.float64))).sum()
        if with_state:
            loss = loss + (hyt * torch.from_numpy(dhy.astype(np.float64))).sum()
            if cyt is not None:
                loss = loss + (cyt * torch.from_numpy(dcy.astype(np.float64))).sum()
        loss.backward()
        dx, dw, dhx, dcx = ro.rnn_backward(desc, dy, cache, dhy if with_state else None,
                                           dcy if (with_state and cell == ro.LSTM) else None)
        assert np.max(np.abs(dx - xt.grad.numpy())) < 1e-5
        assert np.max(np.abs(dw - grads_from_torch(desc, m))) < 2e-5
        if with_state:
            assert np.max(np.abs(dhx - ht.grad.numpy())) < 1e-5
            if cell == ro.LSTM:
                assert np.max(np.abs(dcx - ct.grad.numpy())) < 1e-5


def test_simple_rnn_chain_losses(golden):
    fx = golden["PyTorch_SimpleRNN"]
    before, after = simple_rnn_chain(fx)
    assert abs(before - fx["loss_before"]) < fx["tolerance"], (before, fx["loss_before"])
    assert abs(after - fx["loss_after"]) < fx["tolerance"], (after, fx["loss_after"])


@pytest.mark.parametrize("index", range(13))
def test_zero_weight_layers_reach_the_reference_predictions(golden, oracle, index):
    """SimpleRNN / LSTM / GRU, sequences or last step, one or two directions: the predictions the reference's tests
    store after 10 epochs (tolerance 1e-4 there; reproduced to 1e-6).  Pins the LSTM and GRU cells, both
    directions and the returnSequences handling with the reference's own numbers."""
    fx = golden["ZeroWeightRecurrentLayers"]
    case = fx["cases"][index]
    before, after = zero_weight_chain(fx, case)
    assert np.max(np.abs(before.reshape(-1) - np.array(case["prediction_before"], np.float32).reshape(-1))) <= 1e-6
    assert np.max(np.abs(after.reshape(-1) - np.array(case["prediction_after"], np.float32).reshape(-1))) <= 2e-6, case
