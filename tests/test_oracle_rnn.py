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


def test_philox_known_answers():
    """The three vectors of the Random123 distribution's kat_vectors file for philox4x32 with 10 rounds."""
    kat = [([0, 0, 0, 0], [0, 0], [0x6627e8d5, 0xe169c58d, 0xbc57ac4c, 0x9b00dbd8]),
           ([0xffffffff] * 4, [0xffffffff] * 2, [0x408f276d, 0x41c83b0e, 0xa20bc7c6, 0x6d5451fd]),
           ([0x243f6a88, 0x85a308d3, 0x13198a2e, 0x03707344], [0xa4093822, 0x299f31d0],
            [0xd16cfe09, 0x94fdcceb, 0x5001e420, 0x24126ea1])]
    for counter, key, want in kat:
        got = ro.philox4x32_10([[c] for c in counter], key)
        assert [int(g[0]) for g in got] == want
    # vectorised over counters: the same words as one at a time
    many = ro.philox4x32_10([np.arange(5), np.zeros(5), np.full(5, 2), np.full(5, 7)], [11, 13])
    for i in range(5):
        one = ro.philox4x32_10([[i], [0], [2], [7]], [11, 13])
        assert [int(w[i]) for w in many] == [int(w[0]) for w in one]


def test_dropout_mask_layout_and_statistics():
    """Element e = (t * B + b) * W + u of the step-major numbering takes word e % 4 of counter e // 4; values are 0 or
    1 / (1 - rate); about `rate` of them are zero; call, boundary and seed each select another stream."""
    B, T, W, rate = 3, 5, 6, 0.3
    m = ro.dropout_mask(seed=9, call=4, boundary=1, rate=rate, batch=B, steps=T, width=W)
    assert m.shape == (B, T, W) and m.dtype == np.float32
    scale = np.float32(1.0) / (np.float32(1.0) - np.float32(rate))
    for (b, t, u) in [(0, 0, 0), (2, 4, 5), (1, 3, 2), (0, 4, 1)]:
        e = (t * B + b) * W + u
        word = int(ro.philox4x32_10([[e // 4], [0], [1], [4]], [9, 0])[e % 4][0])
        want = 0.0 if np.float32(word >> 8) * np.float32(2.0 ** -24) < np.float32(rate) else scale
        assert m[b, t, u] == np.float32(want)
    big = ro.dropout_mask(0, 0, 0, rate, 64, 50, 96)
    assert set(np.unique(big)) == {np.float32(0.0), scale}
    frac = float(np.mean(big == 0))
    assert abs(frac - rate) < 4 * np.sqrt(rate * (1 - rate) / big.size)
    for other in (ro.dropout_mask(1, 0, 0, rate, 64, 50, 96), ro.dropout_mask(0, 1, 0, rate, 64, 50, 96),
                  ro.dropout_mask(0, 0, 1, rate, 64, 50, 96)):
        assert 0.3 < float(np.mean(other == big)) < 0.8          # independent streams agree on p^2 + (1-p)^2 = 0.58
    assert np.all(ro.dropout_mask(5, 5, 0, 0.0, 2, 3, 4) == 1.0)


@pytest.mark.parametrize("cell", list(CELLS))
@pytest.mark.parametrize("bidirectional", [False, True])
def test_masks_between_layers_against_a_chain_of_torch_modules(cell, bidirectional):
    """rnn_forward / rnn_backward with masks= on three stacked layers against three one-layer torch modules with the
    masks multiplied in between: outputs, final states, dx and every weight gradient (autograd)."""
    rng = np.random.default_rng(3000 + cell * 2 + int(bidirectional))
    L, H, I, B, T = 3, 4, 5, 3, 6
    desc = ro.RnnDesc(cell, input_size=I, hidden_size=H, num_layers=L, bidirectional=bidirectional, bias_mode=ro.DOUBLE_BIAS)
    K = desc.dirs
    w = np.zeros(ro.weight_space_size(desc), np.float32)
    mods, descs, ws = [], [], []
    for layer in range(L):
        d1 = ro.RnnDesc(cell, input_size=I if layer == 0 else K * H, hidden_size=H, num_layers=1,
                        bidirectional=bidirectional, bias_mode=ro.DOUBLE_BIAS)
        m1 = torch_module(d1)
        w1 = weights_from_torch(d1, m1, rng)
        for k in range(K):
            for lin in range(d1.lin_layer_ids):
                o1, (r, c), b1 = ro.weight_params(d1, k, lin)
                o, (r2, c2), b = ro.weight_params(desc, layer * K + k, lin)
                assert (r, c) == (r2, c2)
                w[o:o + r * c] = w1[o1:o1 + r * c]
                w[b:b + r] = w1[b1:b1 + r]
        mods.append(m1), descs.append(d1), ws.append(w1)
    x = rng.uniform(-1, 1, (B, T, I)).astype(np.float32)
    dy = rng.uniform(-1, 1, (B, T, K * H)).astype(np.float32)
    masks = [ro.dropout_mask(7, 2, b, 0.4, B, T, K * H) for b in range(L - 1)]
    y, hy, cy, cache = ro.rnn_forward(desc, x, w, masks=masks)
    dx, dw, _, _ = ro.rnn_backward(desc, dy, cache)

    xt = torch.from_numpy(x.astype(np.float64)).requires_grad_(True)
    cur, finals = xt, []
    for layer in range(L):
        out, state = mods[layer](cur)
        finals.append(state)
        cur = out * torch.from_numpy(masks[layer].astype(np.float64)) if layer < L - 1 else out
    (cur * torch.from_numpy(dy.astype(np.float64))).sum().backward()
    assert np.max(np.abs(y - cur.detach().numpy())) < 2e-6
    for layer in range(L):
        hyt = finals[layer][0] if cell == ro.LSTM else finals[layer]
        assert np.max(np.abs(hy[layer * K:(layer + 1) * K] - hyt.detach().numpy())) < 2e-6     # states are never masked
        if cell == ro.LSTM:
            assert np.max(np.abs(cy[layer * K:(layer + 1) * K] - finals[layer][1].detach().numpy())) < 2e-6
    assert np.max(np.abs(dx - xt.grad.numpy())) < 1e-5
    for layer in range(L):
        g1 = grads_from_torch(descs[layer], mods[layer])
        for k in range(K):
            for lin in range(descs[layer].lin_layer_ids):
                o1, (r, c), b1 = ro.weight_params(descs[layer], k, lin)
                o, _, b = ro.weight_params(desc, layer * K + k, lin)
                assert np.max(np.abs(dw[o:o + r * c] - g1[o1:o1 + r * c])) < 2e-5
                assert np.max(np.abs(dw[b:b + r] - g1[b1:b1 + r])) < 2e-5
    # without masks the same call differs (the masks act), with masks of ones it does not
    y0, _, _, _ = ro.rnn_forward(desc, x, w)
    y1, _, _, _ = ro.rnn_forward(desc, x, w, masks=[np.ones_like(m) for m in masks])
    assert np.array_equal(y0, y1) and np.max(np.abs(y0 - y)) > 1e-3


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
