"""TEST INFRASTRUCTURE - not part of the product.

Only tests/, ``__graft_entry__.smoke()`` and bench.py's ``cpu_baseline`` leg may
import this module.  Nothing under sharpnet_amd/ does.

CPU restatement (numpy, float64 arithmetic on float32 data) of the recurrent
layers the reference builds on cuDNN: ``cudnnRNNForward`` /
``cudnnRNNBackwardData_v8`` / ``cudnnRNNBackwardWeights_v8`` as called at
Prod/Layers/RecurrentLayer.cs:353-374,456-503 with
``CUDNN_RNN_ALGO_STANDARD``, linear input, batch-major unpacked data
(Prod/GPU/GPUWrapper.cs:538) and full-length sequences.  cuDNN itself is not
part of the reference tree (bound as cudnn64_8, Prod/GPU/CudnnWrapper.cs); its
published cell formulas are restated here:

  RELU / TANH   h' = act(W x + bW + R h + bR)
  LSTM          i, f, o = sigmoid(.), g = tanh(.) of W x + bW + R h + bR;  c' = f c + i g;  h' = o tanh(c')
  GRU           r, z = sigmoid(W x + bW + R h + bR);  n = tanh(Wn x + bWn + r (Rn h + bRn));  h' = (1 - z) n + z h

gate order i, f, g, o and r, z, n (linLayerID 0 .. G-1 input side, G .. 2G-1
recurrent side, as RecurrentLayer.cs:170-184 walks them).

=========================  ======================================  ==================================================
function                   follows                                 pinned by
=========================  ======================================  ==================================================
weight_params /            cudnnGetRNNWeightParams as used at      round trip against rnn_forward with torch's
weight_space_size          RecurrentLayer.cs:170-184; the order    per-gate parameter order (tests/test_oracle_rnn.py)
                           inside the weight space is this
                           build's own (the reference only ever
                           asks for addresses)
rnn_forward                cudnnRNNForward, RecurrentLayer.cs:353  the reference's stored predictions of SimpleRNN /
                                                                   LSTM / GRU networks after 10 epochs of training
                                                                   (TestNetworkPropagation.cs:1193-1330, 13 cases:
                                                                   sequences or last step, one or two directions);
                                                                   SimpleRNN loss before training
                                                                   ParallelRunWithPyTorch.cs:949 (0.48370790481567383);
                                                                   torch.nn.RNN / LSTM / GRU on the CPU (library
                                                                   routine, same parameter convention): all cells,
                                                                   both directions, 1-2 layers, every bias mode,
                                                                   initial states, gate order with non-zero weights
rnn_backward               cudnnRNNBackwardData_v8 +               the same 13 stored predictions (they are reached
                           cudnnRNNBackwardWeights_v8, :456-503    through 10 gradient steps); SimpleRNN loss after
                                                                   10 epochs ParallelRunWithPyTorch.cs:951
                                                                   (0.2722862660884857); torch autograd through the
                                                                   same modules
masks= of rnn_forward /    dropout between stacked layers as       the mask values are an input, so what is pinned is
rnn_backward               cuDNN applies it in training            where they act: a two-layer call with a mask equals
                           (RNNDescriptor.dropoutRate,             torch.nn.LSTM / GRU / RNN modules of one layer each
                           RecurrentLayer.cs:69,123; states        with the mask multiplied in between, values and all
                           seeded with 0, GPUWrapper.cs:460-474)   gradients through autograd (tests/test_oracle_rnn.py)
philox4x32_10 /            the generator the library documents     the three known-answer vectors of the Random123
dropout_mask               for its masks (cuDNN's own stream is    distribution (kat_vectors: zeros, all ones, digits of
                           not reproducible: which units cuDNN     pi); the mask's layout by construction from them
                           would drop is "parity unpinned", and
                           no reference fixture uses a rate > 0)
layer_forward /            RecurrentLayer.ForwardPropagation /     the same stored predictions and losses (last-step
layer_backward             BackwardPropagation :305-520            outputs of uni- and bidirectional layers; a 2-layer
                           (returnSequences == false: last step    bidirectional sequence layer feeding a last-step
                           of the forward direction, first step    layer)
                           of the reverse one)
=========================  ======================================  ==================================================
"""
import numpy as np

RELU, TANH, LSTM, GRU = 0, 1, 2, 3                      # cudnnRNNMode_t, Prod/GPU/CudnnWrapper.cs:313-327
NO_BIAS, SINGLE_INP_BIAS, DOUBLE_BIAS, SINGLE_REC_BIAS = 0, 1, 2, 3   # cudnnRNNBiasMode_t, :396-410
GATES = {RELU: 1, TANH: 1, LSTM: 4, GRU: 3}


class RnnDesc:
    """The fields of Prod/Layers/RNNDescriptor.cs this path uses."""

    def __init__(self, cell, input_size, hidden_size, num_layers=1, bidirectional=False, bias_mode=DOUBLE_BIAS):
        self.cell, self.input_size, self.hidden_size = cell, input_size, hidden_size
        self.num_layers, self.bidirectional, self.bias_mode = num_layers, bidirectional, bias_mode

    @property
    def dirs(self):
        return 2 if self.bidirectional else 1

    @property
    def gates(self):
        return GATES[self.cell]

    @property
    def pseudo_layers(self):                           # RNNDescriptor.cs:67-75
        return self.dirs * self.num_layers

    @property
    def lin_layer_ids(self):                           # RNNDescriptor.cs:84-98
        return 2 * self.gates

    def layer_input_size(self, layer):
        return self.input_size if layer == 0 else self.dirs * self.hidden_size

    def has_bias(self, recurrent_side):
        if self.bias_mode == DOUBLE_BIAS:
            return True
        return self.bias_mode == (SINGLE_REC_BIAS if recurrent_side else SINGLE_INP_BIAS)


def _matrix_floats(desc, pseudo):
    G, H = desc.gates, desc.hidden_size
    return G * H * desc.layer_input_size(pseudo // desc.dirs) + G * H * H


def _bias_floats(desc):
    G, H = desc.gates, desc.hidden_size
    return G * H * (int(desc.has_bias(False)) + int(desc.has_bias(True)))


def weight_space_size(desc):
    """Number of floats of the weight space: all matrices (pseudo-layer by pseudo-layer: the G input matrices, then
    the G recurrent ones, each hidden x inputs, row-major), then all bias vectors in the same order."""
    return sum(_matrix_floats(desc, p) for p in range(desc.pseudo_layers)) + desc.pseudo_layers * _bias_floats(desc)


def weight_params(desc, pseudo, lin_layer_id):
    """(matrix offset, matrix shape, bias offset or None), offsets in floats: what cudnnGetRNNWeightParams hands out."""
    G, H = desc.gates, desc.hidden_size
    recurrent = lin_layer_id >= G
    gate = lin_layer_id - G if recurrent else lin_layer_id
    cols = H if recurrent else desc.layer_input_size(pseudo // desc.dirs)
    base = sum(_matrix_floats(desc, p) for p in range(pseudo))
    if recurrent:
        base += G * H * desc.layer_input_size(pseudo // desc.dirs)
    w_off = base + gate * H * cols
    b_off = None
    if desc.has_bias(recurrent):
        b_base = sum(_matrix_floats(desc, p) for p in range(desc.pseudo_layers)) + pseudo * _bias_floats(desc)
        if recurrent and desc.has_bias(False):
            b_base += G * H
        b_off = b_base + gate * H
    return w_off, (H, cols), b_off


def _stacked(desc, weights, pseudo):
    """W (G*H, in), R (G*H, H), bW (G*H), bR (G*H) of one pseudo-layer as float64 (absent biases: zeros)."""
    G, H = desc.gates, desc.hidden_size
    w0, (_, cols), b0 = weight_params(desc, pseudo, 0)
    r0, _, c0 = weight_params(desc, pseudo, G)
    W = weights[w0:w0 + G * H * cols].reshape(G * H, cols).astype(np.float64)
    R = weights[r0:r0 + G * H * H].reshape(G * H, H).astype(np.float64)
    bW = weights[b0:b0 + G * H].astype(np.float64) if b0 is not None else np.zeros(G * H)
    bR = weights[c0:c0 + G * H].astype(np.float64) if c0 is not None else np.zeros(G * H)
    return W, R, bW, bR


def _sigmoid(x):
    return 1.0 / (1.0 + np.exp(-x))


def _cell_forward(cell, H, gx, h, c, R, bR):
    """One step.  gx = W x + bW (B, G*H).  Returns h', c', saved (what the step's backward needs)."""
    gh = h @ R.T + bR
    if cell in (RELU, TANH):
        pre = gx + gh
        hn = np.maximum(pre, 0.0) if cell == RELU else np.tanh(pre)
        return hn, c, (hn,)
    if cell == LSTM:
        pre = gx + gh
        i, f, g, o = _sigmoid(pre[:, :H]), _sigmoid(pre[:, H:2 * H]), np.tanh(pre[:, 2 * H:3 * H]), _sigmoid(pre[:, 3 * H:])
        cn = f * c + i * g
        return o * np.tanh(cn), cn, (i, f, g, o, c, cn)
    r = _sigmoid(gx[:, :H] + gh[:, :H])
    z = _sigmoid(gx[:, H:2 * H] + gh[:, H:2 * H])
    q = gh[:, 2 * H:]
    n = np.tanh(gx[:, 2 * H:] + r * q)
    return (1.0 - z) * n + z * h, c, (r, z, n, q, h)


def _cell_backward(cell, H, dh, dc, saved):
    """Returns d(gx) (B, G*H), d(gh) (B, G*H), the part of dh_prev that does not pass through R, dc_prev."""
    if cell in (RELU, TANH):
        (hn,) = saved
        dpre = dh * ((hn > 0).astype(np.float64) if cell == RELU else 1.0 - hn * hn)
        return dpre, dpre, np.zeros_like(dh), dc
    if cell == LSTM:
        i, f, g, o, c_prev, cn = saved
        tc = np.tanh(cn)
        dcn = dc + dh * o * (1.0 - tc * tc)
        dg = np.concatenate([dcn * g * i * (1 - i), dcn * c_prev * f * (1 - f), dcn * i * (1 - g * g), dh * tc * o * (1 - o)], 1)
        return dg, dg, np.zeros_like(dh), dcn * f
    r, z, n, q, h_prev = saved
    dn_pre = dh * (1.0 - z) * (1.0 - n * n)
    dz_pre = dh * (h_prev - n) * z * (1 - z)
    dr_pre = dn_pre * q * r * (1 - r)
    return (np.concatenate([dr_pre, dz_pre, dn_pre], 1), np.concatenate([dr_pre, dz_pre, dn_pre * r], 1), dh * z, dc)


def philox4x32_10(counter, key):
    """Philox4x32-10 (Salmon, Moraes, Dror, Shaw: "Parallel random numbers: as easy as 1, 2, 3", SC'11): four arrays of
    32-bit counter words and two key words -> four arrays of 32-bit output words."""
    c0, c1, c2, c3 = (np.asarray(c, np.uint64) for c in counter)
    k0, k1 = (np.uint64(k) for k in key)
    m0, m1, w0, w1 = np.uint64(0xD2511F53), np.uint64(0xCD9E8D57), np.uint64(0x9E3779B9), np.uint64(0xBB67AE85)
    lo, sh = np.uint64(0xFFFFFFFF), np.uint64(32)
    for _ in range(10):
        p0, p1 = m0 * c0, m1 * c2
        c0, c1, c2, c3 = ((p1 >> sh) ^ c1 ^ k0) & lo, p1 & lo, ((p0 >> sh) ^ c3 ^ k1) & lo, p0 & lo
        k0, k1 = (k0 + w0) & lo, (k1 + w1) & lo
    return [c.astype(np.uint32) for c in (c0, c1, c2, c3)]


def dropout_mask(seed, call, boundary, rate, batch, steps, width):
    """The mask the library documents for the activations between layers `boundary` and `boundary + 1` in its
    training-mode forward call number `call`: element e, numbered in (step, sample, unit) order, takes word e % 4 of
    philox(counter = {e // 4 low, e // 4 high, boundary, call}, key = {seed low, seed high}) and is dropped when
    (word >> 8) / 2^24 < rate.  Returned as (batch, steps, width) float32 with values 0 and 1 / (1 - rate)."""
    count = batch * steps * width
    chunk = np.arange((count + 3) // 4, dtype=np.uint64)
    words = philox4x32_10([chunk & np.uint64(0xFFFFFFFF), chunk >> np.uint64(32), np.full_like(chunk, boundary),
                           np.full_like(chunk, call & 0xFFFFFFFF)], [seed & 0xFFFFFFFF, (seed >> 32) & 0xFFFFFFFF])
    bits = np.stack(words, axis=1).reshape(-1)[:count]
    u = (bits >> np.uint32(8)).astype(np.float32) * np.float32(1.0 / 16777216.0)
    scale = np.float32(1.0) / (np.float32(1.0) - np.float32(rate))
    step_major = np.where(u < np.float32(rate), np.float32(0.0), scale).astype(np.float32).reshape(steps, batch, width)
    return np.ascontiguousarray(step_major.transpose(1, 0, 2))


def rnn_forward(desc, x, weights, hx=None, cx=None, masks=None):
    """x (B, T, input) -> y (B, T, dirs*H), hy (pseudo_layers, B, H), cy (same, LSTM only), cache.
    masks (training with dropout): one (B, T, dirs*H) array per layer but the last, multiplied onto that layer's
    outputs on their way into the next layer (values 0 and 1 / (1 - rate)); y, hy, cy are never masked."""
    B, T, _ = x.shape
    H, K = desc.hidden_size, desc.dirs
    inp = x.astype(np.float64)
    hy = np.zeros((desc.pseudo_layers, B, H))
    cy = np.zeros((desc.pseudo_layers, B, H))
    cache = {"desc": desc, "weights": weights, "layers": [], "masks": masks}
    for layer in range(desc.num_layers):
        out = np.zeros((B, T, K * H))
        per_dir = []
        for d in range(K):
            p = layer * K + d
            W, R, bW, bR = _stacked(desc, weights, p)
            h = hx[p].astype(np.float64) if hx is not None else np.zeros((B, H))
            c = cx[p].astype(np.float64) if cx is not None else np.zeros((B, H))
            h0 = h
            steps = range(T) if d == 0 else range(T - 1, -1, -1)
            saved, h_in = {}, {}
            for t in steps:
                h_in[t] = h
                h, c, saved[t] = _cell_forward(desc.cell, H, inp[:, t] @ W.T + bW, h, c, R, bR)
                out[:, t, d * H:(d + 1) * H] = h
            hy[p], cy[p] = h, c
            per_dir.append({"saved": saved, "h_in": h_in, "h0": h0})
        cache["layers"].append({"input": inp, "dirs": per_dir})
        inp = out
        if masks is not None and layer < desc.num_layers - 1:
            inp = out * masks[layer].astype(np.float64)
    return out.astype(np.float32), hy.astype(np.float32), cy.astype(np.float32), cache


def rnn_backward(desc, dy, cache, dhy=None, dcy=None):
    """dy (B, T, dirs*H) -> dx, dweights (flat, the layout of weight_params), dhx, dcx."""
    weights = cache["weights"]
    B, T, _ = dy.shape
    H, K, G = desc.hidden_size, desc.dirs, desc.gates
    dw = np.zeros(weight_space_size(desc))
    dhx = np.zeros((desc.pseudo_layers, B, H))
    dcx = np.zeros((desc.pseudo_layers, B, H))
    dout = dy.astype(np.float64)
    for layer in range(desc.num_layers - 1, -1, -1):
        inp = cache["layers"][layer]["input"]
        dinp = np.zeros_like(inp)
        for d in range(K):
            p = layer * K + d
            W, R, _, _ = _stacked(desc, weights, p)
            rec = cache["layers"][layer]["dirs"][d]
            dh = dhy[p].astype(np.float64) if dhy is not None else np.zeros((B, H))
            dc = dcy[p].astype(np.float64) if dcy is not None else np.zeros((B, H))
            dW, dR, dbW, dbR = np.zeros_like(W), np.zeros_like(R), np.zeros(G * H), np.zeros(G * H)
            steps = range(T - 1, -1, -1) if d == 0 else range(T)
            for t in steps:
                dgx, dgh, direct, dc = _cell_backward(desc.cell, H, dh + dout[:, t, d * H:(d + 1) * H], dc, rec["saved"][t])
                dW += dgx.T @ inp[:, t]
                dR += dgh.T @ rec["h_in"][t]
                dbW += dgx.sum(0)
                dbR += dgh.sum(0)
                dinp[:, t] += dgx @ W
                dh = direct + dgh @ R
            dhx[p], dcx[p] = dh, dc
            w0, (_, cols), b0 = weight_params(desc, p, 0)
            r0, _, c0 = weight_params(desc, p, G)
            dw[w0:w0 + G * H * cols] = dW.ravel()
            dw[r0:r0 + G * H * H] = dR.ravel()
            if b0 is not None:
                dw[b0:b0 + G * H] = dbW
            if c0 is not None:
                dw[c0:c0 + G * H] = dbR
        dout = dinp
        if cache.get("masks") is not None and layer > 0:
            dout = dinp * cache["masks"][layer - 1].astype(np.float64)   # gradient of the outputs of the layer below
    return dinp.astype(np.float32), dw.astype(np.float32), dhx.astype(np.float32), dcx.astype(np.float32)


def layer_forward(desc, x, weights, return_sequences):
    """RecurrentLayer.ForwardPropagation (RecurrentLayer.cs:305-408) without the encoder / decoder variants:
    y = the whole sequence, or (B, dirs*H) = hy laid side by side."""
    y, hy, _, cache = rnn_forward(desc, x, weights)
    cache["return_sequences"] = return_sequences
    if return_sequences:
        return y, cache
    top = hy[(desc.num_layers - 1) * desc.dirs:]                       # (dirs, B, H) -> (B, dirs*H), :376-391
    return np.ascontiguousarray(np.transpose(top, (1, 0, 2))).reshape(x.shape[0], -1), cache


def layer_backward(desc, dy, cache):
    """RecurrentLayer.BackwardPropagation (:410-520): with returnSequences == false dy is scattered to the last step
    (first half) and, when bidirectional, the first step (second half) of a zero sequence (:437-454)."""
    if not cache["return_sequences"]:
        B, T = cache["layers"][0]["input"].shape[:2]
        H, K = desc.hidden_size, desc.dirs
        full = np.zeros((B, T, K * H), np.float32)
        full[:, T - 1, :H] = dy[:, :H]
        if K == 2:
            full[:, 0, H:] = dy[:, H:]
        dy = full
    dx, dw, _, _ = rnn_backward(desc, dy, cache)
    return dx, dw
