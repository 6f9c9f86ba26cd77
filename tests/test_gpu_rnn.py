"""GPU tests of the recurrent layers (snhip_rnn_*): the raw entry points against oracle/rnn_oracle.py for every
cell, direction, depth and bias mode, with and without initial states; the RecurrentLayer mirror through the
reference's stored SimpleRNN losses."""
import ctypes

import numpy as np
import pytest

from oracle import rnn_oracle as ro
from tests.rnn_chain import simple_rnn_chain, zero_weight_chain

pytestmark = pytest.mark.gpu


def T(w, a):
    from sharpnet_amd import GPUTensor
    a = np.asarray(a, np.float32)
    return GPUTensor(list(a.shape), a, w)


def lib_desc(desc, dropout=0.0):
    from sharpnet_amd.hiplib import RnnDesc
    return RnnDesc(cell_mode=desc.cell, bias_mode=desc.bias_mode, bidirectional=desc.bidirectional,
                   num_layers=desc.num_layers, input_size=desc.input_size, hidden_size=desc.hidden_size, dropout=dropout)


def check(st, what):
    from sharpnet_amd.hiplib import check_status
    check_status(st, what)


def run_gpu(w, desc, x, weights, dy, hx=None, cx=None, dhy=None, dcy=None, training=True, want_dstate=True, dropout=0.0,
            between=None):
    """Forward (+ backward when training) through the C ABI; returns dict of numpy arrays.  between: called after the
    forward call and before the backward ones (other work on the same handle)."""
    from sharpnet_amd import GPUTensor
    lib, d = w.lib, lib_desc(desc, dropout)
    B, Tn, _ = x.shape
    H, K, P = desc.hidden_size, desc.dirs, desc.pseudo_layers
    ws, rs = ctypes.c_size_t(), ctypes.c_size_t()
    check(lib.snhip_rnn_temp_space_sizes(ctypes.byref(d), int(training), B, Tn, ctypes.byref(ws), ctypes.byref(rs)), "sizes")
    gws = GPUTensor([ws.value // 4], None, w)
    grs = GPUTensor([max(rs.value // 4, 2)], None, w)
    gws.SetValue(float("nan"))
    grs.SetValue(float("nan"))
    gx, gw = T(w, x), T(w, weights)
    gy = GPUTensor([B, Tn, K * H], None, w)
    ghy, gcy = GPUTensor([P, B, H], None, w), GPUTensor([P, B, H], None, w)
    for t in (gy, ghy, gcy):
        t.SetValue(float("nan"))
    ghx = T(w, hx) if hx is not None else None
    gcx = T(w, cx) if cx is not None else None
    ptr = lambda t: t.Pointer if t is not None else None
    check(lib.snhip_rnn_forward(w.handle, ctypes.byref(d), int(training), B, Tn, gx.Pointer, gy.Pointer, ptr(ghx), ghy.Pointer,
                                ptr(gcx), gcy.Pointer, gw.Pointer, gws.Pointer, ws.value, grs.Pointer if training else None,
                                rs.value), "snhip_rnn_forward")
    out = {"y": gy.ToNumpy(), "hy": ghy.ToNumpy(), "cy": gcy.ToNumpy()}
    if not training:
        return out
    if between is not None:
        between()
    gdy = T(w, dy)
    gdx = GPUTensor(list(x.shape), None, w)
    gdhx, gdcx = GPUTensor([P, B, H], None, w), GPUTensor([P, B, H], None, w)
    for t in (gdx, gdhx, gdcx):
        t.SetValue(float("nan"))
    gdhy = T(w, dhy) if dhy is not None else None
    gdcy = T(w, dcy) if dcy is not None else None
    check(lib.snhip_rnn_backward_data(w.handle, ctypes.byref(d), B, Tn, gy.Pointer, gdy.Pointer, gdx.Pointer, ptr(ghx),
                                      ptr(gdhy), gdhx.Pointer if want_dstate else None, ptr(gcx), ptr(gdcy),
                                      gdcx.Pointer if want_dstate else None, gw.Pointer, gws.Pointer,
                                      ws.value, grs.Pointer, rs.value), "snhip_rnn_backward_data")
    gdw = GPUTensor([weights.size], None, w)
    gdw.ZeroMemory()
    check(lib.snhip_rnn_backward_weights(w.handle, ctypes.byref(d), B, Tn, gx.Pointer, ptr(ghx), gy.Pointer, gdw.Pointer,
                                         gws.Pointer, ws.value, grs.Pointer, rs.value), "snhip_rnn_backward_weights")
    out.update(dx=gdx.ToNumpy(), dw=gdw.ToNumpy(), dhx=gdhx.ToNumpy(), dcx=gdcx.ToNumpy())
    return out


def compare(desc, got, x, weights, dy, hx, cx, dhy, dcy, tol, masks=None):
    y, hy, cy, cache = ro.rnn_forward(desc, x, weights, hx, cx, masks=masks)
    assert np.max(np.abs(got["y"] - y)) <= tol, "y"
    assert np.max(np.abs(got["hy"] - hy)) <= tol, "hy"
    if desc.cell == ro.LSTM:
        assert np.max(np.abs(got["cy"] - cy)) <= tol, "cy"
    if "dx" not in got:
        return
    dx, dw, dhx, dcx = ro.rnn_backward(desc, dy, cache, dhy, dcy if desc.cell == ro.LSTM else None)
    scale = max(1.0, float(np.max(np.abs(dw))))
    assert np.max(np.abs(got["dx"] - dx)) <= tol * max(1.0, float(np.max(np.abs(dx)))), "dx"
    assert np.max(np.abs(got["dw"] - dw)) <= tol * scale, "dw"
    assert np.max(np.abs(got["dhx"] - dhx)) <= tol * max(1.0, float(np.max(np.abs(dhx)))), "dhx"
    if desc.cell == ro.LSTM:
        assert np.max(np.abs(got["dcx"] - dcx)) <= tol * max(1.0, float(np.max(np.abs(dcx)))), "dcx"


@pytest.mark.parametrize("cell", [ro.RELU, ro.TANH, ro.LSTM, ro.GRU])
@pytest.mark.parametrize("bidirectional,layers", [(False, 1), (True, 1), (False, 2), (True, 2)])
@pytest.mark.parametrize("bias_mode", [ro.DOUBLE_BIAS, ro.SINGLE_INP_BIAS, ro.SINGLE_REC_BIAS, ro.NO_BIAS])
def test_cells_small(gpu_wrapper, cell, bidirectional, layers, bias_mode):
    rng = np.random.default_rng(1000 + cell * 100 + layers * 10 + int(bidirectional) + bias_mode)
    desc = ro.RnnDesc(cell, input_size=5, hidden_size=3, num_layers=layers, bidirectional=bidirectional, bias_mode=bias_mode)
    B, Tn = 4, 6
    weights = rng.uniform(-0.6, 0.6, ro.weight_space_size(desc)).astype(np.float32)
    x = rng.uniform(-1, 1, (B, Tn, 5)).astype(np.float32)
    dy = rng.uniform(-1, 1, (B, Tn, desc.dirs * 3)).astype(np.float32)
    st = lambda: rng.uniform(-1, 1, (desc.pseudo_layers, B, 3)).astype(np.float32)
    hx, cx, dhy, dcy = st(), st(), st(), st()
    if cell != ro.LSTM:
        cx = dcy = None
    got = run_gpu(gpu_wrapper, desc, x, weights, dy)
    compare(desc, got, x, weights, dy, None, None, None, None, 2e-5)
    got = run_gpu(gpu_wrapper, desc, x, weights, dy, hx, cx, dhy, dcy)
    compare(desc, got, x, weights, dy, hx, cx, dhy, dcy, 2e-5)


@pytest.mark.parametrize("cell", [ro.TANH, ro.LSTM, ro.GRU])
def test_cells_wider(gpu_wrapper, cell):
    """Sizes at which the GEMMs use full tiles, split-K and the fused column sums; odd batch and widths."""
    rng = np.random.default_rng(50 + cell)
    desc = ro.RnnDesc(cell, input_size=45, hidden_size=68, num_layers=2, bidirectional=True, bias_mode=ro.DOUBLE_BIAS)
    B, Tn = 33, 17
    weights = rng.uniform(-0.12, 0.12, ro.weight_space_size(desc)).astype(np.float32)
    x = rng.uniform(-1, 1, (B, Tn, 45)).astype(np.float32)
    dy = rng.uniform(-1, 1, (B, Tn, 2 * 68)).astype(np.float32)
    got = run_gpu(gpu_wrapper, desc, x, weights, dy)
    compare(desc, got, x, weights, dy, None, None, None, None, 1e-4)


@pytest.mark.parametrize("cell", [ro.RELU, ro.TANH, ro.LSTM, ro.GRU])
@pytest.mark.parametrize("hidden,batch", [(32, 5), (64, 33), (96, 70), (160, 32), (36, 9), (100, 40), (44, 64)])
def test_cells_one_launch_per_step(gpu_wrapper, cell, hidden, batch):
    """Hidden sizes that are multiples of 4 (from 32 up) take the kernel that computes h . R^T and the cell in one launch
    (K split over the wavefronts of a workgroup); checked against the oracle and against the GEMM + cell-kernel form
    selected through snhip_rnn_set_step_mode (different summation orders: 2e-5)."""
    rng = np.random.default_rng(hidden * 10 + batch + cell)
    desc = ro.RnnDesc(cell, input_size=20, hidden_size=hidden, num_layers=2, bidirectional=True, bias_mode=ro.DOUBLE_BIAS)
    Tn = 7
    weights = rng.uniform(-0.15, 0.15, ro.weight_space_size(desc)).astype(np.float32)
    x = rng.uniform(-1, 1, (batch, Tn, 20)).astype(np.float32)
    dy = rng.uniform(-1, 1, (batch, Tn, 2 * hidden)).astype(np.float32)
    st = lambda: rng.uniform(-1, 1, (desc.pseudo_layers, batch, hidden)).astype(np.float32)
    hx, cx, dhy, dcy = st(), st(), st(), st()
    if cell != ro.LSTM:
        cx = dcy = None
    got = run_gpu(gpu_wrapper, desc, x, weights, dy, hx, cx, dhy, dcy)
    compare(desc, got, x, weights, dy, hx, cx, dhy, dcy, 5e-5)
    # without the gradients of the initial states (what a layer inside a network asks for): same dx and dw
    plain = run_gpu(gpu_wrapper, desc, x, weights, dy, hx, cx, dhy, dcy, want_dstate=False)
    assert np.array_equal(plain["dx"], got["dx"]) and np.array_equal(plain["dw"], got["dw"])
    check(gpu_wrapper.lib.snhip_rnn_set_step_mode(gpu_wrapper.handle, 1), "step mode")
    try:
        two = run_gpu(gpu_wrapper, desc, x, weights, dy, hx, cx, dhy, dcy)
    finally:
        check(gpu_wrapper.lib.snhip_rnn_set_step_mode(gpu_wrapper.handle, 0), "step mode")
    compare(desc, two, x, weights, dy, hx, cx, dhy, dcy, 5e-5)
    assert np.max(np.abs(two["y"] - got["y"])) <= 2e-5


@pytest.mark.parametrize("cell", [ro.RELU, ro.LSTM, ro.GRU])
def test_inference_equals_training_forward(gpu_wrapper, cell):
    rng = np.random.default_rng(7 + cell)
    desc = ro.RnnDesc(cell, input_size=9, hidden_size=16, num_layers=2, bidirectional=True, bias_mode=ro.SINGLE_INP_BIAS)
    weights = rng.uniform(-0.3, 0.3, ro.weight_space_size(desc)).astype(np.float32)
    x = rng.uniform(-1, 1, (6, 5, 9)).astype(np.float32)
    a = run_gpu(gpu_wrapper, desc, x, weights, None, training=False)
    b = run_gpu(gpu_wrapper, desc, x, weights, np.zeros((6, 5, 32), np.float32), training=True)
    assert np.array_equal(a["y"], b["y"]) and np.array_equal(a["hy"], b["hy"])


def test_weight_params_match_oracle_layout(gpu_wrapper):
    lib = gpu_wrapper.lib
    for cell in (ro.RELU, ro.TANH, ro.LSTM, ro.GRU):
        for mode in (ro.NO_BIAS, ro.SINGLE_INP_BIAS, ro.DOUBLE_BIAS, ro.SINGLE_REC_BIAS):
            desc = ro.RnnDesc(cell, 7, 5, num_layers=3, bidirectional=True, bias_mode=mode)
            d = lib_desc(desc)
            nbytes = ctypes.c_size_t()
            check(lib.snhip_rnn_weight_space_size(ctypes.byref(d), ctypes.byref(nbytes)), "size")
            assert nbytes.value == 4 * ro.weight_space_size(desc)
            for p in range(desc.pseudo_layers):
                for lin in range(desc.lin_layer_ids):
                    off, rows, cols, boff = ctypes.c_longlong(), ctypes.c_int(), ctypes.c_int(), ctypes.c_longlong()
                    check(lib.snhip_rnn_weight_params(ctypes.byref(d), p, lin, ctypes.byref(off), ctypes.byref(rows),
                                                      ctypes.byref(cols), ctypes.byref(boff)), "params")
                    o, (r, c), b = ro.weight_params(desc, p, lin)
                    assert (off.value, rows.value, cols.value, boff.value) == (o, r, c, -1 if b is None else b)


def test_simple_rnn_training_losses_on_device(golden, gpu_wrapper):
    """Tests/NonReg/ParallelRunWithPyTorch.cs:896-953 with both layers run by the RecurrentLayer mirror: the stored
    losses before and after 10 epochs (the reference's tolerance 1e-6 is for cuDNN against PyTorch; 2e-6 here)."""
    from sharpnet_amd import GPUTensor, recurrent
    fx = golden["PyTorch_SimpleRNN"]
    layers = {}

    def layer_for(desc, return_sequences):
        key = (desc.input_size, desc.num_layers, return_sequences)
        if key not in layers:
            layers[key] = recurrent.RecurrentLayer(gpu_wrapper, desc.input_size, desc.hidden_size, desc.cell, desc.bias_mode,
                                                   return_sequences, desc.bidirectional, desc.num_layers)
        return layers[key]

    def forward(desc, x, weights, return_sequences):
        layer = layer_for(desc, return_sequences)
        layer._weightsAndBiases.InitializeFromHostMemory(weights)
        gx = T(gpu_wrapper, x)
        gy = GPUTensor(layer.OutputShape(x.shape[0], x.shape[1]), None, gpu_wrapper)
        layer.ForwardPropagation(gx, gy, True)
        return gy.ToNumpy(), (layer, gx, gy)

    def backward(desc, dy, cache):
        layer, gx, gy = cache
        gdx = GPUTensor(gx.Shape, None, gpu_wrapper)
        layer.BackwardPropagation(gx, gy, T(gpu_wrapper, dy), gdx)
        return gdx.ToNumpy(), layer._weightsAndBiasesGradients.ToNumpy()

    before, after = simple_rnn_chain(fx, forward, backward)
    assert abs(before - fx["loss_before"]) < 2e-6, (before, fx["loss_before"])
    assert abs(after - fx["loss_after"]) < 2e-6, (after, fx["loss_after"])


def mirror_callbacks(gpu_wrapper):
    """forward / backward in the oracle's signature, run by the RecurrentLayer mirror on the device."""
    from sharpnet_amd import GPUTensor, recurrent
    layers = {}

    def forward(desc, x, weights, return_sequences):
        key = (desc.cell, desc.input_size, desc.hidden_size, desc.num_layers, desc.bidirectional, return_sequences)
        if key not in layers:
            layers[key] = recurrent.RecurrentLayer(gpu_wrapper, desc.input_size, desc.hidden_size, desc.cell, desc.bias_mode,
                                                   return_sequences, desc.bidirectional, desc.num_layers)
        layer = layers[key]
        layer._weightsAndBiases.InitializeFromHostMemory(weights)
        gx = T(gpu_wrapper, x)
        gy = GPUTensor(layer.OutputShape(x.shape[0], x.shape[1]), None, gpu_wrapper)
        layer.ForwardPropagation(gx, gy, True)
        return gy.ToNumpy(), (layer, gx, gy)

    def backward(desc, dy, cache):
        layer, gx, gy = cache
        gdx = GPUTensor(gx.Shape, None, gpu_wrapper)
        layer.BackwardPropagation(gx, gy, T(gpu_wrapper, dy), gdx)
        return gdx.ToNumpy(), layer._weightsAndBiasesGradients.ToNumpy()

    return forward, backward


@pytest.mark.parametrize("index", range(13))
def test_zero_weight_layers_reach_the_reference_predictions_on_device(golden, oracle, gpu_wrapper, index):
    """Tests/NonReg/TestNetworkPropagation.cs:1193-1330 with the recurrent layer run by the mirror on the GPU: the
    stored predictions after 10 epochs, within the reference's own tolerance (1e-4)."""
    fx = golden["ZeroWeightRecurrentLayers"]
    case = fx["cases"][index]
    forward, backward = mirror_callbacks(gpu_wrapper)
    before, after = zero_weight_chain(fx, case, forward, backward)
    assert np.max(np.abs(before.reshape(-1) - np.array(case["prediction_before"], np.float32).reshape(-1))) <= fx["tolerance"]
    assert np.max(np.abs(after.reshape(-1) - np.array(case["prediction_after"], np.float32).reshape(-1))) <= fx["tolerance"], case


def test_rnn_argument_checks(gpu_wrapper):
    from sharpnet_amd.hiplib import CublasStatus, RnnDesc
    lib = gpu_wrapper.lib
    d = RnnDesc(cell_mode=2, bias_mode=2, bidirectional=0, num_layers=1, input_size=4, hidden_size=4)
    ws, rs = ctypes.c_size_t(), ctypes.c_size_t()
    check(lib.snhip_rnn_temp_space_sizes(ctypes.byref(d), 1, 2, 3, ctypes.byref(ws), ctypes.byref(rs)), "sizes")
    x = T(gpu_wrapper, np.zeros((2, 3, 4)))
    y = T(gpu_wrapper, np.zeros((2, 3, 4)))
    wt = T(gpu_wrapper, np.zeros(4 * 4 * 8 + 32))
    buf = T(gpu_wrapper, np.zeros(max(ws.value, rs.value) // 4))
    # a reserve buffer that is too small is refused before anything is launched
    st = lib.snhip_rnn_forward(gpu_wrapper.handle, ctypes.byref(d), 1, 2, 3, x.Pointer, y.Pointer, None, None, None, None,
                               wt.Pointer, buf.Pointer, ws.value, buf.Pointer, rs.value - 4)
    assert st == CublasStatus.CUBLAS_STATUS_INVALID_VALUE
    bad = RnnDesc(cell_mode=4, bias_mode=2, bidirectional=0, num_layers=1, input_size=4, hidden_size=4)
    assert lib.snhip_rnn_temp_space_sizes(ctypes.byref(bad), 1, 2, 3, ctypes.byref(ws), ctypes.byref(rs)) == \
        CublasStatus.CUBLAS_STATUS_INVALID_VALUE
    # empty problems are no-ops
    check(lib.snhip_rnn_forward(gpu_wrapper.handle, ctypes.byref(d), 1, 0, 3, None, None, None, None, None, None, None,
                                None, 0, None, 0), "empty batch")


@pytest.mark.parametrize("cell", [ro.LSTM, ro.GRU])
def test_full_size_layer_properties(gpu_wrapper, cell):
    """Benchmark configuration 4's shape (batch 256, 128 steps, 256 -> 512), too large for the oracle: the two forms
    of the time step (one launch / separate launches) agree on values and on every gradient, the final state equals
    the last step of y, and a second run reproduces the first bit for bit."""
    rng = np.random.default_rng(40 + cell)
    B, Tn, I, H = 256, 128, 256, 512
    desc = ro.RnnDesc(cell, input_size=I, hidden_size=H, num_layers=1, bidirectional=False, bias_mode=ro.DOUBLE_BIAS)
    weights = rng.uniform(-0.04, 0.04, ro.weight_space_size(desc)).astype(np.float32)
    x = rng.uniform(-1, 1, (B, Tn, I)).astype(np.float32)
    dy = rng.uniform(-0.01, 0.01, (B, Tn, H)).astype(np.float32)
    one = run_gpu(gpu_wrapper, desc, x, weights, dy)
    again = run_gpu(gpu_wrapper, desc, x, weights, dy)
    for key in ("y", "hy", "dx", "dw"):
        assert np.array_equal(one[key], again[key]), key
    assert np.array_equal(one["hy"][0], one["y"][:, -1, :])
    check(gpu_wrapper.lib.snhip_rnn_set_step_mode(gpu_wrapper.handle, 1), "step mode")
    try:
        two = run_gpu(gpu_wrapper, desc, x, weights, dy)
    finally:
        check(gpu_wrapper.lib.snhip_rnn_set_step_mode(gpu_wrapper.handle, 0), "step mode")
    assert np.max(np.abs(one["y"] - two["y"])) <= 1e-4
    for key in ("dx", "dw", "dhx"):
        scale = max(1.0, float(np.max(np.abs(two[key]))))
        assert np.max(np.abs(one[key] - two[key])) <= 2e-4 * scale, key


@pytest.mark.parametrize("cell", [ro.TANH, ro.LSTM, ro.GRU])
@pytest.mark.parametrize("batch,steps,hidden", [(1, 1, 32), (3, 1, 5), (1, 4, 64), (2, 2, 32)])
def test_degenerate_sequence_shapes(gpu_wrapper, cell, batch, steps, hidden):
    """One sample, one step, two steps: the first / last step special cases of both step forms."""
    rng = np.random.default_rng(batch * 100 + steps * 10 + hidden + cell)
    desc = ro.RnnDesc(cell, input_size=8, hidden_size=hidden, num_layers=2, bidirectional=True, bias_mode=ro.DOUBLE_BIAS)
    weights = rng.uniform(-0.3, 0.3, ro.weight_space_size(desc)).astype(np.float32)
    x = rng.uniform(-1, 1, (batch, steps, 8)).astype(np.float32)
    dy = rng.uniform(-1, 1, (batch, steps, 2 * hidden)).astype(np.float32)
    st = lambda: rng.uniform(-1, 1, (desc.pseudo_layers, batch, hidden)).astype(np.float32)
    hx, cx, dhy, dcy = st(), st(), st(), st()
    if cell != ro.LSTM:
        cx = dcy = None
    got = run_gpu(gpu_wrapper, desc, x, weights, dy, hx, cx, dhy, dcy)
    compare(desc, got, x, weights, dy, hx, cx, dhy, dcy, 3e-5)
    got = run_gpu(gpu_wrapper, desc, x, weights, dy)
    compare(desc, got, x, weights, dy, None, None, None, None, 3e-5)


@pytest.mark.parametrize("cell", [ro.LSTM, ro.GRU])
def test_encoder_decoder_pair(gpu_wrapper, cell):
    """An encoder (last step only, returns its final hidden and cell states as two blocks of one buffer) feeding a
    decoder's initial states, forward and backward through the RecurrentLayer mirror, against the oracle run with
    hx / cx / dhx / dcx passed by hand (RecurrentLayer.cs:318-319,421-423,526-533)."""
    from sharpnet_amd import GPUTensor, recurrent
    rng = np.random.default_rng(90 + cell)
    B, T1, T2, I1, I2, H = 6, 5, 4, 7, 3, 32
    de = ro.RnnDesc(cell, I1, H, 1, False, ro.DOUBLE_BIAS)
    dd = ro.RnnDesc(cell, I2, H, 1, False, ro.DOUBLE_BIAS)
    we = rng.uniform(-0.3, 0.3, ro.weight_space_size(de)).astype(np.float32)
    wd = rng.uniform(-0.3, 0.3, ro.weight_space_size(dd)).astype(np.float32)
    x1 = rng.uniform(-1, 1, (B, T1, I1)).astype(np.float32)
    x2 = rng.uniform(-1, 1, (B, T2, I2)).astype(np.float32)
    dy2 = rng.uniform(-1, 1, (B, T2, H)).astype(np.float32)
    # oracle
    _, hy1, cy1, c1 = ro.rnn_forward(de, x1, we)
    y2, _, _, c2 = ro.rnn_forward(dd, x2, wd, hy1, cy1 if cell == ro.LSTM else None)
    dx2, dw2, dhx2, dcx2 = ro.rnn_backward(dd, dy2, c2)
    dseq = np.zeros((B, T1, H), np.float32)
    dseq[:, -1, :] = dhx2[0]
    dx1, dw1, _, _ = ro.rnn_backward(de, dseq, c1, None, dcx2 if cell == ro.LSTM else None)
    # device
    w = gpu_wrapper
    enc = recurrent.RecurrentLayer(w, I1, H, cell, ro.DOUBLE_BIAS, False, False, 1, isEncoderThatWillBeFollowedByDecoder=True)
    dec = recurrent.RecurrentLayer(w, I2, H, cell, ro.DOUBLE_BIAS, True, False, 1)
    enc._weightsAndBiases.InitializeFromHostMemory(we)
    dec._weightsAndBiases.InitializeFromHostMemory(wd)
    gx1, gx2, gdy2 = T(w, x1), T(w, x2), T(w, dy2)
    assert enc.OutputShape(B, T1) == [B, 2 * H]
    enc_out, d_enc_out = GPUTensor([B, 2 * H], None, w), GPUTensor([B, 2 * H], None, w)
    gy2, gdx2, gdx1 = GPUTensor([B, T2, H], None, w), GPUTensor([B, T2, I2], None, w), GPUTensor([B, T1, I1], None, w)
    enc_out.ZeroMemory()
    d_enc_out.ZeroMemory()
    enc.ForwardPropagation(gx1, enc_out, True)
    dec.ForwardPropagation(gx2, gy2, True, encoderOutput=enc_out)
    dec.BackwardPropagation(gx2, gy2, gdy2, gdx2, encoderOutput=enc_out, dEncoderOutput=d_enc_out)
    enc.BackwardPropagation(gx1, enc_out, d_enc_out, gdx1)
    eo = enc_out.ToNumpy().reshape(-1)
    assert np.max(np.abs(eo[:B * H].reshape(B, H) - hy1[0])) <= 2e-5
    if cell == ro.LSTM:
        assert np.max(np.abs(eo[B * H:].reshape(B, H) - cy1[0])) <= 2e-5
    assert np.max(np.abs(gy2.ToNumpy() - y2)) <= 2e-5
    assert np.max(np.abs(gdx2.ToNumpy() - dx2)) <= 5e-5 * max(1.0, float(np.max(np.abs(dx2))))
    assert np.max(np.abs(dec._weightsAndBiasesGradients.ToNumpy() - dw2)) <= 5e-5 * max(1.0, float(np.max(np.abs(dw2))))
    assert np.max(np.abs(gdx1.ToNumpy() - dx1)) <= 5e-5 * max(1.0, float(np.max(np.abs(dx1))))
    assert np.max(np.abs(enc._weightsAndBiasesGradients.ToNumpy() - dw1)) <= 5e-5 * max(1.0, float(np.max(np.abs(dw1))))


def dropout_calls(w):
    n = ctypes.c_ulonglong()
    check(w.lib.snhip_rnn_get_dropout_calls(w.handle, ctypes.byref(n)), "snhip_rnn_get_dropout_calls")
    return n.value


@pytest.mark.parametrize("batch,steps,hidden,bidirectional,layers", [(3, 5, 6, False, 2), (4, 3, 5, True, 3), (1, 1, 3, False, 2),
                                                                     (7, 9, 33, True, 2)])
def test_dropout_mask_is_the_documented_generator(gpu_wrapper, batch, steps, hidden, bidirectional, layers):
    """snhip_rnn_dropout_mask against the oracle's restatement of the documented stream (Philox4x32-10, itself pinned
    by the published known-answer vectors): bit for bit, for several seeds, call numbers and boundaries, element counts
    that are and are not multiples of four."""
    from sharpnet_amd import GPUTensor
    w = gpu_wrapper
    desc = ro.RnnDesc(ro.LSTM, input_size=4, hidden_size=hidden, num_layers=layers, bidirectional=bidirectional)
    width = desc.dirs * hidden
    out = GPUTensor([batch, steps, width], None, w)
    try:
        for seed, call, rate in [(0, 0, 0.5), (12345678901234567, 3, 0.2), (2 ** 63 + 5, 2 ** 32 - 1, 0.9)]:
            check(w.lib.snhip_rnn_set_dropout_seed(w.handle, seed), "seed")
            d = lib_desc(desc, rate)
            for boundary in range(layers - 1):
                out.SetValue(float("nan"))
                check(w.lib.snhip_rnn_dropout_mask(w.handle, ctypes.byref(d), batch, steps, call, boundary, out.Pointer), "mask")
                want = ro.dropout_mask(seed, call, boundary, rate, batch, steps, width)
                assert np.array_equal(out.ToNumpy(), want), (seed, call, boundary)
        d = lib_desc(desc, 0.5)
        assert w.lib.snhip_rnn_dropout_mask(w.handle, ctypes.byref(d), batch, steps, 0, layers - 1, out.Pointer) == 7
        assert w.lib.snhip_rnn_dropout_mask(w.handle, ctypes.byref(d), batch, steps, 0, -1, out.Pointer) == 7
    finally:
        check(w.lib.snhip_rnn_set_dropout_seed(w.handle, 0), "seed")
        out.Dispose()


@pytest.mark.parametrize("cell", [ro.TANH, ro.LSTM, ro.GRU])
@pytest.mark.parametrize("bidirectional,layers,hidden", [(False, 2, 5), (True, 3, 4), (False, 3, 32), (True, 2, 36)])
def test_dropout_between_stacked_layers(gpu_wrapper, cell, bidirectional, layers, hidden):
    """Training with RNNDescriptor.dropoutRate > 0 and more than one layer: the call draws the masks numbered by the
    handle's call count; with those masks (regenerated on the host from the documented stream) the oracle gives the same
    outputs, final states and gradients.  The masks belong to the forward call: another layer's training call between
    this layer's forward and backward calls changes nothing.  Inference ignores the rate; so does a repeat of the
    call not ignore the count: the second call draws other masks."""
    w = gpu_wrapper
    rng = np.random.default_rng(5000 + cell * 37 + layers * 5 + hidden + int(bidirectional))
    rate, seed = 0.35, 77
    desc = ro.RnnDesc(cell, input_size=6, hidden_size=hidden, num_layers=layers, bidirectional=bidirectional)
    B, Tn = 5, 7
    width = desc.dirs * hidden
    weights = rng.uniform(-0.5, 0.5, ro.weight_space_size(desc)).astype(np.float32)
    x = rng.uniform(-1, 1, (B, Tn, 6)).astype(np.float32)
    dy = rng.uniform(-1, 1, (B, Tn, width)).astype(np.float32)
    st = lambda: rng.uniform(-1, 1, (desc.pseudo_layers, B, hidden)).astype(np.float32)
    hx, cx, dhy, dcy = st(), st(), st(), st()
    if cell != ro.LSTM:
        cx = dcy = None
    other = ro.RnnDesc(ro.GRU, input_size=3, hidden_size=4, num_layers=2)
    other_w = rng.uniform(-0.5, 0.5, ro.weight_space_size(other)).astype(np.float32)

    def another_layers_training_call():
        run_gpu(w, other, rng.uniform(-1, 1, (2, 3, 3)).astype(np.float32), other_w,
                rng.uniform(-1, 1, (2, 3, 4)).astype(np.float32), dropout=0.5)
    try:
        check(w.lib.snhip_rnn_set_dropout_seed(w.handle, seed), "seed")
        assert dropout_calls(w) == 0
        first = None
        for call in range(2):
            print("rnn dropout", cell, bidirectional, layers, hidden, "call", call, flush=True)
            got = run_gpu(w, desc, x, weights, dy, hx, cx, dhy, dcy, dropout=rate,
                          between=another_layers_training_call if call == 1 else None)
            masks = [ro.dropout_mask(seed, call, b, rate, B, Tn, width) for b in range(layers - 1)]
            compare(desc, got, x, weights, dy, hx, cx, dhy, dcy, 3e-5, masks=masks)
            if first is None:
                first = got
            else:
                assert np.max(np.abs(first["y"] - got["y"])) > 1e-4           # other masks
        assert dropout_calls(w) == 3                                           # two calls here, one of the other layer
        # the masks act: the result without dropout is another one; inference with the same descriptor is that one
        plain = run_gpu(w, desc, x, weights, dy, hx, cx, dhy, dcy)
        assert np.max(np.abs(plain["y"] - first["y"])) > 1e-4
        infer = run_gpu(w, desc, x, weights, dy, hx, cx, training=False, dropout=rate)
        assert np.array_equal(infer["y"], plain["y"]) and np.array_equal(infer["hy"], plain["hy"])
        assert dropout_calls(w) == 3
        # same seed, same call number: the same masks again
        check(w.lib.snhip_rnn_set_dropout_seed(w.handle, seed), "seed")
        again = run_gpu(w, desc, x, weights, dy, hx, cx, dhy, dcy, dropout=rate)
        for k in ("y", "hy", "dx", "dw"):
            assert np.array_equal(again[k], first[k]), k
    finally:
        check(w.lib.snhip_rnn_set_dropout_seed(w.handle, 0), "seed")
