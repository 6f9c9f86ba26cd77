"""The five benchmark configurations at their real shapes, checked through size-independent properties:
sampled rows / columns / batches of the result against the oracle on the same seeded inputs (any row block of
C = op(A) op(B) is itself a Dot of a row block of op(A) with B), NaN-prefilled destinations, and linearity in beta."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu


def bound(K, a, b, extra=0.0):
    return 1e-4 * np.sqrt(max(K, 1)) * float(np.max(np.abs(a))) * float(np.max(np.abs(b))) + extra


def sampled_rows_check(oracle, w, g, a, b, c, nrows=8, seed=0, bf16=False):
    """Runs g on the device and compares `nrows` sampled rows with the oracle."""
    from sharpnet_amd import GPUTensor
    ga, gb = GPUTensor(list(a.shape), a, w), GPUTensor(list(b.shape), b, w)
    gc = GPUTensor([g.M, g.N], c, w) if c is not None else GPUTensor([g.M, g.N], None, w)
    if c is None:
        gc.SetValue(float("nan"))
    gc.Dot(ga, g.tA, gb, g.tB, g.alpha, g.beta)
    got = gc.ToNumpy()
    assert np.all(np.isfinite(got))
    rows = np.sort(np.random.default_rng(seed).choice(g.M, min(nrows, g.M), replace=False))
    opa_rows = np.ascontiguousarray(a[:, rows].T if g.tA else a[rows])       # rows of op(A), as a non-transposed operand
    if bf16:
        opa_rows, bb = oracle.round_to_bf16(opa_rows), oracle.round_to_bf16(b)
    else:
        bb = b
    ref = oracle.dot(opa_rows, False, bb, g.tB, g.alpha, g.beta, c[rows] if c is not None else None)
    err = float(np.max(np.abs(got[rows] - ref)))
    assert err <= bound(g.K, a, b, 1e-6 * (float(np.max(np.abs(c))) if c is not None else 0)), (g.label(), err)
    for t in (ga, gb, gc):
        t.Dispose()
    return got


def test_config2_sweep_all_sizes_transposes_betas(oracle, gpu_wrapper):
    """Square and ragged sweep incl. 8192^3; the same A/B buffers serve all transposes of a square size."""
    from sharpnet_amd import workloads as wl
    rng = np.random.default_rng(2)
    for (M, N, K) in wl.SWEEP_SIZES:
        bufs = {}
        for tA in (False, True):
            for tB in (False, True):
                sa = (K, M) if tA else (M, K)
                sb = (N, K) if tB else (K, N)
                for s in (sa, sb):
                    if s not in bufs:
                        bufs[s] = rng.uniform(-1, 1, s).astype(np.float32)
                a, b = bufs[sa], bufs[sb]
                if a is b:                                     # square sizes: keep A and B distinct
                    b = bufs.setdefault((sb, "b"), rng.uniform(-1, 1, sb).astype(np.float32))
                for beta in (0.0, 1.0):
                    c = rng.uniform(-1, 1, (M, N)).astype(np.float32) if beta else None
                    sampled_rows_check(oracle, gpu_wrapper, wl.Gemm(M, N, K, tA, tB, 1.0, beta), a, b, c, nrows=6)


def test_config2_headline_bf16(oracle, gpu_wrapper):
    """The headline size (8192^3) in bf16-input arithmetic, all four transposes with fp32 storage, and the NT form
    with operands stored as bf16 (the kernel fed by global -> LDS direct loads): sampled rows against the oracle on
    bf16-rounded inputs (fp32 bound) and against the fp32 result (1e-2 relative)."""
    from sharpnet_amd import GPUTensor, workloads as wl
    from sharpnet_amd.hiplib import check_status
    w = gpu_wrapper
    S = 8192
    rng = np.random.default_rng(22)
    a, b = rng.uniform(-1, 1, (S, S)).astype(np.float32), rng.uniform(-1, 1, (S, S)).astype(np.float32)
    try:
        w.set_math_mode(w.MATH_BF16_INPUT)
        for tA, tB in [(False, False), (False, True), (True, False), (True, True)]:
            print("bf16-input 8192^3", tA, tB, flush=True)
            got = sampled_rows_check(oracle, w, wl.Gemm(S, S, S, tA, tB), a, b, None, nrows=6, bf16=True)
            # 1e-2 relative to the fp32 result as well
            rows = slice(0, 4)
            ref32 = oracle.dot(np.ascontiguousarray(a[:, rows].T if tA else a[rows]), False, b, tB)
            assert np.max(np.abs(got[rows] - ref32)) / np.max(np.abs(ref32)) <= 1e-2
            del got
    finally:
        w.set_math_mode(w.MATH_FP32)
    # operands stored as bf16, A plain and B transposed
    print("bf16-stored 8192^3 NT", flush=True)
    ga, gb, gc = GPUTensor([S, S], a, w), GPUTensor([S, S], b, w), GPUTensor([S, S], None, w)
    pa, pb = w.allocate(2 * S * S), w.allocate(2 * S * S)
    check_status(w.lib.snhip_convert_f32_to_bf16(w.handle, ga.Pointer, pa, S * S))
    check_status(w.lib.snhip_convert_f32_to_bf16(w.handle, gb.Pointer, pb, S * S))
    gc.SetValue(float("nan"))
    check_status(w.lib.snhip_dot_bf16_stored(w.handle, pa, S, S, 0, pb, S, S, 1, gc.Pointer, 1.0, 0.0, None))
    kinds = {c["id"]: c["kind"] for c in w.configs()}
    assert kinds[w.last_tuning()[0]] == "bf16-stored-dtl"
    got = gc.ToNumpy()
    assert np.all(np.isfinite(got))
    rows = np.sort(rng.choice(S, 6, replace=False))
    ref = oracle.dot(oracle.round_to_bf16(a[rows]), False, oracle.round_to_bf16(b), True)
    assert np.max(np.abs(got[rows] - ref)) <= bound(S, a, b)
    w.release(pa, 2 * S * S)
    w.release(pb, 2 * S * S)
    for t in (ga, gb, gc):
        t.Dispose()


def test_config3_mlp_step_gemms(oracle, gpu_wrapper):
    """Batch 4096, 3072 -> 4096 -> 4096 -> 1000: every forward (+bias), dW and dX product at full shape."""
    from sharpnet_amd import GPUTensor, workloads as wl
    w = gpu_wrapper
    rng = np.random.default_rng(3)
    for g in wl.mlp_gemms():
        a = rng.uniform(0, 1, g.a_shape).astype(np.float32) if g.name.startswith("fwd") else \
            rng.normal(0, 1e-3, g.a_shape).astype(np.float32)
        lim = np.sqrt(6.0 / (g.N + g.K))
        b = rng.uniform(-lim, lim, g.b_shape).astype(np.float32)
        if not g.bias:
            sampled_rows_check(oracle, w, g, a, b, None, nrows=4)
            continue
        bias = rng.uniform(-1, 1, g.N).astype(np.float32)
        ga, gb, gbias = GPUTensor(list(a.shape), a, w), GPUTensor(list(b.shape), b, w), GPUTensor([g.N], bias, w)
        gc = GPUTensor([g.M, g.N], None, w)
        gc.SetValue(float("nan"))
        gc.DotRowMajor(ga, g.tA, gb, g.tB, 1.0, 0.0, bias=gbias)
        rows = np.array([0, 1, g.M // 2, g.M - 1])
        ref = oracle.dense_forward(a[rows], b, bias)
        assert np.max(np.abs(gc.ToNumpy()[rows] - ref)) <= bound(g.K, a, b, 1e-6), g.label()


def test_config4_lstm_projections(oracle, gpu_wrapper):
    """Input projection (32768,2048,256) once, then sequential recurrent steps (256,2048,512) accumulating with beta=1."""
    from sharpnet_amd import GPUTensor, workloads as wl
    w = gpu_wrapper
    d = wl.lstm_inputs(seed=4)
    proj, rec, _ = wl.lstm_gemms()
    sampled_rows_check(oracle, w, proj, d["x"], d["w"], None, nrows=8)
    _, _, steps = wl.lstm_gemms()
    assert steps == 128                         # the whole chain of sequential beta = 1 products
    rng = np.random.default_rng(44)
    hs = [np.tanh(rng.normal(0, 1, d["h"].shape)).astype(np.float32) for _ in range(steps)]
    gates0 = rng.normal(0, 1, (rec.M, rec.N)).astype(np.float32)
    gg, gu = GPUTensor([rec.M, rec.N], gates0, w), GPUTensor(list(d["u"].shape), d["u"], w)
    ref = gates0.astype(np.float64)
    for h in hs:
        gh = GPUTensor(list(h.shape), h, w)
        gg.Dot(gh, False, gu, False, 1.0, 1.0)
        gh.Dispose()
        ref = oracle.dot_f64(h, False, d["u"], False, 1.0, 1.0, ref)
    assert np.max(np.abs(gg.ToNumpy() - ref)) <= steps * bound(rec.K, hs[0], d["u"], 1e-6)


@pytest.mark.parametrize("bf16", [False, True])
def test_config5_attention_batched(oracle, gpu_wrapper, bf16):
    """512 batches x (256,256,64): S = Q K^T / 8, P = softmax(S) on the host, O = P V; sampled batches vs the oracle."""
    from sharpnet_amd import GPUTensor, workloads as wl
    w = gpu_wrapper
    d = wl.attention_inputs(seed=5)
    q, k, v = d["q"], d["k"], d["v"]
    batch, T, dim = q.shape
    gq, gk, gv = (GPUTensor(list(t.shape), t, w) for t in (q, k, v))
    gs = GPUTensor([batch, T, T], None, w)
    gs.SetValue(float("nan"))
    rnd = oracle.round_to_bf16 if bf16 else (lambda t: t)
    try:
        if bf16:
            w.set_math_mode(w.MATH_BF16_INPUT)
        gs.BatchMatrixMultiplication(gq, False, gk, True, 0.125, 0.0)
        s = gs.ToNumpy()
        sel = [0, 1, 255, 511]
        ref_s = oracle.bmm(rnd(q[sel]), False, rnd(k[sel]), True, 0.125)
        assert np.max(np.abs(s[sel] - ref_s)) <= bound(dim, q, k) * 0.125 + 1e-6
        p = oracle.softmax_last_dim(s)
        gp, go = GPUTensor([batch, T, T], p, w), GPUTensor([batch, T, dim], None, w)
        go.SetValue(float("nan"))
        go.BatchMatrixMultiplication(gp, False, gv, False, 1.0, 0.0)
        o = go.ToNumpy()
        assert np.all(np.isfinite(o)) and np.all(np.isfinite(s))
        ref_o = oracle.bmm(rnd(p[sel]), False, rnd(v[sel]), False)
        assert np.max(np.abs(o[sel] - ref_o)) <= bound(T, p, v)
        if bf16:   # and within 1e-2 relative of the fp32 result
            ref32 = oracle.bmm(p[sel], False, v[sel], False)
            assert np.max(np.abs(o[sel] - ref32)) / np.max(np.abs(ref32)) <= 1e-2
    finally:
        w.set_math_mode(w.MATH_FP32)


def test_calls_can_be_recorded_into_a_hip_graph_and_replayed(oracle, gpu_wrapper):
    """An LSTM forward + backward, a Dense forward (fused bias + ReLU), a split-K product, a fill and the one-launch
    attention, recorded into a HIP graph on a capturing stream and replayed three times with eager work and synchronisations in between: every
    replay must reproduce the eager results (the calls launch kernels only: no allocation once the split-K workspace
    exists, no memset nodes)."""
    import ctypes
    from sharpnet_amd import GPUTensor, linear, attention
    from sharpnet_amd.hiplib import check_status
    from tests.helpers import random_tensor
    w = gpu_wrapper
    rng = np.random.default_rng(77)
    x, W, b = random_tensor(rng, (96, 300), -1, 1), random_tensor(rng, (130, 300), -0.2, 0.2), random_tensor(rng, (130,), -1, 1)
    a2, b2 = random_tensor(rng, (64, 4096), -1, 1), random_tensor(rng, (4096, 48), -1, 1)      # long K: split-K path
    q = random_tensor(rng, (6, 50, 16), -1, 1)
    gx, gW, gb, ga2, gb2, gq = (GPUTensor(list(t.shape), t, w) for t in (x, W, b, a2, b2, q))
    gy, gc2, go, gfill = GPUTensor([96, 130], None, w), GPUTensor([64, 48], None, w), GPUTensor([6, 50, 16], None, w), \
        GPUTensor([1000], None, w)

    # a small LSTM (hidden size 32: the one-launch step kernels) with caller-owned workspace and reserve buffers
    from sharpnet_amd.hiplib import RnnDesc
    rd = RnnDesc(cell_mode=2, bias_mode=2, bidirectional=1, num_layers=1, input_size=12, hidden_size=32)
    nb, wsb, rsb = ctypes.c_size_t(), ctypes.c_size_t(), ctypes.c_size_t()
    check_status(w.lib.snhip_rnn_weight_space_size(ctypes.byref(rd), ctypes.byref(nb)), "rnn weight space")
    check_status(w.lib.snhip_rnn_temp_space_sizes(ctypes.byref(rd), 1, 9, 5, ctypes.byref(wsb), ctypes.byref(rsb)), "rnn sizes")
    rx, rw, rdy = random_tensor(rng, (9, 5, 12), -1, 1), random_tensor(rng, (nb.value // 4,), -0.3, 0.3), \
        random_tensor(rng, (9, 5, 64), -1, 1)
    grx, grw, grdy = (GPUTensor(list(t.shape), t, w) for t in (rx, rw, rdy))
    gry, grdx, grws, grrs = GPUTensor([9, 5, 64], None, w), GPUTensor([9, 5, 12], None, w), \
        GPUTensor([wsb.value // 4], None, w), GPUTensor([rsb.value // 4], None, w)

    def rnn():
        check_status(w.lib.snhip_rnn_forward(w.handle, ctypes.byref(rd), 1, 9, 5, grx.Pointer, gry.Pointer, None, None, None,
                                             None, grw.Pointer, grws.Pointer, wsb.value, grrs.Pointer, rsb.value), "rnn forward")
        check_status(w.lib.snhip_rnn_backward_data(w.handle, ctypes.byref(rd), 9, 5, gry.Pointer, grdy.Pointer, grdx.Pointer,
                                                   None, None, None, None, None, None, grw.Pointer, grws.Pointer, wsb.value,
                                                   grrs.Pointer, rsb.value), "rnn backward")

    def work():
        rnn()
        linear.DenseForwardPropagation(gy, gx, gW, gb, False, activation="CUDNN_ACTIVATION_RELU")
        gc2.Dot(ga2, False, gb2, False, 1.0, 0.0)
        gfill.SetValue(3.5)
        assert attention.fused_attention_forward(gq, gq, gq, go, None, batch=6, heads=1, tq=50, tkv=50, dk=16, dv=16,
                                                 scale=0.25, is_causal=True, packed=False)

    def results():
        return [t.ToNumpy().copy() for t in (gy, gc2, go, gfill, gry, grdx)]

    work()                                   # eager: also sizes the split-K workspace
    w.synchronize()
    assert w.last_tuning() is not None
    eager = results()
    assert np.max(np.abs(eager[0] - oracle.activation_forward(oracle.dense_forward(x, W, b), "relu"))) < 1e-3
    assert np.all(eager[3] == 3.5)

    # the HIP runtime the library itself is linked against (same shared object, found by soname)
    hip = ctypes.CDLL("libamdhip64.so")
    vp = ctypes.c_void_p
    for name, args in (("hipStreamBeginCapture", [vp, ctypes.c_int]), ("hipStreamEndCapture", [vp, ctypes.POINTER(vp)]),
                       ("hipGraphInstantiate", [ctypes.POINTER(vp), vp, vp, vp, ctypes.c_size_t]),
                       ("hipGraphLaunch", [vp, vp]), ("hipGraphExecDestroy", [vp]), ("hipGraphDestroy", [vp])):
        getattr(hip, name).argtypes = args
        getattr(hip, name).restype = ctypes.c_int
    stream = vp()
    check_status(w.lib.snhip_stream_create(ctypes.byref(stream)), "snhip_stream_create")
    check_status(w.lib.snhip_set_stream(w.handle, stream), "snhip_set_stream")
    graph, graph_exec = vp(), vp()
    try:
        assert hip.hipStreamBeginCapture(stream, 0) == 0          # hipStreamCaptureModeGlobal
        try:
            work()
        finally:
            assert hip.hipStreamEndCapture(stream, ctypes.byref(graph)) == 0
        assert hip.hipGraphInstantiate(ctypes.byref(graph_exec), graph, None, None, 0) == 0
        for rep in range(3):
            for t in (gy, gc2, go, gfill, gry, grdx):   # eager work between replays: wipe the outputs on the same stream
                t.SetValue(float("nan"))
            w.synchronize()
            assert hip.hipGraphLaunch(graph_exec, stream) == 0
            w.synchronize()
            for got, want in zip(results(), eager):
                assert np.array_equal(got, want), rep
    finally:
        check_status(w.lib.snhip_set_stream(w.handle, None), "snhip_set_stream")
        if graph_exec:
            hip.hipGraphExecDestroy(graph_exec)
        if graph:
            hip.hipGraphDestroy(graph)
        check_status(w.lib.snhip_stream_destroy(stream), "snhip_stream_destroy")


def test_workspace_can_be_reserved_ahead_of_time(oracle, gpu_wrapper):
    """snhip_reserve_workspace sizes the handle's scratch buffer so that later calls neither synchronise nor allocate:
    a split-K product whose partial sums fit leaves the buffer as reserved, and gives the result it gives otherwise."""
    import ctypes
    from sharpnet_amd import GPUTensor
    from sharpnet_amd.hiplib import check_status, CublasStatus
    from tests.helpers import random_tensor
    w = gpu_wrapper
    size = ctypes.c_size_t()
    check_status(w.lib.snhip_get_workspace_size(w.handle, ctypes.byref(size)))
    want = max(size.value, 48 << 20) + (1 << 20)
    check_status(w.lib.snhip_reserve_workspace(w.handle, want))
    check_status(w.lib.snhip_get_workspace_size(w.handle, ctypes.byref(size)))
    assert size.value == want
    check_status(w.lib.snhip_reserve_workspace(w.handle, 1024))                 # never shrinks
    check_status(w.lib.snhip_get_workspace_size(w.handle, ctypes.byref(size)))
    assert size.value == want
    assert w.lib.snhip_reserve_workspace(w.handle, (1 << 30) + 1) == CublasStatus.CUBLAS_STATUS_INVALID_VALUE
    rng = np.random.default_rng(5)
    a, b = random_tensor(rng, (512, 8192), -1, 1), random_tensor(rng, (8192, 64), -1, 1)
    ga, gb, gc = GPUTensor(a.shape, a, w), GPUTensor(b.shape, b, w), GPUTensor([512, 64], None, w)
    gc.SetValue(float("nan"))
    gc.Dot(ga, False, gb, False, 1.0, 0.0)
    assert w.last_tuning()[1] > 1                                             # split along K: the buffer is in use
    assert np.max(np.abs(gc.ToNumpy() - oracle.dot(a, False, b, False))) <= 1e-4 * np.sqrt(8192)
    check_status(w.lib.snhip_get_workspace_size(w.handle, ctypes.byref(size)))
    assert size.value == want
