"""GPU tests of the callers of Dot: Linear forward/backward and scaled-dot-product attention,
driven through the host mirrors of the reference's layer code and checked against the oracle
and against the losses the reference's own tests store."""
import numpy as np
import pytest

from tests.helpers import numpy_array_for_tests, y_numpy_array_for_tests, random_tensor, sigmoid

pytestmark = pytest.mark.gpu


def T(w, a):
    from sharpnet_amd import GPUTensor
    a = np.asarray(a, np.float32)
    return GPUTensor(list(a.shape), a, w)


def bound(K, a, b, extra=0.0):
    return 1e-4 * np.sqrt(max(K, 1)) * float(np.max(np.abs(a))) * float(np.max(np.abs(b))) + extra


def test_dense_layer_forward_backward_config1(oracle, gpu_wrapper):
    """Single Dense layer fwd+bwd, batch 128, 784 -> 256 (reference layout W:(out,in), Linear.cs:125-191)."""
    from sharpnet_amd import GPUTensor, workloads as wl, linear
    d = wl.dense_layer_inputs(seed=1)
    x, W, dy = d["x"], d["w_out_in"], d["dy"]
    bias = np.linspace(-0.5, 0.5, W.shape[0]).astype(np.float32)
    gx, gW, gb, gdy = T(gpu_wrapper, x), T(gpu_wrapper, W), T(gpu_wrapper, bias), T(gpu_wrapper, dy)
    ref_y = oracle.dense_forward(x, W, bias)
    for fuse in (True, False):
        gy = GPUTensor([x.shape[0], W.shape[0]], None, gpu_wrapper)
        gy.SetValue(float("nan"))
        linear.DenseForwardPropagation(gy, gx, gW, gb, False, fused=fuse)
        assert np.max(np.abs(gy.ToNumpy() - ref_y)) <= bound(x.shape[1], x, W, 1e-6)
    gdW, gdb, gdx = GPUTensor(list(W.shape), None, gpu_wrapper), GPUTensor([W.shape[0]], None, gpu_wrapper), \
        GPUTensor(list(x.shape), None, gpu_wrapper)
    for t in (gdW, gdb, gdx):
        t.SetValue(float("nan"))
    for fused in (True, False):
        for t in (gdW, gdb, gdx):
            t.SetValue(float("nan"))
        linear.DenseBackwardPropagation(gdx, gdW, gdb, gx, gdy, gW, fused=fused)   # SharpNet mode: multiplier 1/batch
        rdW, rdb, rdx = oracle.dense_backward(x, dy, W, multiplier=1.0 / x.shape[0])
        assert np.max(np.abs(gdW.ToNumpy() - rdW)) <= bound(x.shape[0], dy, x) / x.shape[0] + 1e-9
        assert np.max(np.abs(gdb.ToNumpy() - rdb)) <= 1e-5 * np.sqrt(x.shape[0]) * np.max(np.abs(dy)) + 1e-7
        assert np.max(np.abs(gdx.ToNumpy() - rdx)) <= bound(W.shape[0], dy, W)
        # weight decay (PyTorch mode: dW += batch*wd*W, Linear.cs:168-181) and the input-layer shortcut
        gdx.SetValue(7.0)
        linear.DenseBackwardPropagation(gdx, gdW, gdb, gx, gdy, gW, bias_1D=gb, compatibility_mode="PyTorch",
                                        use_weight_decay_in_backpropagation=True, weight_decay=0.01,
                                        prevLayerIsInputLayer=True, fused=fused)
        alpha = 1 * x.shape[0] * 0.01
        rdW2, rdb2, _ = oracle.dense_backward(x, dy, W, multiplier=1.0, weight_decay_alpha=alpha)
        assert np.max(np.abs(gdW.ToNumpy() - rdW2)) <= bound(x.shape[0], dy, x) + 1e-5
        assert np.max(np.abs(gdb.ToNumpy() - (rdb2 + alpha * bias))) <= 1e-4
        assert np.all(gdx.ToNumpy() == 7.0)                              # dx untouched when the previous layer is the input


def test_dense_layer_config1_in_out_layout(oracle, gpu_wrapper):
    """The same layer in the (in, out) weight layout of the benchmark's wording and of the TensorFlow-era vectors
    (Tests/NonReg/TestNetworkPropagation.cs:80-105): Y = X.W + b (NN with the bias in the same launch),
    dW = X^T.dY (TN: 784 x 256 x 128), dX = dY.W^T (NT), at the full shape, NaN-prefilled destinations."""
    from sharpnet_amd import GPUTensor, workloads as wl
    w = gpu_wrapper
    d = wl.dense_layer_inputs(seed=1)
    x, dy = d["x"], d["dy"]
    W = np.ascontiguousarray(d["w_out_in"].T)                       # (784, 256)
    bias = np.linspace(-0.5, 0.5, W.shape[1]).astype(np.float32)
    gx, gW, gb, gdy = T(w, x), T(w, W), T(w, bias), T(w, dy)
    gy, gdW, gdx = GPUTensor([128, 256], None, w), GPUTensor([784, 256], None, w), GPUTensor([128, 784], None, w)
    for t in (gy, gdW, gdx):
        t.SetValue(float("nan"))
    gy.DotRowMajor(gx, False, gW, False, 1.0, 0.0, bias=gb)
    assert np.max(np.abs(gy.ToNumpy() - (oracle.dot(x, False, W, False) + bias))) <= bound(784, x, W, 1e-6)
    # the oracle's Linear forward on the (out, in) copy of the same weights is the same function
    assert np.max(np.abs(gy.ToNumpy() - oracle.dense_forward(x, d["w_out_in"], bias))) <= bound(784, x, W, 1e-6)
    gdW.Dot(gx, True, gdy, False, 1.0 / 128, 0.0)
    assert np.max(np.abs(gdW.ToNumpy() - oracle.dot(x, True, dy, False, 1.0 / 128))) <= bound(128, x, dy) / 128 + 1e-9
    gdx.Dot(gdy, False, gW, True, 1.0, 0.0)
    assert np.max(np.abs(gdx.ToNumpy() - oracle.dot(dy, False, W, True))) <= bound(256, dy, W)
    # consistent with the (out, in) layer: dW here is the transpose of dW there, dX is the same
    _, _, rdx = oracle.dense_backward(x, dy, d["w_out_in"], multiplier=1.0 / 128)
    assert np.max(np.abs(gdx.ToNumpy() - rdx)) <= bound(256, dy, W)


ACTS = [("relu", "CUDNN_ACTIVATION_RELU", 0.0), ("leaky_relu", "CUDNN_ACTIVATION_LEAKY_RELU", 0.1),
        ("leaky_relu", "CUDNN_ACTIVATION_LEAKY_RELU", 0.3), ("sigmoid", "CUDNN_ACTIVATION_SIGMOID", 0.0),
        ("tanh", "CUDNN_ACTIVATION_TANH", 0.0)]


@pytest.mark.parametrize("mode,cudnn,slope", ACTS)
def test_activation_fused_into_forward_and_stand_alone(oracle, gpu_wrapper, mode, cudnn, slope):
    """Linear + ActivationLayer as one launch (write-out of the GEMM), on direct and split-K paths and on a ragged
    shape, against the oracle; then ActivationForward / ActivationBackward by themselves."""
    from sharpnet_amd import GPUTensor, linear
    rng = np.random.default_rng(11)
    try:
        for (rows, fin, fout, tuning) in ((128, 784, 256, (-1, 0)), (77, 301, 130, (-1, 0)), (64, 1024, 96, (6, 4)),
                                          (300, 200, 515, (3, 1)), (256, 64, 512, (0, 1))):
            x, W, b = random_tensor(rng, (rows, fin), -1, 1), random_tensor(rng, (fout, fin), -0.2, 0.2), \
                random_tensor(rng, (fout,), -1, 1)
            gx, gW, gb = T(gpu_wrapper, x), T(gpu_wrapper, W), T(gpu_wrapper, b)
            gy = GPUTensor([rows, fout], None, gpu_wrapper)
            gy.SetValue(float("nan"))
            gpu_wrapper.set_tuning(*tuning)
            linear.DenseForwardPropagation(gy, gx, gW, gb, False, activation=cudnn, activation_parameter=slope)
            want = oracle.activation_forward(oracle.dense_forward(x, W, b), mode, slope)
            assert np.max(np.abs(gy.ToNumpy() - want)) <= bound(fin, x, W, 1e-6), (rows, fin, fout, tuning)
            gy2 = GPUTensor([rows, fout], None, gpu_wrapper)
            linear.DenseForwardPropagation(gy2, gx, gW, gb, False, fused=False, activation=cudnn,
                                           activation_parameter=slope)
            assert np.max(np.abs(gy2.ToNumpy() - want)) <= bound(fin, x, W, 1e-6)
    finally:
        gpu_wrapper.set_tuning(-1, 0)
    v = random_tensor(rng, (5, 3, 41), -3, 3)
    dy = random_tensor(rng, v.shape, -1, 1)
    gv, gdy = T(gpu_wrapper, v), T(gpu_wrapper, dy)
    gout, gdx = GPUTensor(list(v.shape), None, gpu_wrapper), GPUTensor(list(v.shape), None, gpu_wrapper)
    gv.ActivationForward(cudnn, slope, gout)
    yy = oracle.activation_forward(v, mode, slope)
    assert np.max(np.abs(gout.ToNumpy() - yy)) <= 2e-6
    gout.ActivationBackward(cudnn, slope, gdy, gdx)
    assert np.max(np.abs(gdx.ToNumpy() - oracle.activation_backward(gout.ToNumpy(), dy, mode, slope))) <= 2e-6


def test_bias_gradient_rides_along_with_dW_for_every_tile_configuration(oracle, gpu_wrapper):
    """snhip_gemm_ex colsum (= Compute_BiasGradient_from_dy of the dy the dW product reads) with gamma*D (weight decay),
    for each fp32 tile configuration, with and without split-K (the split-K case takes the stand-alone kernel),
    a strided batch, ragged sizes and padded leading dimensions."""
    from sharpnet_amd import GPUTensor
    rng = np.random.default_rng(12)
    w = gpu_wrapper
    fp32_cfgs = [c["id"] for c in w.configs() if c["kind"] == "fp32"]
    try:
        for cfg in fp32_cfgs + [-1]:
            for splitk in ((1, 2) if cfg >= 0 else (0,)):
                for (out_f, in_f, rows, batch) in ((333, 190, 517, 1), (64, 64, 32, 3), (700, 130, 96, 2)):
                    lda, ldb, ldc, ldd = out_f + 3, in_f + 1, in_f + 2, in_f + 5
                    dy = random_tensor(rng, (batch, rows, lda), -1, 1)
                    x = random_tensor(rng, (batch, rows, ldb), -1, 1)
                    Wm = random_tensor(rng, (batch, out_f, ldd), -1, 1)
                    c0 = random_tensor(rng, (batch, out_f, ldc), -1, 1)
                    gdy, gx, gWm, gc = T(w, dy), T(w, x), T(w, Wm), T(w, c0)
                    gcs = GPUTensor([batch, out_f], None, w)
                    gcs.SetValue(float("nan"))
                    w.set_tuning(cfg, splitk)
                    gc.GemmEx(transA=1, M=out_f, N=in_f, K=rows, alpha=0.5, beta=0.25, A=gdy, lda=lda, strideA=rows * lda,
                              B=gx, ldb=ldb, strideB=rows * ldb, ldc=ldc, strideC=out_f * ldc, batch=batch,
                              D=gWm, ldd=ldd, strideD=out_f * ldd, gamma=0.75, colsum=gcs)
                    got, cs = gc.ToNumpy(), gcs.ToNumpy()
                    for z in range(batch):
                        a, b = dy[z][:, :out_f], x[z][:, :in_f]
                        want = oracle.dot(np.ascontiguousarray(a), True, np.ascontiguousarray(b), False, 0.5, 0.25,
                                          np.ascontiguousarray(c0[z][:, :in_f])) + 0.75 * Wm[z][:, :in_f]
                        assert np.max(np.abs(got[z][:, :in_f] - want)) <= bound(rows, a, b, 1e-5), (cfg, splitk, out_f)
                        assert np.array_equal(got[z][:, in_f:], c0[z][:, in_f:])          # padding untouched
                        ref_cs = a.astype(np.float64).sum(axis=0)
                        assert np.max(np.abs(cs[z] - ref_cs)) <= 1e-5 * np.sqrt(rows) + 1e-6, (cfg, splitk, out_f)
    finally:
        w.set_tuning(-1, 0)
    # a column sum cannot be asked for without transposeA
    with pytest.raises(Exception):
        gc.GemmEx(transA=0, M=4, N=4, K=4, A=gdy, lda=4, B=gx, ldb=4, ldc=4, colsum=gcs)


def test_every_shape_of_the_end_of_k_for_every_tile_configuration(oracle, gpu_wrapper):
    """The last k tiles of a block are fetched by pairs of their own kind (a full tile and nothing, the partial tile,
    the tile of zeros that completes a pair, nothing at all), chosen by how K ends: an even or odd number of k tiles
    (of 16 or 32), the last one full or partial, and K shorter than the look-ahead.  Each shape of the end, for each
    fp32 tile configuration, in blocks inside the matrix and at its edge (M, N = 300, 270), with the column sums that
    ride on the staging of A (a stage that is stored twice would be summed twice)."""
    from sharpnet_amd import GPUTensor
    rng = np.random.default_rng(77)
    w = gpu_wrapper
    fp32_cfgs = [c["id"] for c in w.configs() if c["kind"] == "fp32"]
    M, N = 300, 270
    try:
        for K in (5, 16, 33, 60, 64, 70, 80, 90, 96, 100, 128, 136, 150):
            at = random_tensor(rng, (K, M), -1, 1)   # A read transposed: the dW form, the one that carries the sums
            a = random_tensor(rng, (M, K), -1, 1)
            b = random_tensor(rng, (K, N), -1, 1)
            gat, ga, gb = T(w, at), T(w, a), T(w, b)
            want_t = oracle.dot(at, True, b, False)
            want_n = oracle.dot(a, False, b, False)
            want_cs = at.astype(np.float64).sum(axis=0)
            for cfg in fp32_cfgs:
                w.set_tuning(cfg, 1)
                gc = GPUTensor([M, N], None, w)
                gcs = GPUTensor([1, M], None, w)
                gcs.SetValue(float("nan"))
                gc.GemmEx(transA=1, M=M, N=N, K=K, A=gat, lda=M, B=gb, ldb=N, ldc=N, colsum=gcs)
                assert np.max(np.abs(gc.ToNumpy() - want_t)) <= bound(K, at, b, 1e-5), (cfg, K, "TN")
                assert np.max(np.abs(gcs.ToNumpy()[0] - want_cs)) <= 1e-5 * np.sqrt(K) + 1e-6, (cfg, K)
                gc.GemmEx(transA=0, M=M, N=N, K=K, A=ga, lda=K, B=gb, ldb=N, ldc=N)
                assert np.max(np.abs(gc.ToNumpy() - want_n)) <= bound(K, a, b, 1e-5), (cfg, K, "NN")
    finally:
        w.set_tuning(-1, 0)


@pytest.mark.parametrize("rows,in_f,out_f,with_db,wd", [(128, 784, 256, True, 1e-2), (36, 100, 64, False, 0.0),
                                                         (96, 132, 68, True, 0.5), (32, 32, 32, True, 0.0),
                                                         (64, 1000, 128, True, 0.0)])
def test_dense_backward_small_layer_in_one_launch(oracle, gpu_wrapper, rows, in_f, out_f, with_db, wd):
    """snhip_dense_backward on a layer whose dW and dx are each a handful of 32 x 32 tiles (benchmark configuration 1:
    128 x 784 -> 256): both products and the bias gradient leave as one launch.  Checked against the oracle's
    Linear.DenseBackwardPropagation restatement and against the same call with the tile configuration forced (which
    takes the products one by one through the 32 x 32 K-split kernel)."""
    from sharpnet_amd import GPUTensor
    from sharpnet_amd.hiplib import check_status
    w = gpu_wrapper
    rng = np.random.default_rng(rows + in_f + out_f)
    x, dy = random_tensor(rng, (rows, in_f), 0, 1), random_tensor(rng, (rows, out_f), -0.1, 0.1)
    W = random_tensor(rng, (out_f, in_f), -0.07, 0.07)
    gx, gdy, gW = T(w, x), T(w, dy), T(w, W)
    bias = random_tensor(rng, (out_f,), -1, 1)
    gbias = T(w, bias)
    bias_wd = wd if with_db else 0.0          # the PyTorch-mode decay on the bias gradient (Linear.cs:178-181)
    mult = 1.0 / rows
    ksplit = [c["id"] for c in w.configs() if c["kind"] == "fp32-ksplit"][0]
    got = {}
    for form in ("one launch", "forced"):
        gdx, gdW, gdb = (GPUTensor(sh, None, w) for sh in ([rows, in_f], [out_f, in_f], [out_f]))
        for t in (gdx, gdW, gdb):
            t.SetValue(float("nan"))
        print("dense backward", rows, in_f, out_f, with_db, wd, form, flush=True)
        if form == "forced":
            w.set_tuning(ksplit, 1)
        try:
            check_status(w.lib.snhip_dense_backward_ex(w.handle, gdx.Pointer, gdW.Pointer, gdb.Pointer if with_db else None,
                                                       gx.Pointer, gdy.Pointer, gW.Pointer, rows, in_f, out_f, mult, wd,
                                                       gbias.Pointer if bias_wd else None, bias_wd))
        finally:
            w.set_tuning(-1, 0)
        got[form] = (gdx.ToNumpy(), gdW.ToNumpy(), gdb.ToNumpy())
        assert w.last_tuning() == (ksplit, 1)
    dx, dW, db = got["one launch"]
    ref_dW = oracle.dot_f64(dy, True, x, False, mult) + wd * W.astype(np.float64)
    ref_dx = oracle.dot_f64(dy, False, W, False)
    assert np.max(np.abs(dW - ref_dW)) <= bound(rows, dy, x, 1e-6) * mult + 1e-6 * wd
    assert np.max(np.abs(dx - ref_dx)) <= bound(out_f, dy, W, 1e-7)
    if with_db:
        ref_db = dy.astype(np.float64).sum(axis=0) + bias_wd * bias.astype(np.float64)
        assert np.max(np.abs(db - ref_db)) <= 1e-5 * np.sqrt(rows) * 0.1 + 1e-6 * bias_wd + 1e-7
    else:
        assert np.isnan(db).all()
    # against the products issued one by one: the same kernel code per tile, but the one-launch form may give a product
    # 32 x 64 tiles with two K slices where the forced configuration has 32 x 32 tiles with four (another grouping of
    # the same partial sums), and the bias decay is one multiply-add here and a separate pass there
    assert np.allclose(got["one launch"][0], got["forced"][0], rtol=0, atol=bound(out_f, dy, W) / 10)
    assert np.allclose(got["one launch"][1], got["forced"][1], rtol=0, atol=bound(rows, dy, x) * mult / 10 + 1e-7)
    assert np.allclose(got["one launch"][2], got["forced"][2], rtol=0, atol=1e-6, equal_nan=True)


def test_linear_sigmoid_predictions_on_device(golden, gpu_wrapper):
    """Tests/NonReg/TestNetworkPropagation.cs:36-105 predictions through the GPU Dot."""
    from sharpnet_amd import GPUTensor, linear
    fx = golden["Linear_1_1_4_4"]
    x = np.array(fx["x"], np.float32)
    w_in_out = np.array(fx["w_in_out"], np.float32)
    gx, gw = T(gpu_wrapper, x), T(gpu_wrapper, w_in_out)
    gy = GPUTensor([1, 3], None, gpu_wrapper)
    gy.Dot(gx, False, gw, False, 1.0, 0.0)                                # (1,1,4,4) read as (1,16): flatten rule
    assert np.max(np.abs(sigmoid(gy.ToNumpy()) - np.array(fx["sigmoid_prediction"]))) < 2e-6
    gwt = T(gpu_wrapper, np.ascontiguousarray(w_in_out.T))
    linear.DenseForwardPropagation(gy, gx, gwt, None, False)
    assert np.max(np.abs(sigmoid(gy.ToNumpy()) - np.array(fx["sigmoid_prediction"]))) < 2e-6


def test_dense_chain_training_losses_on_device(golden, gpu_wrapper):
    """Tests/NonReg/ParallelRunWithPyTorch.cs:102-138 with every Linear product on the GPU:
    loss 0.297953724861145 before and 0.09050967544317245 after 10 epochs of SGD(0.1, momentum 0.9)."""
    from sharpnet_amd import GPUTensor, linear
    w = gpu_wrapper
    fx = golden["PyTorch_Mse"]
    X = numpy_array_for_tests(*fx["x_shape"])
    Y = y_numpy_array_for_tests(*fx["y_shape"])
    params = [np.array(fx["linear1_weight_out_in"], np.float32), np.zeros(3, np.float32),
              np.array(fx["linear2_weight_out_in"], np.float32), np.zeros(3, np.float32)]
    vel = [np.zeros_like(p) for p in params]
    gX = T(w, X)

    def forward():
        gW1, gb1, gW2, gb2 = (T(w, p) for p in params)
        gh = GPUTensor([2, 3, 4, 3], None, w)
        # flatten on last dimension: (24,5).(5,3); the ReLU layer that follows is folded into the product
        linear.DenseForwardPropagation(gh, gX, gW1, gb1, True, activation="CUDNN_ACTIVATION_RELU")
        h = r = gh.ToNumpy()
        gf = gh.Reshape(2, 36)
        gout = GPUTensor([2, 3], None, w)
        linear.DenseForwardPropagation(gout, gf, gW2, gb2, False)
        return h, r, gf, gout.ToNumpy(), (gW1, gW2)

    mse = lambda out: float(np.mean((out.astype(np.float64) - Y) ** 2))
    assert abs(mse(forward()[3]) - fx["loss_before"]) < fx["tolerance"]
    for _ in range(fx["epochs"]):
        h, r, gf, out, (gW1, gW2) = forward()
        dout = (2.0 * (out - Y) / out.size).astype(np.float32)
        gdW2, gdb2, gdf = GPUTensor([3, 36], None, w), GPUTensor([3], None, w), GPUTensor([2, 36], None, w)
        linear.DenseBackwardPropagation(gdf, gdW2, gdb2, gf, T(w, dout), gW2, compatibility_mode="PyTorch")
        gdh = GPUTensor([2, 36], None, w)
        gf.ActivationBackward("CUDNN_ACTIVATION_RELU", 0.0, gdf, gdh)       # y = relu output, Tensor.ActivationBackward
        gdW1, gdb1 = GPUTensor([3, 5], None, w), GPUTensor([3], None, w)
        linear.DenseBackwardPropagation(None, gdW1, gdb1, gX, gdh.Reshape(2, 3, 4, 3), gW1, compatibility_mode="PyTorch",
                                        prevLayerIsInputLayer=True, flattenInputTensorOnLastDimension=True)
        grads = [gdW1.ToNumpy(), gdb1.ToNumpy(), gdW2.ToNumpy(), gdb2.ToNumpy()]
        for i, g in enumerate(grads):
            vel[i] = (fx["momentum"] * vel[i] + g).astype(np.float32)
            params[i] = (params[i] - fx["lr"] * vel[i]).astype(np.float32)
    assert abs(mse(forward()[3]) - fx["loss_after"]) < fx["tolerance"]


@pytest.mark.parametrize("is_causal", [False, True])
def test_attention_fixture_loss_on_device(golden, oracle, gpu_wrapper, is_causal):
    """Tests/NonReg/ParallelRunWithPyTorch.cs:963-1010 loss_before with QK^T, softmax, PV on the GPU."""
    from sharpnet_amd import GPUTensor, attention, linear
    w = gpu_wrapper
    fx = golden["PyTorch_DotProductAttention"]
    X = numpy_array_for_tests(*fx["x_shape"])
    Y = y_numpy_array_for_tests(*fx["y_shape"])
    Wq, Wk, Wv = [np.array(fx[k], np.float32)[:, :, 0] for k in ("conv_q", "conv_k", "conv_v")]
    Wd = np.array(fx["dense_weight_out_in"], np.float32)
    gX = T(w, X)
    qkv = []
    for Wc in (Wq, Wk, Wv):                       # kernel-1 conv = per-sample (2x4).(4x5): a batched product, W stride 0
        out = GPUTensor([6, 2, 5], None, w)
        st = w.lib.snhip_gemm_rm(w.handle, 0, 0, 2, 5, 4, 1.0, T(w, Wc).Pointer, 4, 0, gX.Pointer, 5, 20, 0.0,
                                 out.Pointer, 5, 10, 6, None)
        assert st == 0
        qkv.append(out)
    gy = GPUTensor([6, 2, 5], None, w)
    attention.ScaledDotProductAttentionForwardPropagation(qkv[0], qkv[1], qkv[2], gy, False, False, is_causal)
    glog = GPUTensor([6, 3], None, w)
    linear.DenseForwardPropagation(glog, gy, T(w, Wd), None, False)
    p = oracle.softmax_last_dim(glog.ToNumpy()).astype(np.float64)
    loss = float(np.mean(-np.sum(Y * np.log(p), axis=1)))
    want = [c for c in fx["cases"] if c["is_causal"] == is_causal][0]["loss_before"]
    assert abs(loss - want) < 2e-6


@pytest.mark.parametrize("is_causal", [False, True])
def test_sdpa_forward_backward_vs_oracle(oracle, gpu_wrapper, is_causal):
    """ScaledDotProductAttentionLayer.cs:46-132: all six batched products (NT, NN, TN, NT, NN, TN) + softmax."""
    from sharpnet_amd import GPUTensor, attention
    w = gpu_wrapper
    rng = np.random.default_rng(41)
    B, Tn, d = 12, 96, 64
    Q, K, V, dy = (rng.normal(0, 1, (B, Tn, d)).astype(np.float32) for _ in range(4))
    gQ, gK, gV, gdy = (T(w, t) for t in (Q, K, V, dy))
    gy = GPUTensor([B, Tn, d], None, w)
    gweights = attention.ScaledDotProductAttentionForwardPropagation(gQ, gK, gV, gy, True, True, is_causal)
    ry, rw = oracle.sdpa_forward(Q, K, V, use_scale=True, is_causal=is_causal)
    assert np.max(np.abs(gweights.ToNumpy() - rw)) <= 2e-5
    assert np.max(np.abs(gy.ToNumpy() - ry)) <= bound(Tn, rw, V, 1e-5)
    gdQ, gdK, gdV = (GPUTensor([B, Tn, d], None, w) for _ in range(3))
    attention.ScaledDotProductAttentionBackwardPropagation(gdQ, gdK, gdV, gQ, gK, gV, gdy, gweights, True)
    rdQ, rdK, rdV = oracle.sdpa_backward(Q, K, V, dy, rw, use_scale=True)
    assert np.max(np.abs(gdV.ToNumpy() - rdV)) <= bound(Tn, rw, dy, 1e-4)
    assert np.max(np.abs(gdQ.ToNumpy() - rdQ)) <= bound(Tn, K, dy, 2e-4)
    assert np.max(np.abs(gdK.ToNumpy() - rdK)) <= bound(Tn, Q, dy, 2e-4)


def test_row_helpers_vs_numpy(gpu_wrapper):
    """Compute_BiasGradient_from_dy, BroadcastAddVectorToOutput, Update_Adding_Alpha_X, softmax, causal mask
    (Tests/TestParallelRunCpuVersusGpu.cs:730-736, 938-944, 651-665, 766)."""
    from sharpnet_amd import GPUTensor
    w = gpu_wrapper
    rng = np.random.default_rng(43)
    for rows, cols in [(1, 1), (7, 130), (300, 65), (1000, 1000)]:
        dy = random_tensor(rng, (rows, cols))
        gdb = GPUTensor([cols], None, w)
        T(w, dy).Compute_BiasGradient_from_dy(gdb)
        assert np.max(np.abs(gdb.ToNumpy() - dy.astype(np.float64).sum(0))) <= 1e-5 * np.sqrt(rows) * 1.5 * 4
        v = random_tensor(rng, (cols,))
        gy = T(w, dy)
        T(w, v).BroadcastAddVectorToOutput(gy)
        assert np.array_equal(gy.ToNumpy(), dy + v[None, :])
        gy.Update_Adding_Alpha_X(-0.5, T(w, dy))
        assert np.max(np.abs(gy.ToNumpy() - ((dy + v[None, :]) - 0.5 * dy))) <= 1e-6
        gs = GPUTensor([rows, cols], None, w)
        T(w, dy).SoftmaxLastDimension(gs)
        e = np.exp(dy.astype(np.float64) - dy.max(1, keepdims=True))
        assert np.max(np.abs(gs.ToNumpy() - e / e.sum(1, keepdims=True))) <= 2e-6
    m = random_tensor(rng, (3, 5, 7))
    gm = T(w, m)
    gm.SetAllElementsAboveMainDiagonal(-1e12)
    want = m.copy()
    for r in range(5):
        want[:, r, r + 1:] = np.float32(-1e12)
    assert np.array_equal(gm.ToNumpy(), want)


def _gpu_mha(gpu_wrapper, heads_in_place):
    """mha_forward / mha_backward with the oracle's signatures, computed by the device mirror."""
    from sharpnet_amd import GPUTensor, attention
    w = gpu_wrapper

    def fwd(Q, K, V, w_Q, w_K, w_V, w_O, H, dk, dv, b_Q=None, b_K=None, b_V=None, b_O=None, is_causal=False,
            use_scale=True):
        opt = lambda a: None if a is None else T(w, a)
        g = dict(Q=T(w, Q), K=T(w, K), V=T(w, V), w_Q=T(w, w_Q), w_K=T(w, w_K), w_V=T(w, w_V), w_O=T(w, w_O),
                 b=[opt(b_Q), opt(b_K), opt(b_V), opt(b_O)])
        gy = GPUTensor(list(V.shape), None, w)
        gy.SetValue(float("nan"))
        st = attention.MultiheadAttentionForwardPropagation(
            g["Q"], g["K"], g["V"], gy, g["w_Q"], g["w_K"], g["w_V"], g["w_O"], H, dk, dv, *g["b"], isTraining=True,
            use_scale=use_scale, is_causal=is_causal, heads_in_place=heads_in_place)
        g["st"], g["use_scale"] = st, use_scale
        return gy.ToNumpy(), g

    def bwd(dy, g):
        has_b = g["b"][0] is not None
        grads, outs = {}, {}
        for key, wt in (("w_Q", g["w_Q"]), ("w_K", g["w_K"]), ("w_V", g["w_V"]), ("out_proj_weight", g["w_O"])):
            gw = GPUTensor(wt.Shape, None, w)
            gb = GPUTensor([wt.Shape[0]], None, w) if has_b else None
            for t in (gw, gb):
                if t is not None:
                    t.SetValue(float("nan"))
            grads[key] = (gw, gb)
        dQ, dK, dV = (GPUTensor(g[k].Shape, None, w) for k in ("Q", "K", "V"))
        attention.MultiheadAttentionBackwardPropagation(dQ, dK, dV, g["Q"], g["K"], g["V"], T(w, dy), g["st"], g["w_Q"],
                                                        g["w_K"], g["w_V"], g["w_O"], grads, use_scale=g["use_scale"])
        outs.update(dQ=dQ.ToNumpy(), dK=dK.ToNumpy(), dV=dV.ToNumpy())
        for key, short in (("w_Q", "Q"), ("w_K", "K"), ("w_V", "V"), ("out_proj_weight", "O")):
            outs["dw_" + short] = grads[key][0].ToNumpy()
            outs["db_" + short] = grads[key][1].ToNumpy() if has_b else None
        return outs
    return fwd, bwd


@pytest.mark.parametrize("heads_in_place", [True, False])
@pytest.mark.parametrize("is_causal", [False, True])
def test_multi_head_attention_forward_backward(oracle, gpu_wrapper, heads_in_place, is_causal):
    """MultiheadAttention forward and backward (MultiheadAttention.cs:178-292) on the device, with the heads
    multiplied in place (two-level strided batch) or through the reference's transposition copies, against the
    oracle; biases on, a batch / step count that leaves ragged tiles (key_dim == value_dim: the reference's attention
    requires K and V of one shape, ScaledDotProductAttentionLayer.cs:48-51)."""
    rng = np.random.default_rng(21)
    B, Tn, H, dk, dv = 3, 37, 4, 16, 16
    E = H * dv
    Q, K, V = (random_tensor(rng, (B, Tn, E), -1, 1) for _ in range(3))
    w_Q, w_K = (random_tensor(rng, (H * dk, E), -0.3, 0.3) for _ in range(2))
    w_V, w_O = (random_tensor(rng, (H * dv, E), -0.3, 0.3) for _ in range(2))
    b_Q, b_K = (random_tensor(rng, (H * dk,), -0.5, 0.5) for _ in range(2))
    b_V, b_O = (random_tensor(rng, (H * dv,), -0.5, 0.5) for _ in range(2))
    dy = random_tensor(rng, (B, Tn, E), -1, 1)
    fwd, bwd = _gpu_mha(gpu_wrapper, heads_in_place)
    y, g = fwd(Q, K, V, w_Q, w_K, w_V, w_O, H, dk, dv, b_Q, b_K, b_V, b_O, is_causal=is_causal)
    ry, cache = oracle.mha_forward(Q, K, V, w_Q, w_K, w_V, w_O, H, dk, dv, b_Q, b_K, b_V, b_O, is_causal=is_causal)
    scale = float(np.max(np.abs(ry)))
    assert np.max(np.abs(y - ry)) <= 2e-4 * scale, np.max(np.abs(y - ry))
    got = bwd(dy, g)
    want = oracle.mha_backward(dy, cache)
    for k, ref in want.items():
        err = float(np.max(np.abs(got[k] - ref)))
        assert err <= 3e-4 * max(float(np.max(np.abs(ref))), 1.0), (k, err)


@pytest.mark.parametrize("B,Tn,H,d,is_causal", [(2, 256, 4, 64, True), (3, 300, 2, 32, False), (2, 130, 8, 64, True),
                                                 (1, 520, 2, 64, False), (2, 516, 3, 32, True)])
def test_multi_head_attention_heads_in_place_against_transposition_copies(gpu_wrapper, B, Tn, H, d, is_causal):
    """MultiheadAttention forward and backward at sizes that take the 16-query attention kernels and the two-level
    batches of the streaming GEMM kernels (heads multiplied in place in the (batch, steps, heads * dim) activations)
    against the same layer run the reference's way, with its transposition copies (MultiheadAttention.cs:178-292); both
    on the device, both fp32."""
    rng = np.random.default_rng(33)
    E = H * d
    Q, K, V, dy = (random_tensor(rng, (B, Tn, E), -1, 1) for _ in range(4))
    w_Q, w_K, w_V, w_O = (random_tensor(rng, (E, E), -0.1, 0.1) for _ in range(4))
    b_Q, b_K, b_V, b_O = (random_tensor(rng, (E,), -0.5, 0.5) for _ in range(4))
    res = []
    for heads_in_place in (True, False):
        fwd, bwd = _gpu_mha(gpu_wrapper, heads_in_place)
        y, g = fwd(Q, K, V, w_Q, w_K, w_V, w_O, H, d, d, b_Q, b_K, b_V, b_O, is_causal=is_causal)
        got = bwd(dy, g)
        got["y"] = y
        res.append(got)
    for k, ref in res[1].items():
        assert np.all(np.isfinite(res[0][k])), k
        err = float(np.max(np.abs(res[0][k] - ref)))
        assert err <= 1e-4 * max(float(np.max(np.abs(ref))), 1.0), (k, err)


@pytest.mark.parametrize("variant,is_causal", [("no_bias", False), ("no_bias", True), ("with_bias", False),
                                               ("with_bias", True)])
def test_multi_head_attention_training_losses_on_device(golden, oracle, gpu_wrapper, variant, is_causal):
    """Tests/NonReg/ParallelRunWithPyTorch.cs:1013-1131: the stored losses before and after 10 epochs with every
    product of the MultiheadAttention layer (projections, per-head scores and outputs, all gradients) on the device,
    heads multiplied in place."""
    from tests.test_oracle import _mha_chain
    fx = golden["PyTorch_MultiHeadAttention"]
    case = [c for c in fx[variant]["cases"] if c["is_causal"] == is_causal][0]
    fwd, bwd = _gpu_mha(gpu_wrapper, True)
    before, after = _mha_chain(oracle, fx, variant, is_causal, mha_fwd=fwd, mha_bwd=bwd)
    assert abs(before - case["loss_before"]) < 2e-6, (before, case)
    assert abs(after - case["loss_after"]) < 5e-6, (after, case)


@pytest.mark.parametrize("B,H,Tq,Tk,dk,dv,causal,packed", [
    (5, 1, 37, 37, 16, 16, False, False), (5, 1, 37, 37, 16, 16, True, False),      # ragged, small tiles
    (2, 3, 256, 256, 64, 64, True, True), (2, 3, 256, 256, 64, 64, False, False),   # the largest supported size
    (3, 2, 200, 130, 24, 40, False, True), (3, 2, 129, 65, 33, 7, True, False),     # Tq != Tk, dk != dv, odd sizes
    # head dimension exactly 64 and 129 to 256 keys (the form with two wavefronts per SIMD): ragged last query tile,
    # keys short of 256, three tiles per matrix; 255 keys (not a multiple of 4) stay on the general kernel
    (3, 2, 200, 132, 64, 64, True, False), (2, 2, 300, 256, 64, 64, False, True), (1, 3, 77, 252, 64, 64, False, False),
    (2, 1, 384, 200, 64, 64, True, True), (1, 3, 77, 255, 64, 64, True, True),
    # ... and 65 to 128 keys
    (4, 2, 128, 128, 64, 64, True, True), (3, 2, 100, 68, 64, 64, False, False), (2, 1, 300, 100, 64, 64, True, False),
    # ... and head dimension exactly 32
    (2, 2, 256, 256, 32, 32, True, True), (3, 1, 200, 132, 32, 32, False, False), (2, 2, 130, 100, 32, 32, True, False),
    # ... more matrices than compute units: a workgroup walks through several, the next one's K and V prefetched
    (75, 8, 130, 132, 64, 64, True, True), (700, 1, 100, 100, 64, 64, False, False), (90, 7, 140, 136, 32, 32, True, False),
    (1, 4, 1, 5, 3, 2, False, True),
    (2, 2, 128, 128, 128, 128, True, True), (3, 1, 70, 100, 96, 128, False, False),  # head dimension up to 128: 128 keys
    # more than 256 keys: the two-pass kernel over key blocks (head dimensions that are multiples of 4, up to 64)
    (2, 2, 512, 512, 64, 64, False, True), (2, 2, 512, 512, 64, 64, True, False),
    (1, 2, 1024, 1024, 32, 32, True, True), (1, 1, 1024, 1024, 64, 64, False, False),
    (1, 3, 300, 700, 24, 40, False, False), (1, 2, 700, 300, 64, 16, True, True), (1, 1, 2048, 2048, 64, 64, True, False),
    (2, 1, 257, 257, 8, 4, True, False),
    # ... head dimension exactly 64 (two wavefronts per SIMD): ragged query tiles and a last key block short of 256,
    # with and without the mask; 770 keys (not a multiple of 4) stay on the general two-pass kernel
    (2, 2, 300, 700, 64, 64, True, False), (1, 3, 650, 516, 64, 64, False, True), (1, 1, 130, 770, 64, 64, True, True),
    # ... and head dimension exactly 32
    (2, 2, 300, 700, 32, 32, True, False), (1, 3, 650, 516, 32, 32, False, True), (40, 8, 128, 512, 32, 32, True, True),
    (1, 2, 260, 260, 32, 32, False, False),
])
def test_fused_attention_forward(oracle, gpu_wrapper, B, H, Tq, Tk, dk, dv, causal, packed):
    """snhip_attention_forward (scores, mask, softmax and P.V in one launch) against the oracle's
    ScaledDotProductAttention, for stacked (batch*heads, steps, dim) operands and for heads addressed in place
    inside (batch, steps, heads*dim) activations; both the output and the softmax weights kept for backward."""
    from sharpnet_amd import GPUTensor, attention
    rng = np.random.default_rng(31)
    Z = B * H
    q, k, v = random_tensor(rng, (Z, Tq, dk), -1, 1), random_tensor(rng, (Z, Tk, dk), -1, 1), \
        random_tensor(rng, (Z, Tk, dv), -1, 1)
    scale = 1.0 / np.sqrt(dk)
    s = np.stack([oracle.dot(q[z], False, k[z], True, scale) for z in range(Z)])
    if causal:
        s[:, np.triu_indices(Tq, 1, Tk)[0], np.triu_indices(Tq, 1, Tk)[1]] = -1e12
    wref = oracle.softmax_last_dim(s)
    oref = oracle.bmm(wref, False, v, False)

    def lay(x, steps, dim):            # (Z, steps, dim) -> what the device sees
        if not packed:
            return x
        return np.ascontiguousarray(x.reshape(B, H, steps, dim).transpose(0, 2, 1, 3)).reshape(B, steps, H * dim)
    gq, gk, gv = T(gpu_wrapper, lay(q, Tq, dk)), T(gpu_wrapper, lay(k, Tk, dk)), T(gpu_wrapper, lay(v, Tk, dv))
    go = GPUTensor(list(lay(oref, Tq, dv).shape), None, gpu_wrapper)
    gw = GPUTensor([Z, Tq, Tk], None, gpu_wrapper)
    go.SetValue(float("nan"))
    gw.SetValue(float("nan"))
    assert attention.fused_attention_forward(gq, gk, gv, go, gw, batch=B, heads=H, tq=Tq, tkv=Tk, dk=dk, dv=dv,
                                             scale=scale, is_causal=causal, packed=packed)
    assert np.max(np.abs(gw.ToNumpy() - wref)) <= 2e-6 + 1e-5 * float(np.max(wref))
    assert np.max(np.abs(go.ToNumpy() - lay(oref, Tq, dv))) <= 1e-5 * max(1.0, float(np.max(np.abs(v))))
    # inference form: no weights requested, same output - bit for bit where the same kernel runs without its stores;
    # beyond 256 keys a call without weights may take a single pass with a running maximum instead (other rounding)
    go2 = GPUTensor(go.Shape, None, gpu_wrapper)
    go2.SetValue(float("nan"))
    assert attention.fused_attention_forward(gq, gk, gv, go2, None, batch=B, heads=H, tq=Tq, tkv=Tk, dk=dk, dv=dv,
                                             scale=scale, is_causal=causal, packed=packed)
    if Tk <= 256:
        assert np.array_equal(go2.ToNumpy(), go.ToNumpy())
    else:
        assert np.max(np.abs(go2.ToNumpy() - lay(oref, Tq, dv))) <= 1e-5 * max(1.0, float(np.max(np.abs(v))))


def test_fused_attention_limits(gpu_wrapper):
    """Beyond 256 keys with a head dimension that is not a multiple of 4 or above 64, beyond 128 keys with a head
    dimension above 64, or with a head dimension above 128, nothing is launched and the caller is told so."""
    from sharpnet_amd import GPUTensor, attention
    w = gpu_wrapper
    big = GPUTensor([1, 300, 6], None, w)
    out = GPUTensor([1, 300, 6], None, w)
    assert attention.fused_attention_forward(big, big, big, out, None, batch=1, heads=1, tq=300, tkv=300, dk=6, dv=6,
                                             scale=1.0, is_causal=False, packed=False) is False
    wide = GPUTensor([1, 16, 160], None, w)
    outw = GPUTensor([1, 16, 160], None, w)
    assert attention.fused_attention_forward(wide, wide, wide, outw, None, batch=1, heads=1, tq=16, tkv=16, dk=160, dv=160,
                                             scale=1.0, is_causal=False, packed=False) is False
    long_wide = GPUTensor([1, 200, 80], None, w)
    outl = GPUTensor([1, 200, 80], None, w)
    assert attention.fused_attention_forward(long_wide, long_wide, long_wide, outl, None, batch=1, heads=1, tq=200, tkv=200,
                                             dk=80, dv=80, scale=1.0, is_causal=False, packed=False) is False
    # ... and the library says the same when asked directly
    import ctypes
    from sharpnet_amd import hiplib
    d = hiplib.AttentionDesc(batch=1, Tq=200, Tk=200, dk=80, dv=80, Q=long_wide.Pointer, K=long_wide.Pointer,
                             V=long_wide.Pointer, O=outl.Pointer, ldq=80, ldk=80, ldv=80, ldo=80)
    assert w.lib.snhip_attention_forward(w.handle, ctypes.byref(d)) == hiplib.CublasStatus.CUBLAS_STATUS_NOT_SUPPORTED
    # the layer mirror falls back to the four-call sequence on its own
    y = GPUTensor([1, 300, 6], None, w)
    big.SetValue(0.5)
    wts = attention.ScaledDotProductAttentionForwardPropagation(big, big, big, y, True, True, False)
    assert abs(float(wts.ToNumpy()[0, 0, 0]) - 1.0 / 300) < 1e-6 and abs(float(y.ToNumpy()[0, 7, 3]) - 0.5) < 1e-6


def test_fused_attention_on_views_at_odd_element_offsets(oracle, gpu_wrapper):
    """Operands that are views starting 1, 2 and 3 floats into their buffers (4-byte alignment only, as tensor
    slices are, GpuTensor.cs:616): the vector loads and stores of the attention kernel must not assume more."""
    from sharpnet_amd import GPUTensor, attention
    rng = np.random.default_rng(41)
    Z, Tn, d = 3, 40, 8
    q, k, v = (random_tensor(rng, (Z, Tn, d), -1, 1) for _ in range(3))
    ref, wref = oracle.sdpa_forward(q, k, v, use_scale=True, is_causal=True)
    bufs = []
    for off, x in zip((1, 2, 3), (q, k, v)):
        flat = np.concatenate([np.full(off, 7.0, np.float32), x.reshape(-1)])
        g = GPUTensor([flat.size], flat, gpu_wrapper)
        bufs.append((g, g.Slice(off, [Z, Tn, d])))
    obuf = GPUTensor([Z * Tn * d + 5], None, gpu_wrapper)
    obuf.SetValue(-3.0)
    wbuf = GPUTensor([Z * Tn * Tn + 2], None, gpu_wrapper)
    wbuf.SetValue(-3.0)
    assert attention.fused_attention_forward(bufs[0][1], bufs[1][1], bufs[2][1], obuf.Slice(1, [Z, Tn, d]),
                                             wbuf.Slice(1, [Z, Tn, Tn]), batch=Z, heads=1, tq=Tn, tkv=Tn, dk=d, dv=d,
                                             scale=1.0 / np.sqrt(d), is_causal=True, packed=False)
    o, wt = obuf.ToNumpy(), wbuf.ToNumpy()
    assert np.max(np.abs(o[1:1 + Z * Tn * d].reshape(Z, Tn, d) - ref)) <= 1e-5
    assert np.max(np.abs(wt[1:1 + Z * Tn * Tn].reshape(Z, Tn, Tn) - wref)) <= 1e-5
    assert o[0] == -3.0 and np.all(o[1 + Z * Tn * d:] == -3.0) and wt[0] == -3.0 and wt[-1] == -3.0


@pytest.mark.parametrize("Tq,Tk,d", [(150, 200, 64), (150, 100, 32), (140, 520, 64)])
def test_fused_attention_inputs_at_odd_element_offsets_outputs_aligned(oracle, gpu_wrapper, Tq, Tk, d):
    """The kernels with two wavefronts per SIMD ask for 16-byte-aligned outputs but read Q, K and V wherever they lie:
    inputs that start 1, 2 and 3 floats into their buffers, outputs at the start of theirs; nothing outside the
    outputs is written."""
    from sharpnet_amd import GPUTensor, attention
    rng = np.random.default_rng(43)
    Z = 3
    q, k, v = random_tensor(rng, (Z, Tq, d), -1, 1), random_tensor(rng, (Z, Tk, d), -1, 1), random_tensor(rng, (Z, Tk, d), -1, 1)
    ref, wref = oracle.sdpa_forward(q, k, v, use_scale=True, is_causal=False)
    views = []
    for off, x in zip((1, 2, 3), (q, k, v)):
        flat = np.concatenate([np.full(off, 7.0, np.float32), x.reshape(-1)])
        g = GPUTensor([flat.size], flat, gpu_wrapper)
        views.append((g, g.Slice(off, list(x.shape))))
    obuf = GPUTensor([Z * Tq * d + 8], None, gpu_wrapper)
    obuf.SetValue(-3.0)
    wbuf = GPUTensor([Z * Tq * Tk + 8], None, gpu_wrapper)
    wbuf.SetValue(-3.0)
    assert attention.fused_attention_forward(views[0][1], views[1][1], views[2][1], obuf.Slice(0, [Z, Tq, d]),
                                             wbuf.Slice(0, [Z, Tq, Tk]), batch=Z, heads=1, tq=Tq, tkv=Tk, dk=d, dv=d,
                                             scale=1.0 / np.sqrt(d), is_causal=False, packed=False)
    o, wt = obuf.ToNumpy(), wbuf.ToNumpy()
    assert np.max(np.abs(o[:Z * Tq * d].reshape(Z, Tq, d) - ref)) <= 1e-5
    assert np.max(np.abs(wt[:Z * Tq * Tk].reshape(Z, Tq, Tk) - wref)) <= 1e-5
    assert np.all(o[Z * Tq * d:] == -3.0) and np.all(wt[Z * Tq * Tk:] == -3.0)
    # without weights (beyond 256 keys: the single-pass form)
    obuf.SetValue(-3.0)
    assert attention.fused_attention_forward(views[0][1], views[1][1], views[2][1], obuf.Slice(0, [Z, Tq, d]), None,
                                             batch=Z, heads=1, tq=Tq, tkv=Tk, dk=d, dv=d, scale=1.0 / np.sqrt(d),
                                             is_causal=False, packed=False)
    o = obuf.ToNumpy()
    assert np.max(np.abs(o[:Z * Tq * d].reshape(Z, Tq, d) - ref)) <= 1e-5
    assert np.all(o[Z * Tq * d:] == -3.0)


def test_gemm_ex_degenerate_products_keep_the_rest_of_the_epilogue(oracle, gpu_wrapper):
    """alpha == 0 or K == 0: A and B are not read (BLAS rule) but bias, beta * C, gamma * D and the activation still apply,
    and a requested column sum is still produced (zeros for K == 0)."""
    from sharpnet_amd import GPUTensor
    w = gpu_wrapper
    rng = np.random.default_rng(51)
    M, N, K = 37, 29, 11
    a, b = random_tensor(rng, (K, M), -1, 1), random_tensor(rng, (K, N), -1, 1)
    c0, d, bias = random_tensor(rng, (M, N), -1, 1), random_tensor(rng, (M, N), -1, 1), random_tensor(rng, (N,), -1, 1)
    want = np.maximum(0.5 * c0 + bias[None, :] + 0.25 * d, 0)
    for alpha, k in ((0.0, K), (1.0, 0)):
        gc, gcs = T(w, c0), GPUTensor([M], None, w)
        gcs.SetValue(float("nan"))
        gc.GemmEx(transA=1, M=M, N=N, K=k, alpha=alpha, beta=0.5, A=T(w, a), lda=M, B=T(w, b), ldb=N, ldc=N, bias=T(w, bias),
                  D=T(w, d), ldd=N, gamma=0.25, activation=1, colsum=gcs)
        assert np.max(np.abs(gc.ToNumpy() - want)) <= 1e-6
        ref_cs = a.astype(np.float64).sum(axis=0) if k else np.zeros(M)
        assert np.max(np.abs(gcs.ToNumpy() - ref_cs)) <= 1e-5


def test_gemm_ex_features_under_bf16_input_math(oracle, gpu_wrapper):
    """The bf16-input kernels have no extended instantiations: addend, ReLU, column sum and the two-level batch are
    then applied by extra passes / one launch per outer step, with the same results (checked against the oracle on
    bf16-rounded operands, fp32 bound)."""
    from sharpnet_amd import GPUTensor
    w = gpu_wrapper
    rng = np.random.default_rng(52)
    Bo, Bi, M, N, K = 2, 3, 70, 90, 130
    a = random_tensor(rng, (Bo, Bi, K, M), -1, 1)      # transposed A: stored K x M
    b = random_tensor(rng, (Bo, Bi, K, N), -1, 1)
    d = random_tensor(rng, (Bo, Bi, M, N), -1, 1)
    bias = random_tensor(rng, (N,), -1, 1)
    gc, gcs = GPUTensor([Bo, Bi, M, N], None, w), GPUTensor([Bo * Bi, M], None, w)
    gc.SetValue(float("nan"))
    gc.GemmEx(transA=1, M=M, N=N, K=K, alpha=0.5, A=T(w, a), lda=M, strideA=K * M, strideA_outer=Bi * K * M, B=T(w, b), ldb=N,
              strideB=K * N, strideB_outer=Bi * K * N, ldc=N, strideC=M * N, strideC_outer=Bi * M * N, batch=Bo * Bi,
              batch_inner=Bi, bias=T(w, bias), D=T(w, d), ldd=N, strideD=M * N, strideD_outer=Bi * M * N, gamma=-0.75,
              activation=2, activation_param=0.1, colsum=gcs, math=1)
    got, cs = gc.ToNumpy(), gcs.ToNumpy().reshape(Bo, Bi, M)
    ar, br = oracle.round_to_bf16(a), oracle.round_to_bf16(b)
    for o in range(Bo):
        for i in range(Bi):
            pre = oracle.dot(ar[o, i], True, br[o, i], False, 0.5) + bias[None, :] - 0.75 * d[o, i]
            want = np.where(pre >= 0, pre, 0.1 * pre)
            assert np.max(np.abs(got[o, i] - want)) <= bound(K, a, b, 1e-5), (o, i)
            assert np.max(np.abs(cs[o, i] - a[o, i].astype(np.float64).sum(axis=0))) <= 1e-5 * np.sqrt(K) + 1e-6


@pytest.mark.parametrize("B,H,Tq,Tk,dk,dv,packed", [
    (5, 1, 37, 37, 16, 16, False), (2, 3, 256, 256, 64, 64, True), (2, 3, 256, 256, 64, 64, False),
    (3, 2, 200, 130, 24, 40, True), (3, 2, 129, 65, 33, 7, False), (1, 4, 1, 5, 3, 2, True),
    (1, 2, 40, 300, 8, 8, False),                                  # beyond 256 keys: the five-launch sequence
    (2, 2, 128, 128, 128, 128, True), (3, 1, 70, 100, 96, 128, False),   # head dimension up to 128
    (1, 2, 60, 200, 80, 80, False),                                # 200 keys x 80: the five-launch sequence
    # head dimension exactly 64, 129 to 256 keys (two wavefronts per SIMD): ragged query tiles, keys short of 256
    (3, 2, 200, 132, 64, 64, False), (2, 2, 300, 256, 64, 64, True), (1, 3, 77, 252, 64, 64, False),
    (2, 1, 384, 200, 64, 64, True), (2, 3, 128, 128, 64, 64, True), (3, 2, 100, 68, 64, 64, False),
    (2, 2, 256, 256, 32, 32, True), (3, 1, 200, 132, 32, 32, False), (2, 2, 130, 100, 32, 32, False),
    (75, 8, 130, 132, 64, 64, True), (700, 1, 100, 100, 64, 64, False), (90, 7, 140, 136, 32, 32, False),
    # beyond 256 keys with head dimension exactly 64 or 32: the two-pass kernel over key blocks (a last block of 4 keys,
    # ragged query tiles, whole blocks, many matrices); 1002 keys and head dimension 48: the five-launch sequence
    (2, 2, 300, 520, 64, 64, False), (1, 3, 130, 1024, 64, 64, True), (2, 1, 257, 260, 64, 64, False),
    (1, 2, 100, 1000, 64, 64, True), (40, 8, 128, 512, 64, 64, True), (1, 2, 100, 1002, 64, 64, False),
    (1, 2, 100, 512, 32, 32, False), (2, 2, 300, 520, 32, 32, True), (30, 8, 130, 772, 32, 32, False),
    (1, 2, 100, 512, 48, 48, False), (1, 1, 300, 2048, 64, 64, False), (1, 2, 130, 1540, 32, 32, True),
])
def test_attention_backward_call(oracle, gpu_wrapper, B, H, Tq, Tk, dk, dv, packed):
    """snhip_attention_backward (dV, score gradient through the softmax, dQ, dK; the middle two from one kernel when
    the sizes allow it) against the oracle's ScaledDotProductAttentionBackwardPropagation, stacked and in-place-head
    layouts, including the score-gradient buffer itself."""
    from sharpnet_amd import GPUTensor, attention
    rng = np.random.default_rng(61)
    Z = B * H
    q, k = random_tensor(rng, (Z, Tq, dk), -1, 1), random_tensor(rng, (Z, Tk, dk), -1, 1)
    v, do = random_tensor(rng, (Z, Tk, dv), -1, 1), random_tensor(rng, (Z, Tq, dv), -1, 1)
    wts = oracle.softmax_last_dim(random_tensor(rng, (Z, Tq, Tk), -3, 3))
    scale = 0.37
    # reference sequence, ScaledDotProductAttentionLayer.cs:117-128
    dv_ref = oracle.bmm(wts, True, do, False)
    ds_ref = oracle.softmax_last_dim_backward(wts, oracle.bmm(do, False, v, True, scale))
    dq_ref = oracle.bmm(ds_ref, False, k, False)
    dk_ref = oracle.bmm(ds_ref, True, q, False)

    def lay(x, steps, dim):
        if not packed:
            return x
        return np.ascontiguousarray(x.reshape(B, H, steps, dim).transpose(0, 2, 1, 3)).reshape(B, steps, H * dim)
    w = gpu_wrapper
    gq, gk, gv, gdo = T(w, lay(q, Tq, dk)), T(w, lay(k, Tk, dk)), T(w, lay(v, Tk, dv)), T(w, lay(do, Tq, dv))
    gw, gds = T(w, wts), GPUTensor([Z, Tq, Tk], None, w)
    gdq, gdk, gdv = (GPUTensor(t.Shape, None, w) for t in (gq, gk, gv))
    for t in (gds, gdq, gdk, gdv):
        t.SetValue(float("nan"))
    attention.attention_backward(gdq, gdk, gdv, gq, gk, gv, gdo, gw, gds, batch=B, heads=H, tq=Tq, tkv=Tk, dk=dk, dv=dv,
                                 scale=scale, packed=packed)
    tol = 2e-5 * np.sqrt(max(Tq, Tk, dk, dv))
    assert np.max(np.abs(gds.ToNumpy() - ds_ref)) <= tol
    assert np.max(np.abs(gdv.ToNumpy() - lay(dv_ref, Tk, dv))) <= tol
    assert np.max(np.abs(gdq.ToNumpy() - lay(dq_ref, Tq, dk))) <= tol
    assert np.max(np.abs(gdk.ToNumpy() - lay(dk_ref, Tk, dk))) <= tol


@pytest.mark.parametrize("B,H,Tq,Tk,d,packed", [
    (2, 2, 1024, 1024, 64, False), (1, 3, 700, 900, 64, True), (2, 1, 1030, 520, 32, False), (1, 2, 300, 1540, 32, True),
    (3, 2, 256, 256, 64, False), (1, 2, 200, 132, 32, True), (1, 1, 520, 516, 48, False)])
def test_attention_backward_with_the_causal_hint(oracle, gpu_wrapper, B, H, Tq, Tk, d, packed):
    """snhip_attention_backward with `causal` set, on weights that a causally masked forward pass produced (zero above
    the diagonal): beyond 256 keys the key blocks above the diagonal are skipped and their score gradients
    zero-filled, and the sums over queries of dV and dK start at the first query that sees a key.  Every output
    against the oracle's ScaledDotProductAttentionBackwardPropagation on the same weights, and against the same call
    without the hint (the hint must not change what comes out).  Sizes: square and ragged, more queries than keys
    and the reverse, both 16-query head dimensions, <= 256 keys (nothing to skip in the kernel), and a head dimension
    that takes the call sequence."""
    from sharpnet_amd import GPUTensor, attention
    rng = np.random.default_rng(6100 + Tq + Tk + d)
    Z = B * H
    q, k = random_tensor(rng, (Z, Tq, d), -1, 1), random_tensor(rng, (Z, Tk, d), -1, 1)
    v, do = random_tensor(rng, (Z, Tk, d), -1, 1), random_tensor(rng, (Z, Tq, d), -1, 1)
    scores = random_tensor(rng, (Z, Tq, Tk), -3, 3)
    scores[:, np.triu_indices(Tq, 1, Tk)[0], np.triu_indices(Tq, 1, Tk)[1]] = -1e12     # SetAllElementsAboveMainDiagonal
    wts = oracle.softmax_last_dim(scores)
    assert np.all(wts[:, np.triu_indices(Tq, 1, Tk)[0], np.triu_indices(Tq, 1, Tk)[1]] == 0.0)
    scale = 0.37
    dv_ref = oracle.bmm(wts, True, do, False)
    ds_ref = oracle.softmax_last_dim_backward(wts, oracle.bmm(do, False, v, True, scale))
    dq_ref = oracle.bmm(ds_ref, False, k, False)
    dk_ref = oracle.bmm(ds_ref, True, q, False)

    def lay(x, steps, dim):
        if not packed:
            return x
        return np.ascontiguousarray(x.reshape(B, H, steps, dim).transpose(0, 2, 1, 3)).reshape(B, steps, H * dim)
    w = gpu_wrapper
    gq, gk, gv, gdo = T(w, lay(q, Tq, d)), T(w, lay(k, Tk, d)), T(w, lay(v, Tk, d)), T(w, lay(do, Tq, d))
    gw = T(w, wts)
    outs = {}
    for causal in (True, False):
        gds = GPUTensor([Z, Tq, Tk], None, w)
        gdq, gdk, gdv = (GPUTensor(t.Shape, None, w) for t in (gq, gk, gv))
        for t in (gds, gdq, gdk, gdv):
            t.SetValue(float("nan"))
        print("attention backward", B, H, Tq, Tk, d, packed, "causal hint", causal, flush=True)
        attention.attention_backward(gdq, gdk, gdv, gq, gk, gv, gdo, gw, gds, batch=B, heads=H, tq=Tq, tkv=Tk, dk=d, dv=d,
                                     scale=scale, packed=packed, is_causal=causal)
        outs[causal] = [t.ToNumpy() for t in (gds, gdv, gdq, gdk)]
        for t in (gds, gdq, gdk, gdv):
            t.Dispose()
    tol = 2e-5 * np.sqrt(max(Tq, Tk, d))
    for got in outs.values():
        assert np.max(np.abs(got[0] - ds_ref)) <= tol
        assert np.max(np.abs(got[1] - lay(dv_ref, Tk, d))) <= tol
        assert np.max(np.abs(got[2] - lay(dq_ref, Tq, d))) <= tol
        assert np.max(np.abs(got[3] - lay(dk_ref, Tk, d))) <= tol
    # the score gradient and dQ come from the same arithmetic with or without the hint; dV and dK leave out exact zeros
    assert np.array_equal(outs[True][0], outs[False][0]) and np.array_equal(outs[True][2], outs[False][2])
    assert np.max(np.abs(outs[True][1] - outs[False][1])) <= tol and np.max(np.abs(outs[True][3] - outs[False][3])) <= tol


@pytest.mark.parametrize("rows,cols", [(33333, 130), (512, 64), (511, 3), (100000, 1), (4096, 4096)])
def test_bias_gradient_tall_matrices(gpu_wrapper, rows, cols):
    """Column sums of matrices much taller than wide are cut into row chunks (two kernels); same result as one pass."""
    from sharpnet_amd import GPUTensor
    rng = np.random.default_rng(rows + cols)
    dy = rng.uniform(-1, 1, (rows, cols)).astype(np.float32)
    g = GPUTensor([cols], None, gpu_wrapper)
    g.SetValue(float("nan"))
    T(gpu_wrapper, dy).Compute_BiasGradient_from_dy(g)
    ref = dy.astype(np.float64).sum(axis=0)
    assert np.max(np.abs(g.ToNumpy() - ref)) <= 1e-5 * np.sqrt(rows) + 1e-6 * rows ** 0.5


def test_fused_attention_agrees_with_the_call_sequence_on_seeded_random_sizes(gpu_wrapper):
    """ScaledDotProductAttention forward (weights kept) and backward through the fused entry points against the
    reference's own sequence of calls (ScaledDotProductAttentionLayer.cs:46-91, 97-135) issued through the same library,
    on 28 seeded random sizes: 1-9 matrices, 1-900 positions, head dimensions 4-64, with and without the mask.  Both
    sides compute in fp32; the bar is the sum of two rounding bounds."""
    from sharpnet_amd import GPUTensor, attention
    rng = np.random.default_rng(2024)
    w = gpu_wrapper
    for case in range(28):
        Z = int(rng.integers(1, 10))
        steps = int(rng.integers(1, 901)) if case % 4 else int(rng.choice([64, 128, 256, 260, 512, 772]))
        d = int(rng.choice([4, 8, 16, 24, 32, 40, 64]))
        causal = bool(rng.integers(0, 2))
        host = [random_tensor(rng, (Z, steps, d), -1, 1) for _ in range(4)]
        results = []
        for fused in (True, False):
            q, k, v, dy = (T(w, x) for x in host)
            y, dq, dk, dv = (GPUTensor([Z, steps, d], None, w) for _ in range(4))
            wts = attention.ScaledDotProductAttentionForwardPropagation(q, k, v, y, True, True, causal, fused=fused)
            out = [y.ToNumpy(), wts.ToNumpy()]
            attention.ScaledDotProductAttentionBackwardPropagation(dq, dk, dv, q, k, v, dy, wts, True, fused=fused)
            out += [dq.ToNumpy(), dk.ToNumpy(), dv.ToNumpy()]
            results.append(out)
            for t in (q, k, v, dy, y, dq, dk, dv):
                t.Dispose()
        tol = 4e-5 * np.sqrt(max(steps, d))
        for name, a, b in zip(("y", "weights", "dQ", "dK", "dV"), results[0], results[1]):
            assert np.all(np.isfinite(a)), (case, Z, steps, d, causal, name)
            assert np.max(np.abs(a - b)) <= tol, (case, Z, steps, d, causal, name, float(np.max(np.abs(a - b))))
