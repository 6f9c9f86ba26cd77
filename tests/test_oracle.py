"""Pins the CPU oracle (oracle/dot_oracle.*) before anything is compared against it.

Each check is chosen so that a plausible slip (a transposed operand, lda/ldb mixed
up, beta applied to the product, C read when beta == 0, a wrong flatten rule)
fails at least one of them:
  * the reference's known answers (Tests/GPU/TestGpuTensor.cs:53-109),
  * brute-force triple loops on tiny ragged shapes,
  * the numpy float64 closed form on random ragged shapes,
  * the QR identity of Tests/CPU/TestCpuTensor.cs:826-866,
  * network-level losses the reference stores (ParallelRunWithPyTorch.cs).
"""
import itertools

import numpy as np
import pytest

from tests.helpers import numpy_array_for_tests, y_numpy_array_for_tests, random_tensor, sigmoid


def test_known_answers_TestDot(golden, oracle):
    for case in golden["TestDot"]["cases"]:
        def arr(v, shape):
            return np.zeros(shape, np.float32) if v == "zeros" else np.array(v, np.float32).reshape(shape)
        a = arr(case["a"], case["a_shape"])
        b = arr(case["b"], case["b_shape"])
        got = oracle.dot(a, False, b, False, 1, 0)
        expected = arr(case["expected"], case["c_shape"]).reshape(got.shape)
        assert np.max(np.abs(got - expected), initial=0.0) <= golden["TestDot"]["tolerance"]


def _brute(a, tA, b, tB, alpha, beta, c):
    aH, aW = a.shape
    bH, bW = b.shape
    M = aW if tA else aH
    N = bH if tB else bW
    K = aH if tA else aW
    out = np.zeros((M, N), np.float64)
    for m in range(M):
        for n in range(N):
            s = 0.0
            for k in range(K):
                av = a[k, m] if tA else a[m, k]
                bv = b[n, k] if tB else b[k, n]
                s += float(av) * float(bv)
            out[m, n] = float(np.float32(alpha)) * s + (float(np.float32(beta)) * float(c[m, n]) if beta != 0 else 0.0)
    return out


@pytest.mark.parametrize("tA,tB", list(itertools.product([False, True], repeat=2)))
def test_brute_force_tiny(oracle, tA, tB):
    rng = np.random.default_rng(7)
    for (M, N, K) in [(1, 1, 1), (3, 2, 5), (5, 7, 3), (2, 9, 4)]:
        a = random_tensor(rng, (K, M) if tA else (M, K))
        b = random_tensor(rng, (N, K) if tB else (K, N))
        c = random_tensor(rng, (M, N))
        for alpha, beta in [(1.0, 0.0), (0.25, 0.0), (-1.0, 1.0), (0.5, 1.0), (1.0, -0.75)]:
            got = oracle.dot(a, tA, b, tB, alpha, beta, c if beta != 0 else None)
            ref = _brute(a, tA, b, tB, alpha, beta, c)
            assert got.shape == (M, N)
            assert np.max(np.abs(got - ref)) <= 2e-6 * max(1.0, np.max(np.abs(ref)))


@pytest.mark.parametrize("tA,tB", list(itertools.product([False, True], repeat=2)))
def test_closed_form_ragged(oracle, tA, tB):
    rng = np.random.default_rng(11)
    for (M, N, K) in [(35, 21, 124), (33, 17, 65), (8, 12, 10), (2, 2, 20000), (129, 257, 63)]:
        a = random_tensor(rng, (K, M) if tA else (M, K))
        b = random_tensor(rng, (N, K) if tB else (K, N))
        c = random_tensor(rng, (M, N))
        for alpha, beta in [(1.0, 0.0), (0.25, 0.0), (-1.0, 1.0)]:
            got = oracle.dot(a, tA, b, tB, alpha, beta, c if beta != 0 else None)
            ref = oracle.dot_f64(a, tA, b, tB, alpha, beta, c)
            # one fp32 rounding of a double-accumulated value
            assert np.max(np.abs(got - ref)) <= 1e-6 * max(1.0, np.max(np.abs(ref)))


def test_beta_zero_does_not_read_c(oracle):
    # the C entry point is handed a NaN-filled destination; beta == 0 must overwrite it
    import ctypes
    rng = np.random.default_rng(3)
    a, b = random_tensor(rng, (4, 6)), random_tensor(rng, (6, 5))
    out = np.full((4, 5), np.nan, np.float32)
    p = lambda x: x.ctypes.data_as(ctypes.POINTER(ctypes.c_float))
    oracle._lib().oracle_dot(p(a), 4, 6, 0, p(b), 6, 5, 0, p(out), 1.0, 0.0)
    assert np.all(np.isfinite(out))
    assert np.allclose(out, a.astype(np.float64) @ b.astype(np.float64), atol=1e-5)


def test_flatten_rule(oracle):
    # operands with more than 2 dims are (Shape[0], MultDim0) matrices: Tests/GPU/TestGpuTensor.cs:84-101
    rng = np.random.default_rng(5)
    a = random_tensor(rng, (10, 1, 4, 7))
    b = random_tensor(rng, (28, 3, 2))
    got = oracle.dot(a, False, b, False)
    assert got.shape == (10, 6)
    assert np.allclose(got, a.reshape(10, 28).astype(np.float64) @ b.reshape(28, 6).astype(np.float64), atol=1e-5)


def test_qr_identity(golden, oracle):
    for case in golden["QR"]["cases"]:
        A = np.array(case["A"], np.float32)
        Q = np.array(case["Q"], np.float32)
        n = A.shape[1]
        R = oracle.dot(Q, True, A, False)           # TN, as QRFactorization's tail does (CpuTensor.cs:3078)
        assert R.shape == (n, n)
        assert np.max(np.abs(np.tril(R, -1))) < 1e-4   # upper triangular
        QR = oracle.dot(Q, False, R, False)         # NN
        assert np.max(np.abs(QR - A)) < 1e-4
        QtQ = oracle.dot(Q, True, Q, False)         # A == B aliasing
        assert np.max(np.abs(QtQ - np.eye(n))) < 1e-6


def test_bmm_is_loop_of_dot(oracle):
    rng = np.random.default_rng(13)
    batch, L, d = 3, 12, 7   # Tests/TestParallelRunCpuVersusGpu.cs:377-401
    dy, V = random_tensor(rng, (batch, L, d)), random_tensor(rng, (batch, L, d))
    S = random_tensor(rng, (batch, L, L))
    for (a, tA, b, tB, alpha) in [(dy, False, V, True, 0.25), (S, False, V, False, 1.0), (S, True, V, False, 1.0)]:
        got = oracle.bmm(a, tA, b, tB, alpha, 0.0)
        for i in range(batch):
            ref = oracle.dot_f64(a[i], tA, b[i], tB, alpha)
            assert np.max(np.abs(got[i] - ref)) <= 1e-6 * max(1.0, np.max(np.abs(ref)))


def test_sgemm_colmajor_identity(oracle):
    # column-major C(m x n) = op(A) op(B)  <=>  row-major C^T = op(B)^T op(A)^T on the same buffers
    rng = np.random.default_rng(17)
    m, n, k = 5, 7, 9
    for ta, tb in itertools.product([0, 1], repeat=2):
        lda = (k if ta else m) + 2
        ldb = (n if tb else k) + 1
        ldc = m + 3
        A = random_tensor(rng, ((m if ta else k), lda))   # row-major view: ld is the row pitch
        B = random_tensor(rng, ((k if tb else n), ldb))
        C = random_tensor(rng, (n, ldc))
        out = oracle.sgemm_colmajor(ta, tb, m, n, k, 0.5, A, lda, B, ldb, -1.0, C, ldc).reshape(n, ldc)
        Acm = A[:, :(k if ta else m)].T.astype(np.float64)   # column-major matrix = transpose of the row-major view
        Bcm = B[:, :(n if tb else k)].T.astype(np.float64)
        opA = Acm.T if ta else Acm
        opB = Bcm.T if tb else Bcm
        ref = 0.5 * (opA @ opB) - C[:, :m].T.astype(np.float64)
        assert np.max(np.abs(out[:, :m].T - ref)) < 1e-5
        assert np.array_equal(out[:, m:], C[:, m:])          # padding untouched


def test_linear_sigmoid_predictions(golden, oracle):
    fx = golden["Linear_1_1_1_1"]
    x = np.array(fx["x"], np.float32)
    w_in_out = np.array(fx["w"], np.float32)                  # (in=1, out=2); layout-independent for 1x1 input
    y = oracle.dense_forward(x, w_in_out.T.copy())
    assert np.max(np.abs(sigmoid(y) - np.array(fx["sigmoid_prediction"]))) < fx["tolerance"]

    fx = golden["Linear_1_1_4_4"]
    x = np.array(fx["x"], np.float32)                          # (1,1,4,4)
    w_in_out = np.array(fx["w_in_out"], np.float32)            # (16, 3)
    y_nn = oracle.dot(x, False, w_in_out, False)               # NN reading of the stored literal
    assert np.max(np.abs(sigmoid(y_nn) - np.array(fx["sigmoid_prediction"]))) < 2e-6
    y_nt = oracle.dense_forward(x, np.ascontiguousarray(w_in_out.T))   # same numbers through the NT path
    assert np.max(np.abs(y_nn - y_nt)) < 1e-6


def test_dense_chain_losses(golden, oracle):
    """Two Linear layers trained for 10 epochs reproduce the stored losses
    (Tests/NonReg/ParallelRunWithPyTorch.cs:102-138): pins NT forward, TN dW, NN dx, bias gradient."""
    fx = golden["PyTorch_Mse"]
    X = numpy_array_for_tests(*fx["x_shape"])
    Y = y_numpy_array_for_tests(*fx["y_shape"])
    W1 = np.array(fx["linear1_weight_out_in"], np.float32)
    W2 = np.array(fx["linear2_weight_out_in"], np.float32)
    b1 = np.zeros(W1.shape[0], np.float32)
    b2 = np.zeros(W2.shape[0], np.float32)
    params = [W1, b1, W2, b2]
    vel = [np.zeros_like(p) for p in params]

    def forward():
        h = oracle.dense_forward(X, params[0], params[1], flatten_last=True)    # (24, 3)
        r = oracle.activation_forward(h, "relu")
        f = r.reshape(X.shape[0], -1)                                            # Flatten -> (2, 36)
        out = oracle.dense_forward(f, params[2], params[3])
        return h, r, f, out

    def mse(out):
        return float(np.mean((out.astype(np.float64) - Y) ** 2))

    loss_before = mse(forward()[3])
    assert abs(loss_before - fx["loss_before"]) < fx["tolerance"]
    for _ in range(fx["epochs"]):
        h, r, f, out = forward()
        dout = (2.0 * (out - Y) / out.size).astype(np.float32)
        dW2, db2, df = oracle.dense_backward(f, dout, params[2])
        dr = df.reshape(r.shape)
        dh = oracle.activation_backward(r, dr, "relu")
        dW1, db1, _ = oracle.dense_backward(X, dh, params[0], prev_is_input=True, flatten_last=True)
        for i, g in enumerate([dW1, db1, dW2, db2]):
            vel[i] = (fx["momentum"] * vel[i] + g).astype(np.float32)
            params[i] = (params[i] - fx["lr"] * vel[i]).astype(np.float32)
    loss_after = mse(forward()[3])
    assert abs(loss_after - fx["loss_after"]) < fx["tolerance"]


def test_activation_functions(golden, oracle):
    """sigmoid against the reference's stored predictions, tanh / leaky relu through identities that tie them to the
    pinned ones, and every gradient (written in terms of the output y) against central differences of the forward."""
    fx = golden["Linear_1_1_4_4"]
    y = oracle.dot(np.array(fx["x"], np.float32), False, np.array(fx["w_in_out"], np.float32), False)
    assert np.max(np.abs(oracle.activation_forward(y, "sigmoid") - np.array(fx["sigmoid_prediction"]))) < 2e-6
    rng = np.random.default_rng(5)
    x = rng.uniform(-3, 3, (7, 33)).astype(np.float32)
    x[np.abs(x) < 1e-2] = 0.5                                   # keep finite differences away from the kinks
    sig = lambda t: oracle.activation_forward(t, "sigmoid").astype(np.float64)
    assert np.max(np.abs(oracle.activation_forward(x, "tanh") - (2 * sig(2 * x) - 1))) < 3e-7
    relu = lambda t: oracle.activation_forward(t, "relu")
    assert np.array_equal(relu(x), np.where(x > 0, x, 0).astype(np.float32))
    for a in (0.1, 0.3):                                        # the slopes the reference tests use
        assert np.allclose(oracle.activation_forward(x, "leaky_relu", a), relu(x) - np.float32(a) * relu(-x), atol=1e-7)
    dy = rng.uniform(-1, 1, x.shape).astype(np.float32)
    for mode, a in (("relu", 0.0), ("leaky_relu", 0.1), ("leaky_relu", 0.3), ("sigmoid", 0.0), ("tanh", 0.0)):
        yy = oracle.activation_forward(x, mode, a)
        h = 1e-3
        num = (oracle.activation_forward(x + np.float32(h), mode, a).astype(np.float64) -
               oracle.activation_forward(x - np.float32(h), mode, a)) / (2 * h) * dy
        assert np.max(np.abs(oracle.activation_backward(yy, dy, mode, a) - num)) < 2e-3, mode
    # weight decay enters dW linearly and nowhere else
    xx, dd, W = rng.uniform(-1, 1, (9, 5)).astype(np.float32), rng.uniform(-1, 1, (9, 4)).astype(np.float32), \
        rng.uniform(-1, 1, (4, 5)).astype(np.float32)
    base = oracle.dense_backward(xx, dd, W)
    wd = oracle.dense_backward(xx, dd, W, weight_decay_alpha=0.5)
    assert np.allclose(wd[0] - base[0], 0.5 * W, atol=1e-6) and np.array_equal(wd[1], base[1]) and \
        np.array_equal(wd[2], base[2])


def test_attention_chain_losses(golden, oracle):
    """loss_before of Test_DotProductAttention (ParallelRunWithPyTorch.cs:963-1010): batched NT -> softmax -> NN."""
    fx = golden["PyTorch_DotProductAttention"]
    X = numpy_array_for_tests(*fx["x_shape"])                  # (6, 4, 5) = (N, C, L)
    Y = y_numpy_array_for_tests(*fx["y_shape"])
    Wq, Wk, Wv = [np.array(fx[k], np.float32)[:, :, 0] for k in ("conv_q", "conv_k", "conv_v")]   # (2, 4)
    Wd = np.array(fx["dense_weight_out_in"], np.float32)      # (3, 10)
    conv = lambda W: np.stack([oracle.dot(W, False, X[n], False) for n in range(X.shape[0])])    # (6, 2, 5)
    Q, K, V = conv(Wq), conv(Wk), conv(Wv)
    for case in fx["cases"]:
        y, _ = oracle.sdpa_forward(Q, K, V, use_scale=False, is_causal=case["is_causal"])
        logits = oracle.dense_forward(y.reshape(X.shape[0], -1), Wd)
        p = oracle.softmax_last_dim(logits).astype(np.float64)
        loss = float(np.mean(-np.sum(Y * np.log(p), axis=1)))
        assert abs(loss - case["loss_before"]) < 2e-6, (case, loss)


def test_mkl_route_matches_closed_form(oracle):
    """The baseline route (the cblas_sgemm call of BlasServices.cs:20) agrees with float64 within the fp32 bound."""
    rng = np.random.default_rng(19)
    for tA, tB in itertools.product([False, True], repeat=2):
        M, N, K = 65, 47, 130
        a = random_tensor(rng, (K, M) if tA else (M, K), -1, 1)
        b = random_tensor(rng, (N, K) if tB else (K, N), -1, 1)
        c = random_tensor(rng, (M, N), -1, 1)
        out = c.copy()
        oracle.mkl_dot(a, tA, b, tB, out, alpha=0.5, beta=1.0)
        ref = oracle.dot_f64(a, tA, b, tB, 0.5, 1.0, c)
        assert np.max(np.abs(out - ref)) <= oracle.tolerance(K, a, b)


def test_mkl_serial_batch_loop_matches_the_batched_oracle(oracle):
    """The batched baseline (one cblas_sgemm per matrix, in order: CpuTensor.cs:3018-3024) agrees with the oracle's bmm."""
    rng = np.random.default_rng(23)
    for tA, tB in itertools.product([False, True], repeat=2):
        n, M, N, K = 5, 33, 18, 40
        a = random_tensor(rng, (n, K, M) if tA else (n, M, K), -1, 1)
        b = random_tensor(rng, (n, N, K) if tB else (n, K, N), -1, 1)
        c = random_tensor(rng, (n, M, N), -1, 1)
        out = c.copy()
        oracle.mkl_bmm_serial(a, tA, b, tB, out, alpha=0.125, beta=1.0)
        ref = oracle.bmm(a, tA, b, tB, 0.125, 1.0, c)
        assert np.max(np.abs(out - ref)) <= oracle.tolerance(K, a, b)


def test_round_to_bf16(oracle):
    """Ties go to the even 8-bit significand; agrees with torch's CPU bfloat16 cast on random data."""
    f = np.float32
    cases = [(1.0, 1.0), (1 + 2.0 ** -8, 1.0), (1 + 2.0 ** -8 + 2.0 ** -20, 1 + 2.0 ** -7),
             (1 + 3 * 2.0 ** -8, 1 + 2.0 ** -6), (-(1 + 2.0 ** -8), -1.0), (0.0, 0.0),
             (2.0 ** -130, 2.0 ** -130)]
    for x, want in cases:
        assert oracle.round_to_bf16(np.array([x], f))[0] == f(want), (x, want)
    import torch
    rng = np.random.default_rng(23)
    x = np.concatenate([rng.normal(0, 1, 20000), rng.uniform(-1e-3, 1e-3, 20000), rng.normal(0, 1e4, 20000)]).astype(f)
    want = torch.from_numpy(x).to(torch.bfloat16).to(torch.float32).numpy()
    assert np.array_equal(oracle.round_to_bf16(x), want)


def test_sdpa_backward_by_finite_differences(oracle):
    """dQ, dK, dV of the attention chain agree with central differences of sum(y * g) (float64 restatement)."""
    rng = np.random.default_rng(29)
    B, T, d = 2, 5, 3
    Q, K, V = (rng.normal(0, 1, (B, T, d)).astype(np.float32) for _ in range(3))
    g = rng.normal(0, 1, (B, T, d)).astype(np.float32)

    def f(q, k, v):
        s = np.einsum("btd,bsd->bts", q, k) / np.sqrt(d)
        e = np.exp(s - s.max(-1, keepdims=True))
        p = e / e.sum(-1, keepdims=True)
        return float(np.sum(np.einsum("bts,bsd->btd", p, v) * g))

    y, w = oracle.sdpa_forward(Q, K, V, use_scale=True, is_causal=False)
    dQ, dK, dV = oracle.sdpa_backward(Q, K, V, g, w, use_scale=True)
    eps = 1e-4
    for name, X, dX in (("Q", Q, dQ), ("K", K, dK), ("V", V, dV)):
        num = np.zeros_like(X, dtype=np.float64)
        for idx in np.ndindex(*X.shape):
            args = {"Q": Q.astype(np.float64), "K": K.astype(np.float64), "V": V.astype(np.float64)}
            xp, xm = args[name].copy(), args[name].copy()
            xp[idx] += eps
            xm[idx] -= eps
            ap, am = dict(args), dict(args)
            ap[name], am[name] = xp, xm
            num[idx] = (f(ap["Q"], ap["K"], ap["V"]) - f(am["Q"], am["K"], am["V"])) / (2 * eps)
        assert np.max(np.abs(num - dX)) < 2e-4, name


def _mha_chain(oracle, fx, variant, is_causal, mha_fwd=None, mha_bwd=None):
    """The network of Tests/NonReg/ParallelRunWithPyTorch.cs:1013-1131 trained exactly as there; returns
    (loss_before, loss_after).  mha_fwd / mha_bwd default to the oracle's (the GPU test passes its own)."""
    mha_fwd = mha_fwd or oracle.mha_forward
    mha_bwd = mha_bwd or oracle.mha_backward
    v = fx[variant]
    use_bias = variant == "with_bias"
    X = numpy_array_for_tests(*fx["x_shape"])                  # (10, C=2, L=6)
    Y = y_numpy_array_for_tests(*fx["y_shape"])
    H, dk, dv = fx["num_heads"], fx["key_dim"], fx["value_dim"]
    E = H * dk
    inw = np.array(v["in_proj_weight"], np.float32)
    P = {"cq": np.array(v["conv_q"], np.float32)[:, :, 0], "ck": np.array(v["conv_k"], np.float32)[:, :, 0],
         "cv": np.array(v["conv_v"], np.float32)[:, :, 0], "cqb": np.zeros(2, np.float32), "ckb": np.zeros(2, np.float32),
         "cvb": np.zeros(2, np.float32), "wq": inw[0:E].copy(), "wk": inw[E:2 * E].copy(), "wv": inw[2 * E:3 * E].copy(),
         "wo": np.array(v["out_proj_weight"], np.float32), "dw": np.array(v["dense_weight_out_in"], np.float32),
         "db": np.zeros(3, np.float32)}
    if use_bias:
        P.update(bq=np.zeros(E, np.float32), bk=np.zeros(E, np.float32), bv=np.zeros(E, np.float32), bo=np.zeros(E, np.float32))
    vel = {k: np.zeros_like(p) for k, p in P.items()}

    def conv(x, W, b):                                         # width-1 Conv1D over (N, C, L)
        return np.stack([oracle.dot(W, False, x[n], False) + b[:, None] for n in range(x.shape[0])]).astype(np.float32)

    def forward(x):
        q, k, vv = conv(x, P["cq"], P["cqb"]), conv(x, P["ck"], P["ckb"]), conv(x, P["cv"], P["cvb"])
        y, cache = mha_fwd(q, k, vv, P["wq"], P["wk"], P["wv"], P["wo"], H, dk, dv, P.get("bq"), P.get("bk"), P.get("bv"),
                           P.get("bo"), is_causal=is_causal)
        flat = y.reshape(x.shape[0], -1)
        logits = oracle.dense_forward(flat, P["dw"], P["db"])
        return oracle.softmax_last_dim(logits), (flat, cache)

    def loss():
        p = forward(X)[0].astype(np.float64)
        return float(np.mean(-np.sum(Y * np.log(p), axis=1)))

    before = loss()
    bs = fx["batch_size"]
    for _ in range(fx["epochs"]):
        for i in range(0, X.shape[0], bs):
            x, y = X[i:i + bs], Y[i:i + bs]
            p, (flat, cache) = forward(x)
            dlogits = (p - y).astype(np.float32)                # Tensor.cs:1389-1395; the 1/batch sits in the update
            G = {}
            G["dw"], G["db"], dflat = oracle.dense_backward(flat, dlogits, P["dw"])
            g = mha_bwd(dflat.reshape(x.shape[0], 2, E), cache)
            G["wq"], G["wk"], G["wv"], G["wo"] = g["dw_Q"], g["dw_K"], g["dw_V"], g["dw_O"]
            if use_bias:
                G["bq"], G["bk"], G["bv"], G["bo"] = g["db_Q"], g["db_K"], g["db_V"], g["db_O"]
            for name, d in (("cq", g["dQ"]), ("ck", g["dK"]), ("cv", g["dV"])):
                G[name] = sum(oracle.dot(d[n], False, x[n], True) for n in range(x.shape[0])).astype(np.float32)
                G[name + "b"] = d.sum(axis=(0, 2)).astype(np.float32)
            for k in P:                                         # Sgd.cs / CpuTensor.cs:470-489, lr / batchSize
                vel[k] = (np.float32(fx["momentum"]) * vel[k] - G[k] * np.float32(fx["lr"] / bs)).astype(np.float32)
                P[k] = (P[k] + vel[k]).astype(np.float32)
    return before, loss()


@pytest.mark.parametrize("variant", ["no_bias", "with_bias"])
@pytest.mark.parametrize("is_causal", [False, True])
def test_multi_head_attention_chain_losses(golden, oracle, variant, is_causal):
    """Both stored losses of Test_MultiHeadAttention_{no,with}_bias: the first pins mha_forward (projections, head
    split, scaled scores, causal mask, softmax, head merge), the second - 50 SGD steps later - mha_backward."""
    fx = golden["PyTorch_MultiHeadAttention"]
    case = [c for c in fx[variant]["cases"] if c["is_causal"] == is_causal][0]
    before, after = _mha_chain(oracle, fx, variant, is_causal)
    assert abs(before - case["loss_before"]) < fx["tolerance"], (before, case)     # the reference's own 1e-6
    assert abs(after - case["loss_after"]) < fx["tolerance"], (after, case)


def test_transpose_and_multiply_tensor(oracle):
    """The Sgeam / Sdgmm restatements against the reference's known transposes (Tests/CPU/TestCpuTensor.cs:82-100) and
    the closed form its MultiplyTensor test asserts (:216-241: expected[i] = a[i] * x[i] and a[i] * x[i / (7*7)])."""
    assert np.array_equal(oracle.transpose(np.array([[1.0]], np.float32)), [[1.0]])
    assert np.array_equal(oracle.transpose(np.arange(6, dtype=np.float32).reshape(1, 6)), np.arange(6).reshape(6, 1))
    assert np.array_equal(oracle.transpose(np.arange(6, dtype=np.float32).reshape(2, 3)).reshape(-1), [0, 3, 1, 4, 2, 5])
    rng = np.random.default_rng(0)
    a = rng.uniform(-10, 10, (4, 9, 7, 7)).astype(np.float32)
    x_same = rng.uniform(-10, 10, a.shape).astype(np.float32)
    assert np.array_equal(oracle.multiply_tensor(a, x_same), a * x_same)
    x = rng.uniform(-10, 10, (4, 9, 1, 1)).astype(np.float32)
    want = (a.reshape(-1) * x.reshape(-1)[np.arange(a.size) // 49]).reshape(a.shape)
    assert np.array_equal(oracle.multiply_tensor(a, x), want)
    # general geam: both operands, both transposes, padded leading dimensions, against numpy
    m, n = 5, 7
    A = rng.uniform(-1, 1, (n + 2) * (m + 3)).astype(np.float32)      # op(A) = A^T: A stored n x m, lda = n + 2
    B = rng.uniform(-1, 1, (m + 1) * n).astype(np.float32)            # B stored m x n, ldb = m + 1
    C0 = rng.uniform(-1, 1, (m + 4) * n).astype(np.float32)
    got = oracle.sgeam_colmajor(True, False, m, n, 0.5, A, n + 2, -2.0, B, m + 1, C0, m + 4)
    Am = np.array([[A[j + i * (n + 2)] for j in range(n)] for i in range(m)])
    Bm = np.array([[B[i + j * (m + 1)] for j in range(n)] for i in range(m)])
    want = C0.copy()
    for j in range(n):
        for i in range(m):
            want[i + j * (m + 4)] = np.float32(0.5 * Am[i, j] - 2.0 * Bm[i, j])
    assert np.allclose(got, want, atol=1e-6) and np.array_equal(got.reshape(n, m + 4)[:, m:], C0.reshape(n, m + 4)[:, m:])
    left = oracle.sdgmm_colmajor(False, 3, 2, np.arange(6, dtype=np.float32), 3, np.array([2, 3, 4], np.float32), 1,
                                 np.zeros(6, np.float32), 3)
    assert np.array_equal(left, [0, 3, 8, 6, 12, 20])
