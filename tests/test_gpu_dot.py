"""GPU parity tests of Tensor.Dot / BatchMatrixMultiplication through the C ABI.

Shaped like the reference's own harness (Tests/TestParallelRunCpuVersusGpu.cs:1449-1465):
the same seeded host inputs go to the oracle and to the device, and every output is
compared.  fp32 bar (written out in `tol`): max|C_gpu - C_ref| <= 1e-4*sqrt(K)*max|a|*max|b|.
"""
import ctypes
import itertools

import numpy as np
import pytest

from tests.helpers import random_tensor

pytestmark = pytest.mark.gpu


def tol(K, a, b, alpha=1.0, beta=0.0, c=None):
    t = 1e-4 * np.sqrt(max(K, 1)) * float(np.max(np.abs(a))) * float(np.max(np.abs(b))) * max(abs(alpha), 1e-30)
    if beta != 0.0 and c is not None:
        t += 1e-6 * abs(beta) * float(np.max(np.abs(c)))
    return max(t, 1e-30)


def gpu_dot(w, a, tA, b, tB, alpha=1.0, beta=0.0, c=None, c_shape=None, prefill=None):
    from sharpnet_amd import GPUTensor
    ga, gb = GPUTensor(a.shape, a, w), GPUTensor(b.shape, b, w)
    if c is not None:
        gc = GPUTensor(c.shape, c, w)
    else:
        gc = GPUTensor(c_shape, None, w)
        if prefill is not None:
            gc.SetValue(prefill)
    gc.Dot(ga, tA, gb, tB, alpha, beta)
    out = gc.ToNumpy()
    for t in (ga, gb, gc):
        t.Dispose()
    return out


def mnk(a, tA, b, tB):
    a2, b2 = a.reshape(a.shape[0], -1), b.reshape(b.shape[0], -1)
    M = a2.shape[1] if tA else a2.shape[0]
    N = b2.shape[0] if tB else b2.shape[1]
    K = a2.shape[0] if tA else a2.shape[1]
    return M, N, K


# ---------------------------------------------------------------------------
# reference known answers
# ---------------------------------------------------------------------------
def test_TestDot_known_answers(golden, gpu_wrapper):
    """Tests/GPU/TestGpuTensor.cs:50-120, tolerance 1e-9."""
    for case in golden["TestDot"]["cases"]:
        def arr(v, shape):
            return np.zeros(shape, np.float32) if v == "zeros" else np.array(v, np.float32).reshape(shape)
        a, b = arr(case["a"], case["a_shape"]), arr(case["b"], case["b_shape"])
        got = gpu_dot(gpu_wrapper, a, False, b, False, 1, 0, c_shape=case["c_shape"], prefill=float("nan"))
        expected = arr(case["expected"], case["c_shape"])
        assert got.shape == expected.shape
        assert np.max(np.abs(got - expected)) <= golden["TestDot"]["tolerance"], case


def test_QR_identity_on_device(golden, gpu_wrapper):
    """Tests/GPU/TestGpuTensor.cs:18-47: Dot(Q,R) ~ A (1e-4), max|QtQ - I| < 1e-6."""
    for case in golden["QR"]["cases"]:
        A, Q = np.array(case["A"], np.float32), np.array(case["Q"], np.float32)
        n = A.shape[1]
        R = gpu_dot(gpu_wrapper, Q, True, A, False, c_shape=[n, n])
        QR = gpu_dot(gpu_wrapper, Q, False, R, False, c_shape=list(A.shape))
        assert np.max(np.abs(QR - A)) < 1e-4
        QtQ = gpu_dot(gpu_wrapper, Q, True, Q, False, c_shape=[n, n])
        assert np.max(np.abs(QtQ - np.eye(n))) < 1e-6


# ---------------------------------------------------------------------------
# CPU-versus-GPU harness cases
# ---------------------------------------------------------------------------
def test_cpu_vs_gpu_TestDot_cases(oracle, gpu_wrapper):
    """TestDot 8x10x12 (:368-375), TestDotV2 (:436-443), TestDotV3 2x20000x2 (:445-456)."""
    rng = np.random.default_rng(0)
    for (M, K, N) in [(8, 10, 12), (8, 10, 12), (2, 20000, 2)]:
        a, b = random_tensor(rng, (M, K)), random_tensor(rng, (K, N))
        got = gpu_dot(gpu_wrapper, a, False, b, False, 1, 0, c_shape=[M, N], prefill=float("nan"))
        ref = oracle.dot(a, False, b, False)
        err = np.max(np.abs(got - ref))
        assert err <= tol(K, a, b), (M, N, K, err)
        assert err <= 1e-2   # the reference's own acceptance (:1440-1447)


def test_cpu_vs_gpu_BatchMatrixMultiplication(oracle, gpu_wrapper):
    """Tests/TestParallelRunCpuVersusGpu.cs:377-401: batch 3, L=12, d=7; NT alpha=0.25, NN, TN."""
    from sharpnet_amd import GPUTensor
    rng = np.random.default_rng(1)
    batch, L, d = 3, 12, 7
    V, dy, K_, Q = (random_tensor(rng, (batch, L, d)) for _ in range(4))
    S = random_tensor(rng, (batch, L, L))
    cases = [((batch, L, L), dy, False, V, True, 0.25),
             ((batch, L, d), S, False, K_, False, 1.0),
             ((batch, L, d), S, True, Q, False, 1.0)]
    for c_shape, a, tA, b, tB, alpha in cases:
        ga, gb = GPUTensor(a.shape, a, gpu_wrapper), GPUTensor(b.shape, b, gpu_wrapper)
        gc = GPUTensor(c_shape, None, gpu_wrapper)
        gc.SetValue(float("nan"))
        gc.BatchMatrixMultiplication(ga, tA, gb, tB, alpha, 0.0)
        got = gc.ToNumpy()
        ref = oracle.bmm(a, tA, b, tB, alpha, 0.0)
        Kdim = a.shape[1] if tA else a.shape[2]
        assert np.max(np.abs(got - ref)) <= tol(Kdim, a, b, alpha)


# ---------------------------------------------------------------------------
# every tile configuration x transpose x alpha/beta on ragged shapes
# ---------------------------------------------------------------------------
SHAPES = [(35, 21, 124), (33, 17, 65), (129, 257, 63), (256, 256, 64), (300, 130, 200), (64, 64, 16), (1, 1, 1),
          (257, 100, 33), (5, 300, 1000)]


@pytest.mark.parametrize("tA,tB", list(itertools.product([False, True], repeat=2)))
def test_all_configs_all_transposes(oracle, gpu_wrapper, tA, tB):
    rng = np.random.default_rng(100 + 2 * tA + tB)
    ncfg = len(gpu_wrapper.configs())
    try:
        for (M, N, K) in SHAPES:
            a = random_tensor(rng, (K, M) if tA else (M, K), -1, 1)
            b = random_tensor(rng, (N, K) if tB else (K, N), -1, 1)
            c = random_tensor(rng, (M, N), -1, 1)
            refs = {}
            for alpha, beta in [(1.0, 0.0), (0.25, 0.0), (-1.0, 1.0), (0.5, 1.0)]:
                refs[(alpha, beta)] = oracle.dot(a, tA, b, tB, alpha, beta, c if beta != 0 else None)
            for cfg in range(ncfg):
                for splitk in (1, 2, 4):
                    if splitk > 1 and K < 64:
                        continue
                    gpu_wrapper.set_tuning(cfg, splitk)
                    for (alpha, beta), ref in refs.items():
                        if beta == 0.0:
                            got = gpu_dot(gpu_wrapper, a, tA, b, tB, alpha, beta, c_shape=[M, N],
                                          prefill=float("nan"))
                        else:
                            got = gpu_dot(gpu_wrapper, a, tA, b, tB, alpha, beta, c=c)
                        err = np.max(np.abs(got - ref))
                        assert np.all(np.isfinite(got)), (M, N, K, cfg, splitk, alpha, beta)
                        assert err <= tol(K, a, b, alpha, beta, c), (M, N, K, cfg, splitk, alpha, beta, err)
    finally:
        gpu_wrapper.set_tuning(-1, 0)


def test_beta_zero_never_reads_destination(oracle, gpu_wrapper):
    """TensorMemoryPool hands out uninitialised memory (Prod/Data/TensorMemoryPool.cs:59-64)."""
    rng = np.random.default_rng(2)
    for (M, N, K) in [(128, 256, 784), (300, 300, 300), (1000, 64, 2048)]:
        a, b = random_tensor(rng, (M, K)), random_tensor(rng, (K, N))
        for fill in (float("nan"), float("inf")):
            got = gpu_dot(gpu_wrapper, a, False, b, False, 1, 0, c_shape=[M, N], prefill=fill)
            assert np.all(np.isfinite(got))
            assert np.max(np.abs(got - oracle.dot(a, False, b, False))) <= tol(K, a, b)


def test_aliased_operands_VanillaSgdOrtho_pattern(oracle, gpu_wrapper):
    """Prod/Optimizers/VanillaSgdOrtho.cs:83: buffer = I - W.W^T via Dot(W,false,W,true,-1,1) on an identity."""
    from sharpnet_amd import GPUTensor
    rng = np.random.default_rng(3)
    m, n = 37, 53
    W = random_tensor(rng, (m, n), -1, 1)
    gW = GPUTensor(W.shape, W, gpu_wrapper)
    gI = GPUTensor([m, m], np.eye(m, dtype=np.float32), gpu_wrapper)
    gI.Dot(gW, False, gW, True, -1.0, 1.0)
    got = gI.ToNumpy()
    ref = oracle.dot(W, False, W, True, -1.0, 1.0, np.eye(m, dtype=np.float32))
    assert np.max(np.abs(got - ref)) <= tol(n, W, W, 1.0, 1.0, np.eye(m))
    # alpha = 0.5, beta = 1 accumulation (:88)
    X = random_tensor(rng, (m, n), -1, 1)
    gX = GPUTensor(X.shape, X, gpu_wrapper)
    gX.Dot(gI, False, gW, False, 0.5, 1.0)
    ref2 = oracle.dot(ref, False, W, False, 0.5, 1.0, X)
    assert np.max(np.abs(gX.ToNumpy() - ref2)) <= tol(m, ref, W, 0.5, 1.0, X) + 1e-5


@pytest.mark.parametrize("m,n", [(37, 53), (64, 256), (130, 70)])
def test_VanillaSgdOrtho_update_all_five_products(oracle, gpu_wrapper, m, n):
    """The whole sequence of Prod/Optimizers/VanillaSgdOrtho.cs:82-88 on the device, buffer for buffer:
    I - W.W^T (NT, alpha -1, beta 1, A == B), (..).dW (NN), W^T.dW (TN, beta 0), -= dW^T.W (TN, alpha -1, beta 1),
    += 0.5 W.(..) (NN, alpha 0.5, beta 1); every intermediate against the oracle fed with the oracle's own chain."""
    from sharpnet_amd import GPUTensor
    w = gpu_wrapper
    rng = np.random.default_rng(300 + m)
    W, dW = random_tensor(rng, (m, n), -1, 1), random_tensor(rng, (m, n), -1, 1)
    gW, gdW = GPUTensor(W.shape, W, w), GPUTensor(dW.shape, dW, w)
    eye = np.eye(m, dtype=np.float32)
    buffer_mm, buffer_mn, buffer_nn = GPUTensor([m, m], eye, w), GPUTensor([m, n], None, w), GPUTensor([n, n], None, w)
    buffer_mn.SetValue(float("nan"))
    buffer_nn.SetValue(float("nan"))
    buffer_mm.Dot(gW, False, gW, True, -1.0, 1.0)
    r_mm = oracle.dot(W, False, W, True, -1.0, 1.0, eye)
    assert np.max(np.abs(buffer_mm.ToNumpy() - r_mm)) <= tol(n, W, W, 1.0, 1.0, eye)
    buffer_mn.Dot(buffer_mm, gdW)                                     # two-argument form: (false, false, 1, 0)
    r_mn = oracle.dot(r_mm, False, dW, False)
    assert np.max(np.abs(buffer_mn.ToNumpy() - r_mn)) <= 2 * tol(m, r_mm, dW)
    buffer_nn.Dot(gW, True, gdW, False, 1.0, 0.0)
    r_nn = oracle.dot(W, True, dW, False, 1.0, 0.0)
    assert np.max(np.abs(buffer_nn.ToNumpy() - r_nn)) <= tol(m, W, dW)
    buffer_nn.Dot(gdW, True, gW, False, -1.0, 1.0)
    r_nn2 = oracle.dot(dW, True, W, False, -1.0, 1.0, r_nn)
    assert np.max(np.abs(buffer_nn.ToNumpy() - r_nn2)) <= 2 * tol(m, dW, W, 1.0, 1.0, r_nn)
    # antisymmetric by construction: W^T dW - (W^T dW)^T
    assert np.max(np.abs(buffer_nn.ToNumpy() + buffer_nn.ToNumpy().T)) <= 4 * tol(m, dW, W)
    buffer_mn.Dot(gW, False, buffer_nn, False, 0.5, 1.0)
    r_fin = oracle.dot(W, False, r_nn2, False, 0.5, 1.0, r_mn)
    assert np.max(np.abs(buffer_mn.ToNumpy() - r_fin)) <= 4 * (tol(n, W, r_nn2, 0.5) + tol(m, r_mm, dW))


def test_views_at_odd_element_offsets(oracle, gpu_wrapper):
    """Slices are views at Pointer + 4*startIndex (GpuTensor.cs:616): only 4-byte alignment may be assumed."""
    from sharpnet_amd import GPUTensor
    rng = np.random.default_rng(4)
    M, N, K = 130, 260, 70
    for off in (1, 2, 3, 5):
        bufA = random_tensor(rng, (M * K + 8,), -1, 1)
        bufB = random_tensor(rng, (K * N + 8,), -1, 1)
        bufC = random_tensor(rng, (M * N + 8,), -1, 1)
        gA, gB, gC = (GPUTensor([x.size], x, gpu_wrapper) for x in (bufA, bufB, bufC))
        a, b, c = gA.Slice(off, [M, K]), gB.Slice(off, [K, N]), gC.Slice(off, [M, N])
        c.Dot(a, False, b, False, 1.0, 1.0)
        out = gC.ToNumpy()
        ref = oracle.dot(bufA[off:off + M * K].reshape(M, K), False, bufB[off:off + K * N].reshape(K, N), False, 1.0,
                         1.0, bufC[off:off + M * N].reshape(M, N))
        assert np.max(np.abs(out[off:off + M * N].reshape(M, N) - ref)) <= tol(K, bufA, bufB, 1, 1, bufC)
        # nothing outside the view was written
        assert np.array_equal(out[:off], bufC[:off]) and np.array_equal(out[off + M * N:], bufC[off + M * N:])
        # transposed operands through views as well
        at, bt = gA.Slice(off, [K, M]), gB.Slice(off, [N, K])
        c.Dot(at, True, bt, True, 1.0, 0.0)
        ref = oracle.dot(bufA[off:off + M * K].reshape(K, M), True, bufB[off:off + K * N].reshape(N, K), True)
        assert np.max(np.abs(c.ToNumpy() - ref)) <= tol(K, bufA, bufB)


def test_colmajor_sgemm_with_padded_leading_dimensions(oracle, gpu_wrapper):
    """snhip_sgemm has cublasSgemm_v2's column-major meaning incl. lda/ldb/ldc > rows; padding stays untouched."""
    from sharpnet_amd import GPUTensor
    lib, h = gpu_wrapper.lib, gpu_wrapper.handle
    rng = np.random.default_rng(5)
    m, n, k = 70, 45, 130
    for ta, tb in itertools.product([0, 1], repeat=2):
        lda = (k if ta else m) + 3
        ldb = (n if tb else k) + 2
        ldc = m + 5
        A = random_tensor(rng, ((m if ta else k), lda), -1, 1)
        B = random_tensor(rng, ((k if tb else n), ldb), -1, 1)
        C = random_tensor(rng, (n, ldc), -1, 1)
        gA, gB, gC = (GPUTensor(list(x.shape), x, gpu_wrapper) for x in (A, B, C))
        al, be = ctypes.c_float(0.5), ctypes.c_float(-1.0)
        st = lib.snhip_sgemm(h, ta, tb, m, n, k, ctypes.byref(al), gA.Pointer, lda, gB.Pointer, ldb, ctypes.byref(be),
                             gC.Pointer, ldc)
        assert st == 0
        got = gC.ToNumpy()
        ref = oracle.sgemm_colmajor(ta, tb, m, n, k, 0.5, A, lda, B, ldb, -1.0, C, ldc).reshape(n, ldc)
        assert np.max(np.abs(got - ref)) <= tol(k, A, B, 0.5, 1.0, C)
        assert np.array_equal(got[:, m:], C[:, m:])


def test_row_major_entry_points_agree(oracle, gpu_wrapper):
    """snhip_dot / snhip_dot_bias / snhip_bmm / snhip_gemm_rm give the oracle's numbers."""
    from sharpnet_amd import GPUTensor
    lib, h = gpu_wrapper.lib, gpu_wrapper.handle
    rng = np.random.default_rng(6)
    M, N, K = 128, 256, 784
    x = rng.uniform(0, 1, (M, K)).astype(np.float32)
    w = random_tensor(rng, (N, K), -0.076, 0.076)
    bias = random_tensor(rng, (N,), -1, 1)
    gx, gw, gb = GPUTensor([M, K], x, gpu_wrapper), GPUTensor([N, K], w, gpu_wrapper), GPUTensor([N], bias, gpu_wrapper)
    gy = GPUTensor([M, N], None, gpu_wrapper)
    gy.SetValue(float("nan"))
    gy.DotRowMajor(gx, False, gw, True, 1.0, 0.0, bias=gb)
    ref = oracle.dense_forward(x, w, bias)
    assert np.max(np.abs(gy.ToNumpy() - ref)) <= tol(K, x, w) + 1e-6
    # inner-dimension mismatch is rejected, not computed
    assert lib.snhip_dot(h, gx.Pointer, M, K, 0, gw.Pointer, N, K, 0, gy.Pointer, 1.0, 0.0) == 7
    # strided batch through snhip_bmm
    batch, T, d = 5, 40, 24
    Q, Kt = random_tensor(rng, (batch, T, d)), random_tensor(rng, (batch, T, d))
    gq, gk = GPUTensor(Q.shape, Q, gpu_wrapper), GPUTensor(Kt.shape, Kt, gpu_wrapper)
    gs = GPUTensor([batch, T, T], None, gpu_wrapper)
    st = lib.snhip_bmm(h, gq.Pointer, T, d, 0, T * d, gk.Pointer, T, d, 1, T * d, gs.Pointer, T * T, batch, 0.125, 0.0)
    assert st == 0
    assert np.max(np.abs(gs.ToNumpy() - oracle.bmm(Q, False, Kt, True, 0.125))) <= tol(d, Q, Kt, 0.125)
    # sub-matrix views with explicit leading dimensions through snhip_gemm_rm
    big = random_tensor(rng, (90, 200), -1, 1)
    gbig = GPUTensor(list(big.shape), big, gpu_wrapper)
    sub_a = big[10:70, 20:120]        # 60 x 100, lda = 200
    sub_b = big[0:50, 60:160]         # 50 x 100, ldb = 200, used transposed -> K=100, N=50
    gout = GPUTensor([60, 64], np.zeros((60, 64), np.float32), gpu_wrapper)
    st = lib.snhip_gemm_rm(h, 0, 1, 60, 50, 100, 1.0, gbig.Pointer + 4 * (10 * 200 + 20), 200, 0,
                           gbig.Pointer + 4 * 60, 200, 0, 0.0, gout.Pointer, 64, 0, 1, None)
    assert st == 0
    got = gout.ToNumpy()
    ref = oracle.dot(np.ascontiguousarray(sub_a), False, np.ascontiguousarray(sub_b), True)
    assert np.max(np.abs(got[:, :50] - ref)) <= tol(100, sub_a, sub_b)
    assert np.all(got[:, 50:] == 0)


def test_degenerate_products(oracle, gpu_wrapper):
    """alpha == 0 or K == 0: C = beta*C and A, B are not referenced; M or N == 0: no-op."""
    from sharpnet_amd import GPUTensor
    lib, h = gpu_wrapper.lib, gpu_wrapper.handle
    rng = np.random.default_rng(7)
    c = random_tensor(rng, (9, 11))
    gc = GPUTensor([9, 11], c, gpu_wrapper)
    nan = np.full((9, 5), np.nan, np.float32)
    ga, gb = GPUTensor([9, 5], nan, gpu_wrapper), GPUTensor([5, 11], np.full((5, 11), np.nan, np.float32), gpu_wrapper)
    gc.Dot(ga, False, gb, False, 0.0, 0.5)
    assert np.allclose(gc.ToNumpy(), 0.5 * c, atol=1e-7)
    gc.Dot(ga, False, gb, False, 0.0, 0.0)
    assert np.all(gc.ToNumpy() == 0)
    assert lib.snhip_dot(h, ga.Pointer, 0, 5, 0, gb.Pointer, 5, 11, 0, gc.Pointer, 1.0, 0.0) == 0
    # invalid arguments come back as status codes, nothing is thrown or aborted
    one = ctypes.c_float(1.0)
    assert lib.snhip_sgemm(h, 5, 0, 4, 4, 4, ctypes.byref(one), ga.Pointer, 4, gb.Pointer, 4, ctypes.byref(one),
                           gc.Pointer, 4) == 7
    assert lib.snhip_sgemm(h, 0, 0, 4, 4, 4, ctypes.byref(one), ga.Pointer, 2, gb.Pointer, 4, ctypes.byref(one),
                           gc.Pointer, 4) == 7
    assert lib.snhip_sgemm(h, 0, 0, -1, 4, 4, ctypes.byref(one), ga.Pointer, 4, gb.Pointer, 4, ctypes.byref(one),
                           gc.Pointer, 4) == 7


def test_run_to_run_determinism(oracle, gpu_wrapper):
    """The reference opts into deterministic cuBLAS (GPUWrapper.cs:78-80); split-K must not use float atomics.
    Both ways of adding the split-K partial sums (second kernel / last workgroup in the GEMM kernel) are covered."""
    rng = np.random.default_rng(8)
    try:
        for mode in (1, 2, 0):
            gpu_wrapper.set_splitk_mode(mode)
            for (M, N, K, cfg, sk) in [(300, 200, 4096, -1, 0), (64, 64, 8192, 6, 8), (512, 512, 512, 0, 1),
                                       (256, 2048, 512, 6, 4), (1000, 64, 4096, 5, 16), (130, 70, 3000, 3, 8)]:
                gpu_wrapper.set_tuning(cfg, sk)
                a, b = random_tensor(rng, (M, K)), random_tensor(rng, (K, N))
                c = random_tensor(rng, (M, N))
                first = gpu_dot(gpu_wrapper, a, False, b, False, 0.5, 1.0, c=c)
                assert np.max(np.abs(first - oracle.dot(a, False, b, False, 0.5, 1.0, c))) <= tol(K, a, b, 0.5, 1.0, c)
                for _ in range(4):
                    assert np.array_equal(first, gpu_dot(gpu_wrapper, a, False, b, False, 0.5, 1.0, c=c))
    finally:
        gpu_wrapper.set_tuning(-1, 0)
        gpu_wrapper.set_splitk_mode(0)


def test_splitk_modes_batched_and_bias(oracle, gpu_wrapper):
    """In-kernel and two-kernel split-K reductions on a strided batch and with the fused bias."""
    from sharpnet_amd import GPUTensor
    from sharpnet_amd.hiplib import check_status
    lib, h = gpu_wrapper.lib, gpu_wrapper.handle
    rng = np.random.default_rng(9)
    try:
        for mode in (1, 2):
            gpu_wrapper.set_splitk_mode(mode)
            for cfg in (0, 3, 6):
                gpu_wrapper.set_tuning(cfg, 4)
                batch, M, N, K = 5, 70, 45, 1030
                a, b = random_tensor(rng, (batch, M, K), -1, 1), random_tensor(rng, (batch, N, K), -1, 1)
                ga, gb = GPUTensor(a.shape, a, gpu_wrapper), GPUTensor(b.shape, b, gpu_wrapper)
                gc = GPUTensor([batch, M, N], None, gpu_wrapper)
                gc.SetValue(float("nan"))
                gc.BatchMatrixMultiplication(ga, False, gb, True, 0.25, 0.0)
                assert gpu_wrapper.last_tuning() == (cfg, 4)
                assert np.max(np.abs(gc.ToNumpy() - oracle.bmm(a, False, b, True, 0.25))) <= tol(K, a, b, 0.25)
                x, w_, bias = random_tensor(rng, (128, 784), 0, 1), random_tensor(rng, (256, 784), -0.07, 0.07), \
                    random_tensor(rng, (256,), -1, 1)
                gx, gw, gbias = (GPUTensor(t.shape, t, gpu_wrapper) for t in (x, w_, bias))
                gy = GPUTensor([128, 256], None, gpu_wrapper)
                gy.SetValue(float("nan"))
                gy.DotRowMajor(gx, False, gw, True, 1.0, 0.0, bias=gbias)
                assert np.max(np.abs(gy.ToNumpy() - oracle.dense_forward(x, w_, bias))) <= tol(784, x, w_) + 1e-6
    finally:
        gpu_wrapper.set_tuning(-1, 0)
        gpu_wrapper.set_splitk_mode(0)


def test_limits_and_user_stream(oracle, gpu_wrapper):
    """Batch counts beyond the grid limit go out in slices; a caller-supplied stream is honoured."""
    from sharpnet_amd import GPUTensor
    from sharpnet_amd.hiplib import check_status
    lib, h = gpu_wrapper.lib, gpu_wrapper.handle
    rng = np.random.default_rng(10)
    tiny = GPUTensor([70000, 1, 1], np.ones(70000, np.float32), gpu_wrapper)
    out = GPUTensor([70000, 1, 1], None, gpu_wrapper)
    # 70000 matrices > 65535 (the grid limit): sliced inside the library, every matrix computed
    vals = np.arange(70000, dtype=np.float32) % 97
    tiny2 = GPUTensor([70000, 1, 1], vals, gpu_wrapper)
    assert lib.snhip_bmm(h, tiny.Pointer, 1, 1, 0, 1, tiny2.Pointer, 1, 1, 0, 1, out.Pointer, 1, 70000, 2.0, 0.0) == 0
    assert np.array_equal(out.ToNumpy().reshape(-1), 2.0 * vals)
    # a two-level batch whose outer strides continue the inner ones is one level to the library: also sliced
    from sharpnet_amd import hiplib
    import ctypes
    out.ZeroMemory()
    d = hiplib.GemmDesc(M=1, N=1, K=1, A=tiny.Pointer, lda=1, strideA=1, strideA_outer=2, B=tiny2.Pointer, ldb=1, strideB=1,
                        strideB_outer=2, C=out.Pointer, ldc=1, strideC=1, strideC_outer=2, batch=70000, batch_inner=2)
    assert lib.snhip_gemm_ex(h, ctypes.byref(d)) == 0
    assert np.array_equal(out.ToNumpy().reshape(-1), vals)
    # a genuine two-level batch that long is refused (status 15): inner stride 0, outer stride 1 for A and B
    d = hiplib.GemmDesc(M=1, N=1, K=1, A=tiny.Pointer, lda=1, strideA=0, strideA_outer=1, B=tiny2.Pointer, ldb=1, strideB=0,
                        strideB_outer=1, C=out.Pointer, ldc=1, strideC=1, strideC_outer=2, batch=70000, batch_inner=2)
    assert lib.snhip_gemm_ex(h, ctypes.byref(d)) == 15
    # K == 0 on a batch: C = beta * C
    c0 = random_tensor(rng, (4, 3, 5))
    gc = GPUTensor([4, 3, 5], c0, gpu_wrapper)
    assert lib.snhip_bmm(h, tiny.Pointer, 3, 0, 0, 0, tiny.Pointer, 0, 5, 0, 0, gc.Pointer, 15, 4, 1.0, 0.5) == 0
    assert np.allclose(gc.ToNumpy(), 0.5 * c0, atol=1e-7)
    # caller-supplied stream
    import ctypes
    st = ctypes.c_void_p()
    check_status(lib.snhip_stream_create(ctypes.byref(st)))
    try:
        check_status(lib.snhip_set_stream(h, st))
        a, b = random_tensor(rng, (300, 500)), random_tensor(rng, (500, 200))
        got = gpu_dot(gpu_wrapper, a, False, b, False, c_shape=[300, 200], prefill=float("nan"))
        assert np.max(np.abs(got - oracle.dot(a, False, b, False))) <= tol(500, a, b)
    finally:
        check_status(lib.snhip_set_stream(h, None))
        check_status(lib.snhip_stream_destroy(st))


def test_random_shapes_offsets_and_pitches(oracle, gpu_wrapper):
    """300 seeded random cases through snhip_gemm_rm: shapes up to 400, all transposes, random alpha/beta, padded
    leading dimensions, element offsets (4-byte alignment only), strided batches, optional bias; automatic tiling."""
    from sharpnet_amd import GPUTensor
    lib, h = gpu_wrapper.lib, gpu_wrapper.handle
    rng = np.random.default_rng(2024)
    for case in range(300):
        M, N, K = (int(rng.integers(1, 400)) for _ in range(3))
        if case % 7 == 0:
            K = int(rng.integers(400, 3000))
        tA, tB = bool(rng.integers(2)), bool(rng.integers(2))
        batch = int(rng.choice([1, 1, 1, 2, 5]))
        alpha = float(rng.choice([1.0, -1.0, 0.5, 0.125, 2.0]))
        beta = float(rng.choice([0.0, 0.0, 1.0, -0.5]))
        use_bias = bool(rng.integers(2)) and batch == 1
        ar, ac = (K, M) if tA else (M, K)
        br, bc = (N, K) if tB else (K, N)
        lda, ldb, ldc = ac + int(rng.integers(0, 4)), bc + int(rng.integers(0, 4)), N + int(rng.integers(0, 4))
        offa, offb, offc = (int(rng.integers(0, 4)) for _ in range(3))
        sA, sB, sC = ar * lda + int(rng.integers(0, 3)), br * ldb + int(rng.integers(0, 3)), M * ldc + int(rng.integers(0, 3))
        bufA = random_tensor(rng, (offa + batch * sA + 4,), -1, 1)
        bufB = random_tensor(rng, (offb + batch * sB + 4,), -1, 1)
        bufC = random_tensor(rng, (offc + batch * sC + 4,), -1, 1)
        bias = random_tensor(rng, (N,), -1, 1) if use_bias else None
        gA, gB, gC = (GPUTensor([x.size], x, gpu_wrapper) for x in (bufA, bufB, bufC))
        gbias = GPUTensor([N], bias, gpu_wrapper) if use_bias else None
        st = lib.snhip_gemm_rm(h, int(tA), int(tB), M, N, K, alpha, gA.Pointer + 4 * offa, lda, sA,
                               gB.Pointer + 4 * offb, ldb, sB, beta, gC.Pointer + 4 * offc, ldc, sC, batch,
                               gbias.Pointer if use_bias else None)
        assert st == 0, (case, st)
        got = gC.ToNumpy()
        want = bufC.copy()
        for i in range(batch):
            a = bufA[offa + i * sA: offa + i * sA + ar * lda].reshape(ar, lda)[:, :ac]
            b = bufB[offb + i * sB: offb + i * sB + br * ldb].reshape(br, ldb)[:, :bc]
            cview = want[offc + i * sC: offc + i * sC + M * ldc].reshape(M, ldc)
            ref = oracle.dot(np.ascontiguousarray(a), tA, np.ascontiguousarray(b), tB, alpha, beta,
                             np.ascontiguousarray(cview[:, :N]) if beta != 0 else None)
            if use_bias:
                ref = ref + bias[None, :]
            gview = got[offc + i * sC: offc + i * sC + M * ldc].reshape(M, ldc)
            err = float(np.max(np.abs(gview[:, :N] - ref)))
            assert err <= tol(K, a, b, alpha, beta, cview) + 1e-6, (case, M, N, K, tA, tB, batch, alpha, beta, err)
            cview[:, :N] = gview[:, :N]
        # everything outside the M x N windows (padding columns, gaps between matrices, offsets) is untouched
        assert np.array_equal(got, want), (case, "padding overwritten")
        for t in (gA, gB, gC):
            t.Dispose()


def test_random_aligned_shapes_every_tiled_configuration(oracle, gpu_wrapper):
    """160 seeded cases on whole, tightly packed tensors (16-byte-aligned rows whenever the extents allow: the
    vector write-out, the branch-free edge loads with and without shifted vectors), sizes up to 1100 with a bias
    towards multiples of 4 and of the tile sizes plus or minus a little, every fp32 tiled configuration in turn with
    split-K 1 or 2, beta 0 / 1 / -0.5.  Reference: the oracle's float64 closed form."""
    from sharpnet_amd import GPUTensor
    w = gpu_wrapper
    tiled = [i for i, c in enumerate(w.configs()) if c["kind"] == "fp32"]
    assert len(tiled) == 10
    rng = np.random.default_rng(77)

    def extent():
        base = int(rng.choice([64, 128, 256, 512, 1024]))
        kind = int(rng.integers(4))
        if kind == 0:
            return base
        if kind == 1:
            return base + int(rng.choice([-8, -4, 4, 8, 12, 40]))      # ragged, multiple of 4
        if kind == 2:
            return base + int(rng.choice([-3, -1, 1, 2, 3, 5]))        # ragged, odd
        return int(rng.integers(1, 1100))
    try:
        for case in range(160):
            M, N, K = extent(), extent(), extent()
            if M * N * K > 6e8:
                K = max(16, K // 4)
            tA, tB = bool(rng.integers(2)), bool(rng.integers(2))
            alpha = float(rng.choice([1.0, -0.5, 2.0]))
            beta = float(rng.choice([0.0, 0.0, 1.0, -0.5]))
            a = random_tensor(rng, (K, M) if tA else (M, K), -1, 1)
            b = random_tensor(rng, (N, K) if tB else (K, N), -1, 1)
            c = random_tensor(rng, (M, N), -1, 1)
            cfg = tiled[case % len(tiled)]
            sk = 2 if (case // len(tiled)) % 3 == 2 and K >= 256 else 1
            w.set_tuning(cfg, sk)
            ga, gb, gc = GPUTensor(a.shape, a, w), GPUTensor(b.shape, b, w), GPUTensor(c.shape, c, w)
            gc.Dot(ga, tA, gb, tB, alpha, beta)
            assert w.last_tuning() == (cfg, sk), (case, w.last_tuning())
            got = gc.ToNumpy()
            ref = oracle.dot_f64(a, tA, b, tB, alpha, beta, c if beta != 0 else None)
            err = float(np.max(np.abs(got - ref)))
            assert err <= tol(K, a, b, alpha, beta, c) + 1e-6, (case, cfg, sk, M, N, K, tA, tB, alpha, beta, err)
            for t in (ga, gb, gc):
                t.Dispose()
    finally:
        w.set_tuning(-1, 0)


def test_sgeam_transpose_and_sdgmm(oracle, gpu_wrapper):
    """Tensor.Transpose (cublasSgeam with the reference's arguments, Tests/TestParallelRunCpuVersusGpu.cs:522-533 sizes and
    larger ones that span several tiles), the general Sgeam form, and Tensor.MultiplyTensor (cublasSdgmm, same file
    :511-519,583-590) against the oracle; bit-exact, these are copies and single products."""
    import ctypes
    from sharpnet_amd import GPUTensor
    w = gpu_wrapper
    rng = np.random.default_rng(8)
    for h in (1, 2, 5, 10, 33, 257):
        for wd in (1, 2, 5, 10, 64, 100):
            a = random_tensor(rng, (h, wd), -1.5, 1.5)
            ga, gt = GPUTensor([h, wd], a, w), GPUTensor([wd, h], None, w)
            gt.SetValue(float("nan"))
            ga.Transpose(gt)
            assert gt.Shape == [wd, h] and np.array_equal(gt.ToNumpy(), oracle.transpose(a)) and \
                np.array_equal(gt.ToNumpy(), a.T)
    # general form: alpha * A^T + beta * B^T into a padded C
    m, n = 45, 70
    A, B, C0 = random_tensor(rng, ((n + 2) * (m + 3),), -1, 1), random_tensor(rng, ((n + 5) * m,), -1, 1), \
        random_tensor(rng, ((m + 4) * n,), -1, 1)
    gA, gB, gC = GPUTensor([A.size], A, w), GPUTensor([B.size], B, w), GPUTensor([C0.size], C0, w)
    al, be = ctypes.c_float(0.5), ctypes.c_float(-2.0)
    st = w.lib.snhip_sgeam(w.handle, 1, 1, m, n, ctypes.byref(al), gA.Pointer, n + 2, ctypes.byref(be), gB.Pointer, n + 5,
                           gC.Pointer, m + 4)
    assert st == 0
    want = oracle.sgeam_colmajor(True, True, m, n, 0.5, A, n + 2, -2.0, B, n + 5, C0, m + 4)
    assert np.max(np.abs(gC.ToNumpy() - want)) <= 1e-6
    assert np.array_equal(gC.ToNumpy().reshape(n, m + 4)[:, m:], C0.reshape(n, m + 4)[:, m:])
    # a zero scalar means "operand not referenced" (cuBLAS): NaN / Inf in that operand, or in the old C, never reach C
    ld = max(m, n) + 1                     # fits either orientation of either operand
    size = ld * max(m, n)
    A2, B2 = random_tensor(rng, (size,), -1, 1), random_tensor(rng, (size,), -1, 1)
    nanA, infB = np.full(size, np.nan, np.float32), np.full(size, np.inf, np.float32)
    gA2, gB2, gNaN, gInf = (GPUTensor([size], x, w) for x in (A2, B2, nanA, infB))
    for (alpha, beta, ta, tb, srcA, srcB, hostA, hostB) in (
            (0.0, 0.0, 1, 0, gNaN, gInf, nanA, infB),          # C = 0 whatever A, B and the old C hold
            (0.0, 1.5, 1, 1, gNaN, gB2, nanA, B2),             # C = 1.5 * B^T, A not read
            (0.0, 1.5, 0, 0, None, gB2, nanA, B2),             # ... A may be NULL
            (-0.75, 0.0, 1, 0, gA2, gInf, A2, infB),           # C = -0.75 * A^T, B not read
            (-0.75, 0.0, 1, 0, gA2, None, A2, infB)):          # ... B may be NULL (the reference's Transpose call)
        gC.SetValue(float("nan"))
        al, be = ctypes.c_float(alpha), ctypes.c_float(beta)
        st = w.lib.snhip_sgeam(w.handle, ta, tb, m, n, ctypes.byref(al), srcA.Pointer if srcA is not None else None, ld,
                               ctypes.byref(be), srcB.Pointer if srcB is not None else None, ld, gC.Pointer, m + 4)
        assert st == 0
        want = oracle.sgeam_colmajor(bool(ta), bool(tb), m, n, alpha, hostA, ld, beta, hostB, ld,
                                     np.full(C0.size, np.nan, np.float32), m + 4)
        got = gC.ToNumpy().reshape(n, m + 4)[:, :m]
        assert np.array_equal(got, want.reshape(n, m + 4)[:, :m]), (alpha, beta, ta, tb)
        assert np.isfinite(got).all()
    # argument errors follow cuBLAS: bad op, short leading dimension, in-place transpose
    assert w.lib.snhip_sgeam(w.handle, 7, 0, m, n, ctypes.byref(al), gA.Pointer, n + 2, ctypes.byref(be), gB.Pointer, n + 5,
                             gC.Pointer, m + 4) == 7
    assert w.lib.snhip_sgeam(w.handle, 1, 1, m, n, ctypes.byref(al), gA.Pointer, n - 1, ctypes.byref(be), gB.Pointer, n + 5,
                             gC.Pointer, m + 4) == 7
    # MultiplyTensor: same shape, and one factor per (batch, channel)
    shape = (4, 9, 7, 7)
    a, x_same, x_bc = random_tensor(rng, shape, -10, 10), random_tensor(rng, shape, -10, 10), \
        random_tensor(rng, (4, 9, 1, 1), -10, 10)
    ga, gc = GPUTensor(list(shape), a, w), GPUTensor(list(shape), None, w)
    gc.MultiplyTensor(ga, GPUTensor(list(shape), x_same, w))
    assert np.array_equal(gc.ToNumpy(), oracle.multiply_tensor(a, x_same))
    gc.MultiplyTensor(ga, GPUTensor([4, 9, 1, 1], x_bc, w))
    assert np.array_equal(gc.ToNumpy(), oracle.multiply_tensor(a, x_bc))
    ga.MultiplyTensor(ga, GPUTensor([4, 9, 1, 1], x_bc, w))             # in place
    assert np.array_equal(ga.ToNumpy(), oracle.multiply_tensor(a, x_bc))


@pytest.mark.parametrize("tA,tB", list(itertools.product([False, True], repeat=2)))
def test_k_split_inside_the_workgroup(oracle, gpu_wrapper, tA, tB):
    """The kernel for products with few output tiles (32 x 32 tiles, K split over a workgroup's wavefronts): ragged
    M and N, K tails that are not multiples of 32, alpha / beta, the fused bias, a strided batch; forced through the
    tuning hook and picked automatically for a Dense layer on a small batch."""
    from sharpnet_amd import GPUTensor
    ks_all = [c["id"] for c in gpu_wrapper.configs() if c["kind"] == "fp32-ksplit"]
    ks = ks_all[0]
    rng = np.random.default_rng(400 + 2 * tA + tB)
    try:
        for (M, N, K) in [(100, 36, 72), (36, 100, 264), (128, 256, 784), (260, 2048, 512), (4, 8, 36), (32, 32, 32),
                          (64, 132, 1000)]:
            a = random_tensor(rng, (K, M) if tA else (M, K), -1, 1)
            b = random_tensor(rng, (N, K) if tB else (K, N), -1, 1)
            c = random_tensor(rng, (M, N), -1, 1)
            for cfg in ks_all:
                gpu_wrapper.set_tuning(cfg, 1)
                for alpha, beta in [(1.0, 0.0), (-0.5, 1.0), (0.25, -2.0)]:
                    ref = oracle.dot(a, tA, b, tB, alpha, beta, c if beta != 0 else None)
                    got = gpu_dot(gpu_wrapper, a, tA, b, tB, alpha, beta, c=c) if beta != 0 else \
                        gpu_dot(gpu_wrapper, a, tA, b, tB, alpha, beta, c_shape=[M, N], prefill=float("nan"))
                    assert gpu_wrapper.last_tuning() == (cfg, 1), (M, N, K)
                    assert np.max(np.abs(got - ref)) <= tol(K, a, b, alpha, beta, c), (M, N, K, cfg, alpha, beta)
        gpu_wrapper.set_tuning(ks, 1)
        # strided batch + bias through the row-major entry point
        batch, M, N, K = 3, 40, 52, 96
        a = random_tensor(rng, (batch, K, M) if tA else (batch, M, K), -1, 1)
        b = random_tensor(rng, (batch, N, K) if tB else (batch, K, N), -1, 1)
        ga, gb = GPUTensor(a.shape, a, gpu_wrapper), GPUTensor(b.shape, b, gpu_wrapper)
        gc = GPUTensor([batch, M, N], None, gpu_wrapper)
        gc.SetValue(float("nan"))
        gc.BatchMatrixMultiplication(ga, tA, gb, tB, 0.5, 0.0)
        assert gpu_wrapper.last_tuning() == (ks, 1)
        assert np.max(np.abs(gc.ToNumpy() - oracle.bmm(a, tA, b, tB, 0.5))) <= tol(K, a, b, 0.5)
        gpu_wrapper.set_tuning(-1, 0)
        # automatic choice: the forward product of benchmark configuration 1's Dense layer (32 tiles of 32 x 32: the
        # 16 x 16-tile kernel), a square product of one 32 x 32 tile per CU (eight K slices; four with a short K), half
        # as many tiles (16 x 16 tiles again), the layer's dx (100 tiles: 16 x 16) and dW (200 tiles, K = 128: four
        # slices); a recurrent step (two 32 x 32 tiles per CU) is left to the tiled kernels
        assert len(ks_all) == 4
        for (M, N, K, want) in [(128, 256, 784, ks_all[3]), (512, 512, 512, ks_all[2]), (512, 512, 256, ks_all[0]),
                                (256, 512, 1024, ks_all[3]), (128, 784, 256, ks_all[3]), (256, 784, 128, ks_all[0]),
                                (256, 2048, 512, None)]:
            a = random_tensor(rng, (K, M) if tA else (M, K), -1, 1)
            b = random_tensor(rng, (N, K) if tB else (K, N), -1, 1)
            got = gpu_dot(gpu_wrapper, a, tA, b, tB, 1.0, 0.0, c_shape=[M, N], prefill=float("nan"))
            if want is None:
                assert gpu_wrapper.last_tuning()[0] not in ks_all
            else:
                assert gpu_wrapper.last_tuning() == (want, 1)
            assert np.max(np.abs(got - oracle.dot(a, tA, b, tB))) <= tol(K, a, b)
        # an operand view at an odd element offset cannot be read in 16-byte pieces: another kernel takes over
        big = GPUTensor([128 * 784 + 1], None, gpu_wrapper)
        big.ZeroMemory()
        view = big.Slice(1, [128, 784])
        w_ = random_tensor(rng, (256, 784), -1, 1)
        gw = GPUTensor(w_.shape, w_, gpu_wrapper)
        gy = GPUTensor([128, 256], None, gpu_wrapper)
        gy.Dot(view, False, gw, True, 1.0, 0.0)
        assert gpu_wrapper.last_tuning()[0] not in ks_all
        assert np.all(gy.ToNumpy() == 0.0)
    finally:
        gpu_wrapper.set_tuning(-1, 0)


@pytest.mark.parametrize("tA,tB", list(itertools.product([False, True], repeat=2)))
def test_streaming_kernel_strided_batches(oracle, gpu_wrapper, tA, tB):
    """The persistent kernel for batches of small matrices with a short K (k panels of 32, one LDS stage): more
    tiles than workgroups so that every workgroup walks through several, ragged M / N, K below, at and above one
    panel with tails, alpha / beta, a single matrix; forced through the tuning hook, and picked automatically for the
    attention-shaped products."""
    from sharpnet_amd import GPUTensor
    w = gpu_wrapper
    st_all = [c["id"] for c in w.configs() if c["kind"] == "fp32-stream"]
    assert len(st_all) == 2
    rng = np.random.default_rng(500 + 2 * tA + tB)
    try:
        for (batch, M, N, K) in [(700, 128, 128, 64), (40, 256, 256, 64), (40, 256, 64, 256), (9, 200, 100, 70),
                                 (5, 130, 257, 130), (3, 64, 40, 7), (1, 300, 200, 129), (1100, 100, 60, 36)]:
            a = random_tensor(rng, (batch, K, M) if tA else (batch, M, K), -1, 1)
            b = random_tensor(rng, (batch, N, K) if tB else (batch, K, N), -1, 1)
            c = random_tensor(rng, (batch, M, N), -1, 1)
            ga, gb = GPUTensor(a.shape, a, w), GPUTensor(b.shape, b, w)
            for cfg in st_all:
                w.set_tuning(cfg, 1)
                for alpha, beta in [(0.125, 0.0), (-0.5, 1.0)]:
                    gc = GPUTensor(c.shape, c, w)
                    if beta == 0.0:
                        gc.SetValue(float("nan"))
                    gc.BatchMatrixMultiplication(ga, tA, gb, tB, alpha, beta)
                    assert w.last_tuning() == (cfg, 1), (batch, M, N, K)
                    got = gc.ToNumpy()
                    gc.Dispose()
                    ref = oracle.bmm(a, tA, b, tB, alpha, beta, c if beta != 0 else None)
                    assert np.all(np.isfinite(got)), (batch, M, N, K, cfg, alpha, beta)
                    assert np.max(np.abs(got - ref)) <= tol(K, a, b, alpha, beta, c), (batch, M, N, K, cfg, alpha, beta)
            ga.Dispose()
            gb.Dispose()
        w.set_tuning(-1, 0)
        # automatic choice: the two attention products of benchmark configuration 5 (fewer matrices, same shape) - the
        # scores (K = 64) stream, the probabilities-times-values product (K = 256) is a few percent faster on the tiled
        # kernels in fp32 - and a K = 128 product with 64 columns
        for (batch, M, N, K, want) in [(256, 256, 256, 64, st_all[0]), (256, 256, 64, 256, None),
                                       (512, 256, 64, 128, st_all[1])]:
            a = random_tensor(rng, (batch, K, M) if tA else (batch, M, K), -1, 1)
            b = random_tensor(rng, (batch, N, K) if tB else (batch, K, N), -1, 1)
            ga, gb, gc = GPUTensor(a.shape, a, w), GPUTensor(b.shape, b, w), GPUTensor([batch, M, N], None, w)
            gc.SetValue(float("nan"))
            gc.BatchMatrixMultiplication(ga, tA, gb, tB, 1.0, 0.0)
            if want is None:
                assert w.last_tuning()[0] not in st_all
            else:
                assert w.last_tuning() == (want, 1)
            assert np.max(np.abs(gc.ToNumpy() - oracle.bmm(a, tA, b, tB, 1.0))) <= tol(K, a, b)
            for t in (ga, gb, gc):
                t.Dispose()
    finally:
        w.set_tuning(-1, 0)


def test_k_split_kernel_padded_pitches_fuzz(oracle, gpu_wrapper):
    """Random small products through the descriptor call with padded row pitches, padded batch strides, bias, addend
    and ReLU, forced onto the K-split kernel; operands sit in NaN-filled buffers so that any read outside a matrix
    shows up in the result."""
    from sharpnet_amd import GPUTensor
    ks_all = [c["id"] for c in gpu_wrapper.configs() if c["kind"] == "fp32-ksplit"]
    rng = np.random.default_rng(77)
    used = 0
    try:
        for it in range(60):
            ks = ks_all[it % len(ks_all)]
            gpu_wrapper.set_tuning(ks, 1)
            tA, tB = bool(rng.integers(2)), bool(rng.integers(2))
            M, N = int(rng.integers(1, 90)), int(rng.integers(1, 90))
            if tA:
                M = 4 * ((M + 3) // 4)
            if not tB:
                N = 4 * ((N + 3) // 4)
            K = 4 * int(rng.integers(8, 80))
            batch = int(rng.integers(1, 4))
            ar, ac = (K, M) if tA else (M, K)
            br, bc = (N, K) if tB else (K, N)
            lda, ldb, ldc, ldd = ac + 4 * int(rng.integers(0, 3)), bc + 4 * int(rng.integers(0, 3)), N + int(rng.integers(0, 5)), \
                N + int(rng.integers(0, 5))
            sA, sB, sC, sD = ar * lda + 4 * int(rng.integers(0, 3)), br * ldb + 4 * int(rng.integers(0, 3)), M * ldc + 3, M * ldd + 1

            def padded(rows, cols, ld, stride, lo=-1.0, hi=1.0):
                buf = np.full(batch * stride + 8, np.nan, np.float32)
                mats = rng.uniform(lo, hi, (batch, rows, cols)).astype(np.float32)
                for z in range(batch):
                    for r in range(rows):
                        buf[z * stride + r * ld: z * stride + r * ld + cols] = mats[z, r]
                return buf, mats
            abuf, a = padded(ar, ac, lda, sA)
            bbuf, b = padded(br, bc, ldb, sB)
            cbuf, c = padded(M, N, ldc, sC)
            dbuf, dmat = padded(M, N, ldd, sD)
            bias = rng.uniform(-1, 1, N).astype(np.float32)
            alpha, beta, gamma = float(rng.uniform(-1, 1)), float(rng.choice([0.0, 1.0, -0.5])), float(rng.choice([0.0, 0.75]))
            relu = bool(rng.integers(2))
            ga, gb, gc, gd, gbias = (GPUTensor([t.size], t, gpu_wrapper) for t in (abuf, bbuf, cbuf, dbuf, bias))
            gc.GemmEx(transA=int(tA), transB=int(tB), M=M, N=N, K=K, alpha=alpha, beta=beta, A=ga, lda=lda, strideA=sA, B=gb,
                      ldb=ldb, strideB=sB, ldc=ldc, strideC=sC, batch=batch, bias=gbias, D=gd, ldd=ldd, strideD=sD, gamma=gamma,
                      activation=1 if relu else 0)
            used += gpu_wrapper.last_tuning()[0] == ks
            out = gc.ToNumpy()
            for z in range(batch):
                ref = oracle.dot_f64(a[z], tA, b[z], tB, alpha, 0.0) + bias[None, :] + beta * c[z] + gamma * dmat[z]
                if relu:
                    ref = np.maximum(ref, 0.0)
                got = np.stack([out[z * sC + r * ldc: z * sC + r * ldc + N] for r in range(M)])
                assert np.all(np.isfinite(got)), (it, tA, tB, M, N, K)
                assert np.max(np.abs(got - ref)) <= tol(K, a, b, alpha) + 1e-5, (it, tA, tB, M, N, K, batch)
                # the gaps between rows stay untouched
                if ldc > N:
                    assert np.all(np.isnan(out[z * sC + N: z * sC + ldc]))
        assert used >= 50, used
    finally:
        gpu_wrapper.set_tuning(-1, 0)


@pytest.mark.parametrize("math,configs", [(0, (16, 17)), (1, (22, 23))])
@pytest.mark.parametrize("tA,tB", [(False, True), (False, False), (True, False)])
def test_streaming_kernels_walk_a_two_level_batch(oracle, gpu_wrapper, math, configs, tA, tB):
    """The persistent streaming kernels (fp32 and bf16-input) on heads addressed in place: entry z of the batch is head
    z % heads of sample z / heads inside (batch, steps, heads * dim) activations, the output a contiguous stack or in
    place as well.  Every product against the oracle (bf16: on rounded operands, the bound of the bf16 tests)."""
    from sharpnet_amd import GPUTensor
    rng = np.random.default_rng(83)
    B, H, M, N, K = 5, 3, 130, 96, 64
    w = gpu_wrapper
    a_rows, a_cols = (K, M) if tA else (M, K)      # per-head operand shapes
    b_rows, b_cols = (N, K) if tB else (K, N)
    a = random_tensor(rng, (B, a_rows, H * a_cols), -1, 1)     # packed: head h is the column block [h*cols, (h+1)*cols)
    b = random_tensor(rng, (B, b_rows, H * b_cols), -1, 1)
    ga, gb = GPUTensor(list(a.shape), a, w), GPUTensor(list(b.shape), b, w)
    want = np.empty((B, H, M, N), np.float32)
    for z, h in itertools.product(range(B), range(H)):
        ah, bh = a[z][:, h * a_cols:(h + 1) * a_cols], b[z][:, h * b_cols:(h + 1) * b_cols]
        if math == 1:
            ah, bh = oracle.round_to_bf16(ah), oracle.round_to_bf16(bh)
        want[z, h] = oracle.dot(np.ascontiguousarray(ah), tA, np.ascontiguousarray(bh), tB, 0.5, 0.0)
    w.set_math_mode(math)
    try:
        for cfg, c_packed in itertools.product(configs, (False, True)):
            gc = GPUTensor([B, M, H * N] if c_packed else [B * H, M, N], None, w)
            gc.SetValue(float("nan"))
            w.set_tuning(cfg, 1)
            gc.GemmEx(transA=int(tA), transB=int(tB), M=M, N=N, K=K, alpha=0.5, beta=0.0, A=ga, lda=H * a_cols, strideA=a_cols,
                      strideA_outer=a_rows * H * a_cols, B=gb, ldb=H * b_cols, strideB=b_cols, strideB_outer=b_rows * H * b_cols,
                      ldc=H * N if c_packed else N, strideC=N if c_packed else M * N,
                      strideC_outer=M * H * N if c_packed else H * M * N, batch=B * H, batch_inner=H)
            assert w.last_tuning() == (cfg, 1)
            got = gc.ToNumpy()
            got = got.reshape(B, M, H, N).transpose(0, 2, 1, 3) if c_packed else got.reshape(B, H, M, N)
            assert np.max(np.abs(got - want)) <= 1e-4 * np.sqrt(K) * 0.5, (cfg, c_packed)
    finally:
        w.set_tuning(-1, 0)
        w.set_math_mode(0)


@pytest.mark.parametrize("tA,tB", list(itertools.product([False, True], repeat=2)))
def test_tall_products_with_few_columns_and_a_long_k(oracle, gpu_wrapper, tA, tB):
    """A tall operand against one of 32 columns or fewer with a long K goes to the kernels that split K inside the
    workgroup (no padding to 64 columns, no second launch): 32 x 32 tiles when those fill the chip, 16 x 16 tiles
    otherwise; likewise a wide operand under 32 rows or fewer (32 x 32 tiles).  Against the oracle, ragged sizes
    included, C prefilled with NaN for beta = 0."""
    from sharpnet_amd import GPUTensor
    w = gpu_wrapper
    rng = np.random.default_rng(9000 + 2 * tA + tB)
    kinds = {c["id"]: (c["kind"], c["BM"]) for c in w.configs()}
    for (M, N, K, want_bm) in [(8192, 32, 2048, 32), (8200, 28, 2052, 32), (4096, 32, 4096, 16), (8192, 8, 2048, 16),
                               (4100, 12, 4096, 16), (32, 8192, 2048, 32), (12, 8200, 2052, 32)]:
        a = random_tensor(rng, (K, M) if tA else (M, K), -1, 1)
        b = random_tensor(rng, (N, K) if tB else (K, N), -1, 1)
        c = random_tensor(rng, (M, N), -1, 1)
        ga, gb = GPUTensor(a.shape, a, w), GPUTensor(b.shape, b, w)
        for alpha, beta in ((1.0, 0.0), (0.5, 1.0)):
            gc = GPUTensor([M, N], c if beta != 0 else None, w)
            if beta == 0:
                gc.SetValue(float("nan"))
            gc.Dot(ga, tA, gb, tB, alpha, beta)
            cfg, splitk = w.last_tuning()
            aligned = (M % 4 == 0 or not tA) and (N % 4 == 0 or tB)      # 16-byte pieces along the contiguous direction
            if aligned:
                assert kinds[cfg] == ("fp32-ksplit", want_bm) and splitk == 1, (M, N, K, cfg, splitk)
            ref = oracle.dot(a, tA, b, tB, alpha, beta, c if beta != 0 else None)
            assert np.max(np.abs(gc.ToNumpy() - ref)) <= 1e-4 * np.sqrt(K) * abs(alpha) + 1e-6, (M, N, K, cfg)
            gc.Dispose()
        ga.Dispose()
        gb.Dispose()
