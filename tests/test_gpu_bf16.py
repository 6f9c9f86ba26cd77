"""GPU parity tests of the bf16-input / fp32-accumulate variant.

Two bars, both written out below:
  * against the fp32 oracle on the unrounded inputs:  max|d| / max|C_ref| <= 1e-2;
  * against the oracle on bf16-rounded inputs (products of two bf16 numbers are exact
    in fp32, so only the summation order differs): the fp32 bound
    max|d| <= 1e-4*sqrt(K)*max|a|*max|b|.
"""
import itertools

import numpy as np
import pytest

from tests.helpers import random_tensor

pytestmark = pytest.mark.gpu

SHAPES = [(35, 21, 124), (129, 257, 63), (256, 256, 64), (300, 130, 200), (64, 64, 16), (1, 1, 1), (257, 100, 33),
          (5, 300, 1000), (512, 384, 512)]


def check(oracle, got, a, tA, b, tB, alpha, beta, c, K):
    ref32 = oracle.dot(a, tA, b, tB, alpha, beta, c if beta != 0 else None)
    refbf = oracle.dot(oracle.round_to_bf16(a), tA, oracle.round_to_bf16(b), tB, alpha, beta, c if beta != 0 else None)
    assert np.all(np.isfinite(got))
    # bar 1: 1e-2 relative to max|C_ref|; where the result cancels to something tiny compared with the operands
    # (e.g. alpha*a*b + beta*c of a 1x1 product) fall back to the rounding envelope 2 * 2^-8 * sqrt(K)*|alpha|*max|a|*max|b|
    scale = max(float(np.max(np.abs(ref32))), 1e-30)
    err32 = float(np.max(np.abs(got - ref32)))
    envelope = 2.0 * 2.0 ** -8 * np.sqrt(max(K, 1)) * abs(alpha) * float(np.max(np.abs(a))) * float(np.max(np.abs(b)))
    assert err32 / scale <= 1e-2 or err32 <= envelope, (err32, scale, envelope)
    tight = 1e-4 * np.sqrt(max(K, 1)) * float(np.max(np.abs(a))) * float(np.max(np.abs(b))) * max(abs(alpha), 1e-30)
    if beta != 0:
        tight += 1e-6 * abs(beta) * float(np.max(np.abs(c)))
    assert float(np.max(np.abs(got - refbf))) <= tight, float(np.max(np.abs(got - refbf)))


@pytest.mark.parametrize("tA,tB", list(itertools.product([False, True], repeat=2)))
def test_bf16_all_configs_all_transposes(oracle, gpu_wrapper, tA, tB):
    from sharpnet_amd import GPUTensor
    from sharpnet_amd.hiplib import check_status
    lib, h = gpu_wrapper.lib, gpu_wrapper.handle
    rng = np.random.default_rng(200 + 2 * tA + tB)
    cfgs = [c["id"] for c in gpu_wrapper.configs() if c["kind"] == "bf16"]
    assert cfgs
    try:
        for (M, N, K) in SHAPES:
            a = random_tensor(rng, (K, M) if tA else (M, K), -1, 1)
            b = random_tensor(rng, (N, K) if tB else (K, N), -1, 1)
            c = random_tensor(rng, (M, N), -1, 1)
            ga, gb = GPUTensor(a.shape, a, gpu_wrapper), GPUTensor(b.shape, b, gpu_wrapper)
            for cfg in cfgs:
                for splitk in (1, 2):
                    if splitk > 1 and K < 128:
                        continue
                    gpu_wrapper.set_tuning(cfg, splitk)
                    for alpha, beta in [(1.0, 0.0), (0.25, 0.0), (-1.0, 1.0)]:
                        gc = GPUTensor([M, N], c if beta != 0 else None, gpu_wrapper)
                        if beta == 0:
                            gc.SetValue(float("nan"))
                        check_status(lib.snhip_dot_bf16(h, ga.Pointer, a.shape[0], a.shape[1], int(tA), gb.Pointer,
                                                        b.shape[0], b.shape[1], int(tB), gc.Pointer, alpha, beta, None))
                        check(oracle, gc.ToNumpy(), a, tA, b, tB, alpha, beta, c, K)
                        gc.Dispose()
    finally:
        gpu_wrapper.set_tuning(-1, 0)


def test_bf16_math_mode_through_reference_shaped_calls(oracle, gpu_wrapper):
    """With the handle in bf16-input mode, Dot / BatchMatrixMultiplication (cuBLAS-shaped entry points) use it."""
    from sharpnet_amd import GPUTensor
    rng = np.random.default_rng(31)
    try:
        gpu_wrapper.set_math_mode(gpu_wrapper.MATH_BF16_INPUT)
        M, N, K = 200, 150, 300
        a, b = random_tensor(rng, (M, K), -1, 1), random_tensor(rng, (N, K), -1, 1)
        ga, gb, gc = GPUTensor(a.shape, a, gpu_wrapper), GPUTensor(b.shape, b, gpu_wrapper), GPUTensor([M, N], None,
                                                                                                         gpu_wrapper)
        gc.Dot(ga, False, gb, True, 1.0, 0.0)
        got = gc.ToNumpy()
        check(oracle, got, a, False, b, True, 1.0, 0.0, None, K)
        # it really is the reduced-precision path: the result differs from the fp32 one
        assert np.max(np.abs(got - oracle.dot(a, False, b, True))) > 1e-5
        batch, T, d = 6, 48, 32
        q, k = random_tensor(rng, (batch, T, d)), random_tensor(rng, (batch, T, d))
        gq, gk, gs = GPUTensor(q.shape, q, gpu_wrapper), GPUTensor(k.shape, k, gpu_wrapper), GPUTensor([batch, T, T],
                                                                                                         None,
                                                                                                         gpu_wrapper)
        gs.BatchMatrixMultiplication(gq, False, gk, True, 0.125, 0.0)
        ref = oracle.bmm(oracle.round_to_bf16(q), False, oracle.round_to_bf16(k), True, 0.125)
        assert np.max(np.abs(gs.ToNumpy() - ref)) <= 1e-4 * np.sqrt(d) * np.max(np.abs(q)) * np.max(np.abs(k))
    finally:
        gpu_wrapper.set_math_mode(gpu_wrapper.MATH_FP32)
    # back in fp32 mode the fp32 bound holds again
    gc.Dot(ga, False, gb, True, 1.0, 0.0)
    assert np.max(np.abs(gc.ToNumpy() - oracle.dot(a, False, b, True))) <= 1e-4 * np.sqrt(K)


def test_bf16_bias_and_batched(oracle, gpu_wrapper):
    from sharpnet_amd import GPUTensor
    from sharpnet_amd.hiplib import check_status
    lib, h = gpu_wrapper.lib, gpu_wrapper.handle
    rng = np.random.default_rng(37)
    M, N, K = 128, 256, 784
    x, w, bias = rng.uniform(0, 1, (M, K)).astype(np.float32), random_tensor(rng, (N, K), -0.07, 0.07), \
        random_tensor(rng, (N,), -1, 1)
    gx, gw, gb, gy = (GPUTensor(t.shape, t, gpu_wrapper) for t in (x, w, bias, np.zeros((M, N), np.float32)))
    check_status(lib.snhip_dot_bf16(h, gx.Pointer, M, K, 0, gw.Pointer, N, K, 1, gy.Pointer, 1.0, 0.0, gb.Pointer))
    ref = oracle.dot(oracle.round_to_bf16(x), False, oracle.round_to_bf16(w), True) + bias
    assert np.max(np.abs(gy.ToNumpy() - ref)) <= 1e-4 * np.sqrt(K) * np.max(np.abs(x)) * np.max(np.abs(w)) + 1e-6
    batch, T, d = 16, 256, 64
    p_, v = rng.uniform(0, 1, (batch, T, T)).astype(np.float32), random_tensor(rng, (batch, T, d))
    gp, gv, go = GPUTensor(p_.shape, p_, gpu_wrapper), GPUTensor(v.shape, v, gpu_wrapper), GPUTensor([batch, T, d],
                                                                                                     None, gpu_wrapper)
    check_status(lib.snhip_bmm_bf16(h, gp.Pointer, T, T, 0, T * T, gv.Pointer, T, d, 0, T * d, go.Pointer, T * d, batch,
                                    1.0, 0.0))
    ref = oracle.bmm(oracle.round_to_bf16(p_), False, oracle.round_to_bf16(v), False)
    assert np.max(np.abs(go.ToNumpy() - ref)) <= 1e-4 * np.sqrt(T) * np.max(np.abs(p_)) * np.max(np.abs(v))
