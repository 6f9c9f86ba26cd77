"""snhip_dot_noalloc: the Dot entry point whose split-K partial sums live in the library's static scratch array.

It must give what snhip_dot gives (same kernels, same tile configuration and split-K factor: bit for bit), on two
calls in a row that share the array, the second on a smaller product; stay within the fp32 bar against the oracle;
and refuse, without launching anything, a product whose partial sums do not fit the array.
"""
import ctypes

import numpy as np
import pytest

pytestmark = pytest.mark.gpu


def _dot(w, entry, a, tA, b, tB, c, alpha, beta):
    """One call of `entry` (snhip_dot or snhip_dot_noalloc) through the C ABI; returns (status, C, tuning)."""
    from sharpnet_amd import GPUTensor
    ga, gb, gc = GPUTensor(a.shape, a, w), GPUTensor(b.shape, b, w), GPUTensor(c.shape, c, w)
    st = entry(w.handle, ga.Pointer, a.shape[0], a.shape[1], int(tA), gb.Pointer, b.shape[0], b.shape[1], int(tB),
               gc.Pointer, alpha, beta)
    out = gc.ToNumpy()
    for t in (ga, gb, gc):
        t.Dispose()
    return st, out, w.last_tuning()


def test_noalloc_matches_dot_on_two_calls_in_a_row(gpu_wrapper, oracle):
    w, lib = gpu_wrapper, gpu_wrapper.lib
    assert lib.snhip_static_scratch_bytes() == 32 << 20
    rng = np.random.default_rng(11)
    # (a shape, tA, b shape, tB, alpha, beta): long-K products with few output tiles, which the library splits along K;
    # the second is smaller than the first in every dimension and reuses the front of the same scratch array
    cases = [((1024, 8192), False, (8192, 64), False, 1.0, 0.0),
             ((4096, 192), True, (4096, 48), False, -0.5, 1.0)]
    for a_shape, tA, b_shape, tB, alpha, beta in cases:
        a = rng.uniform(-1, 1, a_shape).astype(np.float32)
        b = rng.uniform(-1, 1, b_shape).astype(np.float32)
        M = a_shape[1] if tA else a_shape[0]
        N = b_shape[0] if tB else b_shape[1]
        K = a_shape[0] if tA else a_shape[1]
        c0 = rng.uniform(-1, 1, (M, N)).astype(np.float32) if beta != 0.0 else np.full((M, N), np.nan, np.float32)
        print("noalloc case", a_shape, tA, b_shape, tB, alpha, beta, flush=True)
        st, got, tuning = _dot(w, lib.snhip_dot_noalloc, a, tA, b, tB, c0, alpha, beta)
        assert st == 0
        assert tuning[1] > 1, "the case is meant to use split-K (and with it the scratch array): %r" % (tuning,)
        st2, want, tuning2 = _dot(w, lib.snhip_dot, a, tA, b, tB, c0, alpha, beta)
        assert st2 == 0 and tuning2 == tuning
        assert np.array_equal(got, want), "max|d| = %g" % float(np.max(np.abs(got - want)))
        ref = oracle.dot(a, tA, b, tB, alpha, beta, c0 if beta != 0.0 else None)
        bound = 1e-4 * np.sqrt(K) * float(np.max(np.abs(a))) * float(np.max(np.abs(b))) * abs(alpha) + 1e-6
        assert float(np.max(np.abs(got - ref))) <= bound


def test_noalloc_without_split_k_and_refusal_beyond_the_scratch(gpu_wrapper, oracle):
    from sharpnet_amd.hiplib import CublasStatus
    w, lib = gpu_wrapper, gpu_wrapper.lib
    rng = np.random.default_rng(12)
    a = rng.uniform(-1, 1, (1024, 1024)).astype(np.float32)
    b = rng.uniform(-1, 1, (1024, 1024)).astype(np.float32)
    nan = np.full((1024, 1024), np.nan, np.float32)
    # forced to 32 splits, the 1024 x 1024 partial sums take 128 MiB: four times what the array holds
    w.set_tuning(6, 32)
    try:
        st, out, _ = _dot(w, lib.snhip_dot_noalloc, a, False, b, False, nan, 1.0, 0.0)
    finally:
        w.set_tuning(-1, 0)
    assert st == CublasStatus.CUBLAS_STATUS_NOT_SUPPORTED
    assert np.isnan(out).all()                      # nothing was launched
    msg = ctypes.create_string_buffer(256)
    assert lib.snhip_get_last_error_message(w.handle, msg, 256) == 0
    assert b"134217728" in msg.value and b"33554432" in msg.value, msg.value
    # the automatic choice for this product needs no split and therefore no scratch: never refused
    st, out, tuning = _dot(w, lib.snhip_dot_noalloc, a, False, b, False, nan, 1.0, 0.0)
    assert st == 0 and tuning[1] == 1
    ref = oracle.dot(a, False, b, False)
    assert float(np.max(np.abs(out - ref))) <= 1e-4 * np.sqrt(1024)
