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


# ---------------------------------------------------------------------------
# operands stored as bf16 in device memory
# ---------------------------------------------------------------------------
def to_bf16_on_device(w, t):
    """Device buffer holding GPUTensor t converted to bf16 by the library's own pass; returns the raw pointer."""
    from sharpnet_amd.hiplib import check_status
    p = w.allocate(max(2 * t.Count, 8))
    check_status(w.lib.snhip_convert_f32_to_bf16(w.handle, t.Pointer, p, t.Count), "snhip_convert_f32_to_bf16")
    return p


def test_convert_f32_to_bf16_is_round_to_nearest_even(oracle, gpu_wrapper):
    """Bit-exact against the oracle's rounding (itself pinned by hand-computed ties and torch's CPU cast): random
    data, ties, infinities, zeros of both signs, the smallest normals; 16-byte-aligned and odd-offset views."""
    import ctypes
    from sharpnet_amd import GPUTensor
    from sharpnet_amd.hiplib import check_status
    w = gpu_wrapper
    rng = np.random.default_rng(41)
    x = np.concatenate([
        rng.normal(0, 1, 4099).astype(np.float32),
        np.array([1.0, 1 + 2.0 ** -8, 1 + 2.0 ** -8 + 2.0 ** -20, 1 + 3 * 2.0 ** -8, -(1 + 2.0 ** -8), 0.0, -0.0,
                  np.inf, -np.inf, 2.0 ** -126, 3.0e38, -3.0e38, 65504.0, 1e-30], np.float32)])
    gx = GPUTensor([x.size], x, w)
    for off in (0, 1, 3):                                   # element offsets of the source view
        n = x.size - off
        dst = w.allocate(2 * n + 8)
        check_status(w.lib.snhip_convert_f32_to_bf16(w.handle, gx.Pointer + 4 * off, dst, n))
        host = np.empty(n, np.uint16)
        check_status(w.lib.snhip_memcpy_dtoh(w.handle, host.ctypes.data, dst, 2 * n))
        want = (oracle.round_to_bf16(x[off:]).view(np.uint32) >> 16).astype(np.uint16)
        assert np.array_equal(host, want), off
        w.release(dst, 2 * n + 8)


def test_convert_2d_with_pitches_and_transpose(oracle, gpu_wrapper):
    """Matrix form of the conversion: padded row pitches on both sides, with and without transposition, ragged sizes."""
    from sharpnet_amd import GPUTensor
    from sharpnet_amd.hiplib import check_status
    w = gpu_wrapper
    rng = np.random.default_rng(44)
    # (the last four: whole 64-row blocks, 16-byte aligned rows on both sides - the wide transposing kernel - with
    # one, several and partly filled column groups of four wavefronts, padded pitches)
    for rows, cols, pad_s, pad_d in [(1, 1, 0, 0), (33, 65, 3, 2), (100, 31, 0, 5), (256, 128, 4, 0), (64, 32, 0, 0),
                                     (192, 160, 4, 8), (128, 416, 0, 0), (64, 96, 8, 0)]:
        src = random_tensor(rng, (rows, cols + pad_s), -2, 2)
        gs = GPUTensor(src.shape, src, w)
        for transpose in (0, 1):
            dr, dc = (cols, rows) if transpose else (rows, cols)
            ldd = dc + pad_d
            nbytes = 2 * dr * ldd
            dst = w.allocate(nbytes + 8)
            check_status(w.lib.snhip_memset32(w.handle, dst, 0x7fc07fc0, (nbytes + 3) // 4))      # bf16 NaNs
            check_status(w.lib.snhip_convert_f32_to_bf16_2d(w.handle, gs.Pointer, rows, cols, cols + pad_s, transpose, dst,
                                                            ldd))
            host = np.empty(dr * ldd, np.uint16)
            check_status(w.lib.snhip_memcpy_dtoh(w.handle, host.ctypes.data, dst, nbytes))
            host = host.reshape(dr, ldd)
            m = src[:, :cols].T if transpose else src[:, :cols]
            want = (oracle.round_to_bf16(np.ascontiguousarray(m)).view(np.uint32) >> 16).astype(np.uint16)
            assert np.array_equal(host[:, :dc], want), (rows, cols, transpose)
            assert np.all(host[:, dc:] == 0x7fc0)                  # padding untouched
            w.release(dst, nbytes + 8)


def test_transposing_conversion_brings_a_product_into_the_nt_form(oracle, gpu_wrapper):
    """A plain B (K x N) converted with transpose = 1 becomes an (N x K) operand for transposeB = 1, a transposed A
    (K x M) likewise an (M x K) one: the product in the NT form equals the product on the operands as they were, bit
    for bit (same tile configuration, same summation order), ragged even sizes included."""
    from sharpnet_amd import GPUTensor
    from sharpnet_amd.hiplib import check_status
    w = gpu_wrapper
    L, h = w.lib, w.handle
    rng = np.random.default_rng(45)
    for (M, N, K) in [(512, 384, 640), (130, 258, 72), (36, 22, 124)]:
        at = random_tensor(rng, (K, M), -1, 1)     # A stored transposed
        b = random_tensor(rng, (K, N), -1, 1)      # B stored plain
        gat, gb = GPUTensor(at.shape, at, w), GPUTensor(b.shape, b, w)
        pat, pb = w.allocate(2 * K * M), w.allocate(2 * K * N)
        pa_nt, pb_nt = w.allocate(2 * K * M), w.allocate(2 * K * N)
        check_status(L.snhip_convert_f32_to_bf16(h, gat.Pointer, pat, K * M))
        check_status(L.snhip_convert_f32_to_bf16(h, gb.Pointer, pb, K * N))
        check_status(L.snhip_convert_f32_to_bf16_2d(h, gat.Pointer, K, M, M, 1, pa_nt, K))
        check_status(L.snhip_convert_f32_to_bf16_2d(h, gb.Pointer, K, N, N, 1, pb_nt, K))
        c_tn, c_nt = GPUTensor([M, N], None, w), GPUTensor([M, N], None, w)
        for t in (c_tn, c_nt):
            t.SetValue(float("nan"))
        check_status(L.snhip_dot_bf16_stored(h, pat, K, M, 1, pb, K, N, 0, c_tn.Pointer, 1.0, 0.0, None))
        cfg = w.last_tuning()
        w.set_tuning(*cfg)
        try:
            check_status(L.snhip_dot_bf16_stored(h, pa_nt, M, K, 0, pb_nt, N, K, 1, c_nt.Pointer, 1.0, 0.0, None))
        finally:
            w.set_tuning(-1, 0)
        got_tn, got_nt = c_tn.ToNumpy(), c_nt.ToNumpy()
        assert np.array_equal(got_tn, got_nt), (M, N, K)
        ref = oracle.dot(oracle.round_to_bf16(at), True, oracle.round_to_bf16(b), False)
        assert np.max(np.abs(got_nt - ref)) <= 1e-4 * np.sqrt(K), (M, N, K)
        for ptr, n in ((pat, 2 * K * M), (pb, 2 * K * N), (pa_nt, 2 * K * M), (pb_nt, 2 * K * N)):
            w.release(ptr, n)
        for t in (gat, gb, c_tn, c_nt):
            t.Dispose()


EVEN_SHAPES = [(36, 22, 124), (130, 258, 64), (256, 256, 64), (300, 130, 200), (64, 64, 16), (2, 2, 2), (258, 100, 34),
               (6, 300, 1000), (512, 384, 512), (200, 520, 136)]


@pytest.mark.parametrize("tA,tB", list(itertools.product([False, True], repeat=2)))
def test_bf16_stored_all_configs_all_transposes(oracle, gpu_wrapper, tA, tB):
    """bf16 storage: every tile configuration of that kind x transposes x split-K x alpha / beta on ragged shapes with
    even row lengths, NaN-prefilled destinations, against the oracle on bf16-rounded inputs (tight fp32 bound) and the
    fp32 oracle (1e-2); and bit-identical to the fp32-storage bf16-input kernel of the same tile shape is not asked
    for (different k extent per stage), only the bound."""
    from sharpnet_amd import GPUTensor
    from sharpnet_amd.hiplib import check_status
    w = gpu_wrapper
    lib, h = w.lib, w.handle
    rng = np.random.default_rng(600 + 2 * tA + tB)
    cfgs = [c["id"] for c in w.configs() if c["kind"] == "bf16-stored"]
    assert len(cfgs) == 3
    try:
        for (M, N, K) in EVEN_SHAPES:
            a = random_tensor(rng, (K, M) if tA else (M, K), -1, 1)
            b = random_tensor(rng, (N, K) if tB else (K, N), -1, 1)
            c = random_tensor(rng, (M, N), -1, 1)
            ga, gb = GPUTensor(a.shape, a, w), GPUTensor(b.shape, b, w)
            pa, pb = to_bf16_on_device(w, ga), to_bf16_on_device(w, gb)
            for cfg in cfgs:
                for splitk in (1, 2):
                    if splitk > 1 and K < 256:
                        continue
                    w.set_tuning(cfg, splitk)
                    for alpha, beta in [(1.0, 0.0), (0.25, 0.0), (-1.0, 1.0)]:
                        gc = GPUTensor([M, N], c if beta != 0 else None, w)
                        if beta == 0:
                            gc.SetValue(float("nan"))
                        check_status(lib.snhip_dot_bf16_stored(h, pa, a.shape[0], a.shape[1], int(tA), pb, b.shape[0],
                                                               b.shape[1], int(tB), gc.Pointer, alpha, beta, None))
                        assert w.last_tuning() == (cfg, splitk), (M, N, K)
                        check(oracle, gc.ToNumpy(), a, tA, b, tB, alpha, beta, c, K)
                        gc.Dispose()
            w.release(pa, max(2 * ga.Count, 8))
            w.release(pb, max(2 * gb.Count, 8))
            ga.Dispose()
            gb.Dispose()
    finally:
        w.set_tuning(-1, 0)


def test_bf16_stored_batched_bias_and_refusals(oracle, gpu_wrapper):
    from sharpnet_amd import GPUTensor
    from sharpnet_amd.hiplib import check_status, CublasStatus
    w = gpu_wrapper
    lib, h = w.lib, w.handle
    rng = np.random.default_rng(43)
    # Linear forward with bias, automatic configuration
    M, N, K = 128, 256, 784
    x, wt, bias = rng.uniform(0, 1, (M, K)).astype(np.float32), random_tensor(rng, (N, K), -0.07, 0.07), \
        random_tensor(rng, (N,), -1, 1)
    gx, gw, gb, gy = (GPUTensor(t.shape, t, w) for t in (x, wt, bias, np.zeros((M, N), np.float32)))
    px, pw = to_bf16_on_device(w, gx), to_bf16_on_device(w, gw)
    check_status(lib.snhip_dot_bf16_stored(h, px, M, K, 0, pw, N, K, 1, gy.Pointer, 1.0, 0.0, gb.Pointer))
    ref = oracle.dot(oracle.round_to_bf16(x), False, oracle.round_to_bf16(wt), True) + bias
    assert np.max(np.abs(gy.ToNumpy() - ref)) <= 1e-4 * np.sqrt(K) * np.max(np.abs(x)) * np.max(np.abs(wt)) + 1e-6
    # the same operands at fp32 storage through the bf16-input kernel: same rounding, so the two results agree to
    # summation order
    gy2 = GPUTensor([M, N], None, w)
    check_status(lib.snhip_dot_bf16(h, gx.Pointer, M, K, 0, gw.Pointer, N, K, 1, gy2.Pointer, 1.0, 0.0, gb.Pointer))
    assert np.max(np.abs(gy.ToNumpy() - gy2.ToNumpy())) <= 2e-4 * np.sqrt(K) * np.max(np.abs(x)) * np.max(np.abs(wt))
    # strided batch: attention-shaped products, both orders
    batch, T, d = 16, 256, 64
    q, k = random_tensor(rng, (batch, T, d)), random_tensor(rng, (batch, T, d))
    gq, gk, gs = GPUTensor(q.shape, q, w), GPUTensor(k.shape, k, w), GPUTensor([batch, T, T], None, w)
    pq, pk = to_bf16_on_device(w, gq), to_bf16_on_device(w, gk)
    gs.SetValue(float("nan"))
    check_status(lib.snhip_bmm_bf16_stored(h, pq, T, d, 0, T * d, pk, T, d, 1, T * d, gs.Pointer, T * T, batch, 0.125, 0.0,
                                           None))
    ref = oracle.bmm(oracle.round_to_bf16(q), False, oracle.round_to_bf16(k), True, 0.125)
    assert np.max(np.abs(gs.ToNumpy() - ref)) <= 1e-4 * np.sqrt(d) * np.max(np.abs(q)) * np.max(np.abs(k))
    p_ = rng.uniform(0, 1, (batch, T, T)).astype(np.float32)
    gp, go = GPUTensor(p_.shape, p_, w), GPUTensor([batch, T, d], None, w)
    pp = to_bf16_on_device(w, gp)
    check_status(lib.snhip_bmm_bf16_stored(h, pp, T, T, 0, T * T, pk, T, d, 0, T * d, go.Pointer, T * d, batch, 1.0, 0.0,
                                           None))
    ref = oracle.bmm(oracle.round_to_bf16(p_), False, oracle.round_to_bf16(k), False)
    assert np.max(np.abs(go.ToNumpy() - ref)) <= 1e-4 * np.sqrt(T) * np.max(np.abs(p_)) * np.max(np.abs(k))
    # rows that start on odd element offsets cannot be read in aligned pieces: refused, nothing written
    go.SetValue(float("nan"))
    assert lib.snhip_dot_bf16_stored(h, pp, 8, 7, 0, pk, 7, 8, 0, go.Pointer, 1.0, 0.0, None) == \
        CublasStatus.CUBLAS_STATUS_NOT_SUPPORTED
    assert lib.snhip_dot_bf16_stored(h, pp + 2, 8, 8, 0, pk, 8, 8, 0, go.Pointer, 1.0, 0.0, None) == \
        CublasStatus.CUBLAS_STATUS_NOT_SUPPORTED
    assert np.isnan(go.ToNumpy()).all()


def test_bf16_stored_direct_to_lds_kernel(oracle, gpu_wrapper):
    """The bf16-storage kernel fed by global -> LDS direct loads (A plain, B transposed, whole 256 x 256 x 32 tiles):
    forced through the tuning hook on small shapes (one tile, one k panel; fewer k panels than LDS stages; several
    tiles; a strided batch; alpha, beta, bias; NaN-prefilled C for beta = 0), picked by itself for a product with a
    tile per compute unit, and left alone for shapes it does not take.  Bar: the fp32 bound against the oracle on
    bf16-rounded inputs; against the register-staged bf16-storage kernel the results agree to summation order."""
    from sharpnet_amd import GPUTensor
    from sharpnet_amd.hiplib import check_status
    w = gpu_wrapper
    lib, h = w.lib, w.handle
    dtl = [c["id"] for c in w.configs() if c["kind"] == "bf16-stored-dtl"]
    assert len(dtl) == 2                      # 256 x 256 tiles and the same kernel with 128 x 128 tiles
    dtl, dtl_small = dtl
    rng = np.random.default_rng(2700)

    def run(a, b, c0, alpha, beta, bias, force):
        """a: (batch, M, K), b: (batch, N, K) fp32 originals; returns (C, tuning)."""
        batch, M, K = a.shape
        N = b.shape[1]
        ga, gb = GPUTensor(a.shape, a, w), GPUTensor(b.shape, b, w)
        pa, pb = to_bf16_on_device(w, ga), to_bf16_on_device(w, gb)
        gc = GPUTensor([batch, M, N], c0, w)
        if beta == 0.0:
            gc.SetValue(float("nan"))
        gbias = GPUTensor([N], bias, w) if bias is not None else None
        w.set_tuning(force, 1 if force >= 0 else 0)
        try:
            check_status(lib.snhip_bmm_bf16_stored(h, pa, M, K, 0, M * K, pb, N, K, 1, N * K, gc.Pointer, M * N, batch,
                                                   alpha, beta, gbias.Pointer if gbias is not None else None))
        finally:
            w.set_tuning(-1, 0)
        out, tuning = gc.ToNumpy(), w.last_tuning()
        w.release(pa, max(2 * ga.Count, 8))
        w.release(pb, max(2 * gb.Count, 8))
        for t in (ga, gb, gc) + ((gbias,) if gbias is not None else ()):
            t.Dispose()
        return out, tuning

    cases = [(1, 256, 256, 32, 1.0, 0.0, False), (1, 256, 256, 64, -0.5, 1.0, True), (1, 512, 256, 96, 1.0, 0.0, True),
             (1, 256, 768, 1024, 0.25, 0.5, False), (3, 256, 512, 160, 1.0, 1.0, True), (2, 512, 512, 2048, 1.0, 0.0, False)]
    for (batch, M, N, K, alpha, beta, with_bias) in cases:
        print("direct-to-LDS case", batch, M, N, K, alpha, beta, with_bias, flush=True)
        a, b = random_tensor(rng, (batch, M, K), -1, 1), random_tensor(rng, (batch, N, K), -1, 1)
        c0 = random_tensor(rng, (batch, M, N), -1, 1)
        bias = random_tensor(rng, (N,), -1, 1) if with_bias else None
        got, tuning = run(a, b, c0, alpha, beta, bias, dtl)
        assert tuning == (dtl, 1), tuning
        ref = oracle.bmm(oracle.round_to_bf16(a), False, oracle.round_to_bf16(b), True, alpha, beta, c0 if beta else None)
        if bias is not None:
            ref = ref + bias
        bound = 1e-4 * np.sqrt(K) * abs(alpha) + 1e-6 * (abs(beta) + 1)
        assert np.all(np.isfinite(got))
        assert float(np.max(np.abs(got - ref))) <= bound, (batch, M, N, K)
        other, tuning2 = run(a, b, c0, alpha, beta, bias, -1)          # small shapes: the cost model's own choice
        assert tuning2[0] != dtl
        assert float(np.max(np.abs(got - other))) <= bound
    # the 128 x 128 form: one tile and one k panel, fewer k panels than stages, several tiles, a strided batch, a long K
    for (batch, M, N, K, alpha, beta, with_bias) in [(1, 128, 128, 32, 1.0, 0.0, False), (1, 128, 384, 64, -0.5, 1.0, True),
                                                     (1, 384, 128, 96, 1.0, 0.0, True), (3, 128, 256, 160, 1.0, 1.0, True),
                                                     (2, 256, 256, 2048, 1.0, 0.0, False),
                                                     (1, 640, 384, 1024, 0.25, 0.5, False)]:
        print("direct-to-LDS 128 x 128 case", batch, M, N, K, alpha, beta, with_bias, flush=True)
        a, b = random_tensor(rng, (batch, M, K), -1, 1), random_tensor(rng, (batch, N, K), -1, 1)
        c0 = random_tensor(rng, (batch, M, N), -1, 1)
        bias = random_tensor(rng, (N,), -1, 1) if with_bias else None
        got, tuning = run(a, b, c0, alpha, beta, bias, dtl_small)
        assert tuning == (dtl_small, 1), tuning
        ref = oracle.bmm(oracle.round_to_bf16(a), False, oracle.round_to_bf16(b), True, alpha, beta, c0 if beta else None)
        if bias is not None:
            ref = ref + bias
        assert np.all(np.isfinite(got))
        assert float(np.max(np.abs(got - ref))) <= 1e-4 * np.sqrt(K) * abs(alpha) + 1e-6 * (abs(beta) + 1), (batch, M, N, K)
    for (M, N, K) in [(300, 128, 64), (128, 128, 48), (128, 120, 64)]:
        a, b = random_tensor(rng, (1, M, K), -1, 1), random_tensor(rng, (1, N, K), -1, 1)
        got, tuning = run(a, b, None, 1.0, 0.0, None, dtl_small)
        assert tuning[0] != dtl_small
        assert float(np.max(np.abs(got - oracle.bmm(oracle.round_to_bf16(a), False, oracle.round_to_bf16(b), True)))) <= 1e-4 * np.sqrt(K)
    # shapes the kernel does not take run on another configuration even when it is forced
    for (M, N, K) in [(300, 256, 64), (256, 256, 48), (256, 250, 64)]:
        a, b = random_tensor(rng, (1, M, K), -1, 1), random_tensor(rng, (1, N, K), -1, 1)
        got, tuning = run(a, b, None, 1.0, 0.0, None, dtl)
        assert tuning[0] != dtl
        ref = oracle.bmm(oracle.round_to_bf16(a), False, oracle.round_to_bf16(b), True)
        assert float(np.max(np.abs(got - ref))) <= 1e-4 * np.sqrt(K)
    # a tile per compute unit: chosen without being asked for
    M = N = 4096
    K = 256
    a, b = random_tensor(rng, (1, M, K), -1, 1), random_tensor(rng, (1, N, K), -1, 1)
    got, tuning = run(a, b, None, 1.0, 0.0, None, -1)
    assert tuning == (dtl, 1), tuning
    rows = np.sort(rng.choice(M, 8, replace=False))
    ref = oracle.dot(oracle.round_to_bf16(a[0][rows]), False, oracle.round_to_bf16(b[0]), True)
    assert float(np.max(np.abs(got[0][rows] - ref))) <= 1e-4 * np.sqrt(K)


@pytest.mark.parametrize("tA,tB", list(itertools.product([False, True], repeat=2)))
def test_bf16_input_large_products_go_through_one_conversion(oracle, gpu_wrapper, tA, tB):
    """bf16-input arithmetic on a product of whole 256 x 256 tiles with a tile per compute unit: the library rounds both
    fp32 operands to bf16 once (into its workspace, in the k-contiguous form) and multiplies them with the bf16-storage
    kernel, in all four transpose forms.  Sampled rows against
    the oracle on rounded inputs (fp32 bound), alpha / beta / bias, contiguous operands and operands with padded rows
    (snhip_gemm_rm), and the same product again after a smaller one (the workspace is reused)."""
    from sharpnet_amd import GPUTensor
    from sharpnet_amd.hiplib import check_status
    w = gpu_wrapper
    lib, h = w.lib, w.handle
    kinds = {c["id"]: c["kind"] for c in w.configs()}
    rng = np.random.default_rng(880 + 2 * tA + tB)
    M, N, K = 4096, 4096, 256
    want_kind = "bf16-stored-dtl"
    for pad in (0, 8):
        a = random_tensor(rng, (K, M + pad) if tA else (M, K + pad), -1, 1)
        b = random_tensor(rng, (N, K + pad) if tB else (K, N + pad), -1, 1)
        c0, bias = random_tensor(rng, (M, N), -1, 1), random_tensor(rng, (N,), -1, 1)
        ga, gb, gc, gbias = T(w, a), T(w, b), T(w, c0), T(w, bias)
        print("bf16-input via conversion", tA, tB, "padding", pad, flush=True)
        check_status(lib.snhip_gemm_rm(h, int(tA), int(tB), M, N, K, 0.5, ga.Pointer, a.shape[1], 0, gb.Pointer, b.shape[1],
                                       0, -1.0, gc.Pointer, N, 0, 1, gbias.Pointer))     # handle in fp32 mode: reference
        ref32 = gc.ToNumpy()
        gc.InitializeFromHostMemory(c0)
        w.set_math_mode(w.MATH_BF16_INPUT)
        try:
            check_status(lib.snhip_gemm_rm(h, int(tA), int(tB), M, N, K, 0.5, ga.Pointer, a.shape[1], 0, gb.Pointer,
                                           b.shape[1], 0, -1.0, gc.Pointer, N, 0, 1, gbias.Pointer))
        finally:
            w.set_math_mode(w.MATH_FP32)
        assert kinds[w.last_tuning()[0]] == want_kind, (kinds[w.last_tuning()[0]], want_kind)
        got = gc.ToNumpy()
        assert np.all(np.isfinite(got))
        rows = np.sort(rng.choice(M, 6, replace=False))
        opa = np.ascontiguousarray((a[:, :M].T if tA else a[:, :K])[rows])
        opb = np.ascontiguousarray(b[:, :K] if tB else b[:, :N])
        ref = oracle.dot(oracle.round_to_bf16(opa), False, oracle.round_to_bf16(opb), tB, 0.5, -1.0, c0[rows]) + bias
        assert float(np.max(np.abs(got[rows] - ref))) <= 1e-4 * np.sqrt(K) * 0.5 + 2e-6
        assert float(np.max(np.abs(got - ref32))) / float(np.max(np.abs(ref32))) <= 1e-2
        for t in (ga, gb, gc, gbias):
            t.Dispose()


@pytest.mark.parametrize("tA,tB", [(False, False), (True, False), (True, True)])
def test_bf16_stored_large_products_are_brought_into_the_k_contiguous_form(oracle, gpu_wrapper, tA, tB):
    """Operands stored as bf16, a product of whole 256 x 256 tiles with a tile per compute unit, in a form other than
    plain A with transposed B: the library transposes the operand(s) lying the other way once into its workspace
    (bf16 to bf16) and runs the direct-load kernel.  Sampled rows against the oracle on the rounded inputs (fp32
    bound), alpha / beta / bias, contiguous operands and padded rows (snhip_gemm_ex), agreement with the
    register-transposing kernel forced through the tuning hook, and a smaller product of the same form afterwards."""
    from sharpnet_amd.hiplib import check_status, GemmDesc
    import ctypes
    w = gpu_wrapper
    lib, h = w.lib, w.handle
    kinds = {c["id"]: c["kind"] for c in w.configs()}
    staged = [c["id"] for c in w.configs() if c["kind"] == "bf16-stored"][0]
    rng = np.random.default_rng(990 + 2 * tA + tB)
    for (M, N, K, pad) in ((4096, 4096, 256, 0), (4096, 4096, 320, 8), (2048, 8192, 512, 0)):
        a = random_tensor(rng, (K, M + pad) if tA else (M, K + pad), -1, 1)
        b = random_tensor(rng, (N, K + pad) if tB else (K, N + pad), -1, 1)
        c0, bias = random_tensor(rng, (M, N), -1, 1), random_tensor(rng, (N,), -1, 1)
        ga, gb, gbias = T(w, a), T(w, b), T(w, bias)
        pa, pb = to_bf16_on_device(w, ga), to_bf16_on_device(w, gb)
        outs = {}
        for force in (-1, staged):
            gc = T(w, c0)
            d = GemmDesc()
            d.struct_size = ctypes.sizeof(GemmDesc)
            d.transA, d.transB, d.M, d.N, d.K = int(tA), int(tB), M, N, K
            d.alpha, d.beta = 0.5, -1.0
            d.A, d.lda, d.B, d.ldb = pa, a.shape[1], pb, b.shape[1]
            d.C, d.ldc, d.batch = gc.Pointer, N, 1
            d.bias = gbias.Pointer
            d.math = w.MATH_BF16_STORED
            print("bf16-stored via transposition", tA, tB, (M, N, K), "padding", pad, "forced", force, flush=True)
            w.set_tuning(force, 1 if force >= 0 else 0)
            try:
                check_status(lib.snhip_gemm_ex(h, ctypes.byref(d)))
            finally:
                w.set_tuning(-1, 0)
            want_kind = "bf16-stored-dtl" if force < 0 else "bf16-stored"
            assert kinds[w.last_tuning()[0]] == want_kind, (kinds[w.last_tuning()[0]], want_kind)
            outs[force] = gc.ToNumpy()
            gc.Dispose()
        got = outs[-1]
        assert np.all(np.isfinite(got))
        rows = np.sort(rng.choice(M, 6, replace=False))
        opa = np.ascontiguousarray((a[:, :M].T if tA else a[:, :K])[rows])
        opb = np.ascontiguousarray(b[:, :K] if tB else b[:, :N])
        ref = oracle.dot(oracle.round_to_bf16(opa), False, oracle.round_to_bf16(opb), tB, 0.5, -1.0, c0[rows]) + bias
        bound = 1e-4 * np.sqrt(K) * 0.5 + 2e-6
        assert float(np.max(np.abs(got[rows] - ref))) <= bound
        assert float(np.max(np.abs(got - outs[staged]))) <= bound
        w.release(pa, 2 * ga.Count)
        w.release(pb, 2 * gb.Count)
        for t in (ga, gb, gbias):
            t.Dispose()


def T(w, a):
    from sharpnet_amd import GPUTensor
    a = np.asarray(a, np.float32)
    return GPUTensor(list(a.shape), a, w)


@pytest.mark.parametrize("B,H,T,d,K_long", [(3, 2, 96, 64, False), (4, 4, 128, 320, True), (2, 3, 40, 48, False)])
def test_bf16_stored_two_level_batch_through_gemm_ex(oracle, gpu_wrapper, B, H, T, d, K_long):
    """snhip_gemm_ex with math = SNHIP_MATH_BF16_STORED on heads addressed in place: a two-level batch whose outer
    strides do not continue the inner ones, with too few matrices (or too long a K) for the streaming kernels, so the
    library walks the outer level on the host and must offset the 2-byte operands in bytes.  S[b][h] = Q[b][:, h] .
    K[b][:, h]^T; compared with the same call in bf16-input arithmetic on the fp32 originals and with the oracle on
    rounded inputs."""
    from sharpnet_amd import GPUTensor
    w = gpu_wrapper
    rng = np.random.default_rng(4300 + B * 7 + H)
    E = H * d
    q, k = random_tensor(rng, (B, T, E), -1, 1), random_tensor(rng, (B, T, E), -1, 1)
    gq, gk = GPUTensor(q.shape, q, w), GPUTensor(k.shape, k, w)
    pq, pk = to_bf16_on_device(w, gq), to_bf16_on_device(w, gk)
    print("two-level bf16-stored", B, H, T, d, K_long, flush=True)
    fields = dict(transA=0, transB=1, M=T, N=T, K=d, alpha=0.125, beta=0.0, lda=E, ldb=E, ldc=T, batch=B * H,
                  batch_inner=H, strideA=d, strideB=d, strideC=T * T, strideA_outer=T * E, strideB_outer=T * E,
                  strideC_outer=H * T * T)
    got = {}
    for math, a_ptr, b_ptr in ((2, pq, pk), (1, gq.Pointer, gk.Pointer)):
        gs = GPUTensor([B, H, T, T], None, w)
        gs.SetValue(float("nan"))
        gs.GemmEx(A=a_ptr, B=b_ptr, math=math, **fields)
        got[math] = gs.ToNumpy()
        if math == 2:
            # the path under test: not the streaming kernels (which walk both levels themselves)
            kinds = {c["id"]: c["kind"] for c in w.configs()}
            assert kinds[w.last_tuning()[0]] == "bf16-stored", kinds[w.last_tuning()[0]]
        gs.Dispose()
    qr, kr = oracle.round_to_bf16(q).reshape(B, T, H, d), oracle.round_to_bf16(k).reshape(B, T, H, d)
    ref = np.empty((B, H, T, T), np.float32)
    for b in range(B):
        for h in range(H):
            ref[b, h] = oracle.dot(np.ascontiguousarray(qr[b, :, h]), False, np.ascontiguousarray(kr[b, :, h]), True, 0.125)
    bound = 1e-4 * np.sqrt(d) * 0.125
    assert np.all(np.isfinite(got[2]))
    assert float(np.max(np.abs(got[2] - ref))) <= bound
    assert float(np.max(np.abs(got[2] - got[1]))) <= bound
    w.release(pq, max(2 * gq.Count, 8))
    w.release(pk, max(2 * gk.Count, 8))
    gq.Dispose()
    gk.Dispose()


@pytest.mark.parametrize("tA,tB", list(itertools.product([False, True], repeat=2)))
def test_bf16_streaming_kernels_strided_batches(oracle, gpu_wrapper, tA, tB):
    """The persistent streaming kernels in bf16-input arithmetic, fp32 storage and bf16 storage: more tiles than
    workgroups, ragged M / N, K below, at and above one panel, alpha / beta; forced through the tuning hook, and picked
    automatically for the attention-shaped products.  Bar: the fp32 bound against the oracle on bf16-rounded inputs."""
    from sharpnet_amd import GPUTensor
    from sharpnet_amd.hiplib import check_status
    w = gpu_wrapper
    lib, h = w.lib, w.handle
    kinds = {c["kind"]: [] for c in w.configs()}
    for c in w.configs():
        kinds[c["kind"]].append(c["id"])
    assert len(kinds["bf16-stream"]) == 2 and len(kinds["bf16-stored-stream"]) == 2
    rng = np.random.default_rng(700 + 2 * tA + tB)

    def run(stored, pa, pb, a, b, gc, alpha, beta):
        batch = a.shape[0]
        aH, aW, bH, bW = a.shape[1], a.shape[2], b.shape[1], b.shape[2]
        M, N = gc.Shape[1], gc.Shape[2]
        if stored:
            check_status(lib.snhip_bmm_bf16_stored(h, pa, aH, aW, int(tA), aH * aW, pb, bH, bW, int(tB), bH * bW, gc.Pointer,
                                                   M * N, batch, alpha, beta, None))
        else:
            check_status(lib.snhip_bmm_bf16(h, pa, aH, aW, int(tA), aH * aW, pb, bH, bW, int(tB), bH * bW, gc.Pointer, M * N,
                                            batch, alpha, beta))
    try:
        for (batch, M, N, K) in [(600, 128, 128, 64), (40, 256, 256, 64), (40, 256, 64, 256), (9, 200, 100, 72),
                                 (5, 130, 258, 130), (3, 64, 40, 8), (1, 300, 200, 136), (1100, 100, 60, 36)]:
            a = random_tensor(rng, (batch, K, M) if tA else (batch, M, K), -1, 1)
            b = random_tensor(rng, (batch, N, K) if tB else (batch, K, N), -1, 1)
            c = random_tensor(rng, (batch, M, N), -1, 1)
            ar, br = oracle.round_to_bf16(a), oracle.round_to_bf16(b)
            ga, gb = GPUTensor(a.shape, a, w), GPUTensor(b.shape, b, w)
            pa, pb = to_bf16_on_device(w, ga), to_bf16_on_device(w, gb)
            for stored, kind in ((False, "bf16-stream"), (True, "bf16-stored-stream")):
                for cfg in kinds[kind]:
                    w.set_tuning(cfg, 1)
                    for alpha, beta in [(0.125, 0.0), (-0.5, 1.0)]:
                        gc = GPUTensor(c.shape, c, w)
                        if beta == 0.0:
                            gc.SetValue(float("nan"))
                        run(stored, pa if stored else ga.Pointer, pb if stored else gb.Pointer, a, b, gc, alpha, beta)
                        assert w.last_tuning() == (cfg, 1), (batch, M, N, K, kind)
                        got = gc.ToNumpy()
                        gc.Dispose()
                        ref = oracle.bmm(ar, tA, br, tB, alpha, beta, c if beta != 0 else None)
                        bound = 1e-4 * np.sqrt(K) * abs(alpha) + (1e-6 * abs(beta) if beta else 0.0)
                        assert np.all(np.isfinite(got)), (batch, M, N, K, cfg, alpha, beta)
                        assert np.max(np.abs(got - ref)) <= bound, (batch, M, N, K, cfg, alpha, beta)
            w.release(pa, max(2 * ga.Count, 8))
            w.release(pb, max(2 * gb.Count, 8))
            ga.Dispose()
            gb.Dispose()
        w.set_tuning(-1, 0)
        # automatic choice for the two attention products of benchmark configuration 5 (fewer matrices, same shape)
        for (batch, M, N, K, which) in [(256, 256, 256, 64, 0), (256, 256, 64, 256, 1)]:
            a = random_tensor(rng, (batch, K, M) if tA else (batch, M, K), -1, 1)
            b = random_tensor(rng, (batch, N, K) if tB else (batch, K, N), -1, 1)
            ga, gb, gc = GPUTensor(a.shape, a, w), GPUTensor(b.shape, b, w), GPUTensor([batch, M, N], None, w)
            pa, pb = to_bf16_on_device(w, ga), to_bf16_on_device(w, gb)
            ref = oracle.bmm(oracle.round_to_bf16(a), tA, oracle.round_to_bf16(b), tB, 1.0)
            for stored, kind in ((False, "bf16-stream"), (True, "bf16-stored-stream")):
                gc.SetValue(float("nan"))
                run(stored, pa if stored else ga.Pointer, pb if stored else gb.Pointer, a, b, gc, 1.0, 0.0)
                assert w.last_tuning() == (kinds[kind][which], 1)
                assert np.max(np.abs(gc.ToNumpy() - ref)) <= 1e-4 * np.sqrt(K)
            w.release(pa, max(2 * ga.Count, 8))
            w.release(pb, max(2 * gb.Count, 8))
            for t in (ga, gb, gc):
                t.Dispose()
    finally:
        w.set_tuning(-1, 0)


@pytest.mark.parametrize("B,H,Tq,Tk,causal,packed", [(2, 3, 256, 256, True, True), (3, 2, 200, 132, False, False),
                                                       (2, 2, 130, 100, True, False), (70, 8, 130, 136, False, True),
                                                       # more than 256 keys: key blocks, two passes / one pass
                                                       (2, 2, 300, 700, True, False), (1, 3, 650, 516, False, True)])
def test_attention_forward_in_bf16_input_mode(oracle, gpu_wrapper, B, H, Tq, Tk, causal, packed):
    """snhip_attention_forward on a handle in the bf16-input math mode (head dimension 64, up to 256 keys): Q, K, V and
    the probabilities entering the second product are rounded to bf16, sums and softmax stay fp32.
    Two bars: against the fp32 oracle, 1e-2 of max|V| for the output and 1e-2 of the row maximum ... of the weights
    (the scores of |q|,|k| <= 1 at scale 1/8 move by at most 64 * 2 * 2^-9 / 8 = 0.03, their exponentials by 3 %);
    against the same chain on rounded operands: the weights against softmax(scale * Qb . Kb^T) as the fp32 kernels
    are, and the output against round(weights the kernel wrote) . Vb at 2e-5 (the kernel's own weights, because a
    weight that lies next to a bf16 rounding boundary may round either way after a last-bit difference in the
    softmax, and one such flip moves the output by 2^-9 of that weight)."""
    from sharpnet_amd import GPUTensor, attention
    rng = np.random.default_rng(71)
    Z, d = B * H, 64
    q, k, v = random_tensor(rng, (Z, Tq, d), -1, 1), random_tensor(rng, (Z, Tk, d), -1, 1), random_tensor(rng, (Z, Tk, d), -1, 1)
    scale = 1.0 / np.sqrt(d)

    def chain(q_, k_, v_, round_p):
        s = np.stack([oracle.dot(q_[z], False, k_[z], True, scale) for z in range(Z)])
        if causal:
            s[:, np.triu_indices(Tq, 1, Tk)[0], np.triu_indices(Tq, 1, Tk)[1]] = -1e12
        wts = oracle.softmax_last_dim(s)
        return oracle.bmm(oracle.round_to_bf16(wts) if round_p else wts, False, v_, False), wts
    o32, w32 = chain(q, k, v, False)
    obf, wbf = chain(oracle.round_to_bf16(q), oracle.round_to_bf16(k), oracle.round_to_bf16(v), True)

    def lay(x, steps):
        if not packed:
            return x
        return np.ascontiguousarray(x.reshape(B, H, steps, d).transpose(0, 2, 1, 3)).reshape(B, steps, H * d)
    w = gpu_wrapper
    gq, gk, gv = (GPUTensor(list(lay(x, t).shape), lay(x, t), w) for x, t in ((q, Tq), (k, Tk), (v, Tk)))
    go = GPUTensor(list(lay(o32, Tq).shape), None, w)
    gw = GPUTensor([Z, Tq, Tk], None, w)
    go.SetValue(float("nan"))
    gw.SetValue(float("nan"))
    w.set_math_mode(1)
    try:
        assert attention.fused_attention_forward(gq, gk, gv, go, gw, batch=B, heads=H, tq=Tq, tkv=Tk, dk=d, dv=d,
                                                 scale=scale, is_causal=causal, packed=packed)
        got_o, got_w = go.ToNumpy(), gw.ToNumpy()
        go.SetValue(float("nan"))
        assert attention.fused_attention_forward(gq, gk, gv, go, None, batch=B, heads=H, tq=Tq, tkv=Tk, dk=d, dv=d,
                                                 scale=scale, is_causal=causal, packed=packed)
        if Tk <= 256:
            assert np.array_equal(go.ToNumpy(), got_o)      # same kernel without its weight stores
        else:                                               # a single pass with a running maximum instead of two
            assert np.max(np.abs(go.ToNumpy() - lay(o32, Tq))) <= 1e-2 * float(np.max(np.abs(v)))
    finally:
        w.set_math_mode(0)
    assert np.max(np.abs(got_o - lay(o32, Tq))) <= 1e-2 * float(np.max(np.abs(v)))
    assert np.max(np.abs(got_w - w32)) <= 1e-2 * float(np.max(w32)) + 3e-2 * float(np.max(w32))
    assert np.max(np.abs(got_w - wbf)) <= 2e-6 + 1e-5 * float(np.max(wbf))
    o_from_got_w = oracle.bmm(oracle.round_to_bf16(got_w), False, oracle.round_to_bf16(v), False)
    assert np.max(np.abs(got_o - lay(o_from_got_w, Tq))) <= 2e-5 * float(np.max(np.abs(v)))
    assert np.max(np.abs(got_o - lay(obf, Tq))) <= 2.0 ** -8 * float(np.max(np.abs(v)))


@pytest.mark.parametrize("B,H,Tq,Tk,packed", [(2, 3, 256, 256, True), (3, 2, 200, 132, False), (70, 8, 130, 100, False),
                                              (2, 2, 200, 520, True)])
def test_attention_backward_in_bf16_input_mode(oracle, gpu_wrapper, B, H, Tq, Tk, packed):
    """snhip_attention_backward on a handle in the bf16-input math mode (head dimension 64): the batched
    products dV = P^T.dO and dK = dS^T.Q go through the bf16-input GEMMs as every product of such a handle does, and
    up to 256 keys the kernel between them (dP = dO.V^T, softmax gradient, dQ = dS.K) multiplies in bf16 as well (beyond
    256 keys it stays fp32); sums and the softmax gradient stay fp32.  Bar: 1e-2 of the largest reference value of each
    output (the bf16-input bar of the GEMMs)."""
    from sharpnet_amd import GPUTensor, attention
    rng = np.random.default_rng(73)
    Z, d = B * H, 64
    q, k = random_tensor(rng, (Z, Tq, d), -1, 1), random_tensor(rng, (Z, Tk, d), -1, 1)
    v, do = random_tensor(rng, (Z, Tk, d), -1, 1), random_tensor(rng, (Z, Tq, d), -1, 1)
    wts = oracle.softmax_last_dim(random_tensor(rng, (Z, Tq, Tk), -3, 3))
    scale = 0.37
    dv_ref = oracle.bmm(wts, True, do, False)
    ds_ref = oracle.softmax_last_dim_backward(wts, oracle.bmm(do, False, v, True, scale))
    dq_ref = oracle.bmm(ds_ref, False, k, False)
    dk_ref = oracle.bmm(ds_ref, True, q, False)

    def lay(x, steps):
        if not packed:
            return x
        return np.ascontiguousarray(x.reshape(B, H, steps, d).transpose(0, 2, 1, 3)).reshape(B, steps, H * d)
    w = gpu_wrapper
    gq, gk, gv, gdo = (GPUTensor(list(lay(x, t).shape), lay(x, t), w) for x, t in ((q, Tq), (k, Tk), (v, Tk), (do, Tq)))
    gw, gds = GPUTensor(list(wts.shape), wts, w), GPUTensor([Z, Tq, Tk], None, w)
    gdq, gdk, gdv = (GPUTensor(t.Shape, None, w) for t in (gq, gk, gv))
    for t in (gds, gdq, gdk, gdv):
        t.SetValue(float("nan"))
    w.set_math_mode(1)
    try:
        attention.attention_backward(gdq, gdk, gdv, gq, gk, gv, gdo, gw, gds, batch=B, heads=H, tq=Tq, tkv=Tk, dk=d, dv=d,
                                     scale=scale, packed=packed)
        got = [t.ToNumpy() for t in (gds, gdv, gdq, gdk)]
    finally:
        w.set_math_mode(0)
    for name, g, ref in zip(("dS", "dV", "dQ", "dK"), got, (ds_ref, lay(dv_ref, Tk), lay(dq_ref, Tq), lay(dk_ref, Tk))):
        assert np.all(np.isfinite(g)), name
        assert np.max(np.abs(g - ref)) <= 1e-2 * float(np.max(np.abs(ref))), name


@pytest.mark.parametrize("tA,tB", [(False, False), (True, True)])
def test_tall_and_narrow_products_with_a_long_k_are_split_in_every_arithmetic(oracle, gpu_wrapper, tA, tB):
    """A tall operand against a narrow one with a long K (4096 x 64 x 4096 and a ragged neighbour): the host splits K
    over enough workgroups to fill the chip - in fp32, with bf16 MFMAs on fp32 operands and with operands stored as
    bf16 - and the partial sums are added in index order by the reduction kernel.  Result against the oracle at the
    bar of each arithmetic, twice (the same bits both times)."""
    from sharpnet_amd import GPUTensor
    from sharpnet_amd.hiplib import check_status
    w = gpu_wrapper
    lib, h = w.lib, w.handle
    rng = np.random.default_rng(4242 + tA)
    try:
        for (M, N, K) in [(4096, 64, 4096), (4100, 50, 4104)]:
            a = random_tensor(rng, (K, M) if tA else (M, K), -1, 1)
            b = random_tensor(rng, (N, K) if tB else (K, N), -1, 1)
            c = random_tensor(rng, (M, N), -1, 1)
            ga, gb = GPUTensor(a.shape, a, w), GPUTensor(b.shape, b, w)
            # fp32
            w.set_math_mode(w.MATH_FP32)
            outs = []
            for _ in range(2):
                gc = GPUTensor([M, N], c, w)
                gc.Dot(ga, tA, gb, tB, 0.5, 1.0)
                outs.append(gc.ToNumpy())
                gc.Dispose()
            assert w.last_tuning()[1] > 1, w.last_tuning()
            assert np.array_equal(outs[0], outs[1])
            ref = oracle.dot(a, tA, b, tB, 0.5, 1.0, c)
            assert np.max(np.abs(outs[0] - ref)) <= 1e-4 * np.sqrt(K) * 0.5 + 1e-6, (M, N, K)
            # bf16 MFMAs on the fp32 operands
            w.set_math_mode(w.MATH_BF16_INPUT)
            outs = []
            for _ in range(2):
                gc = GPUTensor([M, N], c, w)
                gc.Dot(ga, tA, gb, tB, 0.5, 1.0)
                outs.append(gc.ToNumpy())
                gc.Dispose()
            assert w.last_tuning()[1] > 1, w.last_tuning()
            assert np.array_equal(outs[0], outs[1])
            check(oracle, outs[0], a, tA, b, tB, 0.5, 1.0, c, K)
            w.set_math_mode(w.MATH_FP32)
            # operands stored as bf16
            pa, pb = to_bf16_on_device(w, ga), to_bf16_on_device(w, gb)
            outs = []
            for _ in range(2):
                gc = GPUTensor([M, N], c, w)
                check_status(lib.snhip_dot_bf16_stored(h, pa, a.shape[0], a.shape[1], int(tA), pb, b.shape[0], b.shape[1],
                                                       int(tB), gc.Pointer, 0.5, 1.0, None))
                outs.append(gc.ToNumpy())
                gc.Dispose()
            assert w.last_tuning()[1] > 1, w.last_tuning()
            assert np.array_equal(outs[0], outs[1])
            check(oracle, outs[0], a, tA, b, tB, 0.5, 1.0, c, K)
            w.release(pa, max(2 * ga.Count, 8))
            w.release(pb, max(2 * gb.Count, 8))
            ga.Dispose()
            gb.Dispose()
    finally:
        w.set_math_mode(w.MATH_FP32)
