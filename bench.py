#!/usr/bin/env python3
"""Benchmark of the Tensor.Dot hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--no-cpu] [--no-extra]

A "step" is one Tensor.Dot of the headline workload: fp32, M = N = K = 8192,
no transposes, alpha = 1, beta = 0, A and B ~ U(-1, 1) (seeded), operands resident
in HBM before the timed region.  Prints ONE JSON line on stdout:
  value      TFLOP/s = 2*M*N*K / (wall time of K steps / K), device synchronised on both sides;
  roofline   the same algorithmic flops over the kernel's average launch duration measured with
             HIP events on the stream the kernel runs on, against the 157.3 TFLOP/s fp32 MFMA peak;
  cpu_baseline  the reference's CPU route (MKL cblas_sgemm RowMajor, the call of
             Prod/Data/BlasServices.cs:20) timed on this box's host cores on a bounded sample;
  summary    a handful of figures of the other benchmark configurations.
The line is strict JSON (no NaN tokens) and short (under 4000 characters): it is the LAST line of
stdout.  The per-product figures of the other configurations (dense layer, sweep, MLP step, LSTM
projections, attention matmuls, whole-layer calls) go to stderr and to the JSON file that
--extra-out names.  Every timed product is checked against the oracle on sampled
rows of the timed result; a miss ends the run with an error.
"""
import argparse
import hashlib
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)


MAX_LINE_CHARS = 4000     # the line must fit well inside what a harness keeps of stdout


def log(*a):
    print(*a, file=sys.stderr, flush=True)


def _no_constants(token):
    raise ValueError("non-JSON constant %r in the bench line" % token)


def headline_line(out):
    """The one stdout line: strict JSON (NaN / Infinity refused), short, parsed back before it is returned."""
    line = json.dumps(out, allow_nan=False, separators=(", ", ": "))
    if len(line) >= MAX_LINE_CHARS:
        raise ValueError("bench line has %d characters (limit %d): move detail into the extra file"
                         % (len(line), MAX_LINE_CHARS))
    json.loads(line, parse_constant=_no_constants)
    for key in ("metric", "value", "unit", "n_gpus", "steps", "warmup", "ms_per_step", "dtype", "config", "roofline"):
        if key not in out:
            raise ValueError("bench line lacks %r" % key)
    return line


def source_hash(path):
    """sha256 (first 16 hex digits) of a source file, to tell whether a stored counter figure is still the kernel's."""
    with open(path, "rb") as f:
        return hashlib.sha256(f.read()).hexdigest()[:16]


def traffic_record(root):
    """HBM bytes per launch of the headline kernel: a counter figure from two rocprofv3 --pmc runs, stored under
    profiles/ together with a hash of the kernel source it was measured on.  Returns (bytes or None, source dict)."""
    tpath = os.path.join(root, "profiles", "sgemm_8192_hbm_traffic.json")
    if not os.path.exists(tpath):
        return None, None
    with open(tpath) as f:
        tj = json.load(f)
    kernel_file = tj.get("kernel_source_file", "sharpnet_amd/csrc/sgemm_mfma.hpp")
    kpath = os.path.join(root, kernel_file)
    now = source_hash(kpath) if os.path.exists(kpath) else None
    stale = (tj.get("kernel_source_sha256_16") is None) or (now != tj.get("kernel_source_sha256_16"))
    return tj.get("hbm_bytes_per_launch"), {"file": "profiles/sgemm_8192_hbm_traffic.json",
                                            "measured_in_this_run": False, "stale": bool(stale),
                                            "kernel_source_sha256_16": tj.get("kernel_source_sha256_16"),
                                            "summary": tj.get("source")}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-extra", action="store_true", help="skip the other configurations")
    ap.add_argument("--cpu-reps", type=int, default=3)
    ap.add_argument("--extra-out", default=os.path.join("gpurun_out", "bench_extra.json"), metavar="PATH",
                    help="where the per-product figures of the other configurations are written (JSON)")
    ap.add_argument("--table", default=None, metavar="PATH",
                    help="also write the per-configuration figures of `extra` as a markdown table to PATH")
    ap.add_argument("--pcie", action="store_true",
                    help="also time the headline GEMM with host->device upload of A, B and device->host download of C")
    ap.add_argument("--attention-probe", action="store_true",
                    help="20 launches of the one-launch attention forward of configuration 5 (512 x 256 x 64, weights "
                         "kept), for profilers")
    ap.add_argument("--rnn-probe", choices=["lstm", "gru"], default=None,
                    help="3 forward + backward passes of a recurrent layer at configuration 4's shape (batch 256, 128 "
                         "steps, 256 -> 512), for profilers")
    ap.add_argument("--shapes-probe", action="store_true",
                    help="30 launches each of the skinny, small-M and batched shapes (and the bf16-input headline), in "
                         "the order printed, for profilers")
    ap.add_argument("--bf16-data-probe", action="store_true",
                    help="the bf16-storage product of the headline size (8192^3, A plain, B transposed) on operands of "
                         "different bit activity - U(-1,1), small integers, all ones - 20 launches each through the "
                         "direct-load kernel, then U(-1,1) through the register-staged one: for profilers (the engine "
                         "clock under each load = GRBM_GUI_ACTIVE / duration)")
    ap.add_argument("--dense-probe", action="store_true",
                    help="2000 calls each of the Dense layer of configuration 1 (128 x 784 -> 256) forward (bias + ReLU) "
                         "and backward (bias gradient + weight decay) through the one-launch entry points, for profilers")
    ap.add_argument("--probe", action="store_true",
                    help="counter-collection mode for rocprofv3 --pmc: 3 plain copies of 1 GiB, then 3 headline GEMMs")
    args = ap.parse_args()
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        sys.exit("bench.py: this build runs on ONE GPU only (no collectives, no sharding); run with --gpus 1")

    from sharpnet_amd import GPUWrapper, GPUTensor, workloads as wl
    w = GPUWrapper.FromDeviceId(0)
    info = w.device_info()
    log("[bench] device:", info)

    def upload(arr):
        return GPUTensor(arr.shape, arr, w)

    def time_gemm(g, a, b, c, steps, warmup, bias=None, min_warm_ms=0.0, groups=1):
        """Returns (wall ms/step, event ms/launch, GPUTensor C, launches): C is what `launches` launches in a row
        (warm-up included) made of the seeded C, so a product with beta = 1 still has a closed form.
        groups > 1 (the short products of the other configurations): `steps` launches are timed that many times in a
        row and the median group counts - the interval between two events includes whatever time the host took to
        issue the launches, and one descheduled moment inside a window of 0.2 ms is a factor of ten."""
        ga, gb = upload(a), upload(b)
        gc = upload(c) if c is not None else GPUTensor(g.c_shape, None, w)
        gbias = upload(bias) if bias is not None else None

        launches = [0]

        def launch():
            launches[0] += 1
            if g.batch > 1:
                gc.BatchMatrixMultiplication(ga, g.tA, gb, g.tB, g.alpha, g.beta)
            elif gbias is not None:
                gc.DotRowMajor(ga, g.tA, gb, g.tB, g.alpha, g.beta, bias=gbias)
            else:
                gc.Dot(ga, g.tA, gb, g.tB, g.alpha, g.beta)
        for _ in range(warmup):
            launch()
        if min_warm_ms > 0:
            # short kernels: keep launching until the engine clock has ramped (idle GPUs start slow)
            w.synchronize()
            t_w = time.perf_counter()
            while (time.perf_counter() - t_w) * 1e3 < min_warm_ms:
                for _ in range(10):
                    launch()
                w.synchronize()
        e0, e1 = w.new_event(), w.new_event()
        walls, evs = [], []
        for _ in range(groups):
            w.synchronize()
            t0 = time.perf_counter()
            w.record(e0)
            for _ in range(steps):
                launch()
            w.record(e1)
            w.synchronize()
            walls.append((time.perf_counter() - t0) * 1e3 / steps)
            evs.append(w.elapsed_ms(e0, e1) / steps)
        wall_ms, ev_ms = float(np.median(walls)), float(np.median(evs))
        w.destroy_event(e0)
        w.destroy_event(e1)
        ga.Dispose()
        gb.Dispose()
        if gbias is not None:
            gbias.Dispose()
        return wall_ms, ev_ms, gc, launches[0]

    def check_timed_result(gm, aa, bb, cc, got, steps, bias=None, bf16=False, nrows=6):
        """Sampled rows of a timed result against the oracle.  `got` is C after `steps` launches in a row that started
        from the seeded C (beta is 0 or 1 in every benchmark product: C = steps*(alpha*op(A)op(B) + bias) + C0 for
        beta = 1, and the last launch's result for beta = 0).
        bf16: the oracle multiplies the operands rounded to bf16 (what the reduced-precision kernels compute)."""
        from oracle import dot_oracle
        assert gm.beta in (0.0, 1.0)
        pick = np.random.default_rng(4242)
        reps = steps if gm.beta != 0 else 1
        mats = [None] if gm.batch == 1 else list(np.sort(pick.choice(gm.batch, min(3, gm.batch), replace=False)))
        worst, bound = 0.0, 0.0
        for z in mats:
            a2, b2 = (aa, bb) if z is None else (aa[z], bb[z])
            g2 = got if z is None else got[z]
            rows = np.sort(pick.choice(gm.M, min(nrows, gm.M), replace=False))
            a_sub = np.ascontiguousarray(a2[:, rows] if gm.tA else a2[rows])
            if bf16:
                a_sub, b2 = dot_oracle.round_to_bf16(a_sub), dot_oracle.round_to_bf16(b2)
            ref = dot_oracle.dot_f64(a_sub, gm.tA, b2, gm.tB, gm.alpha) * reps
            if gm.beta != 0:
                ref = ref + (cc if z is None else cc[z])[rows].astype(np.float64)
            if bias is not None:
                ref = ref + bias.reshape(1, -1).astype(np.float64) * reps
            # fp32 rounding of the running sum when C accumulates over many launches
            bound_acc = 0.0 if reps == 1 else reps * 2.0 ** -23 * float(np.max(np.abs(ref)))
            worst = max(worst, float(np.max(np.abs(g2[rows].astype(np.float64) - ref))))
            bound = max(bound, dot_oracle.tolerance(gm.K, a_sub, b2) * abs(gm.alpha) * reps + bound_acc)
        if not worst <= bound:
            sys.exit("bench.py: timed result of %s is outside the parity bound (max|d| = %.3e, bound %.3e)"
                     % (gm.label(), worst, bound))
        return worst, bound

    def run_stored(gm, seed, steps, warmup, to_nt=False):
        """One product with operands stored as bf16.  to_nt (single matrices only): a transposed A / a plain B is
        transposed by the conversion pass, so that the product itself runs in the NT form."""
        from sharpnet_amd.hiplib import check_status
        aa, bb, _ = wl.uniform_operands(gm, seed)
        ga, gb = upload(aa), upload(bb)
        gcs = GPUTensor(gm.c_shape, None, w)
        pa, pb = w.allocate(2 * ga.Count), w.allocate(2 * gb.Count)
        aH, aW = aa.shape[-2:]
        bH, bW = bb.shape[-2:]
        flip_a, flip_b = to_nt and gm.tA, to_nt and not gm.tB
        assert not to_nt or gm.batch == 1

        def convert():
            if flip_a:
                check_status(w.lib.snhip_convert_f32_to_bf16_2d(w.handle, ga.Pointer, aH, aW, aW, 1, pa, aH))
            else:
                check_status(w.lib.snhip_convert_f32_to_bf16(w.handle, ga.Pointer, pa, ga.Count))
            if flip_b:
                check_status(w.lib.snhip_convert_f32_to_bf16_2d(w.handle, gb.Pointer, bH, bW, bW, 1, pb, bH))
            else:
                check_status(w.lib.snhip_convert_f32_to_bf16(w.handle, gb.Pointer, pb, gb.Count))
        if flip_a:
            aH, aW = aW, aH
        if flip_b:
            bH, bW = bW, bH
        tA, tB = (False if flip_a else gm.tA), (True if flip_b else gm.tB)

        def launch():
            check_status(w.lib.snhip_bmm_bf16_stored(w.handle, pa, aH, aW, int(tA), aH * aW, pb, bH, bW, int(tB),
                                                     bH * bW, gcs.Pointer, gm.M * gm.N, gm.batch, gm.alpha, gm.beta,
                                                     None))

        def timed(fn, n, nw):
            for _ in range(nw):
                fn()
            e0, e1 = w.new_event(), w.new_event()
            w.synchronize()
            w.record(e0)
            for _ in range(n):
                fn()
            w.record(e1)
            ms = w.elapsed_ms(e0, e1) / n
            w.destroy_event(e0)
            w.destroy_event(e1)
            return ms
        conv_ms = timed(convert, 5, 2)
        ms = timed(launch, steps, warmup)
        err, bound = check_timed_result(gm, aa, bb, None, gcs.ToNumpy(), steps, bf16=True)
        by = gm.batch * (2.0 * (gm.M * gm.K + gm.K * gm.N) + 4.0 * gm.M * gm.N)
        roof_s = max(gm.flops / (wl.BF16_MFMA_PEAK_TFLOPS * 1e12), by / (wl.HBM_PEAK_GBS * 1e9))
        r = {"gemm": gm.label() + (" (bf16 storage, operands transposed to the NT form by the conversion)" if to_nt
                                 else " (bf16 storage)"), "ms": round(ms, 4), "tflops": round(gm.flops / (ms * 1e-3) / 1e12, 2),
             "frac_of_roofline": round(roof_s * 1e3 / ms, 4), "tile_config": w.last_tuning()[0],
             "splitk": w.last_tuning()[1], "algorithmic_bytes": by, "convert_both_operands_ms": round(conv_ms, 4),
             "max_abs_err": err, "parity_bound": bound}
        w.release(pa, 2 * ga.Count)
        w.release(pb, 2 * gb.Count)
        for t in (ga, gb, gcs):
            t.Dispose()
        return r

    if args.bf16_data_probe:
        from sharpnet_amd.hiplib import check_status
        S = 8192
        rng = np.random.default_rng(2)
        fills = [("U(-1,1)", lambda: rng.uniform(-1, 1, (S, S)).astype(np.float32)),
                 ("integers -2..2", lambda: rng.integers(-2, 3, (S, S)).astype(np.float32)),
                 ("all ones", lambda: np.ones((S, S), np.float32))]
        dtl = [c["id"] for c in w.configs() if c["kind"] == "bf16-stored-dtl"][0]
        staged = [c["id"] for c in w.configs() if c["kind"] == "bf16-stored"][0]
        pa, pb = w.allocate(2 * S * S), w.allocate(2 * S * S)
        gc = GPUTensor([S, S], None, w)
        for name, make, cfg in [(n, m, dtl) for n, m in fills] + [(fills[0][0], fills[0][1], staged)]:
            for host, dst in ((make(), pa), (make(), pb)):
                g = upload(host)
                check_status(w.lib.snhip_convert_f32_to_bf16(w.handle, g.Pointer, dst, S * S))
                g.Dispose()
            w.set_tuning(cfg, 1)
            try:
                def launch():
                    check_status(w.lib.snhip_dot_bf16_stored(w.handle, pa, S, S, 0, pb, S, S, 1, gc.Pointer, 1.0, 0.0, None))
                for _ in range(10):
                    launch()
                e0, e1 = w.new_event(), w.new_event()
                w.synchronize()
                w.record(e0)
                for _ in range(20):
                    launch()
                w.record(e1)
                w.synchronize()
                ms = w.elapsed_ms(e0, e1) / 20
            finally:
                w.set_tuning(-1, 0)
            print(json.dumps({"operands": name, "tile_config": w.last_tuning()[0], "launches": 30, "event_ms": round(ms, 4),
                              "tflops": round(2.0 * S ** 3 / (ms * 1e-3) / 1e12, 1)}), flush=True)
        return
    if args.dense_probe:
        for r in dense_layer_calls(w, wl, upload, timed_calls=2000)["calls"]:
            print(json.dumps(r), flush=True)
        return
    if args.attention_probe:
        from sharpnet_amd import attention
        rng = np.random.default_rng(5)
        Z, Tn, d = 512, 256, 64
        q, k, v = (GPUTensor([Z, Tn, d], rng.uniform(-1, 1, (Z, Tn, d)).astype(np.float32), w) for _ in range(3))
        o, wts = GPUTensor([Z, Tn, d], None, w), GPUTensor([Z, Tn, Tn], None, w)
        for keep in (wts, None):
            for _ in range(20):
                attention.fused_attention_forward(q, k, v, o, keep, batch=Z, heads=1, tq=Tn, tkv=Tn, dk=d, dv=d,
                                                  scale=0.125, is_causal=False, packed=False)
            w.synchronize()
        for t in (q, k, v, o, wts):
            t.Dispose()
        # more than 256 keys: the two-pass kernel over key blocks (64 sequences of 1024 positions, weights kept, then causal)
        Z, Tn = 64, 1024
        q, k, v = (GPUTensor([Z, Tn, d], rng.uniform(-1, 1, (Z, Tn, d)).astype(np.float32), w) for _ in range(3))
        o, wts = GPUTensor([Z, Tn, d], None, w), GPUTensor([Z, Tn, Tn], None, w)
        for causal in (False, True):
            for _ in range(20):
                attention.fused_attention_forward(q, k, v, o, wts, batch=Z, heads=1, tq=Tn, tkv=Tn, dk=d, dv=d,
                                                  scale=0.125, is_causal=causal, packed=False)
            w.synchronize()
        # and the backward call at that size (dV, the two-pass kernel for dS and dQ, dK)
        do, ds = GPUTensor([Z, Tn, d], None, w), GPUTensor([Z, Tn, Tn], None, w)
        dq, dk_, dv_ = (GPUTensor([Z, Tn, d], None, w) for _ in range(3))
        do.SetValue(0.01)
        for _ in range(20):
            attention.attention_backward(dq, dk_, dv_, q, k, v, do, wts, ds, batch=Z, heads=1, tq=Tn, tkv=Tn, dk=d, dv=d,
                                         scale=0.125, packed=False)
        w.synchronize()
        # ... and with the causal hint, on the weights of the causal forward call just above
        for _ in range(20):
            attention.attention_backward(dq, dk_, dv_, q, k, v, do, wts, ds, batch=Z, heads=1, tq=Tn, tkv=Tn, dk=d, dv=d,
                                         scale=0.125, packed=False, is_causal=True)
        w.synchronize()
        for t in (q, k, v, o, wts, do, ds, dq, dk_, dv_):
            t.Dispose()
        # the handle in the bf16-input math mode: 512 x (256 x 64) with and without the weights, then 64 x 1024 keys
        w.set_math_mode(1)
        for Z, Tn in ((512, 256), (64, 1024)):
            q, k, v = (GPUTensor([Z, Tn, d], rng.uniform(-1, 1, (Z, Tn, d)).astype(np.float32), w) for _ in range(3))
            o, wts = GPUTensor([Z, Tn, d], None, w), GPUTensor([Z, Tn, Tn], None, w)
            for keep in (wts, None):
                for _ in range(20):
                    attention.fused_attention_forward(q, k, v, o, keep, batch=Z, heads=1, tq=Tn, tkv=Tn, dk=d, dv=d,
                                                      scale=0.125, is_causal=False, packed=False)
                w.synchronize()
            for t in (q, k, v, o, wts):
                t.Dispose()
        w.set_math_mode(0)
        return
    if args.rnn_probe:
        from sharpnet_amd import recurrent
        rng = np.random.default_rng(4)
        w.use_memory_pool(True)
        B, Tn, I, H = 256, 128, 256, 512
        x = GPUTensor([B, Tn, I], rng.uniform(-1, 1, (B, Tn, I)).astype(np.float32), w)
        dy = GPUTensor([B, Tn, H], rng.uniform(-0.01, 0.01, (B, Tn, H)).astype(np.float32), w)
        y, dx = GPUTensor([B, Tn, H], None, w), GPUTensor([B, Tn, I], None, w)
        cell, bias = ((recurrent.CUDNN_LSTM, recurrent.CUDNN_RNN_SINGLE_INP_BIAS) if args.rnn_probe == "lstm" else
                      (recurrent.CUDNN_GRU, recurrent.CUDNN_RNN_DOUBLE_BIAS))
        layer = recurrent.RecurrentLayer(w, I, H, cell, bias, True, False, 1)
        layer._weightsAndBiases.InitializeFromHostMemory(
            rng.uniform(-0.04, 0.04, layer._weightsAndBiases.Count).astype(np.float32))
        for _ in range(3):
            layer.ForwardPropagation(x, y, True)
            layer.BackwardPropagation(x, y, dy, dx)
        w.synchronize()
        return
    if args.shapes_probe:
        shapes = [("skinny 8192x64x8192 NN", wl.Gemm(8192, 64, 8192), 0), ("skinny 8192x64x8192 TN", wl.Gemm(8192, 64, 8192, True, False), 0)]
        shapes += [("dense " + gm.name, gm, 0) for gm in wl.dense_layer_gemms()]
        proj, rec, _ = wl.lstm_gemms()
        shapes += [("lstm input projection", proj, 0), ("lstm recurrent step (beta=1)", rec, 0)]
        shapes += [("attention " + gm.name, gm, 0) for gm in wl.attention_gemms()]
        shapes += [("bf16-input 8192^3 TN", wl.Gemm(8192, 8192, 8192, True, False), 1),
                   ("bf16-input 8192^3 NN", wl.Gemm(8192, 8192, 8192), 1),
                   ("bf16-input 4096^3 NN", wl.Gemm(4096, 4096, 4096), 1)]
        shapes += [("bf16-input attention " + gm.name, gm, 1) for gm in wl.attention_gemms()]
        shapes += [("square %d^3 NN" % n, wl.Gemm(n, n, n), 0) for n in (1024, 2048, 4096)]
        shapes += [("ragged 1000^3 NN", wl.Gemm(1000, 1000, 1000), 0),
                   ("ragged 4097x3001x2049 NN", wl.Gemm(4097, 3001, 2049), 0)]
        for name, gm, math_mode in shapes:
            w.set_math_mode(math_mode)
            aa, bb, cc = wl.uniform_operands(gm, 2)
            _, ms, gcx, _ = time_gemm(gm, aa, bb, cc, 20, 10)
            gcx.Dispose()
            print(json.dumps({"shape": name, "M": gm.M, "N": gm.N, "K": gm.K, "batch": gm.batch, "launches": 30,
                              "flops": gm.flops, "bytes": gm.bytes, "event_ms": round(ms, 5),
                              "tile_config": w.last_tuning()[0], "splitk": w.last_tuning()[1]}), flush=True)
        w.set_math_mode(0)
        # operands stored as bf16 (converted once, outside the 30 launches of each product)
        stored = [wl.Gemm(8192, 8192, 8192, tA, tB, 1.0, 0.0) for (tA, tB) in ((False, True), (False, False), (True, False))]
        for gm in stored + list(wl.attention_gemms()):
            r = run_stored(gm, 2, 20, 10)
            print(json.dumps({"shape": "bf16-stored " + gm.label(), "M": gm.M, "N": gm.N, "K": gm.K, "batch": gm.batch,
                              "launches": 30, "flops": gm.flops, "bytes": r["algorithmic_bytes"], "event_ms": r["ms"],
                              "tile_config": r["tile_config"], "splitk": r["splitk"]}), flush=True)
        return
    if args.probe:
        # known-size launch: copy_f32_kernel reads 2**30 bytes and writes 2**30 bytes
        n = 1 << 28
        src, dst = GPUTensor([n], None, w), GPUTensor([n], None, w)
        src.SetValue(1.0)
        for _ in range(3):
            from sharpnet_amd.hiplib import check_status
            check_status(w.lib.snhip_copy_f32(w.handle, dst.Pointer, src.Pointer, n), "snhip_copy_f32")
        w.synchronize()
        src.Dispose()
        dst.Dispose()
        g = wl.HEADLINE
        a, b, _ = wl.uniform_operands(g, seed=2)
        _, ev_ms, gc, _ = time_gemm(g, a, b, None, 3, 0)
        log("[bench] probe: 3 x copy of 2^30 bytes, 3 x %s at %.3f ms" % (g.label(), ev_ms))
        return

    # ------------------------------------------------------------------ headline
    g = wl.HEADLINE
    a, b, _ = wl.uniform_operands(g, seed=2)
    wall_ms, ev_ms, gc, _ = time_gemm(g, a, b, None, args.steps, args.warmup)
    cfg, splitk = w.last_tuning()
    tflops = g.flops / (wall_ms * 1e-3) / 1e12
    achieved = g.flops / (ev_ms * 1e-3) / 1e12
    log("[bench] headline %s: wall %.3f ms/step, events %.3f ms/launch, %.1f TFLOP/s, tile config %d split-K %d"
        % (g.label(), wall_ms, ev_ms, tflops, cfg, splitk))

    # parity of the timed configuration: sampled rows and columns against the oracle
    from oracle import dot_oracle
    rng = np.random.default_rng(99)
    rows = np.sort(rng.choice(g.M, 16, replace=False))
    gpu_c = gc.ToNumpy()
    got = gpu_c[rows]
    ref = dot_oracle.dot(np.ascontiguousarray(a[rows]), False, b, False)
    err = float(np.max(np.abs(got - ref)))
    bound = dot_oracle.tolerance(g.K, a, b)
    log("[bench] parity of the timed result (16 sampled rows): max|d| = %.3e, bound %.3e" % (err, bound))
    if not err <= bound:
        sys.exit("bench.py: timed result is outside the parity bound")
    gc.Dispose()

    # HBM traffic per launch is a counter figure (two rocprofv3 --pmc runs); it cannot be collected from inside
    # this process, so the line carries the stored figure together with where and when it was measured.
    traffic, traffic_source = traffic_record(ROOT)

    out = {
        "metric": "fp32 GEMM throughput, Tensor.Dot M=N=K=8192 (GEMM TFLOP/s + % of fp32 MFMA peak at 1 GPU)",
        "value": round(tflops, 2), "unit": "TFLOP/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(wall_ms, 4), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f32", "data": "synthetic",
        "config": {"workload": "configs[1] sweep, headline size: Tensor.Dot fp32 row-major NN, M=N=K=8192, alpha=1, "
                               "beta=0, A,B~U(-1,1) seed 2, operands resident in HBM",
                   "M": g.M, "N": g.N, "K": g.K, "tile_config": cfg, "splitk": splitk,
                   "device": {"cu": info["compute_units"], "clock_mhz": info["clock_khz"] / 1000.0}},
        "roofline": {"bound": "mfma", "achieved": round(achieved, 2), "peak": wl.FP32_MFMA_PEAK_TFLOPS,
                     "unit": "TFLOP/s", "frac": round(achieved / wl.FP32_MFMA_PEAK_TFLOPS, 4), "traffic": traffic,
                     "traffic_source": traffic_source, "flops_per_launch": g.flops,
                     "ms_per_launch_hip_events": round(ev_ms, 4),
                     "kernel": "sgemm_mfma_kernel<TileCfg<4,4,2,2,16>, NN> (256x256x16 tiles)"},
        "parity": {"max_abs_err": err, "bound": bound, "rows_checked": 16},
    }

    if args.pcie:
        # what a caller with host-resident operands would see: upload A and B, multiply, download C (pageable host memory)
        ga, gb = GPUTensor(list(a.shape), None, w), GPUTensor(list(b.shape), None, w)
        gcp = GPUTensor([g.M, g.N], None, w)
        ts = []
        for _ in range(3):
            w.synchronize()
            t0 = time.perf_counter()
            ga.InitializeFromHostMemory(a)
            gb.InitializeFromHostMemory(b)
            gcp.Dot(ga, False, gb, False, 1.0, 0.0)
            gcp.ContentAsFloatArray()
            ts.append(time.perf_counter() - t0)
        t_pcie = float(np.median(ts))
        out["pcie_inclusive"] = {"ms": round(t_pcie * 1e3, 2), "tflops": round(g.flops / t_pcie / 1e12, 2),
                                 "note": "H2D of A and B (2 x 268 MB), kernel, D2H of C (268 MB), pageable host memory"}
        log("[bench] PCIe-inclusive:", out["pcie_inclusive"])
        for t in (ga, gb, gcp):
            t.Dispose()

    # ------------------------------------------------------------------ CPU baseline (bounded sample)
    if not args.no_cpu:
        cores = dot_oracle.mkl_threads()
        cpu_out = np.empty((g.M, g.N), np.float32)
        route = dot_oracle.mkl_dot(a, False, b, False, cpu_out)          # warm-up, also the full-size oracle
        ts = []
        for _ in range(args.cpu_reps):
            t0 = time.perf_counter()
            dot_oracle.mkl_dot(a, False, b, False, cpu_out)
            ts.append(time.perf_counter() - t0)
        cpu_s = float(np.median(ts))
        out["cpu_baseline"] = {
            "value": round(g.flops / cpu_s / 1e12, 4), "unit": "TFLOP/s", "cores": cores, "kind": "port",
            "sample": "%d timed + 1 warm-up calls of the full headline GEMM (8192^3) through %s, "
                      "median %.2f s per call; os.cpu_count()=%d" % (args.cpu_reps, route, cpu_s, os.cpu_count()),
        }
        log("[bench] cpu baseline:", out["cpu_baseline"])
        # the whole timed GPU result against the whole MKL result of the same product
        err_mkl = 0.0
        for r0 in range(0, g.M, 1024):
            err_mkl = max(err_mkl, float(np.max(np.abs(gpu_c[r0:r0 + 1024] - cpu_out[r0:r0 + 1024]))))
        out["parity"]["max_abs_err_vs_mkl_full_result"] = err_mkl
        log("[bench] timed GPU result against the MKL result, all %d x %d elements: max|d| = %.3e (bound %.3e)"
            % (g.M, g.N, err_mkl, bound))
        if not err_mkl <= bound:
            sys.exit("bench.py: timed result differs from the MKL result by more than the parity bound")
        del cpu_out
    del a, b, gpu_c

    # ------------------------------------------------------------------ the other configurations
    # GPU figure and, beside it, the reference's CPU route for the same product on this box's host cores:
    # cblas_sgemm RowMajor through MKL (BlasServices.cs:20), the bias pass of Linear.cs:131 where the layer has
    # one, and the serial per-matrix loop of CpuTensor.cs:3018-3024 for the batched products.  The CPU side is a
    # bounded sample (a few calls per product); its total is logged.
    if not args.no_extra:
        extra = {}
        cpu_on = not args.no_cpu
        cpu_cores = dot_oracle.mkl_threads() if cpu_on else 0
        cpu_spent = [0.0]
        bf16_math = [False]       # set while the handle multiplies in the bf16-input math mode

        def cpu_ms(gm, aa, bb, cc, reps, bias=None):
            """Median ms of the product through MKL after one warm-up call."""
            t_in = time.perf_counter()
            out = np.array(cc, np.float32) if cc is not None else np.empty(gm.c_shape, np.float32)
            ts = []
            for rep in range(reps + 1):
                t0 = time.perf_counter()
                if gm.batch > 1:
                    dot_oracle.mkl_bmm_serial(aa, gm.tA, bb, gm.tB, out, gm.alpha, gm.beta)
                else:
                    dot_oracle.mkl_dot(aa, gm.tA, bb, gm.tB, out, gm.alpha, gm.beta)
                    if bias is not None:
                        np.add(out, bias.reshape(1, -1), out=out)
                if rep > 0:
                    ts.append(time.perf_counter() - t0)
            cpu_spent[0] += time.perf_counter() - t_in
            return float(np.median(ts)) * 1e3

        def run(gm, seed, steps=10, warmup=3, bias=None, cpu_reps=0):
            aa, bb, cc = wl.uniform_operands(gm, seed)
            _, ms, gcx, count = time_gemm(gm, aa, bb, cc, steps, warmup, bias=bias, min_warm_ms=40.0, groups=3)
            err, bound = check_timed_result(gm, aa, bb, cc, gcx.ToNumpy(), count, bias=bias, bf16=bf16_math[0])
            gcx.Dispose()
            tf = gm.flops / (ms * 1e-3) / 1e12
            r = {"gemm": gm.label(), "ms": round(ms, 4), "tflops": round(tf, 2),
                 "frac_of_roofline": round(gm.roofline_seconds() * 1e3 / ms, 4), "tile_config": w.last_tuning()[0],
                 "splitk": w.last_tuning()[1], "max_abs_err": err, "parity_bound": bound}
            if cpu_on and cpu_reps > 0:
                cms = cpu_ms(gm, aa, bb, cc, cpu_reps, bias=bias)
                r["cpu_mkl_ms"] = round(cms, 4)
                r["cpu_mkl_tflops"] = round(gm.flops / (cms * 1e-3) / 1e12, 4)
            return r

        def cpu_summary(rows, gemms, sample):
            """cpu_baseline object of one configuration from its per-product rows."""
            timed = [(r, gm) for r, gm in zip(rows, gemms) if "cpu_mkl_ms" in r]
            if not timed:
                return None
            total_ms = sum(r["cpu_mkl_ms"] for r, _ in timed)
            flops = sum(gm.flops for _, gm in timed)
            return {"value": round(flops / (total_ms * 1e-3) / 1e12, 4), "unit": "TFLOP/s", "cores": cpu_cores,
                    "kind": "port", "ms": round(total_ms, 4),
                    "gpu_ms_same_products": round(sum(r["ms"] for r, _ in timed), 4), "sample": sample}

        dense = wl.dense_layer_gemms()
        rows = [run(gm, 1, 50, 10, bias=np.zeros(gm.N, np.float32) if gm.bias else None, cpu_reps=200) for gm in dense]
        extra["config1_dense_layer"] = {
            "gemms": rows,
            "cpu_baseline": cpu_summary(rows, dense, "forward (cblas_sgemm NT + bias pass), dW (TN), dx (NN) of the "
                                        "128 x 784 -> 256 layer, each the median of 200 calls after a warm-up")}
        extra["config1_dense_layer_calls"] = dense_layer_calls(w, wl, upload)
        if cpu_on:
            # the same three products (and the bias add) back to back on the host, as a layer step runs them
            d = wl.dense_layer_inputs(seed=1)
            x, wt, dyv = d["x"], d["w_out_in"], d["dy"]
            y, dwv, dxv = (np.empty(sh, np.float32) for sh in ((x.shape[0], wt.shape[0]), wt.shape, x.shape))
            bias0 = np.zeros((1, wt.shape[0]), np.float32)

            def cpu_layer():
                dot_oracle.mkl_dot(x, False, wt, True, y)
                np.add(y, bias0, out=y)
                dot_oracle.mkl_dot(dyv, True, x, False, dwv)
                dot_oracle.mkl_dot(dyv, False, wt, False, dxv)
            for _ in range(20):
                cpu_layer()
            t0 = time.perf_counter()
            for _ in range(200):
                cpu_layer()
            cpu_layer_ms = (time.perf_counter() - t0) * 1e3 / 200
            cpu_spent[0] += time.perf_counter() - t0
            lc = extra["config1_dense_layer_calls"]
            extra["config1_dense_layer_fwd_bwd"] = {
                "gpu_ms": round(lc["forward_ms"] + lc["backward_ms"], 4),
                "gpu_forward_ms": lc["forward_ms"], "gpu_backward_ms": lc["backward_ms"],
                "gpu_three_separate_products_ms": round(sum(r["ms"] for r in rows), 4),
                "cpu_mkl_ms": round(cpu_layer_ms, 4), "cpu_cores": cpu_cores,
                "note": "forward + backward of the 128 x 784 -> 256 layer; GPU = snhip_dense_forward + "
                        "snhip_dense_backward_ex (one launch each: dx, dW and db share a grid), beside the sum of the "
                        "three products as separate launches; CPU = cblas_sgemm x 3 + bias add, 200 repetitions"}
        sweep, sweep_gemms = [], []
        for (M, N, K) in wl.SWEEP_SIZES:
            steps, warm = (5, 3) if M * N * K > 1e11 else (50, 20)
            for beta in (0.0, 1.0):
                for tA in (False, True):
                    for tB in (False, True):
                        gm = wl.Gemm(M, N, K, tA, tB, 1.0, beta)
                        # CPU side: one transpose form per size (NN, beta = 0); the 8192^3 one is the headline's
                        cpu_reps = 2 if (not tA and not tB and beta == 0.0 and (M, N, K) != (8192, 8192, 8192)) else 0
                        sweep.append(run(gm, 2, steps, warm, cpu_reps=cpu_reps))
                        sweep_gemms.append(gm)
        if cpu_on and "cpu_baseline" in out:
            for r, gm in zip(sweep, sweep_gemms):
                if (gm.M, gm.N, gm.K, gm.layout, gm.beta) == (8192, 8192, 8192, "NN", 0.0):
                    r["cpu_mkl_tflops"] = out["cpu_baseline"]["value"]
                    r["cpu_mkl_ms"] = round(gm.flops / (out["cpu_baseline"]["value"] * 1e12) * 1e3, 4)
        extra["config2_sweep"] = {
            "gemms": sweep,
            "cpu_baseline": cpu_summary(sweep, sweep_gemms, "the NN beta=0 product of each of the seven sizes through "
                                        "cblas_sgemm, median of 2 calls after a warm-up (8192^3: the headline's "
                                        "cpu_baseline); per-size figures in the rows")}
        mlp_g = wl.mlp_gemms()
        mlp = [run(gm, 3, 20, 10, bias=np.zeros(gm.N, np.float32) if gm.bias else None, cpu_reps=1) for gm in mlp_g]
        extra["config3_mlp_step"] = {"gemms": mlp, "total_ms": round(sum(r["ms"] for r in mlp), 4),
                                     "tflops": round(sum(gm.flops for gm in mlp_g) /
                                                     (sum(r["ms"] for r in mlp) * 1e-3) / 1e12, 2),
                                     "cpu_baseline": cpu_summary(mlp, mlp_g, "all nine products of the step (forward ones "
                                                                 "with the bias pass), one timed call each after a "
                                                                 "warm-up")}
        proj, rec, seq = wl.lstm_gemms()
        lstm_rows = [run(proj, 4, 20, 10, cpu_reps=2), run(rec, 4, seq, 20, cpu_reps=16)]
        cb = cpu_summary(lstm_rows, [proj, rec], "")
        if cb is not None:
            # the whole configuration: one projection + `seq` sequential recurrent products (beta = 1)
            whole_ms = lstm_rows[0]["cpu_mkl_ms"] + seq * lstm_rows[1]["cpu_mkl_ms"]
            cb.update({"value": round((proj.flops + seq * rec.flops) / (whole_ms * 1e-3) / 1e12, 4), "ms": round(whole_ms, 4),
                       "gpu_ms_same_products": round(lstm_rows[0]["ms"] + seq * lstm_rows[1]["ms"], 4),
                       "sample": "input projection: median of 2 calls; recurrent product (beta = 1): median of 16 of the "
                                 "%d sequential calls, scaled to %d" % (seq, seq)})
        extra["config4_lstm"] = {"gemms": lstm_rows, "input_projection": lstm_rows[0], "recurrent_step": lstm_rows[1],
                                 "recurrent_steps": seq, "cpu_baseline": cb}
        att_g = wl.attention_gemms()
        att = [run(gm, 5, 50, 10, cpu_reps=3) for gm in att_g]
        extra["config5_attention_fp32"] = {
            "gemms": att,
            "cpu_baseline": cpu_summary(att, att_g, "serial loop over the 512 matrices, one cblas_sgemm each "
                                        "(CpuTensor.BatchMatrixMultiplication), median of 3 passes after a warm-up")}
        # bf16-input / fp32-accumulate variant (operands stay fp32 in HBM, rounded on the way into LDS)
        w.set_math_mode(w.MATH_BF16_INPUT)
        bf16_math[0] = True
        try:
            bf = [run(gm, 5, 50, 10) for gm in att_g]
            for r, gm in zip(bf, att_g):   # HBM-bound: roofline = bytes / 8 TB/s vs bf16 MFMA peak
                r["frac_of_roofline"] = round(gm.roofline_seconds(wl.BF16_MFMA_PEAK_TFLOPS) * 1e3 / r["ms"], 4)
            extra["config5_attention_bf16_input"] = {
                "gemms": bf, "cpu_baseline": extra["config5_attention_fp32"]["cpu_baseline"],
                "note": "the reference has no reduced-precision CPU route: the CPU figure is the fp32 one"}
            # the headline size, all four forms: transposed A with plain B runs on the fp32-storage kernel, the others
            # through one rounding pass into the workspace and the bf16-storage kernel (the pass is inside the time)
            hbs = []
            for (tA, tB) in ((True, False), (False, False), (False, True), (True, True)):
                hb = run(wl.Gemm(8192, 8192, 8192, tA, tB, 1.0, 0.0), 2, 10, 5)
                hb["frac_of_roofline"] = round(hb["tflops"] / wl.BF16_MFMA_PEAK_TFLOPS, 4)
                hb["gemm"] += " (bf16-input arithmetic, fp32 storage)"
                hbs.append(hb)
            extra["config2_8192_bf16_input"] = hbs
        finally:
            w.set_math_mode(w.MATH_FP32)
            bf16_math[0] = False

        # The same arithmetic on operands STORED as bf16 (2 bytes per element in HBM; algorithmic bytes use s_in = 2).
        # Operands are converted once by the library's own pass (timed separately: it is not part of the product).
        extra["config2_8192_bf16_stored"] = [run_stored(wl.Gemm(8192, 8192, 8192, tA, tB, 1.0, 0.0), 2, 10, 5)
                                            for (tA, tB) in ((False, True), (False, False), (True, False))]
        # the NN and TN products again with their operands brought into the k-contiguous (NT) form by the transposing
        # conversion: what a caller that converts an operand once and multiplies it many times would do
        extra["config2_8192_bf16_stored"] += [run_stored(wl.Gemm(8192, 8192, 8192, tA, tB, 1.0, 0.0), 2, 10, 5, to_nt=True)
                                             for (tA, tB) in ((False, False), (True, False))]
        extra["config5_attention_bf16_stored"] = {"gemms": [run_stored(gm, 5, 50, 10) for gm in att_g],
                                                  "cpu_baseline": extra["config5_attention_fp32"]["cpu_baseline"],
                                                  "note": "CPU figure: the fp32 route (the reference has no other)"}
        if cpu_on:
            extra["cpu_leg_seconds"] = round(cpu_spent[0], 1)
            log("[bench] CPU side of the other configurations took %.1f s" % cpu_spent[0])
        extra["layers_fused_vs_reference_sequence"] = layer_timings(w, wl)
        for k, v in extra.items():
            log("[bench]", k, json.dumps(v, allow_nan=False))
        out["summary"] = summarize(extra)
        full = dict(out)
        full["extra"] = extra
        try:
            d = os.path.dirname(args.extra_out)
            if d:
                os.makedirs(d, exist_ok=True)
            with open(args.extra_out, "w") as f:
                json.dump(full, f, allow_nan=False, indent=1)
            out["summary"]["per_product_figures"] = args.extra_out
        except OSError as e:
            log("[bench] could not write %s: %s" % (args.extra_out, e))
        if args.table:
            write_table(args.table, full)

    print(headline_line(out), flush=True)


def summarize(extra):
    """A few figures of the other configurations for the stdout line (the rest is in the extra file)."""
    def best(rows, key="tflops"):
        return max(r[key] for r in rows)

    def pick(rows, label):
        for r in rows:
            if r["gemm"].startswith(label) or label in r["gemm"]:
                return r
        return None
    s = {}
    fb = extra.get("config1_dense_layer_fwd_bwd")
    if fb:
        s["config1_dense_fwd_bwd_ms"] = {"gpu": fb["gpu_ms"], "gpu_forward": fb["gpu_forward_ms"],
                                         "gpu_backward": fb["gpu_backward_ms"],
                                         "gpu_three_separate_products": fb["gpu_three_separate_products_ms"],
                                         "cpu_mkl": fb["cpu_mkl_ms"], "cpu_cores": fb["cpu_cores"]}
    else:
        lc = extra["config1_dense_layer_calls"]
        s["config1_dense_fwd_bwd_ms"] = {"gpu": round(lc["forward_ms"] + lc["backward_ms"], 4),
                                         "gpu_forward": lc["forward_ms"], "gpu_backward": lc["backward_ms"]}
    sw = extra["config2_sweep"]["gemms"]
    fr = {}
    for r in sw:
        size = r["gemm"].split(")")[0] + ")"
        fr.setdefault(size, []).append(r["frac_of_roofline"])
    s["config2_frac_of_roofline_min_max"] = {k: [min(v), max(v)] for k, v in fr.items()}
    s["config3_mlp_step"] = {"ms": extra["config3_mlp_step"]["total_ms"], "tflops": extra["config3_mlp_step"]["tflops"]}
    s["config4_lstm"] = {"input_projection_frac": extra["config4_lstm"]["input_projection"]["frac_of_roofline"],
                         "recurrent_step_ms": extra["config4_lstm"]["recurrent_step"]["ms"]}
    s["config5_attention_ms"] = {"fp32": [r["ms"] for r in extra["config5_attention_fp32"]["gemms"]],
                                 "bf16_input": [r["ms"] for r in extra["config5_attention_bf16_input"]["gemms"]],
                                 "bf16_stored": [r["ms"] for r in extra["config5_attention_bf16_stored"]["gemms"]]}
    def form(r):
        return r["gemm"].split(")")[1].split()[0]      # "(M,N,K) NT beta=0 ..." -> "NT"
    # fp32 operands rounded on the way (all four forms) and operands stored as bf16 (the first three rows: the operands
    # as the caller laid them out; the rows after them repeat NN / TN with the caller transposing while converting)
    s["bf16_8192_tflops"] = {"input": {form(r): r["tflops"] for r in extra["config2_8192_bf16_input"]},
                             "stored": {form(r): r["tflops"] for r in extra["config2_8192_bf16_stored"][:3]}}
    rows = 0
    for v in extra.values():
        items = v if isinstance(v, list) else (v.get("gemms") or [v]) if isinstance(v, dict) else []
        rows += sum(1 for r in items if isinstance(r, dict) and "max_abs_err" in r)
    s["timed_products_checked_against_oracle"] = rows
    return s


def dense_layer_calls(w, wl, upload, timed_calls=1000):
    """The 128 x 784 -> 256 layer of configuration 1 as the two library calls a Linear layer makes per step
    (Linear.cs:125-132 and :143-191): snhip_dense_forward (bias + ReLU in the write-out) and snhip_dense_backward_ex
    (dx, dW + decay * W and db + decay * bias).  Called straight through the C ABI, HIP events around `timed_calls`
    calls issued back to back (dependent launches: each reads what the one before wrote), and every output of the
    timed calls compared with the float64 result."""
    from sharpnet_amd import GPUTensor
    from sharpnet_amd.hiplib import check_status
    d = wl.dense_layer_inputs(seed=1)
    xs, ws, dys = d["x"], d["w_out_in"], d["dy"]
    bs = np.random.default_rng(11).uniform(-0.1, 0.1, ws.shape[0]).astype(np.float32)  # the workload's bias is all zeros
    rows, fin = xs.shape
    fout = ws.shape[0]
    decay = 0.0128
    x, W, b, dy = upload(xs), upload(ws), upload(bs), upload(dys)
    y, dx, dW, db = (GPUTensor(sh, None, w) for sh in ([rows, fout], [rows, fin], [fout, fin], [fout]))
    calls = (("forward", lambda: w.lib.snhip_dense_forward(w.handle, y.Pointer, x.Pointer, W.Pointer, b.Pointer,
                                                           rows, fin, fout, 1, 0.0)),
             ("backward", lambda: w.lib.snhip_dense_backward_ex(w.handle, dx.Pointer, dW.Pointer, db.Pointer, x.Pointer,
                                                                dy.Pointer, W.Pointer, rows, fin, fout, 1.0, decay,
                                                                b.Pointer, decay)))
    res = []
    for name, call in calls:
        for _ in range(500):
            check_status(call())
        e0, e1 = w.new_event(), w.new_event()
        w.synchronize()
        w.record(e0)
        for _ in range(timed_calls):
            check_status(call())
        w.record(e1)
        w.synchronize()
        res.append({"call": "Dense 128x784->256 " + name, "calls": 500 + timed_calls,
                    "event_us_per_call": round(w.elapsed_ms(e0, e1) * 1e3 / timed_calls, 3)})
        w.destroy_event(e0)
        w.destroy_event(e1)
    x64, w64, b64, dy64 = (a.astype(np.float64) for a in (xs, ws, bs, dys))
    want = {"y": np.maximum(x64 @ w64.T + b64, 0.0), "dx": dy64 @ w64, "dW": dy64.T @ x64 + decay * w64,
            "db": dy64.sum(axis=0) + decay * b64}
    got = {"y": y.ToNumpy(), "dx": dx.ToNumpy(), "dW": dW.ToNumpy(), "db": db.ToNumpy()}
    scale = {"y": np.sqrt(fin), "dx": np.sqrt(fout), "dW": np.sqrt(rows), "db": np.sqrt(rows)}
    parity = {}
    for k in want:
        err = float(np.max(np.abs(got[k].reshape(want[k].shape) - want[k])))
        bound = 1e-4 * float(scale[k]) * max(1.0, float(np.max(np.abs(want[k]))))
        parity[k] = {"max_abs_err": err, "bound": bound}
        if not err <= bound:
            raise RuntimeError("dense layer %s: max|d| = %.3e beyond %.3e" % (k, err, bound))
    for t in (x, W, b, dy, y, dx, dW, db):
        t.Dispose()
    return {"calls": res, "parity": parity,
            "forward_ms": round(res[0]["event_us_per_call"] * 1e-3, 5), "backward_ms": round(res[1]["event_us_per_call"] * 1e-3, 5)}


def layer_timings(w, wl):
    """Linear and multi-head-attention layers as whole calls of the host mirrors: the library's fused forms against
    the reference's own sequence of calls, both on the device, HIP events around `steps` repetitions (host launch
    time included: for the small layer that is most of it)."""
    from sharpnet_amd import GPUTensor, linear, attention
    rng = np.random.default_rng(7)
    w.use_memory_pool(True)

    def T(shape, lo=-1.0, hi=1.0):
        return GPUTensor(list(shape), rng.uniform(lo, hi, shape).astype(np.float32), w)

    def timed(fn, steps, warm):
        t0 = time.perf_counter()
        n = 0
        while n < warm or time.perf_counter() - t0 < 0.06:   # clocks take tens of ms to come up after an idle spell
            fn()
            n += 1
        e0, e1 = w.new_event(), w.new_event()
        groups = []
        for _ in range(3):   # the median of three groups: one moment of the host elsewhere does not count
            w.synchronize()
            w.record(e0)
            for _ in range(steps):
                fn()
            w.record(e1)
            groups.append(w.elapsed_ms(e0, e1) / steps)
        ms = float(np.median(groups))
        w.destroy_event(e0)
        w.destroy_event(e1)
        return round(ms, 4)

    res = []
    for (rows, fin, fout, steps) in ((128, 784, 256, 200), (4096, 4096, 4096, 10)):
        x, W, b, dy = T((rows, fin)), T((fout, fin), -0.05, 0.05), T((fout,)), T((rows, fout))
        y, dx, dW, db = (GPUTensor(sh, None, w) for sh in ([rows, fout], [rows, fin], [fout, fin], [fout]))
        for fused in (True, False):
            f = timed(lambda: linear.DenseForwardPropagation(y, x, W, b, False, fused=fused,
                                                             activation="CUDNN_ACTIVATION_RELU"), steps, steps // 2)
            bwd = timed(lambda: linear.DenseBackwardPropagation(dx, dW, db, x, dy, W, bias_1D=b, compatibility_mode="PyTorch",
                                                                use_weight_decay_in_backpropagation=True, weight_decay=1e-4,
                                                                fused=fused), steps, steps // 2)
            res.append({"layer": "Linear %dx%d->%d: forward with bias + ReLU; backward with bias gradient + weight decay"
                                 % (rows, fin, fout), "form": "fused" if fused else "reference sequence",
                        "forward_ms": f, "backward_ms": bwd})
        for t in (x, W, b, dy, y, dx, dW, db):
            t.Dispose()
    # scaled-dot-product attention of benchmark configuration 5: 512 x (256 x 64), fp32
    Z, Tn, d = 512, 256, 64
    q, k, v = T((Z, Tn, d)), T((Z, Tn, d)), T((Z, Tn, d))
    o = GPUTensor([Z, Tn, d], None, w)
    for fused in (True, False):
        for causal in (False, True):
            def sdpa():
                wts = attention.ScaledDotProductAttentionForwardPropagation(q, k, v, o, True, True, causal, fused=fused)
                wts.Dispose()
            ms = timed(sdpa, 20, 10)
            res.append({"layer": "ScaledDotProductAttention forward 512 x (256 x 64)%s, weights kept" %
                                 (", causal" if causal else ""),
                        "form": "one launch" if fused else "reference sequence (4 calls)", "forward_ms": ms,
                        "backward_ms": None})
    # the same launch on a handle in the bf16-input math mode (Q, K, V and the probabilities rounded to bf16 for the MFMAs)
    w.set_math_mode(1)
    try:
        for training in (True, False):
            def sdpa_bf16():
                wts = attention.ScaledDotProductAttentionForwardPropagation(q, k, v, o, training, True, False, fused=True)
                if wts is not None:
                    wts.Dispose()
            ms = timed(sdpa_bf16, 20, 10)
            res.append({"layer": "ScaledDotProductAttention forward 512 x (256 x 64), bf16-input math, weights %s" %
                                 ("kept" if training else "not kept"),
                        "form": "one launch", "forward_ms": ms, "backward_ms": None})
    finally:
        w.set_math_mode(0)
    dq, dk_, dv_, do = (GPUTensor([Z, Tn, d], None, w) for _ in range(4))
    do.SetValue(0.01)
    for fused in (True, False):
        def sdpa_fb():
            wts = attention.ScaledDotProductAttentionForwardPropagation(q, k, v, o, True, True, True, fused=fused)
            attention.ScaledDotProductAttentionBackwardPropagation(dq, dk_, dv_, q, k, v, do, wts, True, fused=fused,
                                                                   is_causal=True)

        def sdpa_f():
            attention.ScaledDotProductAttentionForwardPropagation(q, k, v, o, True, True, True, fused=fused).Dispose()
        f = timed(sdpa_f, 20, 10)
        fb = timed(sdpa_fb, 20, 10)
        res.append({"layer": "ScaledDotProductAttention forward + backward 512 x (256 x 64), causal",
                    "form": "one launch forward, three backward" if fused else "reference sequence (4 + 5 calls)",
                    "forward_ms": f, "backward_ms": round(fb - f, 4)})
        if fused:
            w.set_math_mode(1)
            try:
                f = timed(sdpa_f, 20, 10)
                fb = timed(sdpa_fb, 20, 10)
            finally:
                w.set_math_mode(0)
            res.append({"layer": "ScaledDotProductAttention forward + backward 512 x (256 x 64), causal, bf16-input math",
                        "form": "one launch forward, three backward", "forward_ms": f, "backward_ms": round(fb - f, 4)})
    for t in (q, k, v, o, dq, dk_, dv_, do):
        t.Dispose()
    # more than 256 keys: 64 matrices of 1024 x 1024, head dimension 64 (key blocks of 256; two passes when the weights
    # are kept, one with a running maximum when they are not)
    Z, Tn, d = 64, 1024, 64
    q, k, v = T((Z, Tn, d)), T((Z, Tn, d)), T((Z, Tn, d))
    o = GPUTensor([Z, Tn, d], None, w)
    for training in (True, False):
        for fused in (True, False):
            for causal in (False, True):
                def sdpa_long():
                    wts = attention.ScaledDotProductAttentionForwardPropagation(q, k, v, o, training, True, causal, fused=fused)
                    if wts is not None:
                        wts.Dispose()
                ms = timed(sdpa_long, 10, 5)
                res.append({"layer": "ScaledDotProductAttention forward 64 x (1024 x 64)%s, weights %s" %
                                     (", causal" if causal else "", "kept" if training else "not kept"),
                            "form": "one launch" if fused else "reference sequence (4 calls)", "forward_ms": ms,
                            "backward_ms": None})
    dq, dk_, dv_, do = (GPUTensor([Z, Tn, d], None, w) for _ in range(4))
    do.SetValue(0.01)
    for fused in (True, False):
        def long_fb():
            wts = attention.ScaledDotProductAttentionForwardPropagation(q, k, v, o, True, True, True, fused=fused)
            attention.ScaledDotProductAttentionBackwardPropagation(dq, dk_, dv_, q, k, v, do, wts, True, fused=fused,
                                                                   is_causal=True)

        def long_f():
            attention.ScaledDotProductAttentionForwardPropagation(q, k, v, o, True, True, True, fused=fused).Dispose()
        f = timed(long_f, 10, 5)
        fb = timed(long_fb, 10, 5)
        res.append({"layer": "ScaledDotProductAttention forward + backward 64 x (1024 x 64), causal",
                    "form": "one launch forward, three backward" if fused else "reference sequence (4 + 5 calls)",
                    "forward_ms": f, "backward_ms": round(fb - f, 4)})
    for t in (q, k, v, o, dq, dk_, dv_, do):
        t.Dispose()
    B, Tn, H, d = 64, 256, 8, 64
    E = H * d
    Q, K, V, dy = T((B, Tn, E)), T((B, Tn, E)), T((B, Tn, E)), T((B, Tn, E))
    wq, wk, wv, wo = (T((E, E), -0.05, 0.05) for _ in range(4))
    y, dQ, dK, dV = (GPUTensor([B, Tn, E], None, w) for _ in range(4))
    grads = {k: (GPUTensor([E, E], None, w), None) for k in ("w_Q", "w_K", "w_V", "out_proj_weight")}
    for in_place, fused_attn in ((True, True), (True, False), (False, False)):
        state = {}

        def fwd():
            if state.get("st") is not None:      # a forward without its backward: give the kept buffers back
                for t in (state["st"].weights_buffer, state["st"].Q_heads, state["st"].K_heads, state["st"].V_heads,
                          state["st"].attention_heads_T):
                    t.Dispose()
            state["st"] = attention.MultiheadAttentionForwardPropagation(Q, K, V, y, wq, wk, wv, wo, H, d, d, is_causal=True,
                                                                         heads_in_place=in_place, fused_attention=fused_attn)

        def fwd_bwd():
            fwd()
            st = state["st"]
            attention.MultiheadAttentionBackwardPropagation(dQ, dK, dV, Q, K, V, dy, st, wq, wk, wv, wo, grads,
                                                            fused_attention=fused_attn)
            for t in (st.weights_buffer, st.Q_heads, st.K_heads, st.V_heads, st.attention_heads_T):
                t.Dispose()
            state["st"] = None

        f = timed(fwd, 10, 5)
        fb = timed(fwd_bwd, 10, 5)
        res.append({"layer": "MultiheadAttention batch %d, %d steps, %d heads x %d, causal" % (B, Tn, H, d),
                    "form": ("heads in place, attention kernels" if fused_attn else "heads in place") if in_place
                    else "reference sequence (transposition copies)",
                    "forward_ms": f, "backward_ms": round(fb - f, 4)})
    for t in (Q, K, V, dy, wq, wk, wv, wo, y, dQ, dK, dV) + tuple(g[0] for g in grads.values()):
        t.Dispose()
    # recurrent layers at the shape of benchmark configuration 4: batch 256, 128 steps, 256 inputs, 512 hidden units
    from sharpnet_amd import recurrent
    B, Tn, I, H = 256, 128, 256, 512
    x, dyr = T((B, Tn, I)), T((B, Tn, H), -0.01, 0.01)
    yr, dxr = GPUTensor([B, Tn, H], None, w), GPUTensor([B, Tn, I], None, w)
    for name, cell, bias, bidir in (("LSTM", recurrent.CUDNN_LSTM, recurrent.CUDNN_RNN_SINGLE_INP_BIAS, False),
                                    ("GRU", recurrent.CUDNN_GRU, recurrent.CUDNN_RNN_DOUBLE_BIAS, False),
                                    ("bidirectional LSTM", recurrent.CUDNN_LSTM, recurrent.CUDNN_RNN_SINGLE_INP_BIAS, True)):
        K = 2 if bidir else 1
        layer = recurrent.RecurrentLayer(w, I, H, cell, bias, True, bidir, 1)
        layer._weightsAndBiases.InitializeFromHostMemory(
            rng.uniform(-0.04, 0.04, layer._weightsAndBiases.Count).astype(np.float32))
        yk = yr if not bidir else GPUTensor([B, Tn, K * H], None, w)
        dyk = dyr if not bidir else T((B, Tn, K * H), -0.01, 0.01)

        def rnn_f():
            layer.ForwardPropagation(x, yk, True)
            layer._reserveSpace.Dispose()

        def rnn_fb():
            layer.ForwardPropagation(x, yk, True)
            layer.BackwardPropagation(x, yk, dyk, dxr)
        gates = 3 if name == "GRU" else 4
        flop = 2.0 * K * B * Tn * gates * H * (I + H)
        for form, mode in (("one launch per step (product with R + cell arithmetic)", 0),
                           ("GEMM + cell kernel per step (+ split-K reduction on the way back)", 1)):
            w.lib.snhip_rnn_set_step_mode(w.handle, mode)
            f = timed(rnn_f, 3, 1)
            fb = timed(rnn_fb, 3, 1)
            w.lib.snhip_rnn_set_step_mode(w.handle, 0)
            res.append({"layer": "%s batch %d, %d steps, %d -> %d (forward %.1f GFLOP: %d sequential steps of %dx%dx%d%s)" %
                                 (name, B, Tn, I, H, flop / 1e9, Tn, B, gates * H, H, " per direction" if bidir else ""),
                        "form": form, "forward_ms": f, "backward_ms": round(fb - f, 4)})
        layer.Dispose()
        if bidir:
            yk.Dispose()
            dyk.Dispose()
    for t in (x, dyr, yr, dxr):
        t.Dispose()
    w.use_memory_pool(False)
    return res


def write_table(path, out):
    """Markdown rendering of the `extra` object (one row per GEMM) plus the headline figures of the same run."""
    rows = []
    layers = out["extra"].get("layers_fused_vs_reference_sequence", [])
    for name, v in out["extra"].items():
        if name in ("layers_fused_vs_reference_sequence", "config1_dense_layer_fwd_bwd", "config1_dense_layer_calls") or not isinstance(v, (list, dict)):
            continue
        items = v if isinstance(v, list) else v.get("gemms") or [v]
        for r in items:
            rows.append("| %s | %s | %.4f | %.1f | %.3f | %d | %d | %s | %s |" % (
                name, r["gemm"], r["ms"], r["tflops"], r["frac_of_roofline"], r["tile_config"], r["splitk"],
                "%.4f" % r["cpu_mkl_ms"] if "cpu_mkl_ms" in r else "", "%.3f" % r["cpu_mkl_tflops"] if "cpu_mkl_ms" in r else ""))
        if isinstance(v, dict) and "total_ms" in v:
            rows.append("| %s | all nine GEMMs | %.4f | %.1f | | | | | |" % (name, v["total_ms"], v["tflops"]))
        cb = v.get("cpu_baseline") if isinstance(v, dict) else None
        if cb:
            rows.append("| %s | CPU baseline of the configuration: %s | %.4f (GPU, same products) | | | | | %.4f | %.3f |" % (
                name, cb["sample"], cb["gpu_ms_same_products"], cb["ms"], cb["value"]))
    cpu = out.get("cpu_baseline")
    with open(path, "w") as f:
        f.write("# Per-configuration GPU figures (MI355X, one GPU, fp32 unless noted)\n\n"
                "Command: `python bench.py --table %s` (the table is the `extra` object of its JSON line). time = HIP events\n"
                "around the timed launches; fraction = max(flops / 157.3 TFLOP/s, bytes / 8 TB/s) / time (bf16-input rows:\n"
                "against the 2.5 PFLOP/s bf16 peak or 8 TB/s); tile config = index into `snhip_config_desc`.\n\n"
                "CPU columns: the same product through MKL cblas_sgemm on the box's host cores (%s threads), the reference's CPU route;\n"
                "batched products as the reference's serial loop over the matrices.\n\n"
                "| configuration | GEMM | ms | TFLOP/s | fraction of roofline | tile config | split-K | CPU (MKL) ms | CPU TFLOP/s |\n"
                "|---|---|---|---|---|---|---|---|---|\n" % (path, cpu["cores"] if cpu else "no"))
        f.write("\n".join(rows) + "\n\n")
        fb = out["extra"].get("config1_dense_layer_fwd_bwd")
        if fb:
            f.write("Dense layer forward + backward (configuration 1): %.4f ms on the GPU (forward call %.4f + backward call "
                    "%.4f, one launch each; the three products as separate launches: %.4f) against %.4f ms through MKL on "
                    "%d host threads.\n\n" % (fb["gpu_ms"], fb["gpu_forward_ms"], fb["gpu_backward_ms"],
                                              fb["gpu_three_separate_products_ms"], fb["cpu_mkl_ms"], fb["cpu_cores"]))
        if layers:
            f.write("Whole layer calls through the host mirrors (HIP events around repeated calls, host launch time included):\n\n"
                    "| layer | form | forward ms | backward ms |\n|---|---|---|---|\n")
            for r in layers:
                f.write("| %s | %s | %.4f | %s |\n" % (r["layer"], r["form"], r["forward_ms"],
                                                         "" if r["backward_ms"] is None else "%.4f" % r["backward_ms"]))
            f.write("\n")
        f.write("Headline line of the same run: %.2f TFLOP/s (%.1f %% of fp32 MFMA peak)" %
                (out["value"], 100.0 * out["roofline"]["frac"]))
        if cpu:
            f.write(", CPU baseline (%d threads): %.2f TFLOP/s" % (cpu["cores"], cpu["value"]))
        f.write(".\n")


if __name__ == "__main__":
    main()
