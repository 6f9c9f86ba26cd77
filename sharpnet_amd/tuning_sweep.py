"""Measure every fp32 tile configuration on a list of shapes and compare the host's automatic choice with the fastest.

    python -m sharpnet_amd.tuning_sweep                      # the built-in shape list, NN form
    python -m sharpnet_amd.tuning_sweep --form TT --json out.json 1024x1024x1024 4097x3001x2049
    python -m sharpnet_amd.tuning_sweep --batch 16 128x128x512 256x256x64     # strided batches of 16 matrices

For each shape (M x N x K; single products through Tensor.Dot, or strided batches through BatchMatrixMultiplication, which
also adds the streaming kernels to the candidates) every tiled fp32 configuration is forced through
snhip_set_tuning with K split 1, 2 and 4 ways (8, 16 and 32 ways too where 64 x 64 tiles would leave the chip mostly idle),
plus the kernels that split K inside the workgroup, and timed on the wall clock over enough launches to hide the host
(the minimum of two runs).  Printed per shape: what the library picks by itself, its time, the fastest
candidate and how far behind the pick is.  The efficiencies and fixed costs of the host's cost model
(estimate_cycles in csrc/sharpnet_hip.hip) are a fit to the JSON this writes.
"""
import argparse
import json
import sys
import time

import numpy as np

DEFAULT_SHAPES = [
    (1024, 1024, 1024), (1000, 1000, 1000), (2048, 2048, 2048), (1536, 1536, 1536), (1280, 1280, 1280), (2560, 2560, 2560),
    (3072, 3072, 3072), (4097, 3001, 2049), (1024, 1024, 4096), (512, 512, 4096), (2048, 2048, 512), (1024, 2048, 1024),
    (768, 768, 768), (4096, 4096, 512), (2048, 512, 2048), (1536, 1024, 1024), (4096, 1024, 1024), (1792, 1792, 1792),
    (1920, 1080, 720), (3000, 2000, 1000), (640, 640, 640), (896, 896, 896), (2304, 2304, 768), (5120, 1280, 1280),
    (4096, 4096, 4096), (8192, 64, 8192), (32768, 2048, 256), (3584, 3584, 3584), (1152, 1152, 2304), (6144, 2048, 1024),
    (256, 256, 8192), (128, 128, 16384), (512, 256, 4096), (384, 384, 3000), (1000, 200, 5000), (300, 300, 300),
    (2000, 2000, 200), (16384, 32, 4096), (8192, 16, 8192), (32, 8192, 2048)]


def main(argv=None):
    ap = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    ap.add_argument("shapes", nargs="*", help="MxNxK, e.g. 1024x1024x1024 (default: a built-in list)")
    ap.add_argument("--form", default="NN", choices=["NN", "NT", "TN", "TT"], help="transposes of A and B")
    ap.add_argument("--batch", type=int, default=1, help="matrices per strided batch (default: single products)")
    ap.add_argument("--json", default=None, metavar="PATH", help="write every measured time to this file")
    args = ap.parse_args(argv)
    from sharpnet_amd import GPUWrapper, GPUTensor
    w = GPUWrapper.FromDeviceId(0)
    rng = np.random.default_rng(0)
    tA, tB = args.form[0] == "T", args.form[1] == "T"
    shapes = [tuple(int(x) for x in s.lower().split("x")) for s in args.shapes] or DEFAULT_SHAPES
    cfgs = w.configs()
    tiled = [c for c in cfgs if c["kind"] == "fp32"]
    inside = [c["id"] for c in cfgs if c["kind"] == "fp32-ksplit"]
    if args.batch > 1:
        inside += [c["id"] for c in cfgs if c["kind"] == "fp32-stream"]
    lead = [args.batch] if args.batch > 1 else []

    def timeit(launch, n):
        for _ in range(max(5, n // 4)):
            launch()
        w.synchronize()
        t0 = time.perf_counter()
        for _ in range(n):
            launch()
        w.synchronize()
        return (time.perf_counter() - t0) / n

    everything, regrets = {}, []
    try:
        for (M, N, K) in shapes:
            a = rng.uniform(-1, 1, lead + ([K, M] if tA else [M, K])).astype(np.float32)
            b = rng.uniform(-1, 1, lead + ([N, K] if tB else [K, N])).astype(np.float32)
            ga, gb = GPUTensor(list(a.shape), a, w), GPUTensor(list(b.shape), b, w)
            gc = GPUTensor(lead + [M, N], None, w)

            def launch():
                if args.batch > 1:
                    gc.BatchMatrixMultiplication(ga, tA, gb, tB, 1.0, 0.0)
                else:
                    gc.Dot(ga, tA, gb, tB, 1.0, 0.0)
            w.set_tuning(-1, 0)
            launch()
            auto = w.last_tuning()
            cands = []
            for c in tiled:
                tiles = -(-M // c["BM"]) * -(-N // c["BN"]) * args.batch
                for s in (1, 2, 4, 8, 16, 32):
                    if s > 4 and -(-M // 64) * -(-N // 64) * s * args.batch > 2048:
                        continue
                    if s > 1 and K // s < 4 * c["BK"]:
                        continue
                    if tiles * s < 100 and (c["id"], s) != auto:
                        continue                      # would leave most of the chip idle
                    cands.append((c["id"], s))
            cands += [(i, 1) for i in inside]
            if auto not in cands:
                cands.append(auto)
            res = {}
            for cand in cands:
                try:
                    w.set_tuning(*cand)
                    launch()
                except Exception:
                    continue                          # a kernel that does not take this shape (alignment)
                if w.last_tuning() != cand:
                    continue
                t = timeit(launch, 20)
                if t < 3 * min(res.values(), default=1e9) or cand == auto:
                    n = max(30, min(300, int(8e-3 / t)))
                    t = min(t, timeit(launch, n), timeit(launch, n))
                res[cand] = t
            w.set_tuning(-1, 0)
            best = min(res, key=res.get)
            regret = res[auto] / res[best] - 1.0
            regrets.append(regret)
            top = sorted(res, key=res.get)[:4]
            print("%6d %6d %6d %s  picked %-9s %8.1f us   fastest %-9s %8.1f us   behind %5.1f %%   %s" % (
                M, N, K, args.form, auto, res[auto] * 1e6, best, res[best] * 1e6, regret * 100,
                " ".join("%s:%.1f" % (c, res[c] * 1e6) for c in top)), flush=True)
            everything["%d,%d,%d" % (M, N, K)] = {"picked": list(auto), "seconds": {"%d,%d" % c: v for c, v in res.items()}}
            for t in (ga, gb, gc):
                t.Dispose()
    finally:
        w.set_tuning(-1, 0)
    print("behind the fastest candidate: %.2f %% on average, %.1f %% at worst (%d shapes)" % (
        100 * sum(regrets) / len(regrets), 100 * max(regrets), len(regrets)))
    if args.json:
        with open(args.json, "w") as f:
            json.dump({"form": args.form, "batch": args.batch, "shapes": everything}, f, indent=1)
    return 0


if __name__ == "__main__":
    sys.exit(main())
