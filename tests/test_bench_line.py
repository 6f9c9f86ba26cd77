"""The stdout line of bench.py: short, strict JSON, with the fields a harness reads (no GPU needed)."""
import json
import os
import sys

import pytest

sys.path.insert(0, os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
import bench  # noqa: E402


def _refuse(token):
    raise AssertionError("non-JSON constant %r" % token)


def _fake_gemm_row(label, frac):
    return {"gemm": label, "ms": 1.2345, "tflops": 123.45, "frac_of_roofline": frac, "tile_config": 0, "splitk": 1,
            "max_abs_err": 1.0e-4, "parity_bound": 9.0e-3, "cpu_mkl_ms": 500.0, "cpu_mkl_tflops": 2.1}


def _fake_extra():
    sizes = [(1024, 1024, 1024), (2048, 2048, 2048), (4096, 4096, 4096), (8192, 8192, 8192), (1000, 1000, 1000),
             (4097, 3001, 2049), (8192, 64, 8192)]
    sweep = [_fake_gemm_row("(%d,%d,%d) %s beta=%g" % (m, n, k, lay, beta), 0.5 + 0.01 * i)
             for i, (m, n, k) in enumerate(sizes) for lay in ("NN", "NT", "TN", "TT") for beta in (0.0, 1.0)]
    att = [_fake_gemm_row("S=QKt/8 512x(256,256,64) NT beta=0", 0.6), _fake_gemm_row("O=PV 512x(256,64,256) NN beta=0", 0.6)]
    layers = [{"layer": "Linear 128x784->256: forward with bias + ReLU; backward with bias gradient + weight decay",
               "form": "fused", "forward_ms": 0.0059, "backward_ms": 0.0141},
              {"layer": "ScaledDotProductAttention forward 512 x (256 x 64), weights kept", "form": "one launch",
               "forward_ms": 0.085, "backward_ms": None}]
    return {
        "config1_dense_layer": {"gemms": [_fake_gemm_row("fwd y=x.Wt+b (128,256,784) NT beta=0", 0.06)] * 3, "cpu_baseline": None},
        "config1_dense_layer_calls": {"calls": [], "parity": {}, "forward_ms": 0.0049, "backward_ms": 0.0067},
        "config1_dense_layer_fwd_bwd": {"gpu_ms": 0.0116, "gpu_forward_ms": 0.0049, "gpu_backward_ms": 0.0067,
                                        "gpu_three_separate_products_ms": 0.0154, "cpu_mkl_ms": 0.2, "cpu_cores": 16,
                                        "note": "x" * 300},
        "config2_sweep": {"gemms": sweep, "cpu_baseline": None},
        "config3_mlp_step": {"gemms": [_fake_gemm_row("fwd0 (4096,4096,3072) NT beta=0", 0.9)] * 9, "total_ms": 5.9,
                             "tflops": 139.0, "cpu_baseline": None},
        "config4_lstm": {"gemms": [], "input_projection": _fake_gemm_row("input proj (32768,2048,256) NN beta=0", 0.76),
                         "recurrent_step": _fake_gemm_row("recurrent step (256,2048,512) NN beta=1", 0.3),
                         "recurrent_steps": 128, "cpu_baseline": None},
        "config5_attention_fp32": {"gemms": att, "cpu_baseline": None},
        "config5_attention_bf16_input": {"gemms": att, "cpu_baseline": None},
        "config5_attention_bf16_stored": {"gemms": att, "cpu_baseline": None},
        "config2_8192_bf16_input": [_fake_gemm_row("(8192,8192,8192) TN beta=0", 0.37)] * 4,
        "config2_8192_bf16_stored": [_fake_gemm_row("(8192,8192,8192) NT beta=0 (bf16 storage)", 0.46)] * 5,
        "layers_fused_vs_reference_sequence": layers,
    }


def _fake_out():
    return {
        "metric": "fp32 GEMM throughput, Tensor.Dot M=N=K=8192 (GEMM TFLOP/s + % of fp32 MFMA peak at 1 GPU)",
        "value": 148.03, "unit": "TFLOP/s", "n_gpus": 1, "steps": 20, "warmup": 5, "ms_per_step": 7.4276,
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "f32", "data": "synthetic",
        "config": {"workload": "configs[1] sweep, headline size: Tensor.Dot fp32 row-major NN, M=N=K=8192, alpha=1, "
                               "beta=0, A,B~U(-1,1) seed 2, operands resident in HBM",
                   "M": 8192, "N": 8192, "K": 8192, "tile_config": 0, "splitk": 1,
                   "device": {"cu": 256, "clock_mhz": 2400.0}},
        "roofline": {"bound": "mfma", "achieved": 149.3, "peak": 157.3, "unit": "TFLOP/s", "frac": 0.9491,
                     "traffic": 3767566749, "traffic_source": bench.traffic_record(bench.ROOT)[1],
                     "flops_per_launch": 2.0 * 8192 ** 3, "ms_per_launch_hip_events": 7.3641,
                     "kernel": "sgemm_mfma_kernel<TileCfg<4,4,2,2,16>, NN> (256x256x16 tiles)"},
        "parity": {"max_abs_err": 1.1e-4, "bound": 9.05e-3, "rows_checked": 16, "max_abs_err_vs_mkl_full_result": 2.0e-4},
        "cpu_baseline": {"value": 1.6, "unit": "TFLOP/s", "cores": 16, "kind": "port",
                         "sample": "3 timed + 1 warm-up calls of the full headline GEMM (8192^3) through "
                                   "libmkl_rt.so cblas_sgemm, median 0.70 s per call; os.cpu_count()=224"},
    }


def test_line_is_short_strict_json_with_the_required_fields():
    out = _fake_out()
    out["summary"] = bench.summarize(_fake_extra())
    out["summary"]["per_product_figures"] = "gpurun_out/bench_extra.json"
    line = bench.headline_line(out)
    assert "\n" not in line and len(line) < 4000
    back = json.loads(line, parse_constant=_refuse)
    for key in ("metric", "value", "unit", "n_gpus", "steps", "warmup", "ms_per_step", "higher_is_better", "scaling",
                "vs_baseline", "dtype", "data", "config", "roofline", "cpu_baseline", "parity"):
        assert key in back
    for key in ("bound", "achieved", "peak", "unit", "frac", "traffic"):
        assert key in back["roofline"]
    for key in ("value", "unit", "cores", "kind", "sample"):
        assert key in back["cpu_baseline"]
    assert "workload" in back["config"] and "model" not in back["config"]
    assert back["summary"]["timed_products_checked_against_oracle"] > 60


def test_line_refuses_nan_and_oversize():
    out = _fake_out()
    out["value"] = float("nan")
    with pytest.raises(ValueError):
        bench.headline_line(out)
    out = _fake_out()
    out["extra"] = _fake_extra()      # the per-product rows do not belong on the line
    with pytest.raises(ValueError):
        bench.headline_line(out)


def test_traffic_record_names_its_kernel_source():
    traffic, src = bench.traffic_record(bench.ROOT)
    assert traffic is None or traffic > 0
    if src is not None:
        assert isinstance(src["stale"], bool)
        if not src["stale"]:
            assert src["kernel_source_sha256_16"] == bench.source_hash(
                os.path.join(bench.ROOT, "sharpnet_amd", "csrc", "sgemm_mfma.hpp"))


def test_tuning_sweep_covers_the_benchmark_shapes_and_parses_its_arguments():
    """The sweep behind the host's cost model: its built-in list holds every fp32 shape of the benchmark's sweep
    configuration and the LSTM input projection, and the command line is understood without touching a GPU."""
    import subprocess
    import sys
    from sharpnet_amd import tuning_sweep
    for shape in [(1024, 1024, 1024), (2048, 2048, 2048), (4096, 4096, 4096), (1000, 1000, 1000), (4097, 3001, 2049),
                  (8192, 64, 8192), (32768, 2048, 256)]:
        assert shape in tuning_sweep.DEFAULT_SHAPES
    out = subprocess.run([sys.executable, "-m", "sharpnet_amd.tuning_sweep", "--help"], capture_output=True, text=True,
                         timeout=120)
    assert out.returncode == 0 and "--batch" in out.stdout and "--form" in out.stdout
