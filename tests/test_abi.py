"""The C-ABI library loads on a machine without a GPU and exports what include/sharpnet_hip.h declares."""
import os
import re

import pytest

from tests.conftest import ROOT


def declared_symbols():
    text = open(os.path.join(ROOT, "include", "sharpnet_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\bint\s+(snhip_\w+)\s*\(", text)))


def test_header_declares_the_reference_shaped_entry_points():
    syms = declared_symbols()
    for required in ("snhip_create", "snhip_destroy", "snhip_sgemm", "snhip_sgemm_strided_batched", "snhip_dot",
                     "snhip_dot_bias", "snhip_bmm"):
        assert required in syms


def test_library_exports_every_declared_symbol():
    from sharpnet_amd import hiplib
    lib = hiplib.load_library()
    for name in declared_symbols():
        assert hasattr(lib, name), name + " is declared in the header but not exported"
    # and the ctypes prototype table covers the whole header
    assert sorted(hiplib.SIGNATURES) == declared_symbols()


def _c_prototypes():
    """name -> list of C parameter type classes, from include/sharpnet_hip.h."""
    text = open(os.path.join(ROOT, "include", "sharpnet_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    protos = {}
    for name, args in re.findall(r"\bint\s+(snhip_\w+)\s*\(([^;{]*?)\)\s*;", text, flags=re.S):
        params = [a.strip() for a in args.replace("\n", " ").split(",")]
        if params == ["void"] or params == [""]:
            params = []
        kinds = []
        for prm in params:
            if "*" in prm:
                kinds.append("ptr")
            elif re.match(r"(unsigned\s+)?long long\b", prm):
                kinds.append("i64")
            elif prm.startswith("size_t"):
                kinds.append("size")
            elif prm.startswith("float"):
                kinds.append("f32")
            elif re.match(r"(unsigned(\s+int)?|int)\b", prm):
                kinds.append("i32")
            else:
                raise AssertionError("unclassified C parameter %r of %s" % (prm, name))
        protos[name] = kinds
    return protos


def _csharp_prototypes():
    """name -> list of parameter type classes, from the DllImport declarations of integration/SharpNetHipWrapper.cs."""
    text = open(os.path.join(ROOT, "integration", "SharpNetHipWrapper.cs")).read()
    text = re.sub(r"//[^\n]*", "", text)
    protos = {}
    for ret, name, args in re.findall(r"\[DllImport\(DLL_NAME\)\]\s*public static extern (\w+) (snhip_\w+)\(([^;]*?)\);",
                                      text, flags=re.S):
        assert ret in ("cublasStatus_t", "int"), (name, ret)
        params = [a.strip() for a in args.replace("\n", " ").split(",") if a.strip()]
        kinds = []
        for prm in params:
            words = prm.split()
            if words[0] in ("ref", "out") or words[0] in ("IntPtr", "System.Text.StringBuilder"):
                kinds.append("ptr")
            elif words[0] in ("long", "ulong"):
                kinds.append("i64")
            elif words[0] in ("UIntPtr", "size_t"):
                kinds.append("size")
            elif words[0] == "float":
                kinds.append("f32")
            elif words[0] in ("int", "uint", "cublasOperation_t", "cublasSideMode_t"):
                kinds.append("i32")
            else:
                raise AssertionError("unclassified C# parameter %r of %s" % (prm, name))
        protos[name] = kinds
    return protos


def test_csharp_shim_matches_the_header():
    """The P/Invoke declarations a SharpNet maintainer would add (the counterpart of Prod/GPU/CublasWrapper.cs:219-252)
    name only functions the header declares, with the same number of arguments and the same class of type in every
    position, and cover the entry points GPUTensor.Dot / BatchMatrixMultiplication and GPUWrapper need."""
    c, cs = _c_prototypes(), _csharp_prototypes()
    assert len(cs) >= 50
    for name, kinds in cs.items():
        assert name in c, name + " is bound in the C# shim but not declared in the header"
        assert kinds == c[name], (name, kinds, c[name])
    for required in ("snhip_create", "snhip_destroy", "snhip_sgemm", "snhip_sgemm_strided_batched", "snhip_sgeam",
                     "snhip_sdgmm", "snhip_dot", "snhip_dot_bias", "snhip_bmm", "snhip_gemm_ex", "snhip_dense_forward",
                     "snhip_dense_backward", "snhip_attention_forward", "snhip_attention_backward", "snhip_rnn_forward",
                     "snhip_dot_noalloc"):
        assert required in cs, required
    # the two cuBLAS-shaped calls keep cuBLAS's argument order (CublasWrapper.cs:229-244)
    assert cs["snhip_sgemm"] == ["ptr", "i32", "i32", "i32", "i32", "i32", "ptr", "ptr", "i32", "ptr", "i32", "ptr", "ptr", "i32"]
    assert cs["snhip_sgemm_strided_batched"] == ["ptr", "i32", "i32", "i32", "i32", "i32", "ptr", "ptr", "i32", "i64", "ptr",
                                                 "i32", "i64", "ptr", "ptr", "i32", "i64", "i32"]
    patch = open(os.path.join(ROOT, "integration", "call_sites.patch")).read()
    for callee in ("snhip_sgemm(", "snhip_sgemm_strided_batched(", "snhip_create(", "snhip_destroy("):
        assert "SharpNetHipWrapper." + callee in patch


def test_no_compute_symbols_from_vendor_blas():
    # the library must not link a vendor GEMM (hipBLAS / rocBLAS / hipBLASLt)
    import subprocess
    from sharpnet_amd import hiplib
    out = subprocess.run(["ldd", hiplib.library_path()], stdout=subprocess.PIPE, text=True).stdout.lower()
    for banned in ("hipblas", "rocblas", "libcublas", "miopen"):
        assert banned not in out


def test_status_codes_match_cublas_numbering():
    from sharpnet_amd.hiplib import CublasStatus
    text = open(os.path.join(ROOT, "include", "sharpnet_hip.h")).read()
    for name, val in re.findall(r"#define SNHIP_STATUS_(\w+) (\d+)", text):
        assert CublasStatus["CUBLAS_STATUS_" + name].value == int(val)


def test_argument_errors_without_gpu():
    """Calls that are rejected before any device work return the cuBLAS-numbered status."""
    import ctypes
    from sharpnet_amd import hiplib
    lib = hiplib.load_library()
    one = ctypes.c_float(1.0)
    # NULL handle -> NOT_INITIALIZED (1), like cuBLAS
    assert lib.snhip_sgemm(None, 0, 0, 1, 1, 1, ctypes.byref(one), None, 1, None, 1, ctypes.byref(one), None, 1) == 1
    assert lib.snhip_dot(None, None, 1, 1, 0, None, 1, 1, 0, None, 1.0, 0.0) == 1
    assert lib.snhip_destroy(None) == 1
    assert lib.snhip_create(None) == 7
    assert lib.snhip_config_count() >= 4
    d = (ctypes.c_int * 6)()
    assert lib.snhip_config_desc(0, d) == 0 and d[0] > 0 and d[1] > 0
    assert lib.snhip_config_desc(999, d) == 7


def test_gemm_descriptor_layout_matches_the_library():
    """The ctypes mirror of snhip_gemm_desc has the size the compiled library reports, and a descriptor whose
    struct_size disagrees is rejected before anything else is looked at."""
    import ctypes
    from sharpnet_amd import hiplib
    lib = hiplib.load_library()
    assert lib.snhip_sizeof_gemm_desc() == ctypes.sizeof(hiplib.GemmDesc)
    d = hiplib.GemmDesc(M=1, N=1, K=1)
    d.struct_size -= 4
    assert lib.snhip_gemm_ex(None, ctypes.byref(d)) == hiplib.CublasStatus.CUBLAS_STATUS_INVALID_VALUE
    assert lib.snhip_gemm_ex(None, None) == hiplib.CublasStatus.CUBLAS_STATUS_INVALID_VALUE
    d = hiplib.GemmDesc(M=1, N=1, K=1)
    assert lib.snhip_gemm_ex(None, ctypes.byref(d)) == hiplib.CublasStatus.CUBLAS_STATUS_NOT_INITIALIZED
    # host-side operand offsets are taken in bytes of the storage type: bf16-stored operands advance 2 bytes an element
    assert [lib.snhip_operand_element_bytes(m) for m in (0, 1, 2, 3, -1)] == [4, 4, 2, 0, 0]
    assert lib.snhip_sizeof_attention_desc() == ctypes.sizeof(hiplib.AttentionDesc)
    a = hiplib.AttentionDesc(batch=1, Tq=1, Tk=1, dk=1, dv=1)
    assert lib.snhip_attention_forward(None, ctypes.byref(a)) == hiplib.CublasStatus.CUBLAS_STATUS_NOT_INITIALIZED
    a.struct_size += 8
    assert lib.snhip_attention_forward(None, ctypes.byref(a)) == hiplib.CublasStatus.CUBLAS_STATUS_INVALID_VALUE
    assert lib.snhip_sizeof_attention_bwd_desc() == ctypes.sizeof(hiplib.AttentionBwdDesc)
    g = hiplib.AttentionBwdDesc(batch=1, Tq=1, Tk=1, dk=1, dv=1)
    assert lib.snhip_attention_backward(None, ctypes.byref(g)) == hiplib.CublasStatus.CUBLAS_STATUS_NOT_INITIALIZED
    g.struct_size -= 4
    assert lib.snhip_attention_backward(None, ctypes.byref(g)) == hiplib.CublasStatus.CUBLAS_STATUS_INVALID_VALUE
    # the descriptor as it was before the `causal` field (its offset as struct_size) is still taken, and means 0
    g.struct_size = hiplib.AttentionBwdDesc.causal.offset
    assert lib.snhip_attention_backward(None, ctypes.byref(g)) == hiplib.CublasStatus.CUBLAS_STATUS_NOT_INITIALIZED
    assert lib.snhip_attention_backward(None, None) == hiplib.CublasStatus.CUBLAS_STATUS_INVALID_VALUE
    assert lib.snhip_sizeof_rnn_desc() == ctypes.sizeof(hiplib.RnnDesc)
    r = hiplib.RnnDesc(cell_mode=2, bias_mode=1, bidirectional=1, num_layers=2, input_size=3, hidden_size=5)
    nbytes = ctypes.c_size_t()
    assert lib.snhip_rnn_weight_space_size(ctypes.byref(r), ctypes.byref(nbytes)) == 0
    # two directions, four gates: layer 0 reads 3 inputs, layer 1 reads 2 * 5; input-side biases only
    assert nbytes.value == 4 * (2 * 4 * 5 * (3 + 5) + 2 * 4 * 5 * (10 + 5) + 4 * 4 * 5)
    assert lib.snhip_rnn_forward(None, ctypes.byref(r), 0, 1, 1, None, None, None, None, None, None, None, None, 0, None,
                                 0) == hiplib.CublasStatus.CUBLAS_STATUS_NOT_INITIALIZED
    r.struct_size += 4
    assert lib.snhip_rnn_weight_space_size(ctypes.byref(r), ctypes.byref(nbytes)) == \
        hiplib.CublasStatus.CUBLAS_STATUS_INVALID_VALUE


def test_rnn_dropout_rate_is_validated():
    """RNNDescriptor.dropoutRate (Prod/Layers/RNNDescriptor.cs:21) travels in snhip_rnn_desc: a rate inside [0, 1) passes
    the descriptor check in every mode (the calls below then stop at the missing handle), anything else is refused."""
    import ctypes
    from sharpnet_amd import hiplib
    lib = hiplib.load_library()
    S = hiplib.CublasStatus

    def fwd(desc, training):
        return lib.snhip_rnn_forward(None, ctypes.byref(desc), training, 1, 1, None, None, None, None, None, None, None,
                                     None, 0, None, 0)
    d = hiplib.RnnDesc(cell_mode=2, bias_mode=2, num_layers=2, input_size=3, hidden_size=5, dropout=0.25)
    assert fwd(d, 1) == S.CUBLAS_STATUS_NOT_INITIALIZED
    assert fwd(d, 0) == S.CUBLAS_STATUS_NOT_INITIALIZED
    d1 = hiplib.RnnDesc(cell_mode=2, bias_mode=2, num_layers=1, input_size=3, hidden_size=5, dropout=0.25)
    assert fwd(d1, 1) == S.CUBLAS_STATUS_NOT_INITIALIZED
    # the reserve buffer grows by the dropped copies of the inter-layer activations (and the generator's position)
    ws, rs, rs0 = ctypes.c_size_t(), ctypes.c_size_t(), ctypes.c_size_t()
    d0 = hiplib.RnnDesc(cell_mode=2, bias_mode=2, num_layers=2, input_size=3, hidden_size=5, dropout=0.0)
    assert lib.snhip_rnn_temp_space_sizes(ctypes.byref(d), 1, 4, 6, ctypes.byref(ws), ctypes.byref(rs)) == 0
    assert lib.snhip_rnn_temp_space_sizes(ctypes.byref(d0), 1, 4, 6, ctypes.byref(ws), ctypes.byref(rs0)) == 0
    assert rs.value == rs0.value + 4 * (4 * 6 * 5 + 4)
    for bad in (-0.1, 1.0, float("nan")):
        db = hiplib.RnnDesc(cell_mode=2, bias_mode=2, num_layers=2, input_size=3, hidden_size=5, dropout=bad)
        assert fwd(db, 0) == S.CUBLAS_STATUS_INVALID_VALUE


def test_host_mirrors_refuse_shapes_that_would_overrun_device_buffers():
    """RecurrentLayer: an encoder / decoder pair exchanges (batch, K*hidden) blocks, which only match the library's
    (K*layers, batch, hidden) states for one layer.  MultiheadAttention: y has the values' shape but one row per query."""
    from sharpnet_amd import recurrent, attention

    with pytest.raises(ValueError):
        recurrent.RecurrentLayer(None, 4, 3, recurrent.CUDNN_LSTM, recurrent.CUDNN_RNN_DOUBLE_BIAS, False, False,
                                 numLayers=2, isEncoderThatWillBeFollowedByDecoder=True)

    class Stub:
        def __init__(self, shape):
            self.Shape = list(shape)
            self.Count = 1
            for s in shape:
                self.Count *= s
    layer = object.__new__(recurrent.RecurrentLayer)
    layer.num_layers, layer.K, layer.hidden_size = 2, 1, 3
    with pytest.raises(ValueError):
        layer._CheckDecoderArguments(Stub((5, 6)), 5)
    layer.num_layers = 1
    layer._CheckDecoderArguments(Stub((5, 6)), 5)                  # 2 blocks of 5 x 3: accepted
    layer._CheckDecoderArguments(None, 5)
    with pytest.raises(ValueError):
        layer._CheckDecoderArguments(Stub((5, 12)), 5)
    q, kv = Stub((2, 9, 8)), Stub((2, 7, 8))
    with pytest.raises(ValueError, match="queries.Shape\\[1\\]"):
        attention.MultiheadAttentionForwardPropagation(q, kv, kv, kv, None, None, None, None, 2, 4, 4)


def test_missing_library_fails_loudly(tmp_path, monkeypatch):
    from sharpnet_amd import hiplib
    with pytest.raises(FileNotFoundError):
        hiplib.load_library(str(tmp_path / "libsharpnet_hip.so"))


def test_tile_choice_model_is_sane_without_gpu():
    """The configuration/split-K choice is pure host arithmetic: check its invariants over many shapes."""
    import ctypes
    import itertools
    from sharpnet_amd import hiplib
    lib = hiplib.load_library()
    ncfg = lib.snhip_config_count()
    descs = []
    for i in range(ncfg):
        d = (ctypes.c_int * 6)()
        assert lib.snhip_config_desc(i, d) == 0
        descs.append(list(d))
    dims = [1, 2, 63, 64, 65, 256, 1000, 1024, 4097, 8192, 32768]
    for math in (0, 1):
        for M, N, K in itertools.product(dims, repeat=3):
            if M * N > (1 << 28):
                continue
            for batch in (1, 7, 512):
                if M * N * batch > (1 << 28):
                    continue
                c, s = ctypes.c_int(-1), ctypes.c_int(-1)
                assert lib.snhip_query_tuning(None, M, N, K, batch, math, ctypes.byref(c), ctypes.byref(s)) == 0
                BM, BN, BK, NT, lds, kind = descs[c.value]
                assert kind == math                                  # a kernel of the requested arithmetic
                assert 1 <= s.value <= 32 and batch * s.value <= 65535
                assert M * N * batch * s.value * 4 <= (1 << 30) or s.value == 1      # workspace cap
                if s.value > 1:
                    kchunk = -(-(-(-K // s.value)) // BK) * BK
                    assert kchunk * (s.value - 1) < K                # no empty split
                    assert K // s.value >= 4 * BK                    # splits keep a few k tiles each
                assert lds <= 160 * 1024
    # the headline shape gets the largest fp32 tile and no split
    c, s = ctypes.c_int(), ctypes.c_int()
    assert lib.snhip_query_tuning(None, 8192, 8192, 8192, 1, 0, ctypes.byref(c), ctypes.byref(s)) == 0
    assert (descs[c.value][0], descs[c.value][1], s.value) == (256, 256, 1)
    # the benchmark's other fp32 shapes go where the sweep of every (configuration, split) pair found the fastest
    # candidate on MI355X: (BM, BN, BK, split)
    measured_best = {(4096, 4096, 4096): (256, 256, 16, 1), (1024, 1024, 1024): (64, 64, 32, 1),
                     (1000, 1000, 1000): (64, 64, 16, 1), (4097, 3001, 2049): (64, 64, 16, 1),
                     (8192, 64, 8192): (128, 64, 32, 4), (32768, 2048, 256): (128, 128, 16, 1),
                     (4096, 3072, 4096): (128, 128, 16, 1), (1280, 1280, 1280): (64, 128, 16, 1)}
    for (M, N, K), want in measured_best.items():
        assert lib.snhip_query_tuning(None, M, N, K, 1, 0, ctypes.byref(c), ctypes.byref(s)) == 0
        assert tuple(descs[c.value][:3]) + (s.value,) == want, (M, N, K, descs[c.value][:3], s.value)
    assert lib.snhip_query_tuning(None, 0, 8, 8, 1, 0, ctypes.byref(c), ctypes.byref(s)) == 7
    assert lib.snhip_query_tuning(None, 8, 8, 8, 1, 5, ctypes.byref(c), ctypes.byref(s)) == 7
