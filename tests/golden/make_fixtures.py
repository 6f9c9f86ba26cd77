"""Writes tests/golden/reference_vectors.json from the literals the reference's own tests hold.

Run once in a container that has the reference tree:  python tests/golden/make_fixtures.py
The reference files are opened as TEXT only (nothing is compiled, imported or
executed); the output holds numbers - inputs and expected outputs - never source.
The GPU box has no reference tree: tests read the committed JSON.
"""
import json
import os
import re
import sys

REF = os.environ.get("SHARPNET_REFERENCE", "/root/reference")
OUT = os.path.join(os.path.dirname(os.path.abspath(__file__)), "reference_vectors.json")


def read(rel):
    with open(os.path.join(REF, rel), encoding="utf-8-sig") as f:
        return f.read()


def lines(text, lo, hi):
    """1-based inclusive line range."""
    return "\n".join(text.split("\n")[lo - 1:hi])


def numpy_literals(block):
    """All FromNumpyArray-style literals in a block of C#: "[[...]]" or "numpy.array([...], numpy.float)"."""
    out = []
    for m in re.finditer(r'"\s*(?:numpy\.array\()?\s*(\[[^"]*?\])\s*(?:,\s*numpy\.float\))?\s*"', block):
        out.append(json.loads(m.group(1)))
    return out


def np_shape(v):
    return (len(v), len(v[0])) if isinstance(v, list) and isinstance(v[0], list) else len(v)


def const_literal(text, name):
    m = re.search(r'const string ' + re.escape(name) + r'\s*=\s*@?"([^"]*)"', text)
    body = m.group(1)
    arr = re.search(r'(\[.*\])', body, re.S).group(1)
    return json.loads(arr)


def main():
    fx = {}

    # ---- Tests/GPU/TestGpuTensor.cs:50-120  TestDot known answers (tolerance 1e-9) ----
    fx["TestDot"] = {
        "source": "Tests/GPU/TestGpuTensor.cs:53-109",
        "tolerance": 1e-9,
        "cases": [
            {"a_shape": [1, 1], "a": [2], "b_shape": [1, 1], "b": [5], "c_shape": [1, 1], "expected": [10]},
            {"a_shape": [2, 2], "a": [1, 2, 3, 4], "b_shape": [2, 2], "b": [1, 2, 3, 4], "c_shape": [2, 2],
             "expected": [7, 10, 15, 22]},
            {"a_shape": [1, 2], "a": [1, 2], "b_shape": [2, 1], "b": [3, 4], "c_shape": [1, 1], "expected": [11]},
            {"a_shape": [2, 1], "a": [1, 2], "b_shape": [1, 2], "b": [3, 4], "c_shape": [2, 2],
             "expected": [3, 4, 6, 8]},
            {"a_shape": [2, 1, 1], "a": [1, 2], "b_shape": [1, 1, 2], "b": [3, 4], "c_shape": [2, 2],
             "expected": [3, 4, 6, 8]},
            {"a_shape": [10, 1, 28, 28], "a": "zeros", "b_shape": [784, 100], "b": "zeros", "c_shape": [10, 1, 1, 100],
             "expected": "zeros"},
            {"a_shape": [35, 124], "a": "zeros", "b_shape": [124, 21], "b": "zeros", "c_shape": [35, 21],
             "expected": "zeros"},
        ],
    }

    # ---- Tests/CPU/TestCpuTensor.cs:826-866  QR factorisation of the Rosetta-code matrix ----
    cpu = read("Tests/CPU/TestCpuTensor.cs")
    qr_cases = []
    for m in re.finditer(r'\[TestCase\("(\[\[[^"]*\]\])",\s*"\s*(\[\[[^"]*\]\])"\)\]', lines(cpu, 855, 870)):
        qr_cases.append({"A": json.loads(m.group(1)), "Q": json.loads(m.group(2))})
    assert len(qr_cases) == 2, qr_cases
    fx["QR"] = {
        "source": "Tests/CPU/TestCpuTensor.cs:826-866 (A at :830, expected Q at :861-863); "
                  "asserts Dot(Q,R)~A within 1e-4 and max|QtQ-I| < 1e-6",
        "cases": qr_cases,
    }

    # ---- Tests/NonReg/TestNetworkPropagation.cs  Linear + sigmoid predictions ----
    tnp = read("Tests/NonReg/TestNetworkPropagation.cs")
    fx["Linear_1_1_1_1"] = {
        "source": "Tests/NonReg/TestNetworkPropagation.cs:36-61",
        "x": [[[[1.0]]]],
        "w": numpy_literals(lines(tnp, 47, 48))[0],
        "sigmoid_prediction": numpy_literals(lines(tnp, 50, 51))[0],
        "tolerance": 1e-6,
    }
    fx["Linear_1_1_4_4"] = {
        "source": "Tests/NonReg/TestNetworkPropagation.cs:24,34,80-105 (weights literal is (in=16, out=3): "
                  "prediction = sigmoid(x[1x16] . W[16x3]))",
        "x": const_literal(tnp, "X_1_1_4_4"),
        "w_in_out": const_literal(tnp, "W_N_1_4_4"),
        "sigmoid_prediction": numpy_literals(lines(tnp, 95, 95))[0],
        "tolerance": 1e-6,
    }

    # ---- Tests/NonReg/ParallelRunWithPyTorch.cs:102-138  two Linear layers, MSE, SGD momentum ----
    prp = read("Tests/NonReg/ParallelRunWithPyTorch.cs")
    blk = lines(prp, 102, 138)
    w = numpy_literals(blk)
    assert len(w) == 2 and len(w[0]) == 3 and len(w[0][0]) == 5 and len(w[1][0]) == 36
    losses = [float(v) for v in re.findall(r'Assert\.AreEqual\(([0-9.eE+-]+), loss_', blk)]
    fx["PyTorch_Mse"] = {
        "source": "Tests/NonReg/ParallelRunWithPyTorch.cs:102-138; inputs numpy_array_for_tests(2,3,4,5) and "
                  "y_numpy_array_for_tests(2,3), Tests/NonReg/TestNetworkPropagation.cs:167-186",
        "x_shape": [2, 3, 4, 5], "y_shape": [2, 3],
        "linear1_weight_out_in": w[0], "linear2_weight_out_in": w[1],
        "lr": 0.1, "momentum": 0.9, "epochs": 10,
        "loss_before": losses[0], "loss_after": losses[1], "tolerance": 1e-6,
    }

    # ---- same file :963-1010  scaled-dot-product attention chain ----
    blk = lines(prp, 961, 1010)
    w = numpy_literals(blk)
    assert len(w) == 4, len(w)
    cases = re.findall(r'\[TestCase\((false|true),\s*([0-9.eE+-]+),\s*([0-9.eE+-]+)\)\]', blk)
    fx["PyTorch_DotProductAttention"] = {
        "source": "Tests/NonReg/ParallelRunWithPyTorch.cs:963-1010 (use_scale=false); X = numpy_array_for_tests(6,4,5) "
                  "read as (N, C=4, L=5); conv1D kernels of width 1 = per-sample (2x4).(4x5) products",
        "x_shape": [6, 4, 5], "y_shape": [6, 3],
        "conv_q": w[0], "conv_k": w[1], "conv_v": w[2], "dense_weight_out_in": w[3],
        "cases": [{"is_causal": c[0] == "true", "loss_before": float(c[1]), "loss_after": float(c[2])} for c in cases],
        "tolerance": 1e-6,
    }

    # ---- same file :1013-1131  multi-head attention chain, without and with bias ----
    mha = {}
    for name, lo, hi in (("no_bias", 1013, 1071), ("with_bias", 1073, 1131)):
        blk = lines(prp, lo, hi)
        w = numpy_literals(blk)
        assert len(w) == 6 and len(w[3]) == 18 and len(w[4]) == 6 and len(w[5]) == 3 and len(w[5][0]) == 12, name
        cases = re.findall(r'\[TestCase\((false|true),\s*([0-9.eE+-]+),\s*([0-9.eE+-]+)\)\]', blk)
        assert len(cases) == 2
        mha[name] = {
            "conv_q": w[0], "conv_k": w[1], "conv_v": w[2], "in_proj_weight": w[3], "out_proj_weight": w[4],
            "dense_weight_out_in": w[5],
            "cases": [{"is_causal": c[0] == "true", "loss_before": float(c[1]), "loss_after": float(c[2])} for c in cases],
        }
    fx["PyTorch_MultiHeadAttention"] = {
        "source": "Tests/NonReg/ParallelRunWithPyTorch.cs:1013-1131; X = numpy_array_for_tests(10,2,6) read as (N, C=2, L=6), "
                  "Y = y_numpy_array_for_tests(10,3); three width-1 Conv1D (with bias, zero at start) feed Q, K, V of a "
                  "MultiheadAttention(num_heads=3, key_dim=value_dim=2), then Flatten, Linear(3, bias), softmax, categorical "
                  "cross-entropy; SGD(0.1, momentum 0.9), batch size 2, 10 epochs, no shuffling; all biases start at zero",
        "x_shape": [10, 2, 6], "y_shape": [10, 3], "num_heads": 3, "key_dim": 2, "value_dim": 2,
        "lr": 0.1, "momentum": 0.9, "epochs": 10, "batch_size": 2, "tolerance": 1e-6,
        "no_bias": mha["no_bias"], "with_bias": mha["with_bias"],
    }

    # ---- same file :896-953  two stacked SimpleRNN layers (cuDNN tanh cells) ----
    blk = lines(prp, 896, 953)
    w = numpy_literals(blk)
    assert len(w) == 10 and len(w[2][0]) == 4 and len(w[8][0]) == 4, [np_shape(v) for v in w]
    losses = [float(v) for v in re.findall(r'Assert\.AreEqual\(([0-9.eE+-]+), loss_', blk)]
    fx["PyTorch_SimpleRNN"] = {
        "source": "Tests/NonReg/ParallelRunWithPyTorch.cs:896-953; X = numpy_array_for_tests(4,2,1), Y = y_numpy_array_for_tests(4,2); "
                  "SimpleRNN(hidden 2, return sequences, bidirectional, 2 layers) then SimpleRNN(hidden 2, last step only); tanh "
                  "cells with two zero-initialised bias vectors (PyTorch compatibility mode); MSE; SGD(0.01, momentum 0.9), "
                  "batch size 2, 10 epochs, no shuffling",
        "x_shape": [4, 2, 1], "y_shape": [4, 2],
        "layer1_weight_ih": w[0:4], "layer1_weight_hh": w[4:8], "layer2_weight_ih": [w[8]], "layer2_weight_hh": [w[9]],
        "lr": 0.01, "momentum": 0.9, "epochs": 10, "batch_size": 2,
        "loss_before": losses[0], "loss_after": losses[1], "tolerance": 1e-6,
    }

    # ---- Tests/NonReg/TestNetworkPropagation.cs:1193-1330  recurrent layers trained from zero weights ----
    rnn_cases = []
    for test, cell in (("Test_SimpleRNN", "tanh"), ("Test_LSTM", "lstm"), ("Test_GRU", "gru")):
        i = tnp.index("public void %s(bool returnSequences" % test)
        blk = tnp[tnp.rindex("\n\n", 0, i):i]
        found = re.findall(r'\[TestCase\((true|false), (true|false), "([^"]*)", "([^"]*)", "([^"]*)"\)\]', blk)
        assert len(found) == 4, (test, len(found))
        for rs, bd, dense, before, after in found:
            rnn_cases.append({"cell": cell, "return_sequences": rs == "true", "bidirectional": bd == "true", "hidden": 2,
                              "dense_weight": json.loads(dense), "prediction_before": json.loads(before),
                              "prediction_after": json.loads(after)})
    blk = lines(tnp, 1198, 1226)
    w = numpy_literals(blk)
    assert len(w) == 3 and len(w[0]) == 3, w
    rnn_cases.append({"cell": "tanh", "return_sequences": False, "bidirectional": False, "hidden": 3, "dense_weight": w[0],
                      "prediction_before": w[1], "prediction_after": w[2]})
    fx["ZeroWeightRecurrentLayers"] = {
        "source": "Tests/NonReg/TestNetworkPropagation.cs:1193-1330 (Test_SimpleRNN_returnSequence_false, Test_SimpleRNN, "
                  "Test_LSTM, Test_GRU): Input(2 steps, 1 feature) -> recurrent layer(hidden, returnSequences, bidirectional), all "
                  "its weights zero -> Linear(1, bias, on the last dimension) with the given weights; Huber loss (delta 1, "
                  "Prod/CPU/CpuTensor.cs:2420-2437), SGD(0.1, momentum 0.9) on the whole batch of 4 for 10 epochs, TensorFlow "
                  "compatibility mode (SimpleRNN and LSTM: one bias vector on the input side, GRU: two, Prod/Networks/Network.cs:188-205)",
        "x": const_literal(tnp, "X_RNN_4_2_1"), "y_sequences": const_literal(tnp, "Y_RNN_4_2_1"),
        "y_last": const_literal(tnp, "Y_RNN_4_1_1"),
        "lr": 0.1, "momentum": 0.9, "epochs": 10, "huber_delta": 1.0, "tolerance": 1e-4, "cases": rnn_cases,
    }

    with open(OUT, "w") as f:
        json.dump(fx, f, indent=1)
    print("wrote", OUT, os.path.getsize(OUT), "bytes")


if __name__ == "__main__":
    sys.exit(main())
