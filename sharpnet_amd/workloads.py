"""Synthetic inputs and algorithmic work figures of the five benchmark configurations.

Dense layer, GEMM sweep, MLP step, LSTM projections, attention matmuls; every generator is
seeded (numpy ``default_rng``) so the oracle and the device see identical data.
Work accounting: flops = 2*M*N*K*batch; bytes = batch*(4*(M*K + K*N) + 4*M*N*(1 + [beta != 0])).
"""
import math

import numpy as np

FP32_MFMA_PEAK_TFLOPS = 157.3   # MI355X dense fp32 matrix peak (256 CU x 256 flop/clk x 2.4 GHz)
BF16_MFMA_PEAK_TFLOPS = 2500.0  # MI355X dense bf16 matrix peak
HBM_PEAK_GBS = 8000.0           # MI355X HBM3E


class Gemm:
    """One row-major GEMM: C[M,N] = alpha*op(A)op(B) + beta*C, `batch` matrices."""

    def __init__(self, M, N, K, tA=False, tB=False, alpha=1.0, beta=0.0, batch=1, bias=False, name=""):
        self.M, self.N, self.K, self.tA, self.tB = M, N, K, tA, tB
        self.alpha, self.beta, self.batch, self.bias, self.name = alpha, beta, batch, bias, name

    @property
    def a_shape(self):
        s = (self.K, self.M) if self.tA else (self.M, self.K)
        return (self.batch,) + s if self.batch > 1 else s

    @property
    def b_shape(self):
        s = (self.N, self.K) if self.tB else (self.K, self.N)
        return (self.batch,) + s if self.batch > 1 else s

    @property
    def c_shape(self):
        return (self.batch, self.M, self.N) if self.batch > 1 else (self.M, self.N)

    @property
    def flops(self):
        return 2.0 * self.M * self.N * self.K * self.batch

    @property
    def bytes(self):
        return self.batch * (4.0 * (self.M * self.K + self.K * self.N) +
                             4.0 * self.M * self.N * (1 + (1 if self.beta != 0 else 0)))

    @property
    def layout(self):
        return ("T" if self.tA else "N") + ("T" if self.tB else "N")

    def roofline_seconds(self, peak_tflops=FP32_MFMA_PEAK_TFLOPS):
        return max(self.flops / (peak_tflops * 1e12), self.bytes / (HBM_PEAK_GBS * 1e9))

    def label(self):
        b = "%dx" % self.batch if self.batch > 1 else ""
        return "%s%s(%d,%d,%d) %s beta=%g" % (self.name + " " if self.name else "", b, self.M, self.N, self.K,
                                              self.layout, self.beta)


def glorot_uniform(rng, fan_in, fan_out, shape):
    lim = math.sqrt(6.0 / (fan_in + fan_out))
    return rng.uniform(-lim, lim, size=shape).astype(np.float32)


# ---- config 1: single Dense layer forward + backward ------------------------
def dense_layer_inputs(seed=1, batch=128, n_in=784, n_out=256):
    rng = np.random.default_rng(seed)
    return {
        "x": rng.uniform(0, 1, (batch, n_in)).astype(np.float32),
        "w_out_in": glorot_uniform(rng, n_in, n_out, (n_out, n_in)),   # reference layout, Linear.cs:22
        "bias": np.zeros(n_out, np.float32),
        "dy": rng.normal(0, 0.01, (batch, n_out)).astype(np.float32),
    }


def dense_layer_gemms(batch=128, n_in=784, n_out=256):
    return [Gemm(batch, n_out, n_in, False, True, bias=True, name="fwd y=x.Wt+b"),
            Gemm(n_out, n_in, batch, True, False, name="dW=dyt.x"),
            Gemm(batch, n_in, n_out, False, False, name="dx=dy.W")]


# ---- config 2: square and ragged sweep ---------------------------------------
SWEEP_SIZES = [(1024, 1024, 1024), (2048, 2048, 2048), (4096, 4096, 4096), (8192, 8192, 8192), (1000, 1000, 1000),
               (4097, 3001, 2049), (8192, 64, 8192)]


def sweep_gemms(sizes=SWEEP_SIZES, betas=(0.0, 1.0)):
    out = []
    for (M, N, K) in sizes:
        for tA in (False, True):
            for tB in (False, True):
                for beta in betas:
                    out.append(Gemm(M, N, K, tA, tB, 1.0, beta))
    return out


def uniform_operands(g, seed=2):
    rng = np.random.default_rng(seed)
    a = rng.uniform(-1, 1, g.a_shape).astype(np.float32)
    b = rng.uniform(-1, 1, g.b_shape).astype(np.float32)
    c = rng.uniform(-1, 1, g.c_shape).astype(np.float32) if g.beta != 0 else None
    return a, b, c


HEADLINE = Gemm(8192, 8192, 8192, False, False, 1.0, 0.0, name="headline")


# ---- config 3: 3-layer MLP training step ---------------------------------------
MLP_WIDTHS = [3072, 4096, 4096, 1000]
MLP_BATCH = 4096


def mlp_gemms(batch=MLP_BATCH, widths=MLP_WIDTHS, skip_first_dx=False):
    fwd, dw, dx = [], [], []
    for i in range(len(widths) - 1):
        n_in, n_out = widths[i], widths[i + 1]
        fwd.append(Gemm(batch, n_out, n_in, False, True, bias=True, name="fwd%d" % i))
        dw.append(Gemm(n_out, n_in, batch, True, False, name="dW%d" % i))
        if not (skip_first_dx and i == 0):
            dx.append(Gemm(batch, n_in, n_out, False, False, name="dX%d" % i))
    return fwd + dw + dx


# ---- config 4: LSTM gate projections ---------------------------------------------
def lstm_gemms(batch=256, seq=128, n_in=256, hidden=512):
    return (Gemm(batch * seq, 4 * hidden, n_in, False, False, name="input proj"),
            Gemm(batch, 4 * hidden, hidden, False, False, 1.0, 1.0, name="recurrent step"), seq)


def lstm_inputs(seed=4, batch=256, seq=128, n_in=256, hidden=512):
    rng = np.random.default_rng(seed)
    lim = 1.0 / math.sqrt(hidden)
    return {
        "x": rng.normal(0, 1, (batch * seq, n_in)).astype(np.float32),
        "w": rng.uniform(-lim, lim, (n_in, 4 * hidden)).astype(np.float32),
        "u": rng.uniform(-lim, lim, (hidden, 4 * hidden)).astype(np.float32),
        "h": np.tanh(rng.normal(0, 1, (batch, hidden))).astype(np.float32),
    }


# ---- config 5: strided-batched attention matmuls -----------------------------------
def attention_gemms(batch=512, seq=256, d=64):
    return [Gemm(seq, seq, d, False, True, 1.0 / math.sqrt(d), 0.0, batch, name="S=QKt/8"),
            Gemm(seq, d, seq, False, False, 1.0, 0.0, batch, name="O=PV")]


def attention_inputs(seed=5, batch=512, seq=256, d=64):
    rng = np.random.default_rng(seed)
    return {k: rng.normal(0, 1, (batch, seq, d)).astype(np.float32) for k in ("q", "k", "v")}
