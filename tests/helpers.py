"""Shared helpers of the parity tests (seeded inputs in the reference's shapes)."""
import numpy as np


def numpy_array_for_tests(*shape):
    """Tests/NonReg/TestNetworkPropagation.cs:167-176: x[i] = 2(i+1)/count * ((i % 2) - 0.5)."""
    count = int(np.prod(shape))
    i = np.arange(count, dtype=np.float64)
    return ((2.0 * (i + 1)) / count * ((i % 2) - 0.5)).astype(np.float32).reshape(shape)


def y_numpy_array_for_tests(rows, cols):
    """TestNetworkPropagation.cs:178-186: one-hot at column row % cols."""
    y = np.zeros((rows, cols), dtype=np.float32)
    for r in range(rows):
        y[r, r % cols] = 1
    return y


def random_tensor(rng, shape, lo=-1.5, hi=1.5):
    """Stand-in for TestParallelRunCpuVersusGpu.RandomTensor (U(-1.5, 1.5), :1421-1424); numpy stream, not .NET's."""
    return rng.uniform(lo, hi, size=shape).astype(np.float32)


def sigmoid(x):
    return 1.0 / (1.0 + np.exp(-np.asarray(x, dtype=np.float64)))
