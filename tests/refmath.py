"""Plain float64 arithmetic the GPU tests check against (the textbook FullyConnected over
dequantised weights, as FullyConnectedReference over MakeWeightsFromInt8 computes it:
common/task/testing_ref_ops.cc:961-988, 2715-2742)."""
import numpy as np


def dequantized_weights(case):
    """float64 [n][k] weights (q - zp) * s of a workloads case."""
    k, groups = case["k"], case["groups"]
    gs = k // groups
    s = np.repeat(case["scale"].astype(np.float64), gs, axis=1)
    q = case["w"].astype(np.float64)
    if case["zero_point"] is not None:
        q = q - np.repeat(case["zero_point"].astype(np.float64), gs, axis=1)
    return q * s


def textbook(case):
    ref = case["act"].astype(np.float64) @ dequantized_weights(case).T
    if case["bias"] is not None:
        ref = ref + case["bias"]
    return ref
