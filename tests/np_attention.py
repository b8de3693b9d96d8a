"""The reference test suite's own double-precision attention checker, restated in numpy
(tests/LayerTest.cpp:89-183): what the CPU checker's and the GPU's attention with options are
both held to."""
import math

import numpy as np


def alibi_slope_f64(head_index, head_count, max_bias):
    """ComputeALiBiSlope of the reference's test (tests/LayerTest.cpp:89-111), in Python floats."""
    if max_bias <= 0.0:
        return 1.0
    head_log2 = 1
    while head_log2 * 2 <= head_count:
        head_log2 *= 2
    m0 = 2.0 ** (-max_bias / head_log2)
    m1 = 2.0 ** (-(max_bias / 2.0) / head_log2)
    if head_index < head_log2:
        return m0 ** (head_index + 1)
    return m1 ** (2 * (head_index - head_log2) + 1)


def attention_ext_expected_f64(q, k, v, scale=1.0, softcap=0.0, mask=None, slope=1.0, sink=None, causal=False,
                               key_off=0, query_off=0):
    """ComputeFlashAttnExpected (tests/LayerTest.cpp:112-183) with every option: scores in double,
    softcap * tanh(score / softcap) with the library tanh (not the f32 exp composition the layer
    lowers to), slope * mask, causal offset mask, the sink joins the maximum and the denominator."""
    q, k, v = (np.asarray(a, np.float64) for a in (q, k, v))
    out = np.zeros((q.shape[0], v.shape[1]), np.float32)
    cols = np.arange(k.shape[0])
    for row in range(q.shape[0]):
        scores = (k @ q[row]) * float(np.float32(scale))
        if softcap != 0.0:
            cap = float(np.float32(softcap))
            scores = cap * np.tanh(scores / cap)
        if mask is not None:
            scores = scores + slope * np.asarray(mask, np.float32).astype(np.float64)[row]
        if causal:
            scores = scores + np.where(key_off + cols > query_off + row, -1.0e9, 0.0)
        top = scores.max() if sink is None else max(scores.max(), float(np.float32(sink)))
        p = np.exp(scores - top)
        denom = p.sum() + (0.0 if sink is None else math.exp(float(np.float32(sink)) - top))
        for col in range(k.shape[0]):
            out[row] += (p[col] / denom * v[col]).astype(np.float32)
    return out
