"""Pins of the CPU checker's dense primitives against the reference's own test vectors,
closed forms and brute force (no GPU)."""
import math

import numpy as np
import pytest

from conftest import rel_l2
from litenn_amd import synth
from litenn_amd.formats import Q4_0, Q4_K, Q6_K, Q8_0, F32, F16
from np_attention import alibi_slope_f64, attention_ext_expected_f64

FORMATS = [Q4_0, Q8_0, Q4_K, Q6_K]


def attention_expected_f64(q, k, v, scale, causal, key_off, query_off):
    """The reference's own independent double-precision checker (ComputeFlashAttnExpected,
    tests/LayerTest.cpp:112-183) without mask/softcap/sinks."""
    q, k, v = (np.asarray(a, np.float64) for a in (q, k, v))
    out = np.zeros((q.shape[0], v.shape[1]), np.float32)
    for row in range(q.shape[0]):
        scores = (k @ q[row]) * float(np.float32(scale))
        if causal:
            cols = np.arange(k.shape[0])
            scores = scores + np.where(key_off + cols > query_off + row, -1.0e9, 0.0)
        p = np.exp(scores - scores.max())
        p = p / p.sum()
        for col in range(k.shape[0]):
            out[row] += (p[col] * v[col]).astype(np.float32)
    return out


def test_matmul_reference_vectors(oracle, golden):
    for case in golden["matmul"]:
        y = oracle.matmul_ikj(case["a"], case["b"])
        assert np.array_equal(y, np.array(case["expected"], np.float32))


def test_matmul_is_sequential_f32_accumulation(oracle):
    """The i-k-j loop accumulates k-ascending in f32: with terms that cancel only in one order
    the result distinguishes it from pairwise, reversed or f64 accumulation."""
    x = np.array([[1e8, 1.0, -1e8, 1.0]], np.float32)
    w = np.ones((4, 1), np.float32)
    assert oracle.matmul_ikj(x, w)[0, 0] == 1.0  # ((1e8 + 1) - 1e8) + 1 in f32 = 1; exact sum is 2
    rng = np.random.default_rng(3)
    a = rng.standard_normal((5, 37)).astype(np.float32)
    b = rng.standard_normal((37, 11)).astype(np.float32)
    want = np.zeros((5, 11), np.float32)
    for kk in range(37):
        want = (want + a[:, kk:kk + 1] * b[kk:kk + 1, :]).astype(np.float32)
    assert np.array_equal(oracle.matmul_ikj(a, b), want)
    assert rel_l2(want, a.astype(np.float64) @ b.astype(np.float64)) < 1e-6
    # identity weights return the input
    assert np.array_equal(oracle.matmul_ikj(a, np.eye(37, dtype=np.float32)), a)


def test_linear_weight_transpose_vector(oracle, golden):
    g = golden["linear_weight_transpose"]
    assert np.array_equal(oracle.transpose(g["imported_nk"]), np.array(g["lowered_kn"], np.float32))


@pytest.mark.parametrize("fmt", FORMATS)
@pytest.mark.parametrize("m", [1, 3])
def test_rowwise_linear_is_bit_identical_to_materialised_path(oracle, fmt, m):
    """dequantise -> transpose -> i-k-j (what the reference executes) versus the memory-bounded
    row-wise form used for the large models: same bits, any thread count."""
    n, k = 40, 512
    wq = synth.quant_weights(fmt, n, k, 7)
    x = synth.activations(m, k, 8)
    a = oracle.mul_mat_q(fmt, wq, n, k, x, rowwise=False)
    for threads in (1, 4):
        oracle.set_threads(threads)
        b = oracle.mul_mat_q(fmt, wq, n, k, x, rowwise=True)
        assert np.array_equal(a.view(np.uint32), b.view(np.uint32))
    # and it is the matmul of the dequantised weight
    w = oracle.dequantize(fmt, wq, n, k)
    assert rel_l2(a, x.astype(np.float64) @ w.astype(np.float64).T) < 1e-5


def test_linear_plain_formats(oracle):
    rng = np.random.default_rng(5)
    w = rng.standard_normal((6, 32)).astype(np.float32)
    x = rng.standard_normal((2, 32)).astype(np.float32)
    y32 = oracle.mul_mat_q(F32, w, 6, 32, x)
    assert np.array_equal(y32, oracle.matmul_ikj(x, w.T.copy()))
    y16 = oracle.mul_mat_q(F16, w.astype(np.float16), 6, 32, x)
    assert np.array_equal(y16, oracle.matmul_ikj(x, w.astype(np.float16).astype(np.float32).T.copy()))


def test_rmsnorm_reference_vectors(oracle, golden):
    c0, c1, c2 = golden["rmsnorm"]
    y = oracle.rmsnorm(c0["x"], c0["w"], c0["eps"])
    assert abs(float(np.mean(y.astype(np.float64) ** 2)) - 1.0) < c0["tol"]
    assert np.allclose(oracle.rmsnorm(c1["x"], c1["w"], c1["eps"]), 0.0, atol=c1["tol"])
    y = oracle.rmsnorm(c2["x"], c2["w"], c2["eps"])[0]
    denom = math.sqrt(14.0 / 3.0 + 1e-6)
    assert np.allclose(y, [2 * v / denom for v in (1, 2, 3)], atol=c2["tol"])


def test_rmsnorm_closed_form_f64(oracle):
    rng = np.random.default_rng(11)
    x = (rng.standard_normal((3, 257)) * 50).astype(np.float32)
    w = rng.standard_normal(257).astype(np.float32)
    eps = float(np.float32(1e-5))
    x64 = x.astype(np.float64)
    want = (x64 / np.sqrt((x64 ** 2).mean(axis=1, keepdims=True) + eps) * w.astype(np.float64)).astype(np.float32)
    got = oracle.rmsnorm(x, w, eps)
    assert np.max(np.abs(got.view(np.int32) - want.view(np.int32))) <= 1  # one ulp at most
    assert np.array_equal(oracle.rmsnorm(x, None, eps), oracle.rmsnorm(x, np.ones(257, np.float32), eps))


def test_rope_reference_vectors(oracle, golden):
    c0, c1, c2 = golden["rope"]
    assert np.allclose(oracle.rope(c0["x"], c0["base"], c0["pos_offset"], c0["freq_scale"]), c0["expected"],
                       atol=c0["tol"])
    y = oracle.rope(c1["x"], c1["base"], c1["pos_offset"], c1["freq_scale"])
    cos1, sin1 = math.cos(1.0), math.sin(1.0)
    assert np.allclose(y[1], [cos1, sin1, -sin1, cos1], atol=c1["tol"])
    assert np.all(y[0] == 0)
    y = oracle.rope(c2["x"], c2["base"], c2["pos_offset"], c2["freq_scale"])
    assert np.allclose(y[1], [cos1, sin1], atol=c2["tol"])  # position (1+1) * scale 0.5 = angle 1


def test_rope_closed_form_and_invariants(oracle):
    rng = np.random.default_rng(12)
    d, m, off, base = 128, 5, 37, 5e5
    x = rng.standard_normal((m, d)).astype(np.float32)
    y = oracle.rope(x, base, off)
    pos = (off + np.arange(m))[:, None].astype(np.float64)
    inv = base ** (-2.0 * np.arange(d // 2) / d)
    ang = pos * inv[None, :]
    c, s = np.cos(ang).astype(np.float32), np.sin(ang).astype(np.float32)
    a, b = x[:, 0::2], x[:, 1::2]
    want = np.empty_like(x)
    want[:, 0::2] = a * c - b * s
    want[:, 1::2] = a * s + b * c
    assert np.array_equal(y.view(np.uint32), want.view(np.uint32))
    # rotation preserves pair norms; composing offsets adds angles
    assert np.allclose((y ** 2).sum(1), (x ** 2).sum(1), rtol=1e-5)
    # partial rotation leaves the tail untouched (rope.dimension_count < headDim)
    yp = oracle.rope(x, base, off, rope_dims=64)
    assert np.array_equal(yp[:, 64:], x[:, 64:])
    assert np.array_equal(yp[:, :64], oracle.rope(x[:, :64].copy(), base, off))


def test_attention_reference_vectors(oracle, golden):
    c0, c1 = golden["attention"]
    scale0 = 1.0 / math.sqrt(2.0)
    got = oracle.attention_head(c0["q"], c0["k"], c0["v"], scale0, True, 0, 0)
    want = attention_expected_f64(c0["q"], c0["k"], c0["v"], scale0, True, 0, 0)
    assert np.allclose(got, want, atol=c0["tol"])
    assert got[0, 0] == 2.0  # first row sees only key 0
    got = oracle.attention_head(c1["q"], c1["k"], c1["v"], 1.0, True, 0, 1)
    want = attention_expected_f64(c1["q"], c1["k"], c1["v"], 1.0, True, 0, 1)
    assert abs(got[0, 0] - want[0, 0]) < c1["tol"]
    assert got[0, 0] < c1["less_than"]  # the key at position 2 (value 1000) is masked


def test_attention_properties(oracle):
    rng = np.random.default_rng(13)
    q = rng.standard_normal((4, 128)).astype(np.float32)
    k = rng.standard_normal((9, 128)).astype(np.float32)
    v = rng.standard_normal((9, 128)).astype(np.float32)
    scale = 1.0 / math.sqrt(128.0)
    got = oracle.attention_head(q, k, v, scale, True, 0, 5)
    want = attention_expected_f64(q, k, v, scale, True, 0, 5)
    assert np.allclose(got, want, atol=1e-5)
    # a single key returns its value exactly
    one = oracle.attention_head(q[:1], k[:1], v[:1], scale, True, 0, 0)
    assert np.array_equal(one, v[:1])
    # constant values => output is that constant (softmax rows sum to one)
    const = oracle.attention_head(q, k, np.full((9, 3), 2.5, np.float32), scale, False)
    assert np.allclose(const, 2.5, atol=1e-6)


def test_attention_options_reference_vector(oracle, golden):
    """The reference's mask + softcap + sinks case (ALiBi slope of head 1 of 4 at maxBias 4), held to
    its own double-precision checker at its own tolerance."""
    c = golden["attention_ext"][0]
    slope = alibi_slope_f64(c["head_index"], c["head_count"], c["max_bias"])
    assert slope == 0.25  # 2^(-4/4) squared
    assert oracle.alibi_slope(c["head_index"], c["head_count"], c["max_bias"]) == slope
    got = oracle.flash_attn_ext(c["q"], c["k"], c["v"], c["scale"], c["logit_softcap"], c["mask"], c["max_bias"],
                                c["head_index"], c["head_count"], c["sink"])
    want = attention_ext_expected_f64(c["q"], c["k"], c["v"], c["scale"], c["logit_softcap"], c["mask"], slope, c["sink"])
    assert np.allclose(got, want, atol=c["tol"])
    # every option matters in this case: dropping one moves the result by far more than the tolerance
    for drop in ("logit_softcap", "mask", "sink", "max_bias"):
        o = dict(c)
        o[drop] = {"logit_softcap": 0.0, "mask": None, "sink": None, "max_bias": 0.0}[drop]
        if o["mask"] is None:
            o["max_bias"] = 0.0
        other = oracle.flash_attn_ext(o["q"], o["k"], o["v"], o["scale"], o["logit_softcap"], o["mask"], o["max_bias"],
                                      o["head_index"], o["head_count"], o["sink"])
        assert np.abs(other - want).max() > 1e-3, drop


def test_attention_options_against_f64_checker(oracle):
    rng = np.random.default_rng(29)
    for case in range(24):
        mq, l, d, dv = int(rng.integers(1, 6)), int(rng.integers(1, 40)), int(rng.choice([2, 16, 64, 128])), int(rng.integers(1, 9))
        q = rng.standard_normal((mq, d)).astype(np.float32)
        k = rng.standard_normal((l, d)).astype(np.float32)
        v = rng.standard_normal((l, dv)).astype(np.float32)
        scale = float(rng.choice([1.0, 1.0 / math.sqrt(d), 1.25])) if d <= 16 else float(rng.choice([1.0, 1.25])) / math.sqrt(d)
        softcap = float(rng.choice([0.0, 0.75, 1.0, 30.0]))
        mask = rng.standard_normal((mq, l)).astype(np.float32) if rng.random() < 0.6 else None
        heads = int(rng.choice([1, 4, 6, 12]))
        head = int(rng.integers(0, heads))
        max_bias = float(rng.choice([0.0, 4.0, 8.0])) if mask is not None else 0.0
        sink = float(rng.standard_normal()) if rng.random() < 0.5 else None
        causal = bool(rng.random() < 0.5)
        key_off = int(rng.integers(0, 3))
        query_off = key_off + int(rng.integers(0, l + 2))  # the first row always sees key 0
        slope = alibi_slope_f64(head, heads, max_bias)
        assert abs(oracle.alibi_slope(head, heads, max_bias) - slope) <= 1e-15 * slope
        got = oracle.flash_attn_ext(q, k, v, scale, softcap, mask, max_bias, head, heads, sink, causal, key_off, query_off)
        want = attention_ext_expected_f64(q, k, v, scale, softcap, mask, slope, sink, causal, key_off, query_off)
        assert np.allclose(got, want, atol=2e-5, rtol=1e-5), case
    # with every option off it is the plain head, bit for bit
    q = rng.standard_normal((3, 64)).astype(np.float32)
    k = rng.standard_normal((17, 64)).astype(np.float32)
    v = rng.standard_normal((17, 64)).astype(np.float32)
    assert np.array_equal(oracle.flash_attn_ext(q, k, v, 0.125, causal=True, query_pos_offset=14),
                          oracle.attention_head(q, k, v, 0.125, True, 0, 14))
    # non-power-of-two head counts: heads past the largest power of two take the interleaved slopes
    assert oracle.alibi_slope(4, 6, 8.0) == 2.0 ** (-(8.0 / 2) / 4)
    assert oracle.alibi_slope(5, 6, 8.0) == (2.0 ** (-(8.0 / 2) / 4)) ** 3
    with pytest.raises(ValueError, match="maxBias requires"):
        oracle.flash_attn_ext(q, k, v, max_bias=4.0)


def test_silu_and_swiglu_reference_vectors(oracle, golden):
    sig = lambda t: 1.0 / (1.0 + math.exp(-t))
    assert abs(float(oracle.silu(golden["silu"]["x"])[0]) - 2.0 * sig(2.0)) < golden["silu"]["tol"]
    for case in golden["swiglu"]:
        x = np.array(case["x"], np.float32)
        gate = oracle.matmul_ikj(x, case["gate_w"])
        up = oracle.matmul_ikj(x, case["up_w"])
        y = oracle.matmul_ikj(oracle.silu_mul(gate, up), case["down_w"])
        e0, e1 = 1 * sig(1) * 1, 2 * sig(2) * 2
        want = [e0, e1] if y.shape[1] == 2 else [e0 + e1]
        assert np.allclose(y[0], want, atol=case["tol"])
    x = np.linspace(-30, 30, 1001).astype(np.float32)
    assert np.allclose(oracle.silu(x), x.astype(np.float64) / (1 + np.exp(-x.astype(np.float64))), atol=1e-6)


def test_get_rows_reference_vector_and_range_check(oracle, golden):
    g = golden["get_rows"]
    assert np.array_equal(oracle.get_rows(g["table"], g["indices"]), np.array(g["expected"], np.float32))
    with pytest.raises(oracle.OracleError, match="out of range"):
        oracle.get_rows(g["table"], [4])
    with pytest.raises(oracle.OracleError, match="out of range"):
        oracle.get_rows(g["table"], [-1])


def test_argmax_first_maximum(oracle):
    assert oracle.argmax([1.0, 5.0, 5.0, 2.0]) == 1
    assert oracle.argmax([-np.inf, -np.inf]) == 0
