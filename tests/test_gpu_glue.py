"""Parity of the decoder's small kernels (through the C ABI) with the CPU checker and with the
reference's own test vectors."""
import math

import numpy as np
import pytest

from conftest import rel_l2
from litenn_amd.formats import DT_F16, DT_F32

pytestmark = pytest.mark.gpu


def T(hip, a, dtype=np.float32):
    return hip.Tensor.from_numpy(np.ascontiguousarray(a, dtype))


def test_rmsnorm(hip, oracle, golden):
    rng = np.random.default_rng(1)
    for m, d in [(1, 4096), (3, 257), (16, 11008)]:
        x = (rng.standard_normal((m, d)) * 7).astype(np.float32)
        w = rng.standard_normal(d).astype(np.float32)
        eps = float(np.float32(1e-5))
        got = hip.rmsnorm(T(hip, x), T(hip, w), eps).numpy()
        want = oracle.rmsnorm(x, w, eps)
        # f64 accumulation on both sides: at most one f32 ulp apart
        assert np.max(np.abs(got.view(np.int32) - want.view(np.int32))) <= 1
        assert np.array_equal(hip.rmsnorm(T(hip, x), None, eps).numpy(), oracle.rmsnorm(x, None, eps)) or \
            rel_l2(hip.rmsnorm(T(hip, x), None, eps).numpy(), oracle.rmsnorm(x, None, eps)) < 1e-7
    c = golden["rmsnorm"][2]
    got = hip.rmsnorm(T(hip, c["x"]), T(hip, c["w"]), c["eps"]).numpy()[0]
    denom = math.sqrt(14.0 / 3.0 + 1e-6)
    assert np.allclose(got, [2 * v / denom for v in (1, 2, 3)], atol=c["tol"])
    zero = golden["rmsnorm"][1]
    assert np.all(hip.rmsnorm(T(hip, zero["x"]), T(hip, zero["w"]), zero["eps"]).numpy() == 0)


def test_rope(hip, oracle, golden):
    rng = np.random.default_rng(2)
    for m, heads, hd, base, off, rd in [(1, 32, 128, 1e4, 0, None), (5, 8, 128, 5e5, 1000, None),
                                         (3, 2, 64, 1e4, 17, 32), (2, 1, 4, 1.0, 1, None)]:
        x = rng.standard_normal((m, heads * hd)).astype(np.float32)
        got = hip.rope_interleaved(T(hip, x), heads, hd, base, off, rope_dims=rd).numpy()
        want = np.concatenate([oracle.rope(x[:, h * hd:(h + 1) * hd].copy(), base, off, rope_dims=rd)
                               for h in range(heads)], axis=1)
        # device f64 cos/sin may differ from the host's by an ulp before rounding to f32
        assert np.allclose(got, want, rtol=0, atol=2e-6 * max(1.0, float(np.abs(x).max())))
    c = golden["rope"][1]
    y = hip.rope_interleaved(T(hip, c["x"]), 1, 4, c["base"], c["pos_offset"]).numpy()
    assert np.allclose(y[1], [math.cos(1), math.sin(1), -math.sin(1), math.cos(1)], atol=c["tol"])
    with pytest.raises(hip.LiteNNHipError, match="even"):
        hip.rope_interleaved(T(hip, np.zeros((2, 3))), 1, 3)


def test_kv_append_f16_uses_litenn_rounding(hip, oracle, golden):
    rng = np.random.default_rng(3)
    cur = np.concatenate([rng.standard_normal(4096) * 30,
                          [1.0 + 2.0**-11, -(2.0 + 2.0**-10), 65520.0, 3.1e-8, 1e-6, -0.0]]).astype(np.float32)
    width = cur.size // 2
    cache = hip.Tensor((8, width), DT_F16)
    hip.DeviceTraits.ZeroFill(hip.HIP(0), cache.ptr, DT_F16, cache.size)
    hip.kv_append(cache, 3, T(hip, cur), width)
    raw = cache.numpy()  # float16 view
    assert np.array_equal(raw[3:5].reshape(-1).view(np.uint16), oracle.f32_to_f16_bits(cur))
    assert np.all(raw[:3] == 0) and np.all(raw[5:] == 0)
    # whole wavefronts of values that land on normal halves (the converter's short path): exact
    # ties over even and odd lower neighbours, near-ties one f32 ulp to either side, both signs,
    # every half exponent, and the run up to the overflow boundary
    exp = rng.integers(113, 143, 8192).astype(np.uint32)
    kept = rng.integers(0, 1024, 8192).astype(np.uint32)
    dropped = rng.choice(np.array([0x1000, 0x0fff, 0x1001, 0x0000, 0x1fff], np.uint32), 8192)
    sign = rng.integers(0, 2, 8192).astype(np.uint32) << 31
    ties = (sign | (exp << 23) | (kept << 13) | dropped).view(np.float32)
    ties[:64] = np.linspace(65472.0, 65535.0, 64, dtype=np.float32)
    cache = hip.Tensor((2, ties.size), DT_F16)
    hip.kv_append(cache, 1, T(hip, ties), ties.size)
    assert np.array_equal(cache.numpy()[1].view(np.uint16), oracle.f32_to_f16_bits(ties))
    g = golden["kv_append"]
    c32 = hip.Tensor((3, 2), DT_F32)
    hip.kv_append(c32, 0, T(hip, g["past_k"]), 2)
    hip.kv_append(c32, 2, T(hip, g["new_k"]), 2)
    assert np.array_equal(c32.numpy(), np.array(g["expected_k"], np.float32))


@pytest.mark.parametrize("cache_dtype", [DT_F32, DT_F16])
def test_attention_decode(hip, oracle, cache_dtype):
    rng = np.random.default_rng(4)
    for m, past, H, KH, hd in [(1, 0, 4, 4, 128), (1, 383, 32, 32, 128), (1, 1023, 32, 8, 128), (6, 10, 8, 2, 64),
                               (2, 1, 2, 1, 2), (3, 0, 4, 2, 80), (1, 100, 32, 32, 128), (1, 4000, 8, 8, 128),
                               (1, 70, 5, 5, 128), (1, 200, 4, 2, 96), (40, 0, 8, 8, 128)]:
        L = past + m
        q = rng.standard_normal((m, H * hd)).astype(np.float32)
        k = rng.standard_normal((L, KH * hd)).astype(np.float32)
        v = rng.standard_normal((L, KH * hd)).astype(np.float32)
        if cache_dtype == DT_F16:
            k = oracle.f16_to_f32(oracle.f32_to_f16_bits(k))
            v = oracle.f16_to_f32(oracle.f32_to_f16_bits(v))
            kc, vc = T(hip, k, np.float16), T(hip, v, np.float16)
        else:
            kc, vc = T(hip, k), T(hip, v)
        got = hip.attn_decode(T(hip, q), kc, vc, m, past, H, KH, hd).numpy()
        want = np.empty_like(got)
        for h in range(H):
            kvh = h // (H // KH)
            want[:, h * hd:(h + 1) * hd] = oracle.attention_head(
                q[:, h * hd:(h + 1) * hd].copy(), k[:, kvh * hd:(kvh + 1) * hd].copy(),
                v[:, kvh * hd:(kvh + 1) * hd].copy(), 1.0 / math.sqrt(hd), True, 0, past)
        assert rel_l2(got, want) < 1e-5, (m, past, H, KH, hd)


@pytest.mark.parametrize("cache_dtype", [DT_F32, DT_F16])
def test_attention_with_large_scores(hip, oracle, cache_dtype):
    """Scores of order 1e3 (a query fifty times unit scale), one key that dominates, keys that all
    tie, and cache entries near the top of Float16's range: the running maximum keeps every
    exponent in range, on one row cut into key chunks and on several rows."""
    rng = np.random.default_rng(41)
    for m, past, H, KH, hd in [(1, 700, 8, 2, 128), (5, 90, 4, 4, 64), (1, 2000, 4, 1, 128)]:
        L = past + m
        q = (rng.standard_normal((m, H * hd)) * 50).astype(np.float32)
        k = rng.standard_normal((L, KH * hd)).astype(np.float32)
        v = np.clip(rng.standard_normal((L, KH * hd)) * 2.0e4, -6.5e4, 6.5e4).astype(np.float32)
        k[L // 3] = q[0, :KH * hd] / 50 * 4       # aligned with the first query heads: dominates their rows
        k[5:9] = k[5]                               # exact ties
        if cache_dtype == DT_F16:
            k = oracle.f16_to_f32(oracle.f32_to_f16_bits(k))
            v = oracle.f16_to_f32(oracle.f32_to_f16_bits(v))
            kc, vc = T(hip, k, np.float16), T(hip, v, np.float16)
        else:
            kc, vc = T(hip, k), T(hip, v)
        got = hip.attn_decode(T(hip, q), kc, vc, m, past, H, KH, hd).numpy()
        want = _attention_want(oracle, q, k, v, past, H, KH, hd)
        assert np.all(np.isfinite(got))
        assert rel_l2(got, want) < 1e-5, (m, past, H, KH, hd)


def _attention_want(oracle, q, k, v, past, H, KH, hd):
    want = np.empty_like(q)
    for h in range(H):
        kvh = h // (H // KH)
        want[:, h * hd:(h + 1) * hd] = oracle.attention_head(
            q[:, h * hd:(h + 1) * hd].copy(), k[:, kvh * hd:(kvh + 1) * hd].copy(),
            v[:, kvh * hd:(kvh + 1) * hd].copy(), 1.0 / math.sqrt(hd), True, 0, past)
    return want


def test_attention_of_a_prompt_on_the_matrix_cores(hip, oracle):
    """litenn_hip_attn_rows: fp16 operands, f32 softmax and accumulation; tolerance 1e-3 relative L2
    (fp16 rounding of q / sqrt(d) and of the softmax weights).  Ragged row and key counts, a filled
    cache before the rows (past > 0), grouped KV heads, outliers in q."""
    rng = np.random.default_rng(14)
    for m, past, H, KH in [(16, 0, 4, 4), (64, 0, 8, 2), (65, 0, 4, 1), (100, 37, 4, 2), (128, 0, 32, 32),
                           (512, 0, 32, 8), (200, 1000, 8, 8), (17, 63, 2, 2), (48, 64, 2, 1)]:
        hd = 128
        L = past + m
        q = rng.standard_normal((m, H * hd)).astype(np.float32)
        q[rng.integers(0, m, 4), rng.integers(0, H * hd, 4)] *= 30.0
        k = oracle.f16_to_f32(oracle.f32_to_f16_bits(rng.standard_normal((L, KH * hd)).astype(np.float32)))
        v = oracle.f16_to_f32(oracle.f32_to_f16_bits(rng.standard_normal((L, KH * hd)).astype(np.float32)))
        kc, vc = T(hip, k, np.float16), T(hip, v, np.float16)
        want = _attention_want(oracle, q, k, v, past, H, KH, hd)
        got = hip.attn_rows(T(hip, q), kc, vc, m, past, H, KH, hd).numpy()
        assert rel_l2(got, want) < 1e-3, (m, past, H, KH, rel_l2(got, want))
        # every row on its own as well: no row may hide behind the others
        row_err = np.linalg.norm(got - want, axis=1) / np.linalg.norm(want, axis=1)
        assert row_err.max() < 3e-3, (m, past, H, KH, int(row_err.argmax()), float(row_err.max()))
        # the precise flag and every other shape keep the f32 row kernel
        exact = hip.attn_rows(T(hip, q), kc, vc, m, past, H, KH, hd, precise=True).numpy()
        assert rel_l2(exact, want) < 1e-5
    # shapes the tiled kernel does not take: f32 cache, other head widths, fewer than 16 rows
    for m, past, H, KH, hd, f16 in [(40, 3, 4, 2, 128, False), (32, 0, 4, 4, 64, True), (8, 20, 4, 4, 128, True)]:
        L = past + m
        q = rng.standard_normal((m, H * hd)).astype(np.float32)
        k = oracle.f16_to_f32(oracle.f32_to_f16_bits(rng.standard_normal((L, KH * hd)).astype(np.float32)))
        v = oracle.f16_to_f32(oracle.f32_to_f16_bits(rng.standard_normal((L, KH * hd)).astype(np.float32)))
        kc, vc = (T(hip, k, np.float16), T(hip, v, np.float16)) if f16 else (T(hip, k), T(hip, v))
        got = hip.attn_rows(T(hip, q), kc, vc, m, past, H, KH, hd).numpy()
        assert rel_l2(got, _attention_want(oracle, q, k, v, past, H, KH, hd)) < 1e-5


def test_prompt_attention_closed_forms_at_full_size(hip):
    """Properties that need no checker, at the prompt sizes of the 7B and 8B configurations:
    a zero query weighs all visible keys equally, so row r returns the mean of the first
    past + r + 1 value rows; one key that dominates the scores returns that key's value row."""
    rng = np.random.default_rng(15)
    hd = 128
    # the last case puts two workgroups on every CU
    for m, past, H, KH in [(128, 0, 32, 32), (512, 0, 32, 8), (512, 512, 32, 8), (1536, 100, 32, 8)]:
        L = past + m
        k = rng.standard_normal((L, KH * hd)).astype(np.float16)
        v = rng.standard_normal((L, KH * hd)).astype(np.float16)
        kc, vc = T(hip, k, np.float16), T(hip, v, np.float16)
        got = hip.attn_rows(T(hip, np.zeros((m, H * hd), np.float32)), kc, vc, m, past, H, KH, hd).numpy()
        prefix_mean = np.cumsum(v.astype(np.float64), axis=0)[past:] / np.arange(past + 1, L + 1)[:, None]
        want = np.concatenate([prefix_mean[:, (h // (H // KH)) * hd:(h // (H // KH) + 1) * hd] for h in range(H)],
                              axis=1)
        # the weights 1/n are rounded to fp16 before the second product: 2^-11 relative at most
        assert np.max(np.abs(got - want)) < 2e-3 * np.max(np.abs(want)) + 1e-4, (m, past)
        # key 5 carries a huge component along dimension 0 and every query points at it
        k2 = k.copy()
        k2[5, :] = 0
        k2[5, 0::hd] = 300.0
        q = np.zeros((m, H * hd), np.float32)
        q[:, 0::hd] = 10.0
        got = hip.attn_rows(T(hip, q), T(hip, k2, np.float16), vc, m, past, H, KH, hd).numpy()
        first = 0 if past >= 5 else 5 - past  # rows that can see key 5
        want = np.concatenate([np.broadcast_to(v[5, (h // (H // KH)) * hd:(h // (H // KH) + 1) * hd], (m, hd))
                               for h in range(H)], axis=1).astype(np.float32)
        assert np.max(np.abs(got[first:] - want[first:])) < 1e-3


def test_attention_reference_vectors(hip, golden):
    c0, c1 = golden["attention"]
    # causal 3x3, head_dim 2 (scale 1/sqrt(2) is the kernel's own 1/sqrt(head_dim))
    # values are [L, 1] in the reference case; widen to head_dim 2 with a zero column
    v2 = np.concatenate([np.array(c0["v"], np.float32), np.zeros((3, 1), np.float32)], axis=1)
    got = hip.attn_decode(T(hip, c0["q"]), T(hip, c0["k"]), T(hip, v2), 3, 0, 1, 1, 2).numpy()
    q, k, v = (np.array(c0[n], np.float64) for n in ("q", "k", "v"))
    for row in range(3):
        s = (k[:row + 1] @ q[row]) / math.sqrt(2.0)
        p = np.exp(s - s.max())
        p /= p.sum()
        assert abs(got[row, 0] - float(p @ v[:row + 1, 0])) < c0["tol"]
        assert got[row, 1] == 0.0


def test_silu_mul_and_argmax(hip, oracle):
    rng = np.random.default_rng(5)
    g = (rng.standard_normal(11008 * 3) * 4).astype(np.float32)
    u = rng.standard_normal(11008 * 3).astype(np.float32)
    got = hip.silu_mul(T(hip, g), T(hip, u)).numpy()
    assert rel_l2(got, oracle.silu_mul(g, u)) < 1e-6
    x = rng.standard_normal((3, 128256)).astype(np.float32)
    x[1, 500] = x[1, 90000] = 99.0  # tie: lowest index wins
    x[2, :] = -np.inf
    idx = hip.argmax(T(hip, x)).numpy()
    assert idx.tolist() == [int(np.argmax(x[0])), 500, 0]
