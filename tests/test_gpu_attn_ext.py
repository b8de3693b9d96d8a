"""litenn_hip_flash_attn_ext: the reference attention layer's options (logit softcap, additive mask
with ALiBi slope, sinks, offset causal mask; src/LiteNN/Layer/FlashAttnExt.h:17-29,100-228) for
every head at once, through the C ABI, against the CPU checker per head and against the
reference's own test cases (tests/LayerTest.cpp:304-440)."""
import ctypes
import math

import numpy as np
import pytest

from conftest import rel_l2
from litenn_amd import _lib
from litenn_amd.formats import DT_F16, DT_F32
from np_attention import alibi_slope_f64, attention_ext_expected_f64

pytestmark = pytest.mark.gpu


def T(hip, a, dtype=np.float32):
    return hip.Tensor.from_numpy(np.ascontiguousarray(a, dtype))


def _want(oracle, q, k, v, H, KH, hd, **o):
    want = np.empty_like(q)
    sinks = o.pop("sinks", None)
    for h in range(H):
        kvh = h // (H // KH)
        want[:, h * hd:(h + 1) * hd] = oracle.flash_attn_ext(
            q[:, h * hd:(h + 1) * hd].copy(), k[:, kvh * hd:(kvh + 1) * hd].copy(),
            v[:, kvh * hd:(kvh + 1) * hd].copy(), head_index=h, head_count=H,
            sink=None if sinks is None else float(sinks[h]), **o)
    return want


def test_reference_cases(hip, golden):
    """The reference's three attention tests, held to its own double-precision checker at its own
    tolerance.  The mask + softcap + sinks case is head 1 of 4: it is placed there, with other
    queries in the other heads."""
    c0, c1 = golden["attention"]
    q, k, v = (np.array(c0[n], np.float32) for n in "qkv")
    # one value feature per key: v is [keys, 1] in the reference, head_dim 2 here, so v is widened
    v2 = np.repeat(v, 2, axis=1)
    got = hip.flash_attn_ext(T(hip, q), T(hip, k), T(hip, v2), 3, 3, 1, 1, 2, scale=1.0 / math.sqrt(2.0), causal=True).numpy()
    want = attention_ext_expected_f64(q, k, v2, 1.0 / math.sqrt(2.0), causal=True)
    assert np.allclose(got, want, atol=c0["tol"]) and got[0, 0] == 2.0
    q, k, v = (np.array(c1[n], np.float32) for n in "qkv")
    v2 = np.repeat(v, 2, axis=1)
    got = hip.flash_attn_ext(T(hip, q), T(hip, k), T(hip, v2), 1, 3, 1, 1, 2, causal=True, query_position_offset=1).numpy()
    want = attention_ext_expected_f64(q, k, v2, causal=True, query_off=1)
    assert abs(got[0, 0] - want[0, 0]) < c1["tol"] and got[0, 0] < c1["less_than"]
    c = golden["attention_ext"][0]
    rng = np.random.default_rng(5)
    H = c["head_count"]
    q = rng.standard_normal((2, H * 2)).astype(np.float32)
    q[:, 2 * c["head_index"]:2 * c["head_index"] + 2] = np.array(c["q"], np.float32)
    k, v2 = np.array(c["k"], np.float32), np.repeat(np.array(c["v"], np.float32), 2, axis=1)
    sinks = rng.standard_normal(H).astype(np.float32)
    sinks[c["head_index"]] = c["sink"]
    got = hip.flash_attn_ext(T(hip, q), T(hip, k), T(hip, v2), 2, 2, H, 1, 2, scale=c["scale"], max_bias=c["max_bias"],
                             logit_softcap=c["logit_softcap"], mask=T(hip, c["mask"]), sinks=T(hip, sinks)).numpy()
    slope = alibi_slope_f64(c["head_index"], H, c["max_bias"])
    want = attention_ext_expected_f64(c["q"], k, v2, c["scale"], c["logit_softcap"], c["mask"], slope, c["sink"])
    assert np.allclose(got[:, 2 * c["head_index"]:2 * c["head_index"] + 2], want, atol=c["tol"])


@pytest.mark.parametrize("cache_dtype", [DT_F32, DT_F16])
def test_options_against_checker(hip, oracle, cache_dtype):
    rng = np.random.default_rng(31 + cache_dtype)
    shapes = [(1, 1, 1, 1, 2), (3, 17, 4, 2, 64), (1, 300, 8, 8, 128), (5, 40, 6, 3, 96), (2, 64, 12, 4, 80),
              (4, 33, 2, 1, 256), (1, 1000, 4, 1, 128), (7, 9, 5, 5, 16)]
    for case, (m, L, H, KH, hd) in enumerate(shapes * 3):
        q = rng.standard_normal((m, H * hd)).astype(np.float32)
        k = rng.standard_normal((L, KH * hd)).astype(np.float32)
        v = rng.standard_normal((L, KH * hd)).astype(np.float32)
        if cache_dtype == DT_F16:
            k = oracle.f16_to_f32(oracle.f32_to_f16_bits(k))
            v = oracle.f16_to_f32(oracle.f32_to_f16_bits(v))
            kc, vc = T(hip, k, np.float16), T(hip, v, np.float16)
        else:
            kc, vc = T(hip, k), T(hip, v)
        # (scale 1 only for narrow heads: the layer's tanh is (exp(2x) - 1) / (exp(2x) + 1) in f32 and
        # turns into NaN once 2x passes 88, in the reference as here)
        o = {"scale": float(rng.choice([1.0 if hd <= 16 else 0.5 / math.sqrt(hd), 1.0 / math.sqrt(hd), 1.25 / math.sqrt(hd)])),
             "softcap": float(rng.choice([0.0, 0.75, 1.0, 30.0])),
             "causal": bool(rng.random() < 0.5)}
        mask = rng.standard_normal((m, L)).astype(np.float32) if rng.random() < 0.6 else None
        max_bias = float(rng.choice([0.0, 4.0, 8.0])) if mask is not None else 0.0
        sinks = rng.standard_normal(H).astype(np.float32) if rng.random() < 0.5 else None
        key_off = int(rng.integers(0, 3))
        query_off = key_off + int(rng.integers(0, L + 2))
        got = hip.flash_attn_ext(T(hip, q), kc, vc, m, L, H, KH, hd, scale=o["scale"], max_bias=max_bias,
                                 logit_softcap=o["softcap"], mask=None if mask is None else T(hip, mask),
                                 sinks=None if sinks is None else T(hip, sinks), causal=o["causal"],
                                 key_position_offset=key_off, query_position_offset=query_off).numpy()
        want = _want(oracle, q, k, v, H, KH, hd, scale=o["scale"], softcap=o["softcap"], mask=mask, max_bias=max_bias,
                     sinks=sinks, causal=o["causal"], key_pos_offset=key_off, query_pos_offset=query_off)
        assert np.all(np.isfinite(got)), case
        assert rel_l2(got, want) < 2e-5, (case, m, L, H, KH, hd, o, max_bias, sinks is not None)


def test_without_options_it_is_the_decoder_attention(hip, oracle):
    rng = np.random.default_rng(33)
    m, past, H, KH, hd = 3, 50, 8, 2, 128
    L = past + m
    q = rng.standard_normal((m, H * hd)).astype(np.float32)
    k = rng.standard_normal((L, KH * hd)).astype(np.float32)
    v = rng.standard_normal((L, KH * hd)).astype(np.float32)
    a = hip.attn_decode(T(hip, q), T(hip, k), T(hip, v), m, past, H, KH, hd).numpy()
    b = hip.flash_attn_ext(T(hip, q), T(hip, k), T(hip, v), m, L, H, KH, hd, scale=1.0 / math.sqrt(hd), causal=True,
                           query_position_offset=past).numpy()
    assert rel_l2(a, b) < 1e-6
    # a null options pointer: scale 1, nothing else
    lib = _lib.load()
    out = hip.Tensor((m, H * hd))
    tq, tk, tv = T(hip, q), T(hip, k), T(hip, v)
    assert lib.litenn_hip_flash_attn_ext(0, tq.ptr, tk.ptr, tv.ptr, DT_F32, m, L, H, KH, hd, None, out.ptr, None) == 0
    want = _want(oracle, q, k, v, H, KH, hd)
    assert rel_l2(out.numpy(), want) < 2e-5


def test_refusals(hip):
    lib = _lib.load()
    one = ctypes.c_void_p(256)  # never dereferenced: the calls fail in validation

    def call(m=1, keys=4, H=2, KH=2, hd=64, dtype=DT_F32, q=one, out=one, **o):
        opts = _lib.AttnExtOpts(o.get("scale", 1.0), o.get("max_bias", 0.0), o.get("softcap", 0.0), o.get("mask"),
                                o.get("sinks"), int(o.get("causal", False)), o.get("key_off", 0), o.get("query_off", 0))
        rc = lib.litenn_hip_flash_attn_ext(0, q, one, one, dtype, m, keys, H, KH, hd, opts, out, None)
        return rc, lib.litenn_hip_last_error().decode()

    rc, msg = call(max_bias=4.0)
    assert rc != 0 and msg == "HIP FlashAttnExt failed: FlashAttnExt maxBias requires an explicit additive mask"
    rc, msg = call(causal=True, key_off=3, query_off=2)
    assert rc != 0 and "hides every key" in msg
    rc, msg = call(keys=0)
    assert rc != 0 and "no keys" in msg
    rc, msg = call(q=None)
    assert rc != 0 and "null" in msg
    rc, msg = call(dtype=2)
    assert rc != 0 and "cache dtype" in msg
    rc, msg = call(H=3, KH=2)
    assert rc != 0 and "multiple of the KV head count" in msg
    rc, msg = call(hd=257)
    assert rc != 0 and "head dimension" in msg
    rc, msg = call(scale=float("nan"))
    assert rc != 0 and "must be numbers" in msg
    assert call(m=0)[0] == 0  # nothing to do
