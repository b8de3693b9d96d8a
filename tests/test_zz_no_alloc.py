"""litenn_hip_attn_decode_noalloc (scratch in a fixed device array inside the library) against
litenn_hip_attn_decode (scratch allocated per call): same kernels, so the outputs must agree bit
for bit.  Calls come in pairs on one GPU, the second with a smaller input, so that whatever the
first call left in the shared array (chunk triples, counters) is there when the second runs."""
import ctypes
import math

import numpy as np
import pytest

from litenn_amd import _lib
from litenn_amd.device import DT_F16, DT_F32, Tensor

pytestmark = pytest.mark.gpu


def T(hip, a, dtype=None):
    return hip.Tensor.from_numpy(np.ascontiguousarray(a if dtype is None else a.astype(dtype)))


def _case(hip, rng, m, past, H, KH, hd, cache_dtype):
    L = past + m
    q = rng.standard_normal((m, H * hd)).astype(np.float32)
    k = rng.standard_normal((L, KH * hd)).astype(np.float32)
    v = rng.standard_normal((L, KH * hd)).astype(np.float32)
    if cache_dtype == DT_F16:
        kc, vc = T(hip, k, np.float16), T(hip, v, np.float16)
        k, v = k.astype(np.float16).astype(np.float32), v.astype(np.float16).astype(np.float32)
    else:
        kc, vc = T(hip, k), T(hip, v)
    return q, k, v, T(hip, q), kc, vc


@pytest.mark.parametrize("cache_dtype", [DT_F16, DT_F32])
def test_two_calls_in_a_row_match_the_allocating_entry_point(hip, oracle, cache_dtype):
    rng = np.random.default_rng(77)
    # (rows, keys before the rows, heads, kv heads, head dim): long single rows are cut into chunks
    # that meet in the scratch; each pair runs the larger case first
    pairs = [((1, 4000, 32, 8, 128), (1, 700, 8, 8, 128)),
             ((1, 2047, 40, 40, 128), (1, 130, 4, 2, 96)),
             ((1, 1023, 48, 8, 256), (1, 64, 5, 5, 128)),
             ((1, 900, 16, 4, 64), (5, 17, 8, 2, 64)),
             ((1, 300, 32, 32, 128), (1, 0, 4, 4, 128))]
    for pair in pairs:
        for (m, past, H, KH, hd) in pair:
            print("case", m, past, H, KH, hd, cache_dtype, flush=True)
            q, k, v, qd, kc, vc = _case(hip, rng, m, past, H, KH, hd, cache_dtype)
            want = hip.attn_decode(qd, kc, vc, m, past, H, KH, hd).numpy()
            out = hip.Tensor.from_numpy(np.full((m, H * hd), np.nan, np.float32))
            got = hip.attn_decode_noalloc(qd, kc, vc, m, past, H, KH, hd, out).numpy()
            assert np.array_equal(got, want), (m, past, H, KH, hd)
            # and both agree with the CPU checker
            ref = np.empty_like(want)
            for h in range(H):
                kvh = h // (H // KH)
                ref[:, h * hd:(h + 1) * hd] = oracle.attention_head(
                    q[:, h * hd:(h + 1) * hd].copy(), k[:, kvh * hd:(kvh + 1) * hd].copy(),
                    v[:, kvh * hd:(kvh + 1) * hd].copy(), 1.0 / math.sqrt(hd), True, 0, past)
            err = np.linalg.norm(got - ref) / np.linalg.norm(ref)
            assert err < 1e-5, (m, past, H, KH, hd, err)


def test_repeated_calls_reuse_the_scratch(hip):
    """The same launch three times, then a smaller one, then the first again: the shared array keeps
    the previous call's contents and none of them may leak into a result."""
    rng = np.random.default_rng(78)
    big = _case(hip, rng, 1, 3000, 32, 8, 128, DT_F16)
    small = _case(hip, rng, 1, 250, 8, 8, 128, DT_F16)
    want_big = hip.attn_decode(big[3], big[4], big[5], 1, 3000, 32, 8, 128).numpy()
    want_small = hip.attn_decode(small[3], small[4], small[5], 1, 250, 8, 8, 128).numpy()
    out_big = hip.Tensor.from_numpy(np.zeros((1, 32 * 128), np.float32))
    out_small = hip.Tensor.from_numpy(np.zeros((1, 8 * 128), np.float32))
    for _ in range(3):
        assert np.array_equal(hip.attn_decode_noalloc(big[3], big[4], big[5], 1, 3000, 32, 8, 128, out_big).numpy(),
                              want_big)
    assert np.array_equal(hip.attn_decode_noalloc(small[3], small[4], small[5], 1, 250, 8, 8, 128, out_small).numpy(),
                          want_small)
    assert np.array_equal(hip.attn_decode_noalloc(big[3], big[4], big[5], 1, 3000, 32, 8, 128, out_big).numpy(),
                          want_big)


def test_sizes_beyond_the_scratch_are_refused(hip):
    """64 heads of 256 features cut into 16 chunks (a cache of 4096 rows) need 64 * 16 * 258 floats,
    more than the fixed array holds: an error return with a clear message, no launch.  The
    allocating entry point takes such heads."""
    lib = _lib.load()
    one = ctypes.c_void_p(256)  # never dereferenced: the call fails in validation
    assert lib.litenn_hip_attn_decode_noalloc(0, one, one, one, DT_F16, 1, 4095, 64, 8, 256, one, None) != 0
    assert b"static scratch" in lib.litenn_hip_last_error()
    rng = np.random.default_rng(79)
    q, k, v, qd, kc, vc = _case(hip, rng, 1, 1023, 64, 8, 256, DT_F16)
    assert np.isfinite(hip.attn_decode(qd, kc, vc, 1, 1023, 64, 8, 256).numpy()).all()
    # null operands and a bad cache type are refused like the allocating entry point refuses them
    assert lib.litenn_hip_attn_decode_noalloc(0, one, None, one, DT_F16, 1, 3, 2, 2, 64, one, None) != 0
    assert b"null" in lib.litenn_hip_last_error()
    assert lib.litenn_hip_attn_decode_noalloc(0, one, one, one, 2, 1, 3, 2, 2, 64, one, None) != 0
    assert b"cache dtype" in lib.litenn_hip_last_error()
