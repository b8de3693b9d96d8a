"""Randomised differential test of the decoder runtime against the CPU checker: model shapes,
formats and sequence lengths are drawn so that every dispatch threshold of the runtime is
crossed (one row / a few rows / sixteen and more rows, head dimensions other than 128, grouped
and full KV heads, partial rotation, both cache types, mixed block formats)."""
import numpy as np
import pytest

from conftest import rel_l2
from litenn_amd import synth
from litenn_amd.formats import (DT_F16, DT_F32, Q2_K, Q3_K, Q4_0, Q4_1, Q4_K, Q5_0, Q5_1, Q5_K, Q6_K, Q8_0)
from llama_util import adopt_device_cache, hip_model, oracle_model

pytestmark = pytest.mark.gpu
SMALL_BLOCK = [Q4_0, Q4_1, Q5_0, Q5_1, Q8_0]
SUPER_BLOCK = [Q2_K, Q3_K, Q4_K, Q5_K, Q6_K]


def draw_config(rng):
    head_dim = int(rng.choice([32, 64, 96, 128, 256]))
    heads = int(rng.choice([1, 2, 4, 6, 8]))
    kv_heads = int(rng.choice([h for h in (1, 2, 3, 4, 6, 8) if heads % h == 0]))
    d_model = heads * head_dim
    super_ok = d_model % 256 == 0
    pool = SMALL_BLOCK + (SUPER_BLOCK if super_ok else [])
    main = int(rng.choice(pool))
    ff = int(rng.choice([256, 512, 768, 1280])) if super_ok else int(rng.choice([96, 352, 512, 800]))
    ff_pool = pool if ff % 256 == 0 else SMALL_BLOCK
    formats = {"default": main}
    for kind in ("attn_v", "attn_k", "ffn_down", "output", "token_embd", "ffn_up"):
        if rng.random() < 0.35:
            # ffn_down's rows are ff wide; everything else here is d_model wide
            formats[kind] = int(rng.choice(ff_pool if kind == "ffn_down" else pool))
    if ff % 256 and formats.get("ffn_down", main) in SUPER_BLOCK:
        formats["ffn_down"] = int(rng.choice(SMALL_BLOCK))
    cfg = synth.tiny_llama(main, block_count=int(rng.integers(1, 3)), d_model=d_model, heads=heads, kv_heads=kv_heads,
                           ff=ff, vocab=int(rng.integers(40, 700)), context_length=96, formats=formats)
    if rng.random() < 0.4:
        cfg.rope_dimension_count = int(rng.choice([d for d in (2, 16, head_dim // 2, head_dim) if d <= head_dim]))
    if rng.random() < 0.3:
        cfg.rope_freq_scale = float(rng.choice([0.5, 0.125]))
    cfg.rope_freq_base = float(rng.choice([1e4, 5e5]))
    return cfg


# Case 53 (d 512, 8/4 heads of 64, ff 512, a Q2_K down projection of exactly 21 pages) once ended
# in a GPU memory fault: the matrix-core kernel fetched a 16-byte piece lying wholly behind the
# tensor.  Fixed in the kernel; tests/test_gpu_gemm.py::test_weights_that_end_on_a_page_boundary.
SEEDS = list(range(64))
# Float16-cache runs, logits of a piece against the checker: [pieces of several rows, whose own rows'
# halves may fall either way; single rows behind a cache the checker shares]
F16_PIECE_TOL = {False: 5e-4, True: 2e-4}  # measured over the 64 cases: at most 1.4e-4 and 7.3e-5


@pytest.mark.parametrize("seed", SEEDS)
def test_random_model_matches_checker(hip, oracle, seed):
    rng = np.random.default_rng(1000 + seed)
    cfg = draw_config(rng)
    kv = DT_F16 if rng.random() < 0.6 else DT_F32
    what = (seed, cfg.embedding_length, cfg.head_count, cfg.head_count_kv, cfg.feed_forward_length, cfg.vocab,
            cfg.formats, cfg.rope_dimension_count, cfg.rope_freq_scale, kv)
    print(what, flush=True)
    ref = oracle_model(oracle, cfg, seed, kv_f16=(kv == DT_F16))
    dev = hip_model(hip, cfg, seed, kv_dtype=kv)
    first = int(rng.choice([1, 2, 3, 5, 15, 16, 17, 33, 40]))
    later = int(rng.choice([2, 4, 9, 16, 21]))
    toks = synth.prompt_tokens(cfg, first + 3 + later + 1, seed)
    # a prompt pass, single-token steps, then several rows on top of a filled cache
    pieces = [toks[:first], toks[first:first + 1], toks[first + 1:first + 2], toks[first + 2:first + 3],
              toks[first + 3:first + 3 + later]]
    synced = 0
    for piece in pieces:
        want = ref.eval(piece)
        got = dev.eval(piece)
        # With the Float16 cache a key or value that lands within an f32 rounding of a half's
        # midpoint rounds the other way on the device (one unit of a half, 5e-4 relative, on a few
        # elements per thousand), and a random block amplifies such a difference several times.  So
        # the checker is handed the device's cache after every piece (every entry held to one half
        # of its own first): a piece then differs from the checker's only by the entries of its own
        # rows that fell the other way, and single rows carry the Float32 cases' sharp bar.
        err = rel_l2(got, want)
        print("piece of %d rows: %.2e" % (len(piece), err), flush=True)
        if kv == DT_F16:
            assert err < F16_PIECE_TOL[len(piece) == 1 and synced > 0], (what, len(piece), dev.past)
            entries, differing = adopt_device_cache(ref, dev, cfg.block_count, slack=2e-5, deeper_slack=2e-2)
            print("  cache: %d of %d entries differ" % (differing, entries), flush=True)
            synced += 1
        else:
            assert err < 5e-5, (what, len(piece), dev.past)
    assert dev.past == ref.past
    kd, vd = dev.get_kv(cfg.block_count - 1)
    kr, vr = ref.get_kv(cfg.block_count - 1)
    assert rel_l2(kd, kr) < 1e-3 and rel_l2(vd, vr) < 1e-3, what
    # the same sequence through the matrix-core prompt path stays within the matmul bar per layer
    dev.reset()
    fast = dev.eval(toks[:first + 3 + later], precise=False)
    ref.reset()
    full = ref.eval(toks[:first + 3 + later])
    # (per row, and every row: the model's attention scores are of order one -- see
    # tests/test_synth_conditioning.py -- so the 3e-4 of the Float16 operands stays a few 1e-4 per
    # matmul and block and no row may stand out.  A wrong tile, row or format shows as errors of
    # order one.)
    rows = np.array([rel_l2(fast[i], full[i]) for i in range(len(full))])
    print("matrix-core rows: median %.2e max %.2e" % (np.median(rows), rows.max()), flush=True)
    assert np.median(rows) < 2e-3 and rows.max() < 5e-3, (what, rows)
    # greedy continuation: device loop and step-by-step evaluation agree with each other
    dev.reset()
    generated = dev.generate(toks[:first], 6)[0]
    dev.reset()
    lg = dev.eval(toks[:first], all_logits=False)
    for t in generated:
        top = np.sort(lg)[-2:]
        if top[1] - top[0] < 1e-4 * max(1.0, abs(top[1])):
            break  # a near-tie may legitimately resolve differently between the two routes
        assert int(np.argmax(lg)) == int(t), what
        lg = dev.eval([int(t)], all_logits=False)
    dev.close()
