"""Decoder runtime (C++ behind the C ABI) against the CPU checker: logits, cache contents,
greedy tokens, the reference's tiny-model vectors and its prefill==decode invariant."""
import math

import numpy as np
import pytest

from conftest import rel_l2
from litenn_amd import synth
from litenn_amd.formats import DT_F16, DT_F32, Q2_K, Q4_0, Q4_K, Q5_0, Q5_K, Q6_K, Q8_0
from llama_util import hip_model, oracle_model, tiny_reference_archive

pytestmark = pytest.mark.gpu


def test_reference_tiny_llama_vectors(hip, golden):
    cfg, tensors = tiny_reference_archive(golden)
    s = 1.0 / math.sqrt(0.25 + 1e-6)
    m = hip_model(hip, cfg, 0, kv_dtype=DT_F32, tensors=tensors)
    logits = m.eval(golden["tiny_llama"]["prefill_tokens"])
    assert np.allclose(logits, [[s, 0, 0], [0, s, 0]], atol=1e-5, rtol=1e-5)
    m.reset()
    m.eval([0])
    assert np.allclose(m.eval([2])[0], [0, 0, s], atol=1e-5)
    k, v = m.get_kv(0)
    assert k.shape == (2, 2) and np.all(k == 0) and np.all(v == 0)
    tied = hip_model(hip, cfg, 0, kv_dtype=DT_F32, tensors=tensors, skip=("output",))
    assert np.allclose(tied.eval([2])[0], [0, 0, s], atol=1e-4)


@pytest.mark.parametrize("fmt", [Q4_0, Q8_0, Q4_K, Q6_K])
@pytest.mark.parametrize("kv", [DT_F16, DT_F32])
def test_logits_and_cache_match_checker(hip, oracle, fmt, kv):
    cfg = synth.tiny_llama(fmt, block_count=3, d_model=512, heads=4, kv_heads=2, ff=1024, vocab=777)
    toks = synth.prompt_tokens(cfg, 9, 1)
    ref = oracle_model(oracle, cfg, 2, kv_f16=(kv == DT_F16))
    dev = hip_model(hip, cfg, 2, kv_dtype=kv)
    want = ref.eval(toks[:6])
    got = dev.eval(toks[:6])
    assert rel_l2(got, want) < 1e-4
    for t in toks[6:]:
        assert rel_l2(dev.eval([t])[0], ref.eval([t])[0]) < 1e-4
    assert dev.past == ref.past == 9
    for layer in (0, 2):
        kd, vd = dev.get_kv(layer)
        kr, vr = ref.get_kv(layer)
        assert rel_l2(kd, kr) < 1e-3 and rel_l2(vd, vr) < 1e-3


def test_prefill_then_decode_matches_full_prefill(hip):
    """The reference's invariant (tests/GGUFImporterTest.cpp:880-908) on the device."""
    cfg = synth.tiny_llama(Q4_K, d_model=256, heads=4, kv_heads=1)
    toks = synth.prompt_tokens(cfg, 8, 4)
    full = hip_model(hip, cfg, 7).eval(toks)
    step = hip_model(hip, cfg, 7)
    step.eval(toks[:1])
    for i in range(1, 8):
        assert rel_l2(step.eval(toks[i:i + 1])[0], full[i]) < 1e-5


@pytest.mark.parametrize("fmt,kvh", [(Q4_0, 4), (Q4_K, 2)])
def test_greedy_tokens_are_exact(hip, oracle, fmt, kvh):
    cfg = synth.tiny_llama(fmt, block_count=4, d_model=512, heads=4, kv_heads=kvh, ff=1024, vocab=2000,
                           context_length=96)
    prompt = synth.prompt_tokens(cfg, 16, 5)
    want, margins = oracle_model(oracle, cfg, 8).generate(prompt, 48)
    dev = hip_model(hip, cfg, 8)
    got, prefill_ms, decode_ms = dev.generate(prompt, 48)
    assert got.tolist() == want.tolist(), (np.nonzero(got != want)[0][:3], margins.min())
    assert dev.past == 16 + 47
    assert decode_ms > 0
    # a second run from a reset cache replays the captured step and must give the same tokens
    dev.reset()
    again, _, _ = dev.generate(prompt, 48)
    assert again.tolist() == want.tolist()
    # graph replay and plain launches agree with eval()-driven decoding
    dev.reset()
    lg = dev.eval(prompt, all_logits=False)
    for i in range(6):
        assert int(np.argmax(lg)) == want[i]
        lg = dev.eval([want[i]], all_logits=False)


def test_mixed_formats_gqa(hip, oracle):
    cfg = synth.tiny_llama(Q4_K, block_count=2, d_model=512, heads=8, kv_heads=2, ff=768, vocab=999,
                           formats={"default": Q4_K, "attn_v": Q6_K, "ffn_down": Q6_K, "output": Q6_K,
                                    "token_embd": Q8_0})
    toks = synth.prompt_tokens(cfg, 5, 6)
    assert rel_l2(hip_model(hip, cfg, 3).eval(toks), oracle_model(oracle, cfg, 3).eval(toks)) < 1e-4


@pytest.mark.parametrize("main_fmt,d_model,ff", [(Q4_K, 512, 768), (Q5_K, 1024, 1024), (Q4_K, 4096, 512)])
def test_single_token_steps_with_a_q6_k_value_projection(hip, oracle, main_fmt, d_model, ff):
    """The K-quant mixes keep attn_v in Q6_K beside Q4_K / Q5_K q and k: the single-token step runs
    the three projections as one launch whose workgroups are shared out between the two formats.
    Logits of every step and the cache against the checker; the tokens of a greedy run exactly."""
    cfg = synth.tiny_llama(main_fmt, block_count=2, d_model=d_model, heads=d_model // 128 * 2, kv_heads=2, ff=ff,
                           vocab=777, formats={"default": main_fmt, "attn_v": Q6_K, "ffn_down": Q6_K, "output": Q6_K})
    toks = synth.prompt_tokens(cfg, 9, 8)
    # Float32 cache: the whole step is held to the checker at a few 1e-6.  Float16 cache: a key or value
    # within an f32 rounding of a half's midpoint lands on the other half on the device (a handful of
    # the 1152 values of a layer do), and this random two-block model amplifies each such 2^-11 about
    # six times per block, so the logits agree to 1e-3 only; what the cache holds is pinned bit for bit
    # by tests/test_gpu_glue.py::test_kv_append_f16_uses_litenn_rounding instead.
    dev32, ref32 = hip_model(hip, cfg, 4, kv_dtype=DT_F32), oracle_model(oracle, cfg, 4, kv_f16=False)
    for t in toks:
        assert rel_l2(dev32.eval([t])[0], ref32.eval([t])[0]) < 3e-5
    for layer in range(cfg.block_count):
        for got, want in zip(dev32.get_kv(layer), ref32.get_kv(layer)):
            assert rel_l2(got, want) < 3e-5
    dev32.close()
    dev, ref = hip_model(hip, cfg, 4), oracle_model(oracle, cfg, 4)
    for t in toks:
        assert rel_l2(dev.eval([t])[0], ref.eval([t])[0]) < 2e-3
    for layer in range(cfg.block_count):
        for got, want in zip(dev.get_kv(layer), ref.get_kv(layer)):
            assert rel_l2(got, want) < 1e-3
    dev.reset()
    ref.reset()
    got, _, _ = dev.generate(toks[:4], 12)
    assert got.tolist() == ref.generate(toks[:4], 12)[0].tolist()


@pytest.mark.parametrize("main_fmt,d_model,rows", [(Q4_K, 512, 5), (Q5_K, 512, 40), (Q5_K, 1024, 352), (Q4_K, 1024, 704)])
def test_prompt_pass_with_a_q6_k_value_projection(hip, oracle, main_fmt, d_model, rows):
    """A prompt's q and k (Q4_K / Q5_K) and v (Q6_K) projections share one matrix-core launch, each
    format's workgroups reading the rows in their decoder's fragment order.  The row counts reach
    the launch's tiles of 16, 32 and 64 rows (the 128-row tile is reached by the 8B shape in
    tests/test_gpu_config5.py).  The Float32 cache holds the k and v projections as the launch left
    them (k after its rotation): they and the logits against the checker."""
    cfg = synth.tiny_llama(main_fmt, block_count=1, d_model=d_model, heads=d_model // 128 * 2, kv_heads=2, ff=512,
                           vocab=333, context_length=rows + 4,
                           formats={"default": main_fmt, "attn_v": Q6_K, "ffn_down": Q6_K, "output": Q6_K})
    toks = synth.prompt_tokens(cfg, rows, 12)
    dev, ref = hip_model(hip, cfg, 6, kv_dtype=DT_F32), oracle_model(oracle, cfg, 6, kv_f16=False)
    got, want = dev.eval(toks, all_logits=False), ref.eval(toks, all_logits=False)
    for got_c, want_c in zip(dev.get_kv(0), ref.get_kv(0)):
        assert got_c.shape == want_c.shape and rel_l2(got_c, want_c) < 1e-3
    assert rel_l2(got, want) < 3e-3
    # and the same rows through the Float32 path
    dev.reset()
    assert rel_l2(dev.eval(toks, all_logits=False, precise=True), want) < 1e-4
    dev.close()


@pytest.mark.parametrize("fmt,ff,rows", [(Q4_K, 5120, 512), (Q4_0, 5024, 500), (Q5_K, 5120, 400), (Q5_0, 5088, 512),
                                        (Q2_K, 5120, 450)])
def test_prompt_pass_with_swiglu_in_the_gate_up_launch(hip, oracle, fmt, ff, rows):
    """With enough rows and a wide enough feed-forward block the gate and up projections of a prompt
    run as one matrix-core launch whose epilogue stores silu(gate) * up.  The second case has a
    feed-forward width that is no multiple of the launch's 128-column strips and a row count that is
    no multiple of its 128-row blocks.  Logits of the last row against the checker, and against the
    Float32 path of the device, which forms the product in its own kernel."""
    cfg = synth.tiny_llama(fmt, block_count=1, d_model=512, heads=8, kv_heads=2, ff=ff, vocab=333,
                           context_length=rows + 4)
    toks = synth.prompt_tokens(cfg, rows, 21)
    dev, ref = hip_model(hip, cfg, 8, kv_dtype=DT_F32), oracle_model(oracle, cfg, 8, kv_f16=False)
    got, want = dev.eval(toks, all_logits=False), ref.eval(toks, all_logits=False)
    assert rel_l2(got, want) < 3e-3
    dev.reset()
    assert rel_l2(dev.eval(toks, all_logits=False, precise=True), want) < 1e-4
    dev.close()


def test_error_paths(hip):
    cfg = synth.tiny_llama(Q4_0, context_length=8)
    m = hip_model(hip, cfg, 1)
    with pytest.raises(hip.LiteNNHipError, match="GetRows index out of range"):
        m.eval([cfg.vocab])
    with pytest.raises(hip.LiteNNHipError, match="context length exceeded"):
        m.eval(np.zeros(9, np.int32))
    with pytest.raises(hip.LiteNNHipError, match="Missing GGUF tensor"):
        hip_model(hip, cfg, 1, skip=("ffn_down",)).eval([0])
    with pytest.raises(hip.LiteNNHipError, match="shape"):
        m.set_tensor("attn_q", 0, Q4_0, np.zeros(18, np.uint8), 1, 32)
    with pytest.raises(hip.LiteNNHipError, match="head counts"):
        hip.LLaMA(1, 64, 4, 3, 64, 10, 8)


# tokens of the 7B-shape fixture that the default (Float16-operand prompt pass) run reproduces before
# its first difference, as measured on an MI355X
DEFAULT_PATH_MATCHING_PREFIX = 256


def _step_figures(logits, probe_indices):
    best = int(np.argmax(logits))
    rest = logits.copy()
    rest[best] = -np.inf
    return best, float(logits[best] - rest.max()), float(np.abs(logits).max()), logits[probe_indices].astype(np.float64)


def test_llama7b_q4_0_greedy_matches_committed_fixture(hip):
    """BASELINE config 4 at full size: the 7B-shape Q4_0 model, prompt 128, 256 greedy tokens, fp16
    KV cache, against tests/golden/llama7b_q4_0_tokens.json (written from the CPU checker by
    tests/golden/make_llama7b_tokens.py; the model and the prompt are rebuilt from the seeds).
    The fixture's continuation is varied (dozens of distinct tokens) and none of its steps is decided
    by less than 1e-3 of the largest logit, so:
      * the device's greedy loop (captured single-token step) must return the same 256 tokens;
      * fed the fixture's tokens step by step, every step's arg-max, top-2 margin and the logits at
        eight fixed vocabulary indices must agree with the checker's to 1e-3 of the largest logit: a
        wrong position, cache row or head mapping at any step shows there even where it would not
        change the token;
      * after a prompt pass on the matrix cores (Float16 operands, about 1e-3 of the logits) the
        same walk holds to 2e-2, and the arg-max wherever the checker's margin is wider than that."""
    import json
    import os
    fx = json.load(open(os.path.join(os.path.dirname(__file__), "golden", "llama7b_q4_0_tokens.json")))
    assert fx["complete"] and fx["new_tokens"] == 256
    tokens, margins = fx["tokens"], np.array(fx["margins"])
    absmax, probes, idx = np.array(fx["logit_absmax"]), np.array(fx["probes"]), fx["probe_indices"]
    # the fixture bites: a varied sequence, no step near a tie
    assert len(set(tokens)) >= 32 and float((margins / absmax).min()) >= 1e-3
    cfg = synth.llama_7b_q4_0(context_length=fx["context_length"])
    assert cfg.name == fx["model"]
    prompt = synth.prompt_tokens(cfg, fx["prompt_length"], fx["prompt_seed"])
    assert prompt[:8].tolist() == fx["prompt_head"]
    dev = hip_model(hip, cfg, fx["seed"])
    # f32-operand prefill (GEMV path), then the captured single-token step
    got, _, _ = dev.generate(prompt, 256)
    assert got.tolist() == tokens, np.nonzero(got != np.array(tokens))[0][:4]
    # the C ABI's default (flags = 0): the prompt pass on the matrix cores with Float16 operands, which
    # is what bench.py times.  Its cache differs from the checker's by about 1e-3, so a step whose
    # margin is that narrow may pick the runner-up, and greedy decoding then follows another path.
    dev.reset()
    fast, _, _ = dev.generate(prompt, 256, precise=False)
    same = fast == np.array(tokens)
    prefix = 256 if same.all() else int(np.argmin(same))
    print("default path (Float16-operand prompt pass): %d of 256 tokens match the fixture, the first %d in a row"
          % (int(same.sum()), prefix), flush=True)
    if prefix < 256:
        print("first difference at step %d: checker margin %.3e of a top logit %.3e"
              % (prefix, margins[prefix], absmax[prefix]), flush=True)
        # a run may leave the fixture's path only at a step the checker itself decided narrowly
        assert margins[prefix] <= 2e-2 * absmax[prefix], (prefix, margins[prefix], absmax[prefix])
    assert prefix >= DEFAULT_PATH_MATCHING_PREFIX, prefix
    for precise, tol in ((True, 1e-3), (False, 2e-2)):
        dev.reset()
        logits = dev.eval(prompt, all_logits=False, precise=precise)
        for step in range(256):
            best, margin, top, pr = _step_figures(logits, idx)
            bar = tol * absmax[step]
            assert abs(top - absmax[step]) <= bar, (precise, step)
            assert np.all(np.abs(pr - probes[step]) <= bar), (precise, step, pr, probes[step])
            if margins[step] > 2 * bar:
                assert best == tokens[step] and abs(margin - margins[step]) <= 2 * bar, (precise, step)
            if step < 255:
                logits = dev.eval([tokens[step]], all_logits=False)
    dev.close()


def test_model_loaded_from_a_gguf_file(hip, oracle, tmp_path):
    """GGUF file -> resident decoder through the library's own reader: same logits as the model built
    tensor by tensor (bit for bit) and as the CPU checker; absent output.weight ties the head to the
    embedding (tools/gguf/LLaMABuilder.cpp:719-733); problems are reported with the reference's texts."""
    import gguf_writer as gw
    from litenn_amd._lib import LiteNNHipError
    cfg = synth.tiny_llama(Q4_K, block_count=2, d_model=512, heads=4, kv_heads=2, ff=768, vocab=333, context_length=48,
                           formats={"default": Q4_K, "attn_v": Q6_K, "ffn_down": Q6_K, "token_embd": Q8_0})
    path = gw.llama_gguf(tmp_path / "m.gguf", cfg, 11)
    toks = synth.prompt_tokens(cfg, 7, 3)
    loaded = hip.LLaMA.from_gguf(str(path))
    built = hip_model(hip, cfg, 11)
    got = loaded.eval(toks)
    assert np.array_equal(got, built.eval(toks))
    assert rel_l2(got, oracle_model(oracle, cfg, 11).eval(toks)) < 1e-4
    assert loaded.past == 7
    loaded.reset()
    built.reset()
    tokens, _, _ = loaded.generate(toks, 5)
    assert tokens.tolist() == built.generate(toks, 5)[0].tolist()
    loaded.close()

    # context override, tied head
    tied_path = gw.llama_gguf(tmp_path / "tied.gguf", cfg, 11, skip=("output",))
    tied = hip.LLaMA.from_gguf(str(tied_path), context_length=16)
    ref_tied = oracle_model(oracle, cfg, 11, skip=("output",))
    assert rel_l2(tied.eval(toks), ref_tied.eval(toks)) < 1e-4
    with pytest.raises(LiteNNHipError):
        tied.eval(list(toks) * 2)  # 7 + 14 > 16 positions
    tied.close()

    with pytest.raises(LiteNNHipError, match="Missing GGUF tensor 'blk.0.ffn_up.weight'"):
        hip.LLaMA.from_gguf(str(gw.llama_gguf(tmp_path / "miss.gguf", cfg, 11, skip=("ffn_up",))))
    with pytest.raises(LiteNNHipError, match="Failed to open GGUF file"):
        hip.LLaMA.from_gguf(str(tmp_path / "absent.gguf"))


def test_model_loaded_from_an_ltnn_archive(hip, oracle, tmp_path):
    """LiteNN model archive (the variable table SaveModel writes for an imported GGUF model,
    Serialization/ModelIO.h:1291-1341) -> resident decoder: the same logits, bit for bit, as the
    same model loaded from a GGUF file, and the CPU checker's within the GEMV bar."""
    import gguf_writer as gw
    import ltnn_writer as lw
    cfg = synth.tiny_llama(Q4_K, block_count=2, d_model=512, heads=4, kv_heads=2, ff=768, vocab=333, context_length=48,
                           formats={"default": Q4_K, "attn_v": Q6_K, "ffn_down": Q6_K, "token_embd": Q8_0})
    toks = synth.prompt_tokens(cfg, 9, 5)
    from_archive = hip.LLaMA.from_gguf(str(lw.llama_ltnn(tmp_path / "m.ltnn", cfg, 13)))
    from_gguf = hip.LLaMA.from_gguf(str(gw.llama_gguf(tmp_path / "m.gguf", cfg, 13)))
    got = from_archive.eval(toks)
    assert np.array_equal(got, from_gguf.eval(toks))
    assert rel_l2(got, oracle_model(oracle, cfg, 13).eval(toks)) < 1e-4
    from_archive.reset()
    from_gguf.reset()
    assert from_archive.generate(toks, 6)[0].tolist() == from_gguf.generate(toks, 6)[0].tolist()
    from_archive.close()
    from_gguf.close()


def test_linear_rope_scaling_and_partial_rotation(hip, oracle, tmp_path):
    """rope.scaling.type = linear (freq_scale = 1 / factor) and rope.dimension_count below the head
    dimension (tools/gguf/LLaMABuilder.cpp:311-348, GGUFImporter.cpp:571-601): prompt pass, single
    steps (fused rotate + append + attention) and the file-loaded model against the CPU checker."""
    import gguf_writer as gw
    cfg = synth.tiny_llama(Q4_0, block_count=2, d_model=512, heads=4, kv_heads=2, ff=768, vocab=300, context_length=40)
    cfg.rope_freq_scale = 0.25
    cfg.rope_dimension_count = 64  # of a head dimension of 128
    toks = synth.prompt_tokens(cfg, 6, 2)
    ref = oracle_model(oracle, cfg, 21)
    dev = hip_model(hip, cfg, 21)
    plain = synth.tiny_llama(Q4_0, block_count=2, d_model=512, heads=4, kv_heads=2, ff=768, vocab=300, context_length=40)
    want = ref.eval(toks)
    assert rel_l2(dev.eval(toks), want) < 1e-4
    assert rel_l2(oracle_model(oracle, plain, 21).eval(toks), want) > 1e-2  # the parameters matter
    for t in (5, 17, 250):  # single-token steps on top of the prompt
        assert rel_l2(dev.eval([t]), ref.eval([t])) < 1e-4
    loaded = hip.LLaMA.from_gguf(str(gw.llama_gguf(tmp_path / "rope.gguf", cfg, 21)))
    dev.reset()
    assert np.array_equal(loaded.eval(toks), dev.eval(toks))
    loaded.close()
    dev.close()


def test_a_context_of_forty_thousand_positions(hip, oracle):
    """Nothing in the runtime holds per-key storage, so the context is bounded by the caches' memory
    only: a model declared with 40000 positions (beyond what an earlier score buffer held) is created,
    evaluates a prompt and single steps like any other (the key chunks of a single row's attention
    follow the cache's current length, not the declared context)."""
    cfg = synth.tiny_llama(Q4_0, block_count=2, d_model=256, heads=4, kv_heads=2, ff=512, vocab=300,
                           context_length=40000)
    toks = synth.prompt_tokens(cfg, 24, 12)
    dev, ref = hip_model(hip, cfg, 5, kv_dtype=DT_F32), oracle_model(oracle, cfg, 5, kv_f16=False)
    assert rel_l2(dev.eval(toks[:20]), ref.eval(toks[:20])) < 5e-5
    for t in toks[20:]:
        assert rel_l2(dev.eval([t])[0], ref.eval([t])[0]) < 5e-5
    dev.reset()
    ref.reset()
    assert dev.generate(toks[:5], 10)[0].tolist() == ref.generate(toks[:5], 10)[0].tolist()
    dev.close()


def test_generation_across_a_doubling_of_the_cache_length(hip, oracle):
    """The number of key chunks a single row's attention is cut into follows the cache length the
    kernel finds on the device, so it changes several times under one captured step: a run that
    starts at 250 rows and ends above 512 must give the checker's tokens, the same tokens as
    evaluation one token at a time (whose launches are sized on the host), and the same cache."""
    cfg = synth.tiny_llama(Q4_0, block_count=2, d_model=256, heads=4, kv_heads=2, ff=512, vocab=300,
                           context_length=2048)
    prompt = synth.prompt_tokens(cfg, 250, 21)
    dev, ref = hip_model(hip, cfg, 6, kv_dtype=DT_F32), oracle_model(oracle, cfg, 6, kv_f16=False)
    got, _, _ = dev.generate(prompt, 280)
    assert dev.past == 250 + 279
    want, _ = ref.generate(prompt, 280)
    assert got.tolist() == want.tolist(), np.nonzero(got != want)[0][:4]
    kv = dev.get_kv(1)
    dev.reset()
    logits = dev.eval(prompt, all_logits=False)
    for step in range(279):
        assert int(np.argmax(logits)) == int(got[step]), step
        logits = dev.eval([int(got[step])], all_logits=False)
    for a, b in zip(dev.get_kv(1), kv):
        assert np.array_equal(a, b)
    dev.close()


@pytest.mark.timeout(300)
def test_generation_through_every_chunk_count(hip, oracle):
    """From 30 cached rows to 3700 under one captured step: the single-row attention goes from one key
    chunk to sixteen on the way.  The device loop must give the checker's tokens and the tokens of
    evaluation one token at a time, and leave the same cache."""
    cfg = synth.tiny_llama(Q4_0, block_count=2, d_model=256, heads=4, kv_heads=2, ff=512, vocab=300,
                           context_length=4096)
    prompt = synth.prompt_tokens(cfg, 30, 22)
    n_new = 3670
    dev, ref = hip_model(hip, cfg, 8, kv_dtype=DT_F32), oracle_model(oracle, cfg, 8, kv_f16=False)
    got, _, _ = dev.generate(prompt, n_new)
    assert dev.past == 30 + n_new - 1
    want, _ = ref.generate(prompt, n_new)
    first_bad = np.nonzero(got != want)[0]
    assert first_bad.size == 0, first_bad[:4]
    kv = dev.get_kv(1)
    dev.reset()
    logits = dev.eval(prompt, all_logits=False)
    for step in range(n_new - 1):
        assert int(np.argmax(logits)) == int(got[step]), step
        logits = dev.eval([int(got[step])], all_logits=False)
    for a, b in zip(dev.get_kv(1), kv):
        assert np.array_equal(a, b)
    dev.close()
