"""Pins of the CPU checker's decoder against the reference's tiny-LLaMA test vectors and the
invariants its tests assert (no GPU)."""
import math

import numpy as np
import pytest

from conftest import rel_l2
from litenn_amd import synth
from litenn_amd.formats import Q4_0, Q4_K, Q6_K, Q8_0
from llama_util import oracle_model, tiny_reference_archive


def test_tiny_llama_reference_golden_logits(oracle, golden):
    cfg, tensors = tiny_reference_archive(golden)
    t = golden["tiny_llama"]
    s = 1.0 / math.sqrt(0.25 + 1e-6)
    m = oracle_model(oracle, cfg, 0, kv_f16=False, materialize=True, tensors=tensors)
    logits = m.eval(t["prefill_tokens"])  # LowerLLaMACausalLM(archive, 2)
    want = np.array([[s, 0, 0], [0, s, 0]], np.float32)
    assert np.allclose(logits, want, atol=t["tol_abs"], rtol=t["tol_rel"])
    # decode graph (seq 1, past 1) with a zero cache: token 2 -> [0, 0, s]
    m.reset()
    m.eval([0])
    assert np.allclose(m.eval([t["decode_token"]])[0], [0, 0, s], atol=t["tol_abs"])
    k, v = m.get_kv(0)
    assert k.shape == (2, 2) and v.shape == (2, 2)  # [past + 1, kvHeads * headDim]
    assert np.all(k == 0) and np.all(v == 0)
    # prefill-then-decode equals the second row of the full prefill (GGUFImporterTest.cpp:880-908)
    m.reset()
    m.eval([0])
    second = m.eval([1])[0]
    assert np.allclose(second, logits[1], atol=t["tol_abs"])
    # tied head: dropping output.weight falls back to token_embd (GGUFImporterTest.cpp:782-798)
    tied = oracle_model(oracle, cfg, 0, kv_f16=False, tensors=tensors, skip=("output",))
    assert np.allclose(tied.eval([2])[0], [0, 0, s], atol=1e-4)


def test_decoder_block_is_identity_with_zero_projections(oracle, golden):
    """GGUFImporterTest.cpp:705-728: with all projections zero the block returns its input, so
    the logits are rmsnorm(embedding) . output for any sequence."""
    cfg, tensors = tiny_reference_archive(golden)
    m = oracle_model(oracle, cfg, 0, kv_f16=False, tensors=tensors)
    logits = m.eval([2, 2, 1, 0])
    s = 1.0 / math.sqrt(0.25 + 1e-6)
    assert np.allclose(logits, np.eye(3, dtype=np.float32)[[2, 2, 1, 0]] * s, atol=1e-5)


@pytest.mark.parametrize("fmt", [Q4_0, Q8_0, Q4_K, Q6_K])
def test_materialised_and_rowwise_models_agree_bitwise(oracle, fmt):
    cfg = synth.tiny_llama(fmt)
    toks = synth.prompt_tokens(cfg, 6, 1)
    a = oracle_model(oracle, cfg, 3, kv_f16=False, materialize=True).eval(toks)
    b = oracle_model(oracle, cfg, 3, kv_f16=False, materialize=False).eval(toks)
    assert np.array_equal(a.view(np.uint32), b.view(np.uint32))
    assert np.all(np.isfinite(a))


@pytest.mark.parametrize("kv_f16", [False, True])
def test_prefill_then_decode_matches_full_prefill(oracle, kv_f16):
    """The reference's own invariant (GGUFImporterTest.cpp:880-908) on a random quantised model
    with GQA: evaluating tokens one at a time against the cache gives the rows of one prefill."""
    cfg = synth.tiny_llama(Q4_K, kv_heads=2, heads=4)
    toks = synth.prompt_tokens(cfg, 7, 2)
    full = oracle_model(oracle, cfg, 4, kv_f16=kv_f16).eval(toks)
    step = oracle_model(oracle, cfg, 4, kv_f16=kv_f16)
    rows = [step.eval(toks[:3])[-1]] + [step.eval([t])[0] for t in toks[3:]]
    assert step.past == 7
    for i, row in enumerate(rows):
        assert rel_l2(row, full[2 + i]) < 1e-5


def test_fp16_cache_holds_litenn_rounded_values(oracle):
    cfg = synth.tiny_llama(Q4_0)
    toks = synth.prompt_tokens(cfg, 5, 3)
    m32 = oracle_model(oracle, cfg, 5, kv_f16=False)
    m16 = oracle_model(oracle, cfg, 5, kv_f16=True)
    m32.eval(toks)
    m16.eval(toks)
    k32, v32 = m32.get_kv(0)  # layer 0 sees identical inputs in both models
    k16, v16 = m16.get_kv(0)
    assert np.array_equal(k16, oracle.f16_to_f32(oracle.f32_to_f16_bits(k32)))
    assert np.array_equal(v16, oracle.f16_to_f32(oracle.f32_to_f16_bits(v32)))
    assert not np.array_equal(k16, k32)


def test_generate_is_argmax_of_eval(oracle):
    cfg = synth.tiny_llama(Q8_0)
    prompt = synth.prompt_tokens(cfg, 4, 9)
    toks, margins = oracle_model(oracle, cfg, 6).generate(prompt, 5)
    m = oracle_model(oracle, cfg, 6)
    lg = m.eval(prompt, all_logits=False)
    for i in range(5):
        assert toks[i] == int(np.argmax(lg))
        srt = np.sort(lg)
        assert abs(margins[i] - (srt[-1] - srt[-2])) < 1e-6
        if i < 4:
            lg = m.eval([toks[i]], all_logits=False)


def test_error_paths(oracle):
    cfg = synth.tiny_llama(Q4_0, context_length=8)
    m = oracle_model(oracle, cfg, 1)
    with pytest.raises(oracle.OracleError, match="out of range"):
        m.eval([cfg.vocab])
    with pytest.raises(oracle.OracleError, match="context length"):
        m.eval(np.zeros(9, np.int32))
    missing = oracle_model(oracle, cfg, 1, skip=("ffn_down",))
    with pytest.raises(oracle.OracleError, match="missing"):
        missing.eval([0])
    with pytest.raises(oracle.OracleError, match="shape"):
        m.set_tensor(2, 0, Q4_0, np.zeros(18, np.uint8), 1, 32)


@pytest.mark.parametrize("fmt,heads,kv_heads,rope_dims,freq_scale", [
    (Q4_0, 8, 2, 0, 1.0), (Q8_0, 6, 3, 0, 1.0), (Q4_K, 4, 1, 32, 0.5), (Q6_K, 4, 4, 0, 1.0)])
def test_block_wiring_against_a_numpy_recomposition_of_the_lowering(oracle, fmt, heads, kv_heads, rope_dims, freq_scale):
    """The checker's decoder against tests/np_llama.py, a float64 recomposition of
    AddLLaMADecoderBlockDecode written from tools/gguf/LLaMABuilder.cpp:568-668 with its own block
    decoders: random non-zero weights, grouped KV heads, several calls so that rows sit at
    positions past + i against a filled cache.  Then the power of the comparison: five plausible
    wiring mistakes planted in the numpy model must all be far outside the tolerance."""
    from np_llama import NumpyLLaMA
    d = 64 * heads if fmt in (Q4_0, Q8_0) else 256
    cfg = synth.LLaMAConfig("wiring", 2, d, heads, kv_heads, 512, 96, 32, formats={"default": fmt},
                            rope_freq_scale=freq_scale, rope_dimension_count=rope_dims)
    if fmt in (Q4_K, Q6_K):
        cfg.feed_forward_length = 512
    tensors = list(synth.llama_tensors(cfg, 31))
    toks = synth.prompt_tokens(cfg, 9, 6)
    pieces = [toks[:5], toks[5:8], toks[8:]]

    def run(model):
        return np.concatenate([np.asarray(model.eval(p), np.float64).reshape(len(p), -1) for p in pieces])

    ref = oracle_model(oracle, cfg, 31, kv_f16=False, tensors=tensors)
    want = run(NumpyLLaMA(cfg, tensors))
    got = run(ref)
    assert rel_l2(got, want) < 1e-5
    # the cache holds rotated keys and plain values at rows 0 .. past
    nm = NumpyLLaMA(cfg, tensors)
    run(nm)
    for layer in range(cfg.block_count):
        k, v = ref.get_kv(layer)
        assert rel_l2(k, nm.k[layer]) < 1e-5 and rel_l2(v, nm.v[layer]) < 1e-5
    mistakes = ["keys_not_rotated", "residual_from_norm", "gate_up_swapped", "positions_from_zero"]
    if kv_heads not in (1, heads):
        mistakes.append("kv_head_modulo")
    for mistake in mistakes:
        assert rel_l2(run(NumpyLLaMA(cfg, tensors, mistake=mistake)), want) > 1e-2, mistake
