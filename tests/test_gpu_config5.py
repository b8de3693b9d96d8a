"""The 8B-shape grouped-query decoder with mixed Q4_K / Q6_K weights (Q6_K for attn_v, ffn_down and
output, Q4_K elsewhere; 32 query heads over 8 KV heads of 128, FFN 14336, vocabulary 128256, RoPE
base 5e5, Float16 cache), prompt of 512 tokens then 512 decoded tokens at a context of 4096:
  * at reduced depth (2 blocks, every matrix at its full size) against the CPU checker: the prompt
    pass on the matrix cores and through the Float32 path, the cache of both blocks, then 16
    single-token steps;
  * at full depth (32 blocks) through properties that need no checker: the device's greedy loop
    (captured step) and evaluation one token at a time give the same 512 tokens and the same cache,
    the two prompt paths agree, the cache ends at 1023 rows.
Lowering being matched: tools/gguf/LLaMABuilder.cpp:568-668,761-800; shapes and metadata:
tools/gguf/GGUFImporter.cpp:505-642."""
import numpy as np
import pytest

from conftest import rel_l2
from litenn_amd import synth
from litenn_amd.formats import DT_F16, DT_F32, Q4_K, Q6_K
from llama_util import adopt_device_cache, hip_model, oracle_model

pytestmark = pytest.mark.gpu

# a single-token step against the checker once both read the same Float16 cache
F16_TWIN_TOL = 1e-4

MIXED = {"default": Q4_K, "attn_v": Q6_K, "ffn_down": Q6_K, "output": Q6_K}


@pytest.mark.timeout(600)
def test_8b_gqa_shape_two_blocks_against_checker(hip, oracle):
    cfg = synth.LLaMAConfig("llama-8b-gqa-shape-2-blocks", 2, 4096, 32, 8, 14336, 128256, 1024, rope_freq_base=5e5,
                            formats=MIXED)
    tensors = list(synth.llama_tensors(cfg, 11))
    prompt = synth.prompt_tokens(cfg, 512, 3)
    # Float32 cache first: nothing is rounded on the way into the cache, so the Float32 path (prompt
    # rows one by one through the GEMV, then 16 single-token steps fed the checker's greedy tokens)
    # is held to the checker at 1e-4.  With the Float16 cache a key or value within a Float32
    # rounding of a half's midpoint lands on the other half on the device; over 512 keys a few do,
    # and the softmax of this random model turns such a 2^-11 into a few 1e-3 of a step's logits.
    # That those entries, and nothing else, are the difference is shown by a second checker that is
    # handed the device's cache before every step (every entry within one half of its own, counted):
    # its logits agree with the device's as closely as with the Float32 cache (measured: 6e-6 to 1e-5
    # where the checker on its own cache is 4e-5 to 8e-4 away).
    for kv, tol in ((DT_F32, 1e-4), (DT_F16, 1e-2)):
        ref = oracle_model(oracle, cfg, 11, kv_f16=(kv == DT_F16), tensors=tensors)
        dev = hip_model(hip, cfg, 11, kv_dtype=kv, tensors=tensors)
        print("checker: prompt of 512, cache dtype %d" % kv, flush=True)
        want = ref.eval(prompt, all_logits=False)
        got = dev.eval(prompt, all_logits=False, precise=True)
        print("Float32 prompt pass: %.2e" % rel_l2(got, want), flush=True)
        assert rel_l2(got, want) < tol
        assert int(np.argmax(got)) == int(np.argmax(want))
        twin = None
        if kv == DT_F16:
            # the checker again, from here on reading the device's cache
            twin = oracle_model(oracle, cfg, 11, kv_f16=True, tensors=tensors)
            for layer in range(2):
                twin.set_kv(layer, *ref.get_kv(layer))
            twin.set_past(512)
            entries, differing = adopt_device_cache(twin, dev, 2, deeper_slack=1e-2)
            print("cache after the prompt: %d of %d entries differ" % (differing, entries), flush=True)
            assert 0 < differing < entries // 4
        tok = int(np.argmax(want))
        fed = []
        for step in range(16):
            fed.append(tok)
            w = ref.eval([tok], all_logits=False)
            g = dev.eval([tok], all_logits=False)
            err = rel_l2(g, w)
            assert err < tol, step
            if twin is not None:
                err_twin = rel_l2(g, twin.eval([tok], all_logits=False))
                entries, differing = adopt_device_cache(twin, dev, 2, deeper_slack=2e-4)
                print("step %d: %.2e against the checker, %.2e against the checker reading the device's cache "
                      "(%d entries of its new rows differ)" % (step, err, err_twin, differing), flush=True)
                assert err_twin < F16_TWIN_TOL, step
            else:
                print("step %d: %.2e" % (step, err), flush=True)
            top2 = np.sort(w)[-2:]
            if top2[1] - top2[0] > 4 * tol * np.abs(w).max():
                assert int(np.argmax(g)) == int(np.argmax(w))
            tok = int(np.argmax(w))
        assert dev.past == ref.past == 528
        ref_kv = [ref.get_kv(layer) for layer in range(2)]
        for layer in range(2):
            for g, w in zip(dev.get_kv(layer), ref_kv[layer]):
                assert g.shape == (528, 1024) and rel_l2(g, w) < (1e-4 if kv == DT_F32 else 1e-3)
        if kv == DT_F32:
            dev.close()
    # the same on the matrix cores (Float16 operands, tiled attention over 512 rows): every product
    # carries about 4e-4, which two blocks and the softmax over 512 keys turn into a few 1e-3 of
    # the logits; the steps behind it read that cache, so they carry its error, not one of their own
    dev.reset()
    fast = dev.eval(prompt, all_logits=False, precise=False)
    print("matrix-core prompt pass: %.2e" % rel_l2(fast, want), flush=True)
    assert rel_l2(fast, want) < 5e-3
    for layer in range(2):
        for g, w in zip(dev.get_kv(layer), ref_kv[layer]):
            assert rel_l2(g, w[:512]) < 3e-3
    for step, tok in enumerate(fed[:4]):
        g = dev.eval([tok], all_logits=False)
        assert np.all(np.isfinite(g))
    assert dev.past == 516
    dev.close()


@pytest.mark.timeout(600)
def test_8b_gqa_shape_full_depth_prompt_512_then_512_tokens(hip):
    cfg = synth.llama_8b_gqa_mixed(context_length=4096)
    assert (cfg.block_count, cfg.head_count, cfg.head_count_kv, cfg.feed_forward_length, cfg.vocab) == \
        (32, 32, 8, 14336, 128256) and cfg.formats == MIXED
    prompt = synth.prompt_tokens(cfg, 512, 5)
    dev = hip_model(hip, cfg, 9)
    print("model resident", flush=True)
    # the device's own loop: prompt pass on the matrix cores, then the captured single-token step
    tokens, _, _ = dev.generate(prompt, 512, precise=False)
    assert dev.past == 1023  # the last token is returned, not fed
    kv_loop = dev.get_kv(31)
    assert kv_loop[0].shape == (1023, 1024)
    assert len(set(tokens.tolist())) >= 32, "the continuation repeats itself"
    # the same run driven from the host, one evaluation per token
    dev.reset()
    logits = dev.eval(prompt, all_logits=False, precise=False)
    fast_prompt_logits = logits.copy()
    stepped = []
    for step in range(512):
        tok = int(np.argmax(logits))
        stepped.append(tok)
        if step < 511:
            logits = dev.eval([tok], all_logits=False)
    assert stepped == tokens.tolist(), np.nonzero(np.array(stepped) != tokens)[0][:4]
    assert dev.past == 1023
    for a, b in zip(dev.get_kv(31), kv_loop):
        assert np.array_equal(a, b)
    # the two prompt paths (Float16 operands on the matrix cores, Float32 through the GEMV) agree
    dev.reset()
    precise = dev.eval(prompt[:64], all_logits=False, precise=True)
    dev.reset()
    fast = dev.eval(prompt[:64], all_logits=False, precise=False)
    assert rel_l2(fast, precise) < 2e-2
    assert np.all(np.isfinite(fast_prompt_logits))
    dev.close()
