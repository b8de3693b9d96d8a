"""The attention half of a decoder block as one launch (RMSNorm + q/k/v rows, rotation + cache append +
attention, output projection; csrc/attn_block.inc) in the single-token step of 4096-wide models
with 32 heads of 128: against the CPU checker, against the same model run through the separate
launches, and with its bounded waits made to run out from the host.
Operator sequence being matched: tools/gguf/LLaMABuilder.cpp:588-653."""
import os

import numpy as np
import pytest

from conftest import rel_l2
from litenn_amd import synth
from litenn_amd.formats import DT_F16, DT_F32, Q4_0, Q4_1, Q4_K, Q5_0, Q5_1, Q5_K, Q6_K, Q8_0
from llama_util import adopt_device_cache, hip_model, oracle_model

pytestmark = pytest.mark.gpu

CASES = {
    # the 7B shape's attention half: every matrix Q4_0, as many KV heads as heads
    "q4_0-32kv": dict(fmt=Q4_0, kv_heads=32, ff=1024, formats=None),
    # the 8B shape's: grouped KV heads, Q4_K with a Q6_K value projection and a Q6_K down projection
    "q4_k-q6_k-8kv": dict(fmt=Q4_K, kv_heads=8, ff=2048,
                          formats={"default": Q4_K, "attn_v": Q6_K, "ffn_down": Q6_K, "output": Q6_K}),
    "q4_k-16kv": dict(fmt=Q4_K, kv_heads=16, ff=1024, formats=None),
}


def make_cfg(case, blocks=2, context=96, **extra):
    c = CASES[case]
    kw = dict(block_count=blocks, d_model=4096, heads=32, kv_heads=c["kv_heads"], ff=c["ff"], vocab=555,
              context_length=context)
    if c["formats"]:
        kw["formats"] = c["formats"]
    rope_dims = extra.pop("rope_dimension_count", 0)
    kw.update(extra)
    cfg = synth.tiny_llama(c["fmt"], **kw)
    if rope_dims:
        cfg.rope_dimension_count = rope_dims
    return cfg


@pytest.fixture
def block_launch_env():
    """Restores the switches the library reads when a model's step is first built."""
    saved = {k: os.environ.get(k) for k in ("LITENN_HIP_ATTN_BLOCK", "LITENN_HIP_ATTN_BLOCK_SPINS")}
    yield
    for k, v in saved.items():
        if v is None:
            os.environ.pop(k, None)
        else:
            os.environ[k] = v


@pytest.mark.parametrize("case", list(CASES))
def test_single_token_steps_match_the_checker(hip, oracle, case, block_launch_env):
    cfg = make_cfg(case)
    toks = synth.prompt_tokens(cfg, 40, 7)
    os.environ.pop("LITENN_HIP_ATTN_BLOCK", None)
    dev = hip_model(hip, cfg, 21)
    ref = oracle_model(oracle, cfg, 21)
    # from an empty cache (the new row is the only key), then on top of a prompt
    for t in toks[:3]:
        got, want = dev.eval([t], all_logits=False), ref.eval([t], all_logits=False)
        assert rel_l2(got, want) < 2e-4, (case, dev.past)
        adopt_device_cache(ref, dev, cfg.block_count, slack=2e-5, deeper_slack=2e-2)
    assert dev.block_form == 1, "the one-launch attention half did not take this shape"
    got, want = dev.eval(toks[3:30]), ref.eval(toks[3:30])
    assert rel_l2(got, want) < 5e-4
    adopt_device_cache(ref, dev, cfg.block_count, slack=2e-5, deeper_slack=2e-2)
    worst = 0.0
    for t in toks[30:]:
        got, want = dev.eval([t], all_logits=False), ref.eval([t], all_logits=False)
        worst = max(worst, rel_l2(got, want))
        adopt_device_cache(ref, dev, cfg.block_count, slack=2e-5, deeper_slack=2e-2)
    print("%s: single-token steps against the checker reading the same cache: %.2e" % (case, worst), flush=True)
    assert worst < 5e-4  # a key or value of the new row itself that rounds the other way shows in its own step
    assert dev.past == ref.past == 40
    # the same model through the separate launches: same cache (bit for bit where the rounding did
    # not fall the other way), same logits to summation order
    os.environ["LITENN_HIP_ATTN_BLOCK"] = "0"
    plain = hip_model(hip, cfg, 21)
    plain.eval(toks[:30], all_logits=False)
    dev.reset()
    dev.eval(toks[:30], all_logits=False)
    for t in toks[30:]:
        a, b = dev.eval([t], all_logits=False), plain.eval([t], all_logits=False)
        assert rel_l2(a, b) < 2e-3
    assert plain.block_form == -1 and dev.block_form == 1
    for layer in range(cfg.block_count):
        for a, b in zip(dev.get_kv(layer), plain.get_kv(layer)):
            assert rel_l2(a, b) < 1e-3
    dev.close()
    plain.close()


@pytest.mark.parametrize("fmt,mix", [(Q4_1, None), (Q5_0, None), (Q5_1, None), (Q5_K, None), (Q5_K, Q6_K)])
def test_the_other_formats_with_an_instance(hip, oracle, fmt, mix):
    formats = {"default": fmt}
    if mix is not None:
        formats.update({"attn_v": mix, "ffn_down": mix, "output": mix})
    cfg = synth.tiny_llama(fmt, block_count=2, d_model=4096, heads=32, kv_heads=8, ff=2048, vocab=444, context_length=48,
                           formats=formats)
    toks = synth.prompt_tokens(cfg, 24, 2)
    dev = hip_model(hip, cfg, 17)
    ref = oracle_model(oracle, cfg, 17)
    dev.eval(toks[:18], all_logits=False)
    ref.eval(toks[:18], all_logits=False)
    adopt_device_cache(ref, dev, 2, slack=2e-5, deeper_slack=2e-2)
    for t in toks[18:]:
        got, want = dev.eval([t], all_logits=False), ref.eval([t], all_logits=False)
        assert rel_l2(got, want) < 5e-4, (fmt, mix, dev.past)
        adopt_device_cache(ref, dev, 2, slack=2e-5, deeper_slack=2e-2)
    assert dev.block_form == 1
    dev.close()


def test_greedy_loop_is_token_exact_and_replays(hip, oracle):
    """The captured step with the one-launch attention half: the device's greedy tokens equal the
    checker's, a second run replays the graph, and stepping from the host gives the same tokens."""
    cfg = make_cfg("q4_0-32kv", blocks=3, context=128)
    prompt = synth.prompt_tokens(cfg, 24, 5)
    want, margins = oracle_model(oracle, cfg, 8).generate(prompt, 40)
    dev = hip_model(hip, cfg, 8)
    got, _, _ = dev.generate(prompt, 40)
    assert dev.block_form == 1
    assert got.tolist() == want.tolist(), (np.nonzero(got != want)[0][:3], margins.min())
    dev.reset()
    again, _, _ = dev.generate(prompt, 40)
    assert again.tolist() == want.tolist()
    dev.reset()
    lg = dev.eval(prompt, all_logits=False)
    for i in range(8):
        assert int(np.argmax(lg)) == want[i]
        lg = dev.eval([want[i]], all_logits=False)
    dev.close()


@pytest.mark.parametrize("case,past,rope_dims", [("q4_0-32kv", 7, 0), ("q4_0-32kv", 8, 64), ("q4_k-q6_k-8kv", 9, 0),
                                                 ("q4_k-16kv", 65, 32), ("q4_k-q6_k-8kv", 1100, 0)])
def test_cache_lengths_around_the_chunk_boundaries_and_partial_rotation(hip, oracle, case, past, rope_dims):
    """A head's cached keys are cut into eight chunks of ceil(len / 8): lengths below, at and just above
    eight keys leave chunks empty or one key long, 65 keys put a second step into the key loop's last
    lanes, 1100 walk several steps per chunk (the 8B shape's lengths); with rope.dimension_count below
    the head width some lanes rotate nothing.  One block, logits against the checker reading the
    device's cache, for the steps that take the cache from `past` to `past + 4` rows."""
    cfg = make_cfg(case, blocks=1, context=past + 8, **({"rope_dimension_count": rope_dims} if rope_dims else {}))
    toks = synth.prompt_tokens(cfg, past + 4, 3)
    dev = hip_model(hip, cfg, 13)
    ref = oracle_model(oracle, cfg, 13)
    dev.eval(toks[:past], all_logits=False)
    ref.eval(toks[:past], all_logits=False)
    adopt_device_cache(ref, dev, 1, slack=2e-5)
    for t in toks[past:]:
        got, want = dev.eval([t], all_logits=False), ref.eval([t], all_logits=False)
        assert rel_l2(got, want) < 3e-4, (case, dev.past)
        adopt_device_cache(ref, dev, 1, slack=2e-5)
    assert dev.block_form == 1 and dev.past == past + 4
    dev.close()


def test_waits_that_run_out_send_the_model_down_the_separate_launches(hip, oracle, block_launch_env):
    """With no polls allowed every wait inside the launch gives up at once (nothing hangs: a
    workgroup that gives up walks on): the step's result is void, the runtime notices, switches to
    the separate launches and repeats the step, so the caller still gets the right logits."""
    cfg = make_cfg("q4_0-32kv", blocks=2)
    toks = synth.prompt_tokens(cfg, 12, 9)
    os.environ["LITENN_HIP_ATTN_BLOCK_SPINS"] = "0"
    dev = hip_model(hip, cfg, 4)
    ref = oracle_model(oracle, cfg, 4)
    want = ref.eval(toks[:8], all_logits=False)
    got = dev.eval(toks[:8], all_logits=False)
    assert rel_l2(got, want) < 2e-4
    for t in toks[8:]:
        got, want = dev.eval([t], all_logits=False), ref.eval([t], all_logits=False)
        assert rel_l2(got, want) < 2e-3
    # either a wait really ran out (and the model gave the launch up) or every flag was already up
    # at the first poll; both leave correct results
    assert dev.block_form in (1, -1)
    print("block form after zero-poll waits:", dev.block_form, flush=True)
    dev.reset()
    ref.reset()
    tokens, _, _ = dev.generate(toks[:8], 10)
    assert tokens.tolist() == ref.generate(toks[:8], 10)[0].tolist()
    dev.close()


def test_shapes_the_launch_is_not_built_for_keep_the_separate_launches(hip, oracle):
    for kw in (dict(fmt=Q8_0, d_model=4096, heads=32, kv_heads=32),   # row slots that do not fit the CU's LDS
               dict(fmt=Q6_K, d_model=4096, heads=32, kv_heads=8),    # column segments of 420 bytes
               dict(fmt=Q4_0, d_model=2048, heads=16, kv_heads=16),   # another width
               dict(fmt=Q4_0, d_model=4096, heads=32, kv_heads=4)):   # KV heads not a multiple of 8
        fmt = kw.pop("fmt")
        cfg = synth.tiny_llama(fmt, block_count=1, ff=512, vocab=333, context_length=16, **kw)
        dev = hip_model(hip, cfg, 2)
        ref = oracle_model(oracle, cfg, 2)
        toks = synth.prompt_tokens(cfg, 4, 1)
        for t in toks:
            assert rel_l2(dev.eval([t], all_logits=False), ref.eval([t], all_logits=False)) < 2e-3
        assert dev.block_form == -1
        dev.close()
    # a Float32 cache as well
    cfg = make_cfg("q4_0-32kv", blocks=1)
    dev = hip_model(hip, cfg, 2, kv_dtype=DT_F32)
    dev.eval([1], all_logits=False)
    assert dev.block_form == -1
    dev.close()


def test_two_instances_stepping_at_once(hip, oracle):
    """Two models of a shape that takes the one-launch attention half, stepping from two host threads
    on their own streams.  Either launch may find only part of its workgroups resident while the
    other runs; its waits are bounded, and a model whose wait ran out falls back to the separate
    launches.  Whatever happened, both must produce the tokens they produce alone."""
    import threading
    cfg = make_cfg("q4_0-32kv", blocks=2, context=96)
    prompts = [synth.prompt_tokens(cfg, 16, s) for s in (3, 4)]
    alone = []
    for i, p in enumerate(prompts):
        dev = hip_model(hip, cfg, 30 + i)
        alone.append(dev.generate(p, 48)[0].tolist())
        assert dev.block_form == 1
        dev.close()
    models = [hip_model(hip, cfg, 30 + i) for i in range(2)]
    got, errors = [None, None], []

    def body(i):
        try:
            got[i] = models[i].generate(prompts[i], 48)[0].tolist()
        except Exception as e:  # reported in the main thread
            errors.append((i, repr(e)))

    threads = [threading.Thread(target=body, args=(i,)) for i in range(2)]
    for t in threads:
        t.start()
    for t in threads:
        t.join(timeout=100)
    assert not any(t.is_alive() for t in threads), "a worker did not finish"
    assert not errors, errors
    print("block forms after stepping side by side:", [m.block_form for m in models], flush=True)
    for i in range(2):
        assert models[i].block_form in (1, -1)
        assert got[i] == alone[i], i
        models[i].close()
