"""Helpers shared by the decoder tests: build the same synthetic model in the CPU checker and
in the HIP runtime."""
import numpy as np

from litenn_amd import synth
from litenn_amd.formats import F32

ORACLE_IDS = {"token_embd": 0, "output": 1, "attn_q": 2, "attn_k": 3, "attn_v": 4, "attn_output": 5, "ffn_gate": 6,
              "ffn_up": 7, "ffn_down": 8, "output_norm": 9, "attn_norm": 10, "ffn_norm": 11}


def oracle_model(oracle, cfg, seed, kv_f16=True, materialize=False, tensors=None, skip=()):
    m = oracle.LLaMA(cfg.block_count, cfg.embedding_length, cfg.head_count, cfg.head_count_kv,
                     cfg.feed_forward_length, cfg.vocab, cfg.context_length, rms_eps=cfg.rms_eps,
                     rope_base=cfg.rope_freq_base, rope_freq_scale=cfg.rope_freq_scale,
                     rope_dims=cfg.rope_dimension_count, kv_f16=kv_f16, materialize=materialize)
    for kind, layer, fmt, payload, n, k in (tensors if tensors is not None else synth.llama_tensors(cfg, seed)):
        if kind in skip:
            continue
        m.set_tensor(ORACLE_IDS[kind], layer, fmt, payload, n, k)
    return m


def hip_model(hip, cfg, seed, kv_dtype=None, tensors=None, skip=()):
    from litenn_amd.formats import DT_F16
    m = hip.LLaMA.from_config(cfg, kv_dtype=DT_F16 if kv_dtype is None else kv_dtype)
    for kind, layer, fmt, payload, n, k in (tensors if tensors is not None else synth.llama_tensors(cfg, seed)):
        if kind in skip:
            continue
        m.set_tensor(kind, layer, fmt, payload, n, k)
    return m


def tiny_reference_archive(golden):
    """The reference's BuildTinyLLaMAArchive (tests/GGUFImporterTest.cpp:220-290) as GGUF-layout
    [out, in] f32 tensors: its token_embd is feature-major [d, vocab] and its linears are stored
    [in, out], so both are transposed here."""
    t = golden["tiny_llama"]
    hp = t["hparams"]
    cfg = synth.LLaMAConfig("reference-tiny", hp["block_count"], hp["embedding_length"], hp["head_count"],
                            hp["head_count_kv"], hp["feed_forward_length"], 3, hp["context_length"],
                            rms_eps=hp["rms_eps"], rope_freq_base=hp["rope_freq_base"], formats={"default": F32})
    d, hd = cfg.embedding_length, cfg.head_dim
    tensors = [
        ("token_embd", -1, F32, np.array(t["token_embd_feature_major_4x3"], np.float32).T.copy(), 3, d),
        ("output", -1, F32, np.array(t["output_in_out_4x3"], np.float32).T.copy(), 3, d),
        ("output_norm", -1, F32, np.full(d, t["norm_weights"], np.float32), 1, d),
    ]
    shapes = cfg.tensor_shapes()
    for kind in synth.TENSOR_KINDS:
        n, k = shapes[kind]
        tensors.append((kind, 0, F32, np.full((n, k), t["all_block_projections"], np.float32), n, k))
    tensors.append(("attn_norm", 0, F32, np.full(d, t["norm_weights"], np.float32), 1, d))
    tensors.append(("ffn_norm", 0, F32, np.full(d, t["norm_weights"], np.float32), 1, d))
    return cfg, tensors


def adopt_device_cache(ref, dev, layers, slack=1e-5, deeper_slack=None):
    """Float16 caches: the device and the checker add a projection's products in different orders, so a
    key or value reaches the conversion a few 1e-6 of the tensor's size apart, and one that falls
    that close to the midpoint between two halves lands on the other half.  Holds every entry of
    the two caches to one half (of the larger magnitude) plus `slack` times the tensor's rms
    (`deeper_slack` for the blocks behind the first, whose inputs already carry the first block's
    differences), then puts the device's rows into the checker's cache (oracle_llama_set_kv), so
    that the checker's next rows are computed against exactly what the device attends to.
    Returns (entries, entries that differ)."""
    entries = differing = 0
    for layer in range(layers):
        kd, vd = dev.get_kv(layer)
        kr, vr = ref.get_kv(layer)
        allow = slack if layer == 0 or deeper_slack is None else deeper_slack
        for got, want in ((kd, kr), (vd, vr)):
            assert np.array_equal(got.astype(np.float16).astype(np.float32), got)  # the cache holds halves
            apart = np.abs(got - want)
            half = np.spacing(np.maximum(np.abs(got), np.abs(want)).astype(np.float16)).astype(np.float32)
            bound = half + allow * float(np.sqrt(np.mean(np.square(want, dtype=np.float64))))
            assert np.all(apart <= bound), (layer, float((apart / bound).max()), int((apart > bound).sum()))
            entries += apart.size
            differing += int(np.count_nonzero(apart))
        ref.set_kv(layer, kd, vd)
    return entries, differing
