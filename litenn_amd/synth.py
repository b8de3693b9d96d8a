"""Seeded synthetic GGUF-layout tensors and LLaMA-shape models.

The laws follow the benchmark configurations: every fp16 scale is
|N(0,1)| * 0.02, every packed quant byte is uniform, activations are N(0,1).
The tensors of a decoder model (llama_tensors) draw their scales with a random
sign, as a quantiser produces them (ggml's Q4_0 scale is the extreme value
/ -8, of either sign): with positive scales only, uniform codes give every
matrix a common offset (Q4_0: -0.5 d per weight) whose rank-one part outweighs
the random part, the hidden state collapses onto the all-ones direction after
a few blocks and greedy decoding repeats one token.  Their spread is
N(0,1) / (CODE_RMS[format] * sqrt(k)), so that a dequantised [n, k] matrix has
entries of root mean square 1/sqrt(k) like an initialised linear layer
whatever its format (0.02 would make a Q4_K weight about 250 times that, the
attention scores of such a model saturate the softmax, and the smallest
rounding difference then picks another key).  The scales of the K-quant
formats land in the fp16 subnormal range, where a trained model's lie too.
Norm weights are drawn from [0.5, 1.5] so that a dropped or misplaced norm
weight changes the result.
Payloads are produced in exactly the byte layout a .gguf file stores
(row-major [n, k/block] blocks), i.e. what LiteNN's importer keeps as a UInt8
variable (tools/gguf/GGUFImporter.cpp:478-491).
"""
from __future__ import annotations

import numpy as np

from .formats import Q4_0, Q4_1, Q5_0, Q5_1, Q8_0, Q2_K, Q3_K, Q4_K, Q5_K, Q6_K, F32, block_layout, row_bytes


def _rng(seed, *stream) -> np.random.Generator:
    return np.random.default_rng([int(seed), *[int(s) for s in stream]])


def _uniform_bytes(rng: np.random.Generator, shape) -> np.ndarray:
    n = int(np.prod(shape))
    return np.frombuffer(rng.bytes(n), np.uint8).reshape(shape)


def _scales_f16(rng: np.random.Generator, shape, signed: bool = False, sigma: float = 0.02) -> np.ndarray:
    d = rng.standard_normal(shape, dtype=np.float32) * np.float32(sigma)
    if not signed:
        d = np.abs(d)
    return d.astype(np.float16).view(np.uint16)


def _put_u16(blocks: np.ndarray, offset: int, values: np.ndarray) -> None:
    blocks[..., offset] = (values & 0xFF).astype(np.uint8)
    blocks[..., offset + 1] = (values >> 8).astype(np.uint8)


def quant_weights(fmt: int, n: int, k: int, seed, *stream, signed_scales: bool = False,
                  scale_sigma: float = 0.02) -> np.ndarray:
    """Random payload of an [n, k] tensor in block format `fmt`: uint8 [n, row_bytes].  Scales are
    |N(0,1)| * scale_sigma, or N(0,1) * scale_sigma with signed_scales."""
    elems, nbytes = block_layout(fmt)
    if k % elems:
        raise ValueError(f"k={k} is not a multiple of the block size {elems}")
    rng = _rng(seed, *stream)
    nb = k // elems
    blocks = np.empty((n, nb, nbytes), np.uint8)
    if fmt == Q8_0:
        _put_u16(blocks, 0, _scales_f16(rng, (n, nb), signed_scales, scale_sigma))
        q = _uniform_bytes(rng, (n, nb, 32)).view(np.int8)
        q = np.where(q == -128, np.int8(-127), q)  # uniform on [-127, 127] up to one remapped code
        blocks[..., 2:] = q.view(np.uint8)
    elif fmt == Q4_0:
        _put_u16(blocks, 0, _scales_f16(rng, (n, nb), signed_scales, scale_sigma))
        blocks[..., 2:] = _uniform_bytes(rng, (n, nb, 16))
    elif fmt == Q4_K:
        _put_u16(blocks, 0, _scales_f16(rng, (n, nb), signed_scales, scale_sigma))
        _put_u16(blocks, 2, _scales_f16(rng, (n, nb), signed_scales, scale_sigma))
        blocks[..., 4:] = _uniform_bytes(rng, (n, nb, 140))
    elif fmt == Q6_K:
        blocks[..., :208] = _uniform_bytes(rng, (n, nb, 208))
        _put_u16(blocks, 208, _scales_f16(rng, (n, nb), signed_scales, scale_sigma))
    elif fmt in (Q4_1, Q5_0, Q5_1, Q5_K):
        # fp16 d [, fp16 m / dmin] first, everything after them uniform bytes
        heads = {Q4_1: 2, Q5_0: 1, Q5_1: 2, Q5_K: 2}[fmt]
        for h in range(heads):
            _put_u16(blocks, 2 * h, _scales_f16(rng, (n, nb), signed_scales, scale_sigma))
        blocks[..., 2 * heads:] = _uniform_bytes(rng, (n, nb, nbytes - 2 * heads))
    elif fmt == Q2_K:
        blocks[..., :80] = _uniform_bytes(rng, (n, nb, 80))
        _put_u16(blocks, 80, _scales_f16(rng, (n, nb), signed_scales, scale_sigma))
        _put_u16(blocks, 82, _scales_f16(rng, (n, nb), signed_scales, scale_sigma))
    elif fmt == Q3_K:
        blocks[..., :108] = _uniform_bytes(rng, (n, nb, 108))
        _put_u16(blocks, 108, _scales_f16(rng, (n, nb), signed_scales, scale_sigma))
    else:
        raise ValueError(f"unsupported format {fmt}")
    return blocks.reshape(n, nb * nbytes)


def activations(m: int, k: int, seed, *stream) -> np.ndarray:
    return _rng(seed, *stream).standard_normal((m, k), dtype=np.float32)


class LLaMAConfig:
    """Shape of a LLaMA-family decoder (tools/gguf/GGUFImporter.cpp:505-642 field names)."""

    def __init__(self, name, block_count, embedding_length, head_count, head_count_kv, feed_forward_length,
                 vocab, context_length, rms_eps=float(np.float32(1e-5)), rope_freq_base=1e4, formats=None,
                 rope_freq_scale=1.0, rope_dimension_count=0):
        self.name = name
        self.block_count = block_count
        self.embedding_length = embedding_length
        self.head_count = head_count
        self.head_count_kv = head_count_kv
        self.feed_forward_length = feed_forward_length
        self.vocab = vocab
        self.context_length = context_length
        self.rms_eps = rms_eps
        self.rope_freq_base = rope_freq_base
        self.rope_freq_scale = rope_freq_scale            # 1 / factor of linear scaling
        self.rope_dimension_count = rope_dimension_count  # 0: the whole head
        # tensor-kind -> block format
        self.formats = formats or {}

    @property
    def head_dim(self) -> int:
        return self.embedding_length // self.head_count

    def fmt(self, kind: str) -> int:
        return self.formats.get(kind, self.formats.get("default", Q4_0))

    def tensor_shapes(self):
        d, hd = self.embedding_length, self.head_dim
        qw, kvw, ff = self.head_count * hd, self.head_count_kv * hd, self.feed_forward_length
        return {
            "attn_q": (qw, d), "attn_k": (kvw, d), "attn_v": (kvw, d), "attn_output": (d, qw),
            "ffn_gate": (ff, d), "ffn_up": (ff, d), "ffn_down": (d, ff),
            "token_embd": (self.vocab, d), "output": (self.vocab, d),
        }

    def matmul_weight_bytes_per_token(self) -> int:
        shapes = self.tensor_shapes()
        per_layer = sum(shapes[k][0] * row_bytes(self.fmt(k), shapes[k][1])
                        for k in ("attn_q", "attn_k", "attn_v", "attn_output", "ffn_gate", "ffn_up", "ffn_down"))
        out = shapes["output"][0] * row_bytes(self.fmt("output"), shapes["output"][1])
        return per_layer * self.block_count + out


def llama_7b_q4_0(context_length: int = 512) -> LLaMAConfig:
    return LLaMAConfig("llama-7b-shape-q4_0", 32, 4096, 32, 32, 11008, 32000, context_length,
                       rope_freq_base=1e4, formats={"default": Q4_0})


def llama_8b_gqa_mixed(context_length: int = 4096) -> LLaMAConfig:
    return LLaMAConfig("llama-8b-gqa-shape-q4_k-q6_k", 32, 4096, 32, 8, 14336, 128256, context_length,
                       rope_freq_base=5e5,
                       formats={"default": Q4_K, "attn_v": Q6_K, "ffn_down": Q6_K, "output": Q6_K})


def tiny_llama(fmt: int = Q4_0, block_count: int = 2, d_model: int = 256, heads: int = 4, kv_heads: int = 2,
               ff: int = 512, vocab: int = 320, context_length: int = 64, formats=None) -> LLaMAConfig:
    return LLaMAConfig("tiny", block_count, d_model, heads, kv_heads, ff, vocab, context_length,
                       formats=formats or {"default": fmt})


TENSOR_KINDS = ("attn_q", "attn_k", "attn_v", "attn_output", "ffn_gate", "ffn_up", "ffn_down")


# root mean square of a dequantised weight at unit scales and uniform code bytes
CODE_RMS = {Q4_0: 4.64, Q4_1: 8.9, Q5_0: 9.3, Q5_1: 18.2, Q8_0: 74.0, Q2_K: 18.7, Q3_K: 43.5, Q4_K: 325.0, Q5_K: 670.0,
            Q6_K: 1355.0}


def model_weights(fmt: int, n: int, k: int, seed, *stream) -> np.ndarray:
    """Payload of a decoder matrix: signed scales sized so that its entries have rms 1/sqrt(k)."""
    return quant_weights(fmt, n, k, seed, *stream, signed_scales=True,
                         scale_sigma=1.0 / (CODE_RMS[fmt] * float(np.sqrt(k))))


def norm_weights(d: int, seed, *stream) -> np.ndarray:
    """f32 [d], uniform on [0.5, 1.5]."""
    return (_rng(seed, *stream).random(d, dtype=np.float32) + np.float32(0.5)).astype(np.float32)


def llama_tensors(cfg: LLaMAConfig, seed: int):
    """Yield (kind, layer, fmt, payload, n, k); matrices follow model_weights, norm weights are f32
    drawn from [0.5, 1.5]."""
    shapes = cfg.tensor_shapes()
    d = cfg.embedding_length
    for kind_id, kind in enumerate(("token_embd", "output")):
        n, k = shapes[kind]
        f = cfg.fmt(kind)
        yield kind, -1, f, model_weights(f, n, k, seed, 1000 + kind_id), n, k
    yield "output_norm", -1, F32, norm_weights(d, seed, 2000), 1, d
    for layer in range(cfg.block_count):
        for kind_id, kind in enumerate(TENSOR_KINDS):
            n, k = shapes[kind]
            f = cfg.fmt(kind)
            yield kind, layer, f, model_weights(f, n, k, seed, layer, kind_id), n, k
        yield "attn_norm", layer, F32, norm_weights(d, seed, 2001, layer), 1, d
        yield "ffn_norm", layer, F32, norm_weights(d, seed, 2002, layer), 1, d


def prompt_tokens(cfg: LLaMAConfig, n: int, seed: int) -> np.ndarray:
    return _rng(seed, 777).integers(0, cfg.vocab, size=n, dtype=np.int32)
