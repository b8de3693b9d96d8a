"""The reference's LLaMA lowering recomposed in numpy float64, written from the graph builders
themselves and sharing no code with oracle/: a second opinion on the CPU checker's block wiring.

Followed, line by line:
  tools/gguf/LLaMABuilder.cpp:738-759   token embedding = GetRows of the [vocab, d] table
  tools/gguf/LLaMABuilder.cpp:568-668   AddLLaMADecoderBlockDecode: norm, q/k/v, rotate keys per KV
                                        head at positionOffset, append to the cache, per query head
                                        attention against kv head = head / groups, concat, output
                                        projection + residual, norm, SwiGLU + residual
  tools/gguf/LLaMABuilder.cpp:311-348   AddLLaMARoPE: first rope.dimension_count features rotate, tail kept
  src/LiteNN/Layer/RoPE.h:24-117        interleaved pairs (2i, 2i+1), angle = pos * base^(-2i/n) * scale
  tools/gguf/LLaMABuilder.cpp:376-404   scale 1/sqrt(headDim), causal, query position = offset + row
  src/LiteNN/Layer/SwiGLU.h:59-69       down(silu(gate(x)) * up(x))
  src/LiteNN/Layer/RMSNorm.h:41-57      x / sqrt(mean(x^2) + eps) * w
  tools/gguf/LLaMABuilder.cpp:761-800   final norm, lm head (tied to token_embd when output is absent)
A linear layer of the lowered graph multiplies by the dequantised GGUF tensor transposed
(tools/gguf/LLaMABuilder.cpp:225-230), i.e. y = x . W^T for W stored [out, in]."""
from __future__ import annotations

import numpy as np

import np_decoders
from litenn_amd.formats import F32


def _weights(tensors):
    """{(kind, layer): float64 [n, k]} from (kind, layer, fmt, payload, n, k) records."""
    out = {}
    for kind, layer, fmt, payload, n, k in tensors:
        if fmt == F32:
            w = np.asarray(payload, np.float32).reshape(n, k) if n > 1 else np.asarray(payload, np.float32).reshape(-1)
        else:
            w = np_decoders.decode(fmt, np.ascontiguousarray(payload).view(np.uint8).reshape(n, -1), k)
        out[(kind, layer)] = w.astype(np.float64)
    return out


def _rmsnorm(x, w, eps):
    return x / np.sqrt(np.mean(x * x, axis=-1, keepdims=True) + eps) * w


def _rope(x, offset, base, scale, rope_dims):
    """x [rows, head_dim]; rows sit at positions offset, offset + 1, ..."""
    rows, hd = x.shape
    n = rope_dims if rope_dims else hd
    half = n // 2
    pos = (offset + np.arange(rows, dtype=np.float64))[:, None]
    inv = np.power(base, -2.0 * np.arange(half, dtype=np.float64) / n)[None, :]
    ang = pos * inv * scale
    c, s = np.cos(ang), np.sin(ang)
    first, second = x[:, 0:n:2], x[:, 1:n:2]
    out = x.copy()
    out[:, 0:n:2] = first * c - second * s
    out[:, 1:n:2] = first * s + second * c
    return out


def _silu(x):
    return x / (1.0 + np.exp(-x))


class NumpyLLaMA:
    """Keeps a float64 KV cache per block; eval() is LowerLLaMACausalLMDecode(sequenceLength = len(tokens),
    pastLength = positionOffset = past)."""

    def __init__(self, cfg, tensors, mistake=None):
        """mistake: None, or one of the wiring errors the comparison has to notice --
        "kv_head_modulo" (kv head = head % kvHeads), "keys_not_rotated", "residual_from_norm"
        (residual taken after the norm), "gate_up_swapped", "positions_from_zero" (rows of a later
        call rotated as if the cache were empty)."""
        self.mistake = mistake
        self.trace = None  # a list here receives (layer, head, scores [rows, keys]) of every attention
        self.cfg = cfg
        self.w = _weights(tensors)
        self.past = 0
        kvw = cfg.head_count_kv * cfg.head_dim
        self.k = [np.zeros((0, kvw)) for _ in range(cfg.block_count)]
        self.v = [np.zeros((0, kvw)) for _ in range(cfg.block_count)]

    def eval(self, tokens):
        cfg, w = self.cfg, self.w
        hd, heads, kvh = cfg.head_dim, cfg.head_count, cfg.head_count_kv
        groups = heads // kvh
        offset = self.past
        rope_offset = 0 if self.mistake == "positions_from_zero" else offset
        h = w[("token_embd", -1)][np.asarray(tokens, np.int64)]
        rows = h.shape[0]
        for layer in range(cfg.block_count):
            xn = _rmsnorm(h, w[("attn_norm", layer)], cfg.rms_eps)
            q = xn @ w[("attn_q", layer)].T
            k = xn @ w[("attn_k", layer)].T
            v = xn @ w[("attn_v", layer)].T
            k_rot = np.concatenate([_rope(k[:, j * hd:(j + 1) * hd], rope_offset, cfg.rope_freq_base,
                                          cfg.rope_freq_scale, cfg.rope_dimension_count) for j in range(kvh)], axis=1)
            if self.mistake == "keys_not_rotated":
                k_rot = k
            self.k[layer] = np.concatenate([self.k[layer], k_rot], axis=0)
            self.v[layer] = np.concatenate([self.v[layer], v], axis=0)
            total = offset + rows
            ctx = []
            for head in range(heads):
                kv_head = head % kvh if self.mistake == "kv_head_modulo" else head // groups
                qh = _rope(q[:, head * hd:(head + 1) * hd], rope_offset, cfg.rope_freq_base, cfg.rope_freq_scale,
                           cfg.rope_dimension_count)
                kk = self.k[layer][:, kv_head * hd:(kv_head + 1) * hd]
                vv = self.v[layer][:, kv_head * hd:(kv_head + 1) * hd]
                scores = qh @ kk.T / np.sqrt(float(hd))
                # causal: the query at position offset + i sees keys at positions 0 .. offset + i
                visible = np.arange(total)[None, :] <= (offset + np.arange(rows))[:, None]
                scores = np.where(visible, scores, -np.inf)
                if self.trace is not None:
                    self.trace.append((layer, head, scores.copy()))
                p = np.exp(scores - scores.max(axis=1, keepdims=True))
                p /= p.sum(axis=1, keepdims=True)
                ctx.append(p @ vv)
            merged = np.concatenate(ctx, axis=1)
            h = (xn if self.mistake == "residual_from_norm" else h) + merged @ w[("attn_output", layer)].T
            xn = _rmsnorm(h, w[("ffn_norm", layer)], cfg.rms_eps)
            gate, up = xn @ w[("ffn_gate", layer)].T, xn @ w[("ffn_up", layer)].T
            if self.mistake == "gate_up_swapped":
                gate, up = up, gate
            gated = _silu(gate) * up
            h = h + gated @ w[("ffn_down", layer)].T
        self.past += rows
        xn = _rmsnorm(h, w[("output_norm", -1)], cfg.rms_eps)
        head_w = w.get(("output", -1), w[("token_embd", -1)])
        return xn @ head_w.T
