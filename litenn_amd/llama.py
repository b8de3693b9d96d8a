"""Decoder runtime front end: the counterpart of lowering with LowerLLaMACausalLMDecode and
running the graph (tools/gguf/LLaMABuilder.cpp:826-872), backed by the C++ runtime in the
library.  Weights are uploaded once in their GGUF block layout and never dequantised in memory.
"""
from __future__ import annotations

import ctypes as C

import numpy as np

from . import _lib
from ._lib import LlamaParams, check
from .device import HIP, Tensor, MATMUL_PRECISE
from .formats import DT_F16, DT_F32, DT_U8, F32

TENSOR_IDS = {"token_embd": 0, "output": 1, "attn_q": 2, "attn_k": 3, "attn_v": 4, "attn_output": 5, "ffn_gate": 6,
              "ffn_up": 7, "ffn_down": 8, "output_norm": 9, "attn_norm": 10, "ffn_norm": 11}


class LLaMA:
    def __init__(self, block_count, embedding_length, head_count, head_count_kv, feed_forward_length, vocab_size,
                 context_length, rms_norm_epsilon=1e-5, rope_freq_base=10000.0, rope_freq_scale=1.0,
                 rope_dimension_count=0, kv_dtype=DT_F16, device: HIP = HIP()):
        self.device = device
        self.vocab_size = vocab_size
        self.kv_width = head_count_kv * (embedding_length // max(head_count, 1))
        self._tensors = []  # device buffers referenced by the runtime
        self._h = C.c_void_p()
        p = LlamaParams(block_count, embedding_length, head_count, head_count_kv, feed_forward_length, vocab_size,
                        context_length, rope_dimension_count, rms_norm_epsilon, rope_freq_base, rope_freq_scale,
                        kv_dtype)
        check(_lib.load().litenn_hip_llama_create(device.deviceIndex, C.byref(p), C.byref(self._h)))

    @classmethod
    def from_config(cls, cfg, kv_dtype=DT_F16, device: HIP = HIP()) -> "LLaMA":
        return cls(cfg.block_count, cfg.embedding_length, cfg.head_count, cfg.head_count_kv,
                   cfg.feed_forward_length, cfg.vocab, cfg.context_length, cfg.rms_eps, cfg.rope_freq_base,
                   rope_freq_scale=getattr(cfg, "rope_freq_scale", 1.0),
                   rope_dimension_count=getattr(cfg, "rope_dimension_count", 0), kv_dtype=kv_dtype, device=device)

    @classmethod
    def from_gguf(cls, path: str, kv_dtype=DT_F16, context_length: int = 0, device: HIP = HIP()) -> "LLaMA":
        """Read a GGUF file (or a LiteNN .ltnn archive of an imported model), upload its decoder
        tensors and return the resident model (the library owns the uploaded buffers).
        context_length > 0 overrides the file's."""
        from .gguf import GGUFFile
        with GGUFFile(path) as f:
            p = f.llama_params()
        self = cls.__new__(cls)
        self.device = device
        self.vocab_size = p.vocab_size
        self.kv_width = p.head_count_kv * (p.embedding_length // max(p.head_count, 1))
        self._tensors = []
        self._h = C.c_void_p()
        check(_lib.load().litenn_hip_llama_load_gguf(device.deviceIndex, str(path).encode(), kv_dtype, context_length,
                                                     C.byref(self._h)))
        return self

    def close(self) -> None:
        if self._h:
            _lib.load().litenn_hip_llama_free(self._h)
            self._h = C.c_void_p()
        for t in self._tensors:
            t.free()
        self._tensors = []

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    def set_tensor(self, kind: str, layer: int, fmt: int, payload: np.ndarray, n: int, k: int) -> None:
        """Upload a host payload (raw GGUF bytes, or f32 for norm weights) and register it."""
        if fmt == F32:
            t = Tensor.from_numpy(np.ascontiguousarray(payload, np.float32).reshape(-1), self.device)
        else:
            t = Tensor.from_numpy(np.ascontiguousarray(payload).view(np.uint8).reshape(-1), self.device)
        self._tensors.append(t)
        check(_lib.load().litenn_hip_llama_set_tensor(self._h, TENSOR_IDS[kind], layer, fmt, t.ptr, n, k))

    def load(self, tensors) -> None:
        for kind, layer, fmt, payload, n, k in tensors:
            self.set_tensor(kind, layer, fmt, payload, n, k)

    @property
    def past(self) -> int:
        return _lib.load().litenn_hip_llama_past(self._h)

    @property
    def block_form(self) -> int:
        """1: a block's attention half runs as one launch in the single-token step; -1: as separate
        launches; 0: not decided yet."""
        return _lib.load().litenn_hip_llama_block_form(self._h)

    def reset(self) -> None:
        check(_lib.load().litenn_hip_llama_reset(self._h))

    def eval(self, tokens, all_logits: bool = True, precise: bool = True) -> np.ndarray:
        t = np.ascontiguousarray(tokens, np.int32).reshape(-1)
        flags = MATMUL_PRECISE if precise else 0
        if all_logits:
            out = np.empty((t.size, self.vocab_size), np.float32)
            check(_lib.load().litenn_hip_llama_eval(self._h, t.ctypes.data, t.size, out.ctypes.data, None, flags))
        else:
            out = np.empty((self.vocab_size,), np.float32)
            check(_lib.load().litenn_hip_llama_eval(self._h, t.ctypes.data, t.size, None, out.ctypes.data, flags))
        return out

    def generate(self, prompt, n_new: int, precise: bool = True):
        """Greedy decode on the device; returns (tokens, prefill_ms, decode_ms)."""
        t = np.ascontiguousarray(prompt, np.int32).reshape(-1)
        out = np.empty((n_new,), np.int32)
        pre, dec = C.c_double(), C.c_double()
        check(_lib.load().litenn_hip_llama_generate(self._h, t.ctypes.data, t.size, n_new, out.ctypes.data,
                                                    MATMUL_PRECISE if precise else 0, C.byref(pre), C.byref(dec)))
        return out, pre.value, dec.value

    def get_kv(self, layer: int):
        k = np.empty((self.past, self.kv_width), np.float32)
        v = np.empty((self.past, self.kv_width), np.float32)
        check(_lib.load().litenn_hip_llama_get_kv(self._h, layer, k.ctypes.data, v.ctypes.data))
        return k, v
