"""ctypes binding of the CPU checker in this folder (test infrastructure only).

Only tests, the smoke check and the benchmark's cpu_baseline leg import this
module; the shipped package never does.
"""
from __future__ import annotations

import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, "liblitenn_oracle.so")

Q4_0, Q8_0, Q4_K, Q6_K, F16, F32 = 1, 5, 9, 11, 25, 27

T_TOKEN_EMBD, T_OUTPUT, T_ATTN_Q, T_ATTN_K, T_ATTN_V, T_ATTN_OUTPUT = 0, 1, 2, 3, 4, 5
T_FFN_GATE, T_FFN_UP, T_FFN_DOWN, T_OUTPUT_NORM, T_ATTN_NORM, T_FFN_NORM = 6, 7, 8, 9, 10, 11


def build(force: bool = False) -> str:
    """Compile liblitenn_oracle.so with the Makefile next to this file."""
    if force or not os.path.exists(_SO) or any(
        os.path.getmtime(os.path.join(_HERE, f)) > os.path.getmtime(_SO)
        for f in ("litenn_oracle.c", "litenn_oracle.h", "Makefile")
    ):
        subprocess.check_call(["make", "-C", _HERE, "-B", "liblitenn_oracle.so"], stdout=subprocess.DEVNULL)
    return _SO


_lib = None


def lib() -> C.CDLL:
    global _lib
    if _lib is None:
        if not os.path.exists(_SO):
            build()
        L = C.CDLL(_SO)
        vp, sz, i32, f64 = C.c_void_p, C.c_size_t, C.c_int, C.c_double
        L.oracle_last_error.restype = C.c_char_p
        L.oracle_f16_to_f32.restype = C.c_float
        L.oracle_f16_to_f32.argtypes = [C.c_uint16]
        L.oracle_f32_to_f16.restype = C.c_uint16
        L.oracle_f32_to_f16.argtypes = [C.c_float]
        L.oracle_f16_to_f32_array.argtypes = [vp, vp, sz]
        L.oracle_f32_to_f16_array.argtypes = [vp, vp, sz]
        L.oracle_block_elements.argtypes = [i32]
        L.oracle_block_bytes.argtypes = [i32]
        L.oracle_row_bytes.restype = sz
        L.oracle_row_bytes.argtypes = [i32, sz]
        L.oracle_dequantize_row.argtypes = [i32, vp, vp, sz]
        L.oracle_dequantize.argtypes = [i32, vp, vp, sz, sz]
        L.oracle_transpose.argtypes = [vp, vp, sz, sz]
        L.oracle_matmul_ikj.argtypes = [vp, vp, vp, sz, sz, sz]
        L.oracle_mul_mat_q.argtypes = [i32, vp, sz, sz, vp, sz, vp]
        L.oracle_mul_mat_q_rowwise.argtypes = [i32, vp, sz, sz, vp, sz, vp]
        L.oracle_rmsnorm.argtypes = [vp, vp, f64, sz, sz, vp]
        L.oracle_rope.argtypes = [vp, vp, sz, sz, sz, f64, f64, sz]
        L.oracle_attention_head.argtypes = [vp, sz, vp, vp, sz, sz, sz, f64, i32, sz, sz, vp]
        L.oracle_alibi_slope.argtypes = [sz, sz, f64]
        L.oracle_alibi_slope.restype = f64
        L.oracle_flash_attn_ext.argtypes = [vp, sz, vp, vp, sz, sz, sz, f64, f64, vp, f64, vp, i32, sz, sz, vp]
        L.oracle_silu.argtypes = [vp, vp, sz]
        L.oracle_silu_mul.argtypes = [vp, vp, vp, sz]
        L.oracle_get_rows.argtypes = [vp, sz, sz, vp, sz, vp]
        L.oracle_argmax.restype = C.c_int32
        L.oracle_argmax.argtypes = [vp, sz]
        L.oracle_llama_new.restype = vp
        L.oracle_llama_new.argtypes = [i32] * 8 + [f64] * 3 + [i32, i32]
        L.oracle_llama_free.argtypes = [vp]
        L.oracle_llama_set_tensor.argtypes = [vp, i32, i32, i32, vp, sz, sz]
        L.oracle_llama_past.argtypes = [vp]
        L.oracle_llama_reset.argtypes = [vp]
        L.oracle_llama_eval.argtypes = [vp, vp, i32, vp, vp]
        L.oracle_llama_generate.argtypes = [vp, vp, i32, i32, vp, vp]
        L.oracle_llama_get_kv.argtypes = [vp, i32, vp, vp]
        L.oracle_llama_set_kv.argtypes = [vp, i32, i32, vp, vp]
        L.oracle_llama_set_past.argtypes = [vp, i32]
        L.oracle_set_threads.argtypes = [i32]
        _lib = L
    return _lib


class OracleError(RuntimeError):
    pass


def _check(rc: int) -> None:
    if rc != 0:
        raise OracleError(lib().oracle_last_error().decode())


def _p(a: np.ndarray) -> C.c_void_p:
    return C.c_void_p(a.ctypes.data)


def _f32(a) -> np.ndarray:
    return np.ascontiguousarray(a, dtype=np.float32)


def _u8(a) -> np.ndarray:
    a = np.ascontiguousarray(a)
    return a.view(np.uint8).reshape(-1)


def set_threads(n: int) -> None:
    lib().oracle_set_threads(n)


def f16_to_f32(bits) -> np.ndarray:
    b = np.ascontiguousarray(bits, dtype=np.uint16)
    out = np.empty(b.shape, np.float32)
    lib().oracle_f16_to_f32_array(_p(b), _p(out), b.size)
    return out


def f32_to_f16_bits(x) -> np.ndarray:
    x = _f32(x)
    out = np.empty(x.shape, np.uint16)
    lib().oracle_f32_to_f16_array(_p(x), _p(out), x.size)
    return out


def block_layout(fmt: int) -> tuple[int, int]:
    return lib().oracle_block_elements(fmt), lib().oracle_block_bytes(fmt)


def row_bytes(fmt: int, k: int) -> int:
    return lib().oracle_row_bytes(fmt, k)


def dequantize(fmt: int, raw, rows: int, k: int) -> np.ndarray:
    raw = _u8(raw)
    rb = row_bytes(fmt, k)
    if rb == 0 or raw.size != rows * rb:
        raise OracleError("payload size does not match [rows, k] for this format")
    out = np.empty((rows, k), np.float32)
    _check(lib().oracle_dequantize(fmt, _p(raw), _p(out), rows, k))
    return out


def transpose(a) -> np.ndarray:
    a = _f32(a)
    out = np.empty((a.shape[1], a.shape[0]), np.float32)
    lib().oracle_transpose(_p(a), _p(out), a.shape[0], a.shape[1])
    return out


def matmul_ikj(x, w) -> np.ndarray:
    x, w = _f32(x), _f32(w)
    m, k = x.shape
    k2, n = w.shape
    assert k == k2
    y = np.empty((m, n), np.float32)
    lib().oracle_matmul_ikj(_p(x), _p(w), _p(y), m, k, n)
    return y


def mul_mat_q(fmt: int, wq, n: int, k: int, x, rowwise: bool = True) -> np.ndarray:
    wq, x = _u8(wq), _f32(x).reshape(-1, k)
    if wq.size != n * row_bytes(fmt, k):
        raise OracleError("payload size does not match [n, k] for this format")
    y = np.empty((x.shape[0], n), np.float32)
    fn = lib().oracle_mul_mat_q_rowwise if rowwise else lib().oracle_mul_mat_q
    _check(fn(fmt, _p(wq), n, k, _p(x), x.shape[0], _p(y)))
    return y


def rmsnorm(x, w, eps: float) -> np.ndarray:
    x = _f32(x)
    m, d = x.shape
    y = np.empty_like(x)
    wp = None
    if w is not None:
        w = _f32(w).reshape(-1)
        wp = _p(w)
    lib().oracle_rmsnorm(_p(x), wp, eps, m, d, _p(y))
    return y


def rope(x, base: float = 10000.0, pos_offset: int = 0, freq_scale: float = 1.0, rope_dims: int | None = None) -> np.ndarray:
    x = _f32(x)
    m, d = x.shape
    y = np.empty_like(x)
    lib().oracle_rope(_p(x), _p(y), m, d, d if rope_dims is None else rope_dims, base, freq_scale, pos_offset)
    return y


def attention_head(q, k, v, scale: float = 1.0, causal: bool = False, key_pos_offset: int = 0,
                   query_pos_offset: int = 0) -> np.ndarray:
    q, k, v = _f32(q), _f32(k), _f32(v)
    mq, d = q.shape
    l, dv = v.shape
    assert k.shape == (l, d)
    out = np.empty((mq, dv), np.float32)
    lib().oracle_attention_head(_p(q), mq, _p(k), _p(v), l, d, dv, scale, int(causal), key_pos_offset,
                                query_pos_offset, _p(out))
    return out


def alibi_slope(head_index: int, head_count: int, max_bias: float) -> float:
    return float(lib().oracle_alibi_slope(head_index, head_count, max_bias))


def flash_attn_ext(q, k, v, scale: float = 1.0, softcap: float = 0.0, mask=None, max_bias: float = 0.0,
                   head_index: int = 0, head_count: int = 1, sink=None, causal: bool = False,
                   key_pos_offset: int = 0, query_pos_offset: int = 0) -> np.ndarray:
    """One head of the reference's AddFlashAttnExt with its options (FlashAttnExt.h:17-29,100-228)."""
    q, k, v = _f32(q), _f32(k), _f32(v)
    mq, d = q.shape
    l, dv = v.shape
    assert k.shape == (l, d)
    if max_bias > 0.0 and mask is None:
        raise ValueError("FlashAttnExt maxBias requires an explicit additive mask")
    m_arr = None if mask is None else _f32(mask)
    assert m_arr is None or m_arr.shape == (mq, l)
    s_arr = None if sink is None else np.array([sink], np.float32)
    out = np.empty((mq, dv), np.float32)
    lib().oracle_flash_attn_ext(_p(q), mq, _p(k), _p(v), l, d, dv, scale, softcap,
                                None if m_arr is None else _p(m_arr), alibi_slope(head_index, head_count, max_bias),
                                None if s_arr is None else _p(s_arr), int(causal), key_pos_offset, query_pos_offset,
                                _p(out))
    return out


def silu(x) -> np.ndarray:
    x = _f32(x)
    y = np.empty_like(x)
    lib().oracle_silu(_p(x), _p(y), x.size)
    return y


def silu_mul(gate, up) -> np.ndarray:
    gate, up = _f32(gate), _f32(up)
    y = np.empty_like(gate)
    lib().oracle_silu_mul(_p(gate), _p(up), _p(y), gate.size)
    return y


def get_rows(table, idx) -> np.ndarray:
    table = _f32(table)
    idx = np.ascontiguousarray(idx, dtype=np.int32)
    out = np.empty((idx.size, table.shape[1]), np.float32)
    _check(lib().oracle_get_rows(_p(table), table.shape[0], table.shape[1], _p(idx), idx.size, _p(out)))
    return out


def argmax(x) -> int:
    x = _f32(x)
    return int(lib().oracle_argmax(_p(x), x.size))


class LLaMA:
    """Decoder restatement; holds numpy references so tensor memory stays alive."""

    def __init__(self, n_layer, d_model, n_head, n_kv_head, d_ff, vocab, ctx, rms_eps=1e-5, rope_base=10000.0,
                 rope_freq_scale=1.0, rope_dims=0, kv_f16=False, materialize=False):
        self.vocab, self.d_model, self.n_layer = vocab, d_model, n_layer
        self.n_kv_head, self.head_dim = n_kv_head, d_model // n_head
        self._keep = []
        self._h = lib().oracle_llama_new(n_layer, d_model, n_head, n_kv_head, d_ff, vocab, ctx, rope_dims,
                                         float(rms_eps), float(rope_base), float(rope_freq_scale), int(kv_f16),
                                         int(materialize))
        if not self._h:
            raise OracleError(lib().oracle_last_error().decode())

    def __del__(self):
        if getattr(self, "_h", None):
            lib().oracle_llama_free(self._h)
            self._h = None

    def set_tensor(self, which: int, layer: int, fmt: int, data, n: int, k: int) -> None:
        if fmt == F32:
            arr = _f32(data).reshape(-1)
        else:
            arr = _u8(data)
        self._keep.append(arr)
        _check(lib().oracle_llama_set_tensor(self._h, which, layer, fmt, _p(arr), n, k))

    @property
    def past(self) -> int:
        return lib().oracle_llama_past(self._h)

    def reset(self) -> None:
        lib().oracle_llama_reset(self._h)

    def eval(self, tokens, all_logits: bool = True) -> np.ndarray:
        t = np.ascontiguousarray(tokens, dtype=np.int32).reshape(-1)
        if all_logits:
            out = np.empty((t.size, self.vocab), np.float32)
            _check(lib().oracle_llama_eval(self._h, _p(t), t.size, _p(out), None))
        else:
            out = np.empty((self.vocab,), np.float32)
            _check(lib().oracle_llama_eval(self._h, _p(t), t.size, None, _p(out)))
        return out

    def generate(self, prompt, n_new: int):
        t = np.ascontiguousarray(prompt, dtype=np.int32).reshape(-1)
        out = np.empty((n_new,), np.int32)
        margins = np.empty((n_new,), np.float32)
        _check(lib().oracle_llama_generate(self._h, _p(t), t.size, n_new, _p(out), _p(margins)))
        return out, margins

    def get_kv(self, layer: int):
        w = self.n_kv_head * self.head_dim
        k = np.empty((self.past, w), np.float32)
        v = np.empty((self.past, w), np.float32)
        _check(lib().oracle_llama_get_kv(self._h, layer, _p(k), _p(v)))
        return k, v

    def set_kv(self, layer: int, k, v) -> None:
        """Puts back rows that get_kv returned (bit for bit); set_past then sets the position."""
        k, v = _f32(k), _f32(v)
        _check(lib().oracle_llama_set_kv(self._h, layer, k.shape[0], _p(k), _p(v)))

    def set_past(self, past: int) -> None:
        _check(lib().oracle_llama_set_past(self._h, past))
