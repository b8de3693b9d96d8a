"""Loads lib/liblitenn_hip.so and declares the C ABI of include/litenn_hip.h for ctypes."""
from __future__ import annotations

import ctypes as C
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "lib", "liblitenn_hip.so")
HEADER_PATH = os.path.join(os.path.dirname(_HERE), "include", "litenn_hip.h")


class LiteNNHipError(RuntimeError):
    """Raised with the text of litenn_hip_last_error() when an entry point fails."""


class Exec(C.Structure):
    _fields_ = [("stream", C.c_void_p), ("synchronize", C.c_int)]


class LlamaParams(C.Structure):
    _fields_ = [
        ("block_count", C.c_int32), ("embedding_length", C.c_int32), ("head_count", C.c_int32),
        ("head_count_kv", C.c_int32), ("feed_forward_length", C.c_int32), ("vocab_size", C.c_int32),
        ("context_length", C.c_int32), ("rope_dimension_count", C.c_int32),
        ("rms_norm_epsilon", C.c_double), ("rope_freq_base", C.c_double), ("rope_freq_scale", C.c_double),
        ("kv_dtype", C.c_int32),
    ]


class AttnExtOpts(C.Structure):
    """litenn_hip_attn_ext_opts: the reference layer's FlashAttnExtOptions for all heads of one call."""
    _fields_ = [
        ("scale", C.c_double), ("max_bias", C.c_double), ("logit_softcap", C.c_double), ("mask", C.c_void_p),
        ("sinks", C.c_void_p), ("causal", C.c_int), ("key_position_offset", C.c_size_t),
        ("query_position_offset", C.c_size_t),
    ]


class GgufTensor(C.Structure):
    _fields_ = [
        ("name", C.c_char_p), ("ggml_type", C.c_int), ("fmt", C.c_int), ("dtype", C.c_int), ("quantized", C.c_int),
        ("rank", C.c_size_t), ("shape", C.c_size_t * 4), ("file_offset", C.c_size_t), ("bytes", C.c_size_t),
        ("data", C.c_void_p),
    ]


_vp, _sz, _i, _u, _d = C.c_void_p, C.c_size_t, C.c_int, C.c_uint, C.c_double
_szp = C.POINTER(C.c_size_t)
_ex = C.POINTER(Exec)

# name -> argtypes; every function returns int except where noted in _RESTYPES
SIGNATURES = {
    "litenn_hip_last_error": [],
    "litenn_hip_device_count": [],
    "litenn_hip_device_info": [_i, C.c_char_p, _sz],
    "litenn_hip_alloc": [_i, _i, _sz, C.POINTER(_vp)],
    "litenn_hip_free": [_i, _vp, _i, _sz],
    "litenn_hip_zero": [_i, _vp, _i, _sz],
    "litenn_hip_copy_to_host": [_i, _i, _vp, _sz, _i, _vp, _ex],
    "litenn_hip_copy_from_host": [_i, _i, _vp, _i, _vp, _sz, _ex],
    "litenn_hip_convert": [_i, _i, _vp, _sz, _i, _vp, _ex],
    "litenn_hip_unary": [_i, _i, _vp, _i, _szp, _sz, _vp, _ex],
    "litenn_hip_binary": [_i, _i, _vp, _i, _szp, _sz, _vp, _i, _szp, _sz, _vp, _ex],
    "litenn_hip_reduce": [_i, _i, _vp, _i, _szp, _sz, _vp, _sz, _ex],
    "litenn_hip_concat": [_i, _vp, _i, C.POINTER(_vp), _szp, _sz, _sz, _sz, _ex],
    "litenn_hip_slice": [_i, _vp, _i, _szp, _sz, _vp, _sz, _sz, _sz, _ex],
    "litenn_hip_get_rows": [_i, _vp, _i, _szp, _sz, _vp, _i, _szp, _sz, _vp, _ex],
    "litenn_hip_permute": [_i, _vp, _i, _szp, _sz, _vp, _szp, _ex],
    "litenn_hip_mul_mat_q": [_i, _i, _vp, _sz, _sz, _vp, _i, _sz, _vp, _vp, _u, _ex],
    "litenn_hip_mul_mat_q_workspace_bytes": [_sz, _sz],
    "litenn_hip_gemv_last_launch": [C.c_char_p, _sz],
    "litenn_hip_gemm_last_launch": [C.c_char_p, _sz],
    "litenn_hip_mul_mat_q_ws": [_i, _i, _vp, _sz, _sz, _vp, _i, _sz, _vp, _vp, _u, _vp, _sz, _ex],
    "litenn_hip_linear_group": [_i, _i, _sz, C.POINTER(_vp), _szp, _sz, _vp, C.POINTER(_vp), _vp, _vp, _d, _u, _ex],
    "litenn_hip_dequantize": [_i, _i, _vp, _sz, _sz, _vp, _ex],
    "litenn_hip_get_rows_q": [_i, _i, _vp, _sz, _sz, _vp, _sz, _vp, _ex],
    "litenn_hip_rmsnorm": [_i, _vp, _vp, _d, _sz, _sz, _vp, _ex],
    "litenn_hip_rope_interleaved": [_i, _vp, _vp, _sz, _sz, _sz, _sz, _d, _d, _sz, _ex],
    "litenn_hip_kv_append": [_i, _vp, _i, _sz, _vp, _sz, _sz, _ex],
    "litenn_hip_attn_decode": [_i, _vp, _vp, _vp, _i, _sz, _sz, _sz, _sz, _sz, _vp, _ex],
    "litenn_hip_attn_decode_noalloc": [_i, _vp, _vp, _vp, _i, _sz, _sz, _sz, _sz, _sz, _vp, _ex],
    "litenn_hip_attn_rows": [_i, _vp, _vp, _vp, _i, _sz, _sz, _sz, _sz, _sz, _vp, _u, _ex],
    "litenn_hip_flash_attn_ext": [_i, _vp, _vp, _vp, _i, _sz, _sz, _sz, _sz, _sz, C.POINTER(AttnExtOpts), _vp, _ex],
    "litenn_hip_silu_mul": [_i, _vp, _vp, _vp, _sz, _ex],
    "litenn_hip_argmax": [_i, _vp, _sz, _sz, _vp, _ex],
    "litenn_hip_llama_create": [_i, C.POINTER(LlamaParams), C.POINTER(_vp)],
    "litenn_hip_llama_free": [_vp],
    "litenn_hip_llama_set_tensor": [_vp, _i, _i, _i, _vp, _sz, _sz],
    "litenn_hip_llama_reset": [_vp],
    "litenn_hip_llama_past": [_vp],
    "litenn_hip_llama_block_form": [_vp],
    "litenn_hip_llama_eval": [_vp, _vp, _sz, _vp, _vp, _u],
    "litenn_hip_llama_generate": [_vp, _vp, _sz, _sz, _vp, _u, C.POINTER(_d), C.POINTER(_d)],
    "litenn_hip_llama_get_kv": [_vp, _i, _vp, _vp],
    "litenn_gguf_open": [C.c_char_p, C.POINTER(_vp)],
    "litenn_gguf_close": [_vp],
    "litenn_gguf_version": [_vp],
    "litenn_gguf_tensor_count": [_vp],
    "litenn_gguf_metadata_count": [_vp],
    "litenn_gguf_tensor_info": [_vp, _sz, C.POINTER(GgufTensor)],
    "litenn_gguf_find_tensor": [_vp, C.c_char_p, C.POINTER(GgufTensor)],
    "litenn_gguf_metadata_key": [_vp, _sz],
    "litenn_gguf_metadata_u64": [_vp, C.c_char_p, C.POINTER(C.c_uint64)],
    "litenn_gguf_metadata_f64": [_vp, C.c_char_p, C.POINTER(_d)],
    "litenn_gguf_metadata_str": [_vp, C.c_char_p, C.POINTER(C.c_char_p)],
    "litenn_gguf_metadata_bool": [_vp, C.c_char_p, C.POINTER(_i)],
    "litenn_gguf_metadata_array": [_vp, C.c_char_p, C.POINTER(_u), C.POINTER(_sz)],
    "litenn_gguf_llama_params": [_vp, C.POINTER(LlamaParams)],
    "litenn_hip_llama_load_gguf": [_i, C.c_char_p, _i, C.c_int32, C.POINTER(_vp)],
}
_RESTYPES = {
    "litenn_hip_last_error": C.c_char_p, "litenn_hip_mul_mat_q_workspace_bytes": C.c_size_t,
    "litenn_gguf_close": None, "litenn_gguf_version": C.c_uint, "litenn_gguf_tensor_count": C.c_size_t,
    "litenn_gguf_metadata_count": C.c_size_t, "litenn_gguf_metadata_key": C.c_char_p,
}

_lib = None


def load() -> C.CDLL:
    """Return the loaded backend library; raises if it has not been built.

    There is deliberately no fallback: without the HIP library nothing in this package computes.
    """
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise LiteNNHipError(
                f"{LIB_PATH} is missing: build it with `python -m litenn_amd.build` (needs hipcc); "
                "this package has no CPU implementation")
        lib = C.CDLL(LIB_PATH)
        for name, argtypes in SIGNATURES.items():
            fn = getattr(lib, name)
            fn.argtypes = argtypes
            fn.restype = _RESTYPES.get(name, C.c_int)
        _lib = lib
    return _lib


def check(status: int) -> None:
    if status != 0:
        raise LiteNNHipError(load().litenn_hip_last_error().decode())
