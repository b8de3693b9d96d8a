"""MI355X (gfx950) backend for LiteNN's GGUF-quantised LLaMA path.

The package is a thin ctypes front end over lib/liblitenn_hip.so (hand-written HIP kernels and a
C++ decoder runtime behind the C ABI of include/litenn_hip.h).  Importing it does not touch the
GPU; the first call that needs the library loads it and raises if it has not been built.
"""
from . import formats, synth
from ._lib import LiteNNHipError, LIB_PATH
from .device import (HIP, DeviceTraits, HIPDeviceCount, IsHIPDeviceAvailable, Tensor, argmax, attn_decode, attn_decode_noalloc,
                     attn_rows, flash_attn_ext,
                     dequantize, get_rows_q, kv_append, linear_group, mul_mat_q, rmsnorm, rope_interleaved, silu_mul,
                     MATMUL_PRECISE)
from .llama import LLaMA
from .gguf import GGUFFile

__all__ = ["formats", "synth", "LiteNNHipError", "LIB_PATH", "HIP", "DeviceTraits", "HIPDeviceCount",
           "IsHIPDeviceAvailable", "Tensor", "argmax", "attn_decode", "attn_decode_noalloc", "attn_rows", "flash_attn_ext", "dequantize", "get_rows_q", "kv_append",
           "mul_mat_q", "linear_group", "rmsnorm", "rope_interleaved", "silu_mul", "MATMUL_PRECISE", "LLaMA", "GGUFFile"]
