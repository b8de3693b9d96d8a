"""ctypes front end of the HIP backend, named after the reference's device interface.

`HIP` plays the role of the reference's device tag (cf. `struct CUDA { int deviceIndex; }`,
src/LiteNN/Device/CUDA.h:16-25) and `DeviceTraits` carries the same static operations as
`DeviceTraits<D>` (src/LiteNN/Device.h:17-69) with the same argument meaning: sizes are element
counts, destinations are preallocated, failures raise with the backend's message.  Everything
here forwards to the C ABI; nothing is computed in Python.
"""
from __future__ import annotations

import ctypes as C
from dataclasses import dataclass

import numpy as np

from . import _lib
from ._lib import Exec, LiteNNHipError, check
from .formats import (DT_BF16, DT_BOOL, DT_F8E4M3, DT_F8E5M2, DT_F16, DT_F32, DT_F64, DT_I8, DT_I32, DT_I64, DT_U8,
                      DTYPE_SIZE, F32,
                      row_bytes)

_NP_TO_DT = {np.dtype(np.float32): DT_F32, np.dtype(np.float64): DT_F64, np.dtype(np.int32): DT_I32,
             np.dtype(np.int64): DT_I64, np.dtype(np.bool_): DT_BOOL, np.dtype(np.float16): DT_F16,
             np.dtype(np.int8): DT_I8, np.dtype(np.uint8): DT_U8}
_DT_TO_NP = {v: k for k, v in _NP_TO_DT.items()}
_DT_TO_NP[DT_BF16] = np.dtype(np.uint16)  # raw bits
_DT_TO_NP[DT_F8E4M3] = np.dtype(np.uint8)  # raw bits
_DT_TO_NP[DT_F8E5M2] = np.dtype(np.uint8)  # raw bits


@dataclass(frozen=True)
class HIP:
    deviceIndex: int = 0


def HIPDeviceCount() -> int:
    return _lib.load().litenn_hip_device_count()


def IsHIPDeviceAvailable(deviceIndex: int = 0) -> bool:
    return 0 <= deviceIndex < HIPDeviceCount()


def _shape_arr(shape):
    arr = (C.c_size_t * max(len(shape), 1))(*shape)
    return arr, len(shape)


def _opts(stream, synchronize):
    if stream is None and synchronize:
        return None
    return C.byref(Exec(stream, int(synchronize)))


class DeviceTraits:
    """Static operations of the backend; first argument is always the `HIP` device tag."""

    @staticmethod
    def Name() -> str:
        return "HIP"

    @staticmethod
    def Info(device: HIP) -> str:
        buf = C.create_string_buffer(256)
        check(_lib.load().litenn_hip_device_info(device.deviceIndex, buf, 256))
        return buf.value.decode()

    @staticmethod
    def Allocate(device: HIP, dtype: int, size: int) -> int:
        out = C.c_void_p()
        check(_lib.load().litenn_hip_alloc(device.deviceIndex, dtype, size, C.byref(out)))
        return out.value or 0

    @staticmethod
    def Deallocate(device: HIP, ptr: int, dtype: int, size: int) -> None:
        check(_lib.load().litenn_hip_free(device.deviceIndex, ptr, dtype, size))

    @staticmethod
    def ZeroFill(device: HIP, ptr: int, dtype: int, size: int) -> None:
        check(_lib.load().litenn_hip_zero(device.deviceIndex, ptr, dtype, size))

    @staticmethod
    def CopyToCPU(device: HIP, srcType: int, src: int, size: int, dstType: int, dst: np.ndarray) -> None:
        assert dst.flags.c_contiguous and dst.nbytes >= size * DTYPE_SIZE[dstType]
        check(_lib.load().litenn_hip_copy_to_host(device.deviceIndex, srcType, src, size, dstType,
                                                  dst.ctypes.data, None))

    @staticmethod
    def CopyFromCPU(device: HIP, dstType: int, dst: int, srcType: int, src: np.ndarray, size: int) -> None:
        assert src.flags.c_contiguous and src.nbytes >= size * DTYPE_SIZE[srcType]
        check(_lib.load().litenn_hip_copy_from_host(device.deviceIndex, dstType, dst, srcType, src.ctypes.data,
                                                    size, None))

    @staticmethod
    def ConvertTo(device: HIP, srcType: int, src: int, size: int, dstType: int, dst: int) -> None:
        check(_lib.load().litenn_hip_convert(device.deviceIndex, srcType, src, size, dstType, dst, None))

    @staticmethod
    def DoUnaryOp(device: HIP, unaryOp: int, dst: int, dtype: int, shape, src: int) -> None:
        arr, rank = _shape_arr(shape)
        check(_lib.load().litenn_hip_unary(device.deviceIndex, unaryOp, dst, dtype, arr, rank, src, None))

    @staticmethod
    def DoBinaryOp(device: HIP, binaryOp: int, dst: int, type1: int, shape1, src1: int, type2: int, shape2,
                   src2: int) -> None:
        a1, r1 = _shape_arr(shape1)
        a2, r2 = _shape_arr(shape2)
        check(_lib.load().litenn_hip_binary(device.deviceIndex, binaryOp, dst, type1, a1, r1, src1, type2, a2, r2,
                                            src2, None))

    @staticmethod
    def DoReduceOp(device: HIP, reduceOp: int, dst: int, dtype: int, shape, src: int, axis: int) -> None:
        arr, rank = _shape_arr(shape)
        check(_lib.load().litenn_hip_reduce(device.deviceIndex, reduceOp, dst, dtype, arr, rank, src, axis, None))

    @staticmethod
    def DoConcatOp(device: HIP, dst: int, dtype: int, srcPtrs, srcShapes, axis: int) -> None:
        n = len(srcPtrs)
        rank = len(srcShapes[0])
        ptrs = (C.c_void_p * n)(*srcPtrs)
        flat = (C.c_size_t * (n * rank))(*[d for s in srcShapes for d in s])
        check(_lib.load().litenn_hip_concat(device.deviceIndex, dst, dtype, ptrs, flat, rank, n, axis, None))

    @staticmethod
    def DoSliceOp(device: HIP, dst: int, dtype: int, srcShape, src: int, axis: int, start: int, length: int) -> None:
        arr, rank = _shape_arr(srcShape)
        check(_lib.load().litenn_hip_slice(device.deviceIndex, dst, dtype, arr, rank, src, axis, start, length, None))

    @staticmethod
    def DoGetRowsOp(device: HIP, dst: int, dataType: int, dataShape, data: int, indexType: int, indexShape,
                    indices: int) -> None:
        a1, r1 = _shape_arr(dataShape)
        a2, r2 = _shape_arr(indexShape)
        check(_lib.load().litenn_hip_get_rows(device.deviceIndex, dst, dataType, a1, r1, data, indexType, a2, r2,
                                              indices, None))

    @staticmethod
    def DoPermuteOp(device: HIP, dst: int, dtype: int, srcShape, src: int, permutation) -> None:
        a1, r1 = _shape_arr(srcShape)
        a2, _ = _shape_arr(permutation)
        check(_lib.load().litenn_hip_permute(device.deviceIndex, dst, dtype, a1, r1, src, a2, None))


class Tensor:
    """Owning, contiguous device tensor (the role of Tensor<D>, src/LiteNN/Tensor.h:15-592)."""

    def __init__(self, shape, dtype: int = DT_F32, device: HIP = HIP()):
        self.shape = tuple(int(d) for d in shape)
        self.dtype = dtype
        self.device = device
        self.size = int(np.prod(self.shape)) if self.shape else 1
        self.ptr = DeviceTraits.Allocate(device, dtype, self.size)

    @classmethod
    def from_numpy(cls, array: np.ndarray, device: HIP = HIP()) -> "Tensor":
        array = np.ascontiguousarray(array)
        t = cls(array.shape, _NP_TO_DT[array.dtype], device)
        if t.size:
            DeviceTraits.CopyFromCPU(device, t.dtype, t.ptr, t.dtype, array, t.size)
        return t

    def numpy(self, dtype: int | None = None) -> np.ndarray:
        dt = self.dtype if dtype is None else dtype
        out = np.empty(self.shape, _DT_TO_NP[dt])
        if self.size:
            DeviceTraits.CopyToCPU(self.device, self.dtype, self.ptr, self.size, dt, out)
        return out

    def free(self) -> None:
        if self.ptr:
            DeviceTraits.Deallocate(self.device, self.ptr, self.dtype, self.size)
            self.ptr = 0

    def __del__(self):
        try:
            self.free()
        except Exception:
            pass


# ---- quantised extensions ------------------------------------------------------------------------

MATMUL_PRECISE = 1


def mul_mat_q(fmt: int, wq: Tensor, n: int, k: int, x: Tensor, y: Tensor | None = None, residual: Tensor | None = None,
              flags: int = 0, stream=None, synchronize: bool = True) -> Tensor:
    """y[m, n] = x[m, k] . deq(wq)[n, k]^T (+ residual); wq holds the raw GGUF payload."""
    m = x.size // k if k else 0
    try:
        expected = n * row_bytes(fmt, k)
    except ValueError:
        expected = None  # unknown format or ragged row: the C ABI reports it
    if expected is not None and wq.size * DTYPE_SIZE[wq.dtype] != expected:
        raise LiteNNHipError("HIP quantized matmul failed: payload size does not match [n, k] for this format")
    if y is None:
        y = Tensor((m, n), DT_F32, x.device)
    check(_lib.load().litenn_hip_mul_mat_q(x.device.deviceIndex, fmt, wq.ptr, n, k, x.ptr, x.dtype, m, y.ptr,
                                           residual.ptr if residual is not None else None, flags,
                                           _opts(stream, synchronize)))
    return y


GROUP_SILU_MUL = 1


def linear_group(fmt: int, weights, ns, k: int, x: Tensor, residual: Tensor | None = None,
                 norm_w: Tensor | None = None, eps: float = 1e-5, silu_mul: bool = False):
    """[RMSNorm] -> 1..3 linears of one format over one activation row -> [residual | SwiGLU].

    Returns the list of outputs (one per matrix; a single tensor list for SwiGLU)."""
    count = len(weights)
    outs = [Tensor((1, ns[0]), DT_F32, x.device)] if silu_mul else [Tensor((1, n), DT_F32, x.device) for n in ns]
    wptrs = (C.c_void_p * count)(*[w.ptr for w in weights])
    yptrs = (C.c_void_p * count)(*[(outs[i].ptr if i < len(outs) else None) for i in range(count)])
    narr = (C.c_size_t * count)(*ns)
    check(_lib.load().litenn_hip_linear_group(x.device.deviceIndex, fmt, count, wptrs, narr, k, x.ptr, yptrs,
                                              residual.ptr if residual is not None else None,
                                              norm_w.ptr if norm_w is not None else None, eps,
                                              GROUP_SILU_MUL if silu_mul else 0, None))
    return outs


def dequantize(fmt: int, wq: Tensor, rows: int, k: int) -> Tensor:
    out = Tensor((rows, k), DT_F32, wq.device)
    check(_lib.load().litenn_hip_dequantize(wq.device.deviceIndex, fmt, wq.ptr, rows, k, out.ptr, None))
    return out


def get_rows_q(fmt: int, table: Tensor, rows: int, k: int, ids: Tensor) -> Tensor:
    out = Tensor((ids.size, k), DT_F32, table.device)
    check(_lib.load().litenn_hip_get_rows_q(table.device.deviceIndex, fmt, table.ptr, rows, k, ids.ptr, ids.size,
                                            out.ptr, None))
    return out


def rmsnorm(x: Tensor, w: Tensor | None, eps: float) -> Tensor:
    m, d = x.shape
    y = Tensor((m, d), DT_F32, x.device)
    check(_lib.load().litenn_hip_rmsnorm(x.device.deviceIndex, x.ptr, w.ptr if w is not None else None, eps, m, d,
                                         y.ptr, None))
    return y


def rope_interleaved(x: Tensor, n_heads: int, head_dim: int, base: float = 10000.0, pos_offset: int = 0,
                     freq_scale: float = 1.0, rope_dims: int | None = None) -> Tensor:
    m = x.size // (n_heads * head_dim)
    y = Tensor(x.shape, DT_F32, x.device)
    check(_lib.load().litenn_hip_rope_interleaved(x.device.deviceIndex, x.ptr, y.ptr, m, n_heads, head_dim,
                                                  head_dim if rope_dims is None else rope_dims, base, freq_scale,
                                                  pos_offset, None))
    return y


def kv_append(cache: Tensor, past: int, cur: Tensor, width: int) -> None:
    m = cur.size // width
    check(_lib.load().litenn_hip_kv_append(cache.device.deviceIndex, cache.ptr, cache.dtype, past, cur.ptr, m, width,
                                           None))


def attn_decode(q: Tensor, kcache: Tensor, vcache: Tensor, m: int, past: int, n_head: int, n_kv_head: int,
                head_dim: int) -> Tensor:
    out = Tensor((m, n_head * head_dim), DT_F32, q.device)
    check(_lib.load().litenn_hip_attn_decode(q.device.deviceIndex, q.ptr, kcache.ptr, vcache.ptr, kcache.dtype, m,
                                             past, n_head, n_kv_head, head_dim, out.ptr, None))
    return out


def attn_decode_noalloc(q: Tensor, kcache: Tensor, vcache: Tensor, m: int, past: int, n_head: int, n_kv_head: int,
                        head_dim: int, out: Tensor) -> Tensor:
    """attn_decode through the entry point that allocates nothing: the caller brings `out`."""
    check(_lib.load().litenn_hip_attn_decode_noalloc(q.device.deviceIndex, q.ptr, kcache.ptr, vcache.ptr,
                                                     kcache.dtype, m, past, n_head, n_kv_head, head_dim, out.ptr,
                                                     None))
    return out


def attn_rows(q: Tensor, kcache: Tensor, vcache: Tensor, m: int, past: int, n_head: int, n_kv_head: int,
              head_dim: int, precise: bool = False) -> Tensor:
    """attn_decode for a prompt's rows: on the matrix cores when the shape allows and precise is False."""
    out = Tensor((m, n_head * head_dim), DT_F32, q.device)
    check(_lib.load().litenn_hip_attn_rows(q.device.deviceIndex, q.ptr, kcache.ptr, vcache.ptr, kcache.dtype, m, past,
                                           n_head, n_kv_head, head_dim, out.ptr, MATMUL_PRECISE if precise else 0,
                                           None))
    return out


def flash_attn_ext(q: Tensor, k: Tensor, v: Tensor, m: int, keys: int, n_head: int, n_kv_head: int, head_dim: int,
                   scale: float = 1.0, max_bias: float = 0.0, logit_softcap: float = 0.0, mask: Tensor | None = None,
                   sinks: Tensor | None = None, causal: bool = False, key_position_offset: int = 0,
                   query_position_offset: int = 0) -> Tensor:
    """The reference's AddFlashAttnExt with its options, every head at once: q [m, n_head * head_dim],
    k / v [keys, n_kv_head * head_dim] (Float16 or Float32), mask [m, keys] and sinks [n_head] Float32."""
    out = Tensor((m, n_head * head_dim), DT_F32, q.device)
    o = _lib.AttnExtOpts(scale, max_bias, logit_softcap, mask.ptr if mask is not None else None,
                         sinks.ptr if sinks is not None else None, int(causal), key_position_offset,
                         query_position_offset)
    check(_lib.load().litenn_hip_flash_attn_ext(q.device.deviceIndex, q.ptr, k.ptr, v.ptr, k.dtype, m, keys, n_head,
                                                n_kv_head, head_dim, o, out.ptr, None))
    return out


def silu_mul(gate: Tensor, up: Tensor) -> Tensor:
    y = Tensor(gate.shape, DT_F32, gate.device)
    check(_lib.load().litenn_hip_silu_mul(gate.device.deviceIndex, gate.ptr, up.ptr, y.ptr, gate.size, None))
    return y


def argmax(x: Tensor) -> Tensor:
    rows, n = x.shape
    out = Tensor((rows,), DT_I32, x.device)
    check(_lib.load().litenn_hip_argmax(x.device.deviceIndex, x.ptr, rows, n, out.ptr, None))
    return out


__all__ = ["HIP", "HIPDeviceCount", "IsHIPDeviceAvailable", "DeviceTraits", "Tensor", "mul_mat_q", "linear_group",
           "dequantize",
           "get_rows_q", "rmsnorm", "rope_interleaved", "kv_append", "attn_decode", "attn_decode_noalloc", "flash_attn_ext", "silu_mul", "argmax",
           "MATMUL_PRECISE", "LiteNNHipError", "F32"]
