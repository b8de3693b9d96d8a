"""Checker for the generic device primitives: a numpy restatement of the reference's CPU loops.

TEST INFRASTRUCTURE ONLY -- imported by tests, never by the product.  Each function follows the
loop of `DeviceTraits<CPU>` it names; where the evaluation order changes the result (sums along an
axis) the order is kept, everything else is the obvious elementwise numpy expression.  Pinned by
the reference's own vectors in tests/test_oracle_ops.py (tests/TensorTest.cpp:114-191,
tests/LayerTest.cpp:186-214) and by hand-computed cases there.
"""
from __future__ import annotations

import math

import numpy as np

# UnaryOp / BinaryOp / ReduceOp positional values (src/LiteNN/Operators.h:12-51,237-242)
(UN_NEGATE, UN_ABS, UN_SQRT, UN_EXP, UN_LOG, UN_SIN, UN_COS, UN_TAN, UN_ARCSIN, UN_ARCCOS, UN_ARCTAN, UN_TRANSPOSE,
 UN_LOGICAL_NEGATION, UN_ERF) = range(14)
(BIN_ADD, BIN_SUBTRACT, BIN_MULTIPLY, BIN_DIVIDE, BIN_MATMUL, BIN_POW, BIN_MAX, BIN_MIN, BIN_LESS, BIN_GREATER,
 BIN_EQUAL) = range(11)
RED_SUM, RED_MEAN, RED_MAX = range(3)

_UNARY = {UN_SQRT: np.sqrt, UN_EXP: np.exp, UN_LOG: np.log, UN_SIN: np.sin, UN_COS: np.cos, UN_TAN: np.tan,
          UN_ARCSIN: np.arcsin, UN_ARCCOS: np.arccos, UN_ARCTAN: np.arctan}


def unary(op: int, x: np.ndarray) -> np.ndarray:
    """DoUnaryOp (src/LiteNN/Device.h:393-532): the result keeps the input's dtype and shape;
    Transpose swaps the axes of a matrix (:500-511); LogicalNegation is Bool -> Bool."""
    x = np.asarray(x)
    if op == UN_TRANSPOSE:
        assert x.ndim == 2
        return np.ascontiguousarray(x.T)
    if op == UN_LOGICAL_NEGATION:
        assert x.dtype == np.bool_
        return ~x
    if op == UN_NEGATE:
        return (-x).astype(x.dtype)
    if op == UN_ABS:
        return np.abs(x).astype(x.dtype)
    if op == UN_ERF:
        return np.vectorize(math.erf, otypes=[np.float64])(x.astype(np.float64)).astype(x.dtype)
    with np.errstate(all="ignore"):
        if op == UN_SQRT and x.dtype == np.float32:
            return np.sqrt(x)  # IEEE: exactly rounded in float32 as well
        # Evaluated in double and rounded once: integers really go that way (std::sqrt(int) etc.);
        # for Float32 this is the correctly rounded value, which the host's float routines (and
        # the device's) approach to within a few units in the last place.
        return _UNARY[op](x.astype(np.float64)).astype(x.dtype)


def broadcast_shapes(shape1, shape2):
    """DefaultBinaryOpTraits::ResultShape (src/LiteNN/Operators.h:173-188): axes pair up from the
    FRONT; a missing axis counts as extent 1."""
    rank = max(len(shape1), len(shape2))
    out = []
    for i in range(rank):
        d1 = shape1[i] if i < len(shape1) else 1
        d2 = shape2[i] if i < len(shape2) else 1
        if d1 != d2 and d1 != 1 and d2 != 1:
            raise ValueError("BinaryOp requires input shapes to be compatible for broadcasting")
        out.append(max(d1, d2))
    return tuple(out)


def binary(op: int, a: np.ndarray, b: np.ndarray) -> np.ndarray:
    """DoBinaryOp (src/LiteNN/Device.h:534-689) for operands of equal rank, where an extent of 1
    repeats (:560-601).  Comparisons give Bool; MatMul is the zero-filled i-k-j loop (:645-658)."""
    a, b = np.asarray(a), np.asarray(b)
    assert a.dtype == b.dtype
    if op == BIN_MATMUL:
        m, k = a.shape
        k2, n = b.shape
        assert k == k2
        y = np.zeros((m, n), a.dtype)
        for kk in range(k):  # y[i, :] += x[i, k] * w[k, :] with k ascending, each step rounded
            y += (a[:, kk:kk + 1] * b[kk:kk + 1, :]).astype(a.dtype)
        return y
    assert a.ndim == b.ndim
    shape = broadcast_shapes(a.shape, b.shape)
    x, y = np.broadcast_to(a, shape), np.broadcast_to(b, shape)
    with np.errstate(all="ignore"):
        if op == BIN_ADD:
            r = x + y
        elif op == BIN_SUBTRACT:
            r = x - y
        elif op == BIN_MULTIPLY:
            r = x * y
        elif op == BIN_DIVIDE:
            if np.issubdtype(a.dtype, np.integer):
                r = np.trunc(x.astype(np.float64) / y.astype(np.float64))  # C++ integer division truncates
            else:
                r = x / y
        elif op == BIN_POW:
            r = np.power(x.astype(np.float64), y.astype(np.float64))
        elif op == BIN_MAX:
            r = np.where(x < y, y, x)  # std::max(a, b)
        elif op == BIN_MIN:
            r = np.where(y < x, y, x)  # std::min(a, b)
        elif op == BIN_LESS:
            return np.ascontiguousarray(x < y)
        elif op == BIN_GREATER:
            return np.ascontiguousarray(x > y)
        elif op == BIN_EQUAL:
            return np.ascontiguousarray(x == y)
        else:
            raise ValueError("unknown binary op")
    return np.ascontiguousarray(r.astype(a.dtype))


def reduce(op: int, x: np.ndarray, axis: int) -> np.ndarray:
    """DoReduceOp (src/LiteNN/Device.h:691-759): the accumulator has the input's type and walks
    the axis front to back; Mean divides the finished sum by the extent; the axis is removed
    (a scalar result has shape [1], Operators.h:255-275)."""
    x = np.asarray(x)
    if op == RED_MAX:
        r = np.max(x, axis=axis)
    else:
        with np.errstate(all="ignore"):
            r = np.take(np.cumsum(x, axis=axis, dtype=x.dtype), -1, axis=axis)  # cumsum adds in order
            if op == RED_MEAN:
                # static_cast<ResultType>(reduceDim) (:750): an extent beyond the type's range wraps
                n = np.array(x.shape[axis], np.int64).astype(x.dtype)
                if np.issubdtype(x.dtype, np.integer):
                    r = np.trunc(r.astype(np.float64) / np.float64(n)).astype(x.dtype)
                else:
                    r = (r / n).astype(x.dtype)
    r = np.asarray(r, dtype=x.dtype)
    return r.reshape(1) if r.ndim == 0 else np.ascontiguousarray(r)


def concat(parts, axis: int) -> np.ndarray:
    """DoConcatOp (src/LiteNN/Device.h:761-792)."""
    return np.ascontiguousarray(np.concatenate(parts, axis=axis))


def slice_(x: np.ndarray, axis: int, start: int, length: int) -> np.ndarray:
    """DoSliceOp (src/LiteNN/Device.h:794-823)."""
    index = [slice(None)] * x.ndim
    index[axis] = slice(start, start + length)
    return np.ascontiguousarray(x[tuple(index)])


def get_rows(data: np.ndarray, indices: np.ndarray) -> np.ndarray:
    """DoGetRowsOp (src/LiteNN/Device.h:825-883): rows of the first axis, result shape =
    index shape + data shape[1:]; an index outside [0, rows) is an error."""
    indices = np.asarray(indices)
    if indices.size and (indices.min() < 0 or indices.max() >= data.shape[0]):
        raise IndexError("GetRows index out of range")
    return np.ascontiguousarray(data[indices.reshape(-1)].reshape(indices.shape + data.shape[1:]))


def permute(x: np.ndarray, permutation) -> np.ndarray:
    """DoPermuteOp (src/LiteNN/Device.h:885-966): result axis d is source axis permutation[d]."""
    return np.ascontiguousarray(np.transpose(x, permutation))


def convert(x: np.ndarray, dtype) -> np.ndarray:
    """ConvertTo (src/LiteNN/Device.h:372-391): static_cast element by element (Float16 through
    float with the reference's own rounding is checked elsewhere; this covers the plain types)."""
    with np.errstate(all="ignore"):
        return x.astype(dtype)


# ---- Float8E4M3 / Float8E5M2 (src/LiteNN/DType.h:148-229, 290-344) ---------------------------------
F8_LAYOUTS = {"e4m3": (4, 3, 7), "e5m2": (5, 2, 15)}  # exponent bits, mantissa bits, bias


def _ldexp_f32(value: np.float32, exponent: int) -> np.float32:
    """Detail::Ldexp (DType.h:34-51): repeated multiplication by 2 or 0.5 in Float32."""
    if value == 0:
        return np.float32(0.0)
    value = np.float32(value)
    while exponent > 0:
        value = np.float32(value * np.float32(2.0))
        exponent -= 1
    while exponent < 0:
        value = np.float32(value * np.float32(0.5))
        exponent += 1
    return value


def _round_to_uint(value: np.float32) -> int:
    """Detail::RoundToUInt (DType.h:53-56): static_cast<uint32>(value + 0.5F), the sum in Float32."""
    return int(np.float32(np.float32(value) + np.float32(0.5)))


def f8_bits_to_f32(bits, kind: str) -> np.ndarray:
    """Float8BitsToFloat32 (DType.h:203-229), element by element."""
    ebits, mbits, bias = F8_LAYOUTS[kind]
    flat = np.asarray(bits, np.uint8).reshape(-1)
    out = np.empty(flat.shape, np.float32)
    exp_mask = (1 << ebits) - 1
    scale = np.float32(1 << mbits)
    for i, b in enumerate(flat.tolist()):
        sign = np.float32(-1.0 if b & 0x80 else 1.0)
        e = (b >> mbits) & exp_mask
        mant = b & ((1 << mbits) - 1)
        if e == 0:
            out[i] = sign * np.float32(0.0) if mant == 0 else sign * _ldexp_f32(np.float32(mant) / scale, 1 - bias)
        elif e == exp_mask:
            out[i] = sign * np.float32(np.inf) if mant == 0 else np.float32(np.nan)
        else:
            out[i] = sign * _ldexp_f32(np.float32(1.0) + np.float32(mant) / scale, e - bias)
    return out.reshape(np.shape(bits))


def f32_to_f8_bits(values, kind: str) -> np.ndarray:
    """Float32ToFloat8Bits (DType.h:148-201), element by element, every step in Float32."""
    ebits, mbits, bias = F8_LAYOUTS[kind]
    flat = np.asarray(values, np.float32).reshape(-1)
    out = np.empty(flat.shape, np.uint8)
    max_exp = (1 << ebits) - 1
    scale = np.float32(1 << mbits)
    with np.errstate(all="ignore"):
        for i, v in enumerate(flat):
            sign = 0x80 if np.signbit(v) else 0
            mag = np.float32(-v) if v < 0 else np.float32(v)
            if mag == 0:
                out[i] = sign
                continue
            if not np.isfinite(mag):
                out[i] = sign | (max_exp << mbits)
                continue
            exponent = 0
            while mag >= 2:
                mag = np.float32(mag * np.float32(0.5))
                exponent += 1
            while mag < 1:
                mag = np.float32(mag * np.float32(2.0))
                exponent -= 1
            stored = exponent + bias
            if stored >= max_exp:
                out[i] = sign | (max_exp << mbits)
                continue
            if stored <= 0:
                sub = _ldexp_f32(mag, exponent + bias - 1)
                out[i] = sign | min(_round_to_uint(np.float32(sub * scale)), (1 << mbits) - 1)
                continue
            mant = _round_to_uint(np.float32(np.float32(mag - np.float32(1.0)) * scale))
            e = stored
            if mant == (1 << mbits):
                mant = 0
                e = min(e + 1, max_exp)
            out[i] = sign | (e << mbits) | mant
    return out.reshape(np.shape(values))
