"""Parity of the generic device primitives (DoUnaryOp, DoBinaryOp, DoReduceOp, DoConcatOp,
DoSliceOp, DoGetRowsOp, DoPermuteOp, ConvertTo) through the C ABI with the numpy checker of the
reference's CPU loops.  Bit-exact wherever the operation is exact or IEEE-defined (integer work,
copies, comparisons, +, -, *, /, sqrt, sums in the reference's order); transcendental float
functions within 4 units in the last place of the host library's result."""
import numpy as np
import pytest

from litenn_amd import LiteNNHipError
from litenn_amd.device import HIP, DeviceTraits, _NP_TO_DT
from litenn_amd.formats import (DT_BF16, DT_BOOL, DT_F8E4M3, DT_F8E5M2, DT_F16, DT_F32, DT_F64, DT_I8, DT_I32, DT_I64,
                                DT_U8)
from oracle import primitives as P

pytestmark = pytest.mark.gpu
DEV = HIP()
NUMERIC = [np.float32, np.float64, np.int32, np.int64, np.int8, np.uint8]


def dt(a):
    return _NP_TO_DT[np.dtype(a)]


def random_array(rng, shape, dtype, lo=-50, hi=50):
    if np.issubdtype(dtype, np.floating):
        return (rng.standard_normal(shape) * 3).astype(dtype)
    if dtype == np.uint8:
        lo = 0
    return rng.integers(lo, hi, shape).astype(dtype)


def ulp_close(got, want, ulps):
    got, want = np.asarray(got), np.asarray(want)
    same_nan = np.isnan(got) == np.isnan(want)
    step = np.spacing(np.abs(np.where(np.isfinite(want), want, 1)).astype(want.dtype))
    ok = np.where(np.isfinite(want), np.abs(got - want) <= ulps * step, (got == want) | np.isnan(want))
    return bool(same_nan.all() and ok.all())


def run_unary(hip, op, x, out_dtype=None):
    src = hip.Tensor.from_numpy(x)
    shape = x.shape[::-1] if op == P.UN_TRANSPOSE else x.shape
    dst = hip.Tensor(shape, dt(out_dtype or x.dtype))
    DeviceTraits.DoUnaryOp(DEV, op, dst.ptr, src.dtype, x.shape, src.ptr)
    return dst.numpy()


def run_binary(hip, op, a, b):
    ta, tb = hip.Tensor.from_numpy(a), hip.Tensor.from_numpy(b)
    if op == P.BIN_MATMUL:
        shape = (a.shape[0], b.shape[1])
    else:
        shape = P.broadcast_shapes(a.shape, b.shape)
    dst = hip.Tensor(shape, DT_BOOL if op >= P.BIN_LESS else ta.dtype)
    DeviceTraits.DoBinaryOp(DEV, op, dst.ptr, ta.dtype, a.shape, ta.ptr, tb.dtype, b.shape, tb.ptr)
    return dst.numpy()


def test_reference_vectors_on_the_device(hip):
    t = np.array([[1, 2, 3], [4, 5, 6]], np.float32)
    assert np.array_equal(run_binary(hip, P.BIN_ADD, t, t), [[2, 4, 6], [8, 10, 12]])
    tt = run_unary(hip, P.UN_TRANSPOSE, t)
    assert np.array_equal(tt.reshape(-1), [1, 4, 2, 5, 3, 6])
    assert np.array_equal(run_binary(hip, P.BIN_MATMUL, t, tt), [[14, 32], [32, 77]])
    assert np.array_equal(run_binary(hip, P.BIN_ADD, t, np.array([[10], [20]], np.float32)),
                          [[11, 12, 13], [24, 25, 26]])
    less = run_binary(hip, P.BIN_LESS, t, t + t)
    assert less.dtype == np.bool_ and less.all()
    assert not run_unary(hip, P.UN_LOGICAL_NEGATION, less).any()
    assert not run_binary(hip, P.BIN_EQUAL, t, t + t).any()


@pytest.mark.parametrize("dtype", NUMERIC)
def test_unary_ops(hip, dtype):
    rng = np.random.default_rng(11)
    for shape in [(1,), (7, 33), (2, 3, 65), (4096,)]:
        x = random_array(rng, shape, dtype)
        exact = [P.UN_NEGATE, P.UN_ABS, P.UN_SQRT]
        if dtype == np.uint8:
            exact = [P.UN_ABS, P.UN_SQRT]
        for op in exact:
            arg = np.abs(x) if op == P.UN_SQRT else x
            assert np.array_equal(run_unary(hip, op, arg), P.unary(op, arg), equal_nan=True), (op, shape)
        if np.issubdtype(dtype, np.floating):
            small = (x / 8).astype(dtype)
            unit = np.clip(small, -1, 1)
            for op, arg in [(P.UN_EXP, small), (P.UN_LOG, np.abs(x) + dtype(0.01)), (P.UN_SIN, x), (P.UN_COS, x),
                            (P.UN_TAN, small), (P.UN_ARCSIN, unit), (P.UN_ARCCOS, unit), (P.UN_ARCTAN, x),
                            (P.UN_ERF, small)]:
                assert ulp_close(run_unary(hip, op, arg), P.unary(op, arg), 4), (op, shape)
    m = random_array(rng, (5, 9), dtype)
    assert np.array_equal(run_unary(hip, P.UN_TRANSPOSE, m), m.T)


def test_unary_special_values_and_refusals(hip):
    x = np.array([-1.0, 0.0, -0.0, np.inf, -np.inf, np.nan], np.float32)
    for op in (P.UN_NEGATE, P.UN_ABS, P.UN_SQRT, P.UN_EXP, P.UN_LOG):
        got, want = run_unary(hip, op, x), P.unary(op, x)
        assert np.array_equal(got, want, equal_nan=True), op
        assert np.array_equal(np.signbit(got), np.signbit(want)) or op in (P.UN_SQRT, P.UN_LOG), op
    with pytest.raises(LiteNNHipError, match="2D"):
        run_unary(hip, P.UN_TRANSPOSE, np.zeros((2, 3, 4), np.float32))
    flags = np.array([True, False, True])
    assert np.array_equal(run_unary(hip, P.UN_LOGICAL_NEGATION, flags), ~flags)


@pytest.mark.parametrize("dtype", NUMERIC)
def test_binary_ops_with_broadcast(hip, dtype):
    rng = np.random.default_rng(12)
    shapes = [((6,), (6,)), ((1,), (9,)), ((5, 7), (5, 7)), ((5, 7), (5, 1)), ((5, 7), (1, 7)), ((1, 1), (4, 3)),
              ((3, 1, 5), (1, 4, 5)), ((2, 3, 4, 5), (2, 1, 4, 1)), ((130, 70), (130, 70))]
    for s1, s2 in shapes:
        a, b = random_array(rng, s1, dtype), random_array(rng, s2, dtype)
        nz = np.where(b == 0, dtype(1), b)
        for op, rhs in [(P.BIN_ADD, b), (P.BIN_SUBTRACT, b), (P.BIN_MULTIPLY, b), (P.BIN_DIVIDE, nz), (P.BIN_MAX, b),
                        (P.BIN_MIN, b), (P.BIN_LESS, b), (P.BIN_GREATER, b), (P.BIN_EQUAL, b)]:
            if dtype == np.int8 and op == P.BIN_DIVIDE:
                rhs = np.where(nz == -1, dtype(1), nz)  # -128 / -1 overflows in C++ too
            got, want = run_binary(hip, op, a, rhs), P.binary(op, a, rhs)
            assert got.dtype == want.dtype and np.array_equal(got, want), (op, s1, s2)
    if np.issubdtype(dtype, np.floating):
        base = np.abs(random_array(rng, (5, 7), dtype)) + dtype(0.5)
        expo = (random_array(rng, (5, 1), dtype) / 4).astype(dtype)
        assert ulp_close(run_binary(hip, P.BIN_POW, base, expo), P.binary(P.BIN_POW, base, expo), 4)
    else:
        base = rng.integers(0, 4, (5, 7)).astype(dtype)
        expo = rng.integers(0, 4, (5, 1)).astype(dtype)
        assert np.array_equal(run_binary(hip, P.BIN_POW, base, expo), P.binary(P.BIN_POW, base, expo))


def test_binary_refusals(hip):
    a = hip.Tensor.from_numpy(np.zeros((2, 3), np.float32))
    b = hip.Tensor.from_numpy(np.zeros((3,), np.float32))
    c = hip.Tensor.from_numpy(np.zeros((2, 3), np.float64))
    flags = hip.Tensor.from_numpy(np.zeros((2, 3), np.bool_))
    with pytest.raises(LiteNNHipError, match="compatible for broadcasting"):
        DeviceTraits.DoBinaryOp(DEV, P.BIN_ADD, a.ptr, DT_F32, (2, 3), a.ptr, DT_F32, (2, 2), a.ptr)
    with pytest.raises(LiteNNHipError, match="same data type"):
        DeviceTraits.DoBinaryOp(DEV, P.BIN_ADD, a.ptr, DT_F32, (2, 3), a.ptr, DT_F64, (2, 3), c.ptr)
    with pytest.raises(LiteNNHipError, match="boolean"):
        DeviceTraits.DoBinaryOp(DEV, P.BIN_ADD, flags.ptr, DT_BOOL, (2, 3), flags.ptr, DT_BOOL, (2, 3), flags.ptr)
    with pytest.raises(LiteNNHipError, match="inner dimensions"):
        DeviceTraits.DoBinaryOp(DEV, P.BIN_MATMUL, a.ptr, DT_F32, (2, 3), a.ptr, DT_F32, (2, 3), a.ptr)
    with pytest.raises(LiteNNHipError, match="2D"):
        DeviceTraits.DoBinaryOp(DEV, P.BIN_MATMUL, a.ptr, DT_F32, (2, 3), a.ptr, DT_F32, (3,), b.ptr)


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
def test_matmul_is_the_host_loop_bit_for_bit(hip, dtype):
    rng = np.random.default_rng(13)
    for m, k, n in [(1, 1, 1), (2, 3, 2), (17, 33, 19), (64, 300, 48), (5, 1000, 7)]:
        a = rng.standard_normal((m, k)).astype(dtype)
        b = rng.standard_normal((k, n)).astype(dtype)
        assert np.array_equal(run_binary(hip, P.BIN_MATMUL, a, b), P.binary(P.BIN_MATMUL, a, b)), (m, k, n)
    a = np.array([[1e8, 1.0, -1e8]], dtype)
    if dtype == np.float32:
        assert run_binary(hip, P.BIN_MATMUL, a, np.ones((3, 1), dtype))[0, 0] == 0.0


@pytest.mark.parametrize("dtype", NUMERIC)
def test_reduce_ops(hip, dtype):
    rng = np.random.default_rng(14)
    for shape in [(9,), (4, 300), (300, 4), (3, 5, 7), (2, 1, 6), (2, 3, 4, 5)]:
        x = random_array(rng, shape, dtype, -9, 9)
        src = hip.Tensor.from_numpy(x)
        for axis in range(len(shape)):
            for op in (P.RED_SUM, P.RED_MEAN, P.RED_MAX):
                want = P.reduce(op, x, axis)
                dst = hip.Tensor(want.shape, src.dtype)
                DeviceTraits.DoReduceOp(DEV, op, dst.ptr, src.dtype, shape, src.ptr, axis)
                assert np.array_equal(dst.numpy(), want), (op, shape, axis)
    # the order of a float sum is the reference's: front to back
    x = np.array([[1.0, 1e8, -1e8]], np.float32)
    src, dst = hip.Tensor.from_numpy(x), hip.Tensor((1,), DT_F32)
    DeviceTraits.DoReduceOp(DEV, P.RED_SUM, dst.ptr, DT_F32, (1, 3), src.ptr, 1)
    assert dst.numpy()[0] == 0.0
    with pytest.raises(LiteNNHipError):
        DeviceTraits.DoReduceOp(DEV, P.RED_SUM, dst.ptr, DT_F32, (1, 3), src.ptr, 2)
    flags = hip.Tensor.from_numpy(np.zeros((2, 2), np.bool_))
    with pytest.raises(LiteNNHipError, match="boolean"):
        DeviceTraits.DoReduceOp(DEV, P.RED_SUM, flags.ptr, DT_BOOL, (2, 2), flags.ptr, 0)


@pytest.mark.parametrize("dtype", NUMERIC + [np.bool_, np.float16])
def test_concat_slice_permute_get_rows_move_bytes_exactly(hip, dtype):
    rng = np.random.default_rng(15)
    make = lambda shape: (rng.integers(0, 2, shape).astype(np.bool_) if dtype == np.bool_
                          else random_array(rng, shape, dtype) if dtype != np.float16
                          else rng.standard_normal(shape).astype(np.float16))
    # concat along every axis, uneven parts, an empty part
    for axis, extents in [(0, (2, 5, 1)), (1, (3, 0, 4)), (2, (1, 1, 6))]:
        shapes = [tuple(e if d == axis else (3, 4, 5)[d] for d in range(3)) for e in extents]
        parts = [make(s) for s in shapes]
        tensors = [hip.Tensor.from_numpy(p) for p in parts]
        want = P.concat(parts, axis)
        dst = hip.Tensor(want.shape, tensors[0].dtype)
        DeviceTraits.DoConcatOp(DEV, dst.ptr, dst.dtype, [t.ptr for t in tensors], shapes, axis)
        assert np.array_equal(dst.numpy(), want), axis
    x = make((4, 6, 10))
    src = hip.Tensor.from_numpy(x)
    for axis, start, length in [(0, 1, 2), (1, 0, 6), (1, 5, 1), (2, 3, 4), (2, 9, 1)]:
        want = P.slice_(x, axis, start, length)
        dst = hip.Tensor(want.shape, src.dtype)
        DeviceTraits.DoSliceOp(DEV, dst.ptr, src.dtype, x.shape, src.ptr, axis, start, length)
        assert np.array_equal(dst.numpy(), want), (axis, start, length)
    with pytest.raises(LiteNNHipError):
        DeviceTraits.DoSliceOp(DEV, src.ptr, src.dtype, x.shape, src.ptr, 2, 8, 3)
    for perm in [(0, 1, 2), (2, 0, 1), (1, 2, 0), (0, 2, 1), (2, 1, 0)]:
        want = P.permute(x, perm)
        dst = hip.Tensor(want.shape, src.dtype)
        DeviceTraits.DoPermuteOp(DEV, dst.ptr, src.dtype, x.shape, src.ptr, perm)
        assert np.array_equal(dst.numpy(), want), perm
    with pytest.raises(LiteNNHipError, match="valid permutation"):
        DeviceTraits.DoPermuteOp(DEV, src.ptr, src.dtype, x.shape, src.ptr, (0, 0, 1))
    for index_dtype in (np.int32, np.int64):
        idx = rng.integers(0, 4, (3, 2)).astype(index_dtype)
        want = P.get_rows(x, idx)
        ti = hip.Tensor.from_numpy(idx)
        dst = hip.Tensor(want.shape, src.dtype)
        DeviceTraits.DoGetRowsOp(DEV, dst.ptr, src.dtype, x.shape, src.ptr, ti.dtype, idx.shape, ti.ptr)
        assert np.array_equal(dst.numpy(), want)
        bad = hip.Tensor.from_numpy(np.array([0, 4], index_dtype))
        with pytest.raises(LiteNNHipError, match="out of range"):
            DeviceTraits.DoGetRowsOp(DEV, dst.ptr, src.dtype, x.shape, src.ptr, bad.dtype, (2,), bad.ptr)
        bad = hip.Tensor.from_numpy(np.array([-1], index_dtype))
        with pytest.raises(LiteNNHipError, match="out of range"):
            DeviceTraits.DoGetRowsOp(DEV, dst.ptr, src.dtype, x.shape, src.ptr, bad.dtype, (1,), bad.ptr)


def test_conversions_between_plain_types(hip):
    rng = np.random.default_rng(16)
    values = np.concatenate([np.clip(rng.standard_normal(500) * 40, -120, 120),
                             [0.0, -0.0, 0.5, -0.5, 1.5, 2.5, -2.5, 126.9, -127.9]])
    for src_dtype in NUMERIC + [np.bool_]:
        if src_dtype == np.bool_:
            x = values > 0
        elif src_dtype == np.uint8:
            x = np.abs(values).astype(src_dtype)
        else:
            x = values.astype(src_dtype)
        src = hip.Tensor.from_numpy(x)
        for dst_dtype in NUMERIC + [np.bool_]:
            if np.issubdtype(src_dtype, np.floating) and dst_dtype == np.uint8:
                x_ok = np.abs(x)  # a negative float to an unsigned type is undefined in C++
                s2 = hip.Tensor.from_numpy(x_ok)
            else:
                x_ok, s2 = x, src
            dst = hip.Tensor(x.shape, dt(dst_dtype))
            DeviceTraits.ConvertTo(DEV, s2.dtype, s2.ptr, s2.size, dst.dtype, dst.ptr)
            assert np.array_equal(dst.numpy(), P.convert(x_ok, dst_dtype)), (src_dtype, dst_dtype)
    # an Int64 beyond 2^53 reaches Float32 in one rounding: 2^60 + 2^36 + 1 lies above the midpoint
    # of two floats and goes up; rounded to double first it would sit on the midpoint and go down
    big = np.array([(1 << 60) + (1 << 36) + 1, -((1 << 60) + (1 << 36) + 1)], np.int64)
    src, dst = hip.Tensor.from_numpy(big), hip.Tensor((2,), DT_F32)
    DeviceTraits.ConvertTo(DEV, DT_I64, src.ptr, 2, DT_F32, dst.ptr)
    assert np.array_equal(dst.numpy(), np.array([2.0**60 + 2.0**37, -(2.0**60 + 2.0**37)], np.float32))
    # copies with a type change at the host boundary take the same route
    assert np.array_equal(src.numpy(DT_F32), dst.numpy())


def test_low_precision_conversions(hip, oracle):
    rng = np.random.default_rng(17)
    x = np.concatenate([rng.standard_normal(4000) * 8, [0.0, -0.0, 65504.0, 65520.0, 1e-8, 6e-5, np.inf, -np.inf]])
    x = x.astype(np.float32)
    src = hip.Tensor.from_numpy(x)
    half = hip.Tensor(x.shape, DT_F16)
    DeviceTraits.ConvertTo(DEV, DT_F32, src.ptr, src.size, DT_F16, half.ptr)
    assert np.array_equal(half.numpy().view(np.uint16), oracle.f32_to_f16_bits(x))
    back = hip.Tensor(x.shape, DT_F32)
    DeviceTraits.ConvertTo(DEV, DT_F16, half.ptr, half.size, DT_F32, back.ptr)
    assert np.array_equal(back.numpy(), oracle.f16_to_f32(oracle.f32_to_f16_bits(x)))
    # BFloat16: round to nearest even on the upper 16 bits (src/LiteNN/DType.h:136-141)
    bf = hip.Tensor(x.shape, DT_BF16)
    DeviceTraits.ConvertTo(DEV, DT_F32, src.ptr, src.size, DT_BF16, bf.ptr)
    bits = x.view(np.uint32).astype(np.uint64)
    want = ((bits + 0x7FFF + ((bits >> 16) & 1)) >> 16).astype(np.uint16)
    assert np.array_equal(bf.numpy(), want)
    DeviceTraits.ConvertTo(DEV, DT_BF16, bf.ptr, bf.size, DT_F32, back.ptr)
    assert np.array_equal(back.numpy().view(np.uint32), want.astype(np.uint32) << 16)


@pytest.mark.parametrize("kind,dtype", [("e4m3", DT_F8E4M3), ("e5m2", DT_F8E5M2)])
def test_float8_conversions(hip, kind, dtype):
    """ConvertTo with Float8E4M3 / Float8E5M2 on either side (src/LiteNN/Device.h:372-391 through the
    constructors and conversion operators of src/LiteNN/DType.h:148-229, 290-344), bit for bit
    against the checker's restatement: every code decoded, Float32 inputs that land on values,
    midpoints, both sides of midpoints, the subnormal range, overflow, infinities and NaN, and the
    other element types through their conversion to float."""
    from litenn_amd.formats import DT_BF16, DT_F16, DT_F64, DT_I32

    def as_tensor(raw_bits):
        t = hip.Tensor(raw_bits.shape, dtype)
        DeviceTraits.CopyFromCPU(DEV, dtype, t.ptr, dtype, np.ascontiguousarray(raw_bits, np.uint8), t.size)
        return t

    def convert(src, dst_dtype):
        dst = hip.Tensor(src.shape, dst_dtype)
        DeviceTraits.ConvertTo(DEV, src.dtype, src.ptr, src.size, dst_dtype, dst.ptr)
        return dst.numpy()

    codes = np.arange(256, dtype=np.uint8)
    table = P.f8_bits_to_f32(codes, kind)
    got = convert(as_tensor(codes), DT_F32)
    assert np.array_equal(got.view(np.uint32)[~np.isnan(table)], table.view(np.uint32)[~np.isnan(table)])
    assert np.all(np.isnan(got[np.isnan(table)]))
    finite = np.isfinite(table)
    assert np.array_equal(convert(as_tensor(codes[finite]), DT_F64), table[finite].astype(np.float64))
    assert np.array_equal(convert(as_tensor(codes[finite]), DT_I32), table[finite].astype(np.int32))
    assert np.array_equal(convert(as_tensor(codes[finite]), DT_F16).view(np.uint16),
                          table[finite].astype(np.float16).view(np.uint16))  # every value is exact in a half
    # Float32 -> Float8
    rng = np.random.default_rng(23)
    pos = np.sort(table[np.isfinite(table) & ~np.signbit(table)]).astype(np.float64)
    mids = (pos[1:] + pos[:-1]) / 2
    x = np.concatenate([pos, mids, np.nextafter(mids.astype(np.float32), np.float32(0)),
                        np.nextafter(mids.astype(np.float32), np.float32(np.inf)),
                        [pos[-1] * 1.03, pos[-1] * 1.07, pos[-1] * 2, 1e30, 1e-30, 1e-40, np.inf, np.nan, 0.0],
                        rng.standard_normal(3000) * 3, rng.standard_normal(1000) * pos[-1] / 2,
                        rng.standard_normal(1000) * pos[2]]).astype(np.float32)
    x = np.concatenate([x, -x])
    want = P.f32_to_f8_bits(x, kind)
    assert np.array_equal(convert(hip.Tensor.from_numpy(x), dtype), want)
    # other sources reach Float8 through their conversion to float
    xd = np.concatenate([mids, pos, rng.standard_normal(500)]).astype(np.float64)
    assert np.array_equal(convert(hip.Tensor.from_numpy(xd), dtype), P.f32_to_f8_bits(xd.astype(np.float32), kind))
    xi = rng.integers(-300, 300, 500).astype(np.int32)
    assert np.array_equal(convert(hip.Tensor.from_numpy(xi), dtype), P.f32_to_f8_bits(xi.astype(np.float32), kind))
    xh = (rng.standard_normal(500) * 4).astype(np.float16)
    assert np.array_equal(convert(hip.Tensor.from_numpy(xh), dtype), P.f32_to_f8_bits(xh.astype(np.float32), kind))
    # and a host copy with a type change takes the same route
    t = hip.Tensor.from_numpy(x[:64])
    assert np.array_equal(t.numpy(dtype), want[:64])
