"""The numpy checker of the generic device primitives (oracle/primitives.py) against the
reference's own vectors (tests/TensorTest.cpp:114-191, tests/LayerTest.cpp:186-214,
tests/CUDADeviceTest.cpp:108-125) and hand-computed cases that a wrong axis, order or rounding
rule would fail.  No GPU."""
import numpy as np
import pytest

from oracle import primitives as P

T23 = np.array([[1, 2, 3], [4, 5, 6]], np.float32)


def test_basic_operations_vectors():
    assert np.array_equal(P.binary(P.BIN_ADD, T23, T23), [[2, 4, 6], [8, 10, 12]])
    t = P.unary(P.UN_TRANSPOSE, T23)
    assert np.array_equal(t.reshape(-1), [1, 4, 2, 5, 3, 6])
    assert np.array_equal(P.binary(P.BIN_MATMUL, T23, t), [[14, 32], [32, 77]])


def test_comparison_and_logical_vectors():
    twice = P.binary(P.BIN_ADD, T23, T23)
    less = P.binary(P.BIN_LESS, T23, twice)
    assert less.dtype == np.bool_ and less.all()
    assert not P.unary(P.UN_LOGICAL_NEGATION, less).any()
    assert not P.binary(P.BIN_EQUAL, T23, twice).any()
    assert P.binary(P.BIN_GREATER, twice, T23).all()


def test_broadcast_vector_and_front_aligned_shapes():
    col = np.array([[10], [20]], np.float32)
    assert np.array_equal(P.binary(P.BIN_ADD, T23, col), [[11, 12, 13], [24, 25, 26]])
    assert P.broadcast_shapes((2, 3), (2,)) == (2, 3)  # a missing axis is a trailing 1
    with pytest.raises(ValueError):
        P.broadcast_shapes((2, 3), (3,))  # numpy would accept this; the reference pairs axes from the front


def test_get_rows_vector():
    table = np.array([[10, 11], [20, 21], [30, 31], [40, 41]], np.float32)
    assert np.array_equal(P.get_rows(table, np.array([2, 0, 3], np.int32)), [[30, 31], [10, 11], [40, 41]])
    with pytest.raises(IndexError):
        P.get_rows(table, np.array([4], np.int32))
    idx = np.array([[1, 1], [0, 3]], np.int64)
    assert P.get_rows(table, idx).shape == (2, 2, 2)


def test_reduce_order_type_and_shape():
    # front to back in float32: (1 + 1e8) - 1e8 = 0, not 1
    x = np.array([[1.0, 1e8, -1e8]], np.float32)
    assert P.reduce(P.RED_SUM, x, 1)[0] == 0.0
    assert P.reduce(P.RED_SUM, x.T.copy(), 0)[0] == 0.0
    # Mean divides the finished sum; integers divide like C++ (towards zero)
    assert P.reduce(P.RED_MEAN, np.array([2, 4, 9], np.int32), 0).tolist() == [5]
    assert P.reduce(P.RED_MEAN, np.array([-7, 2], np.int64), 0).tolist() == [-2]
    assert P.reduce(P.RED_MEAN, np.array([[1.0, 2.0], [4.0, 8.0]], np.float64), 0).tolist() == [2.5, 5.0]
    assert P.reduce(P.RED_MAX, np.array([[1, 9, 3], [7, 2, 8]], np.int32), 1).tolist() == [9, 8]
    # ... and so does the divisor: 300 as int8 is 44; the sum of 300 ones wraps to 44 as well
    assert P.reduce(P.RED_MEAN, np.ones(300, np.int8), 0).tolist() == [1]
    assert P.reduce(P.RED_MEAN, np.full(300, 2, np.int8), 0).tolist() == [2]  # 600 -> 88, 88 / 44
    # an int8 accumulator wraps
    assert P.reduce(P.RED_SUM, np.array([100, 100], np.int8), 0).tolist() == [-56]
    # a fully reduced vector keeps one axis of extent 1
    assert P.reduce(P.RED_SUM, np.array([1.0, 2.0], np.float32), 0).shape == (1,)
    assert P.reduce(P.RED_SUM, np.zeros((2, 3, 4), np.float32), 1).shape == (2, 4)


def test_integer_arithmetic_follows_cpp():
    a, b = np.array([-7, 7, 9], np.int32), np.array([2, -2, 4], np.int32)
    assert P.binary(P.BIN_DIVIDE, a, b).tolist() == [-3, -3, 2]
    assert P.binary(P.BIN_MAX, a, b).tolist() == [2, 7, 9]
    assert P.binary(P.BIN_MIN, a, b).tolist() == [-7, -2, 4]
    assert P.binary(P.BIN_POW, np.array([2, 3], np.int64), np.array([10, 3], np.int64)).tolist() == [1024, 27]
    assert P.unary(P.UN_SQRT, np.array([16, 17], np.int32)).tolist() == [4, 4]
    assert P.unary(P.UN_ABS, np.array([-3, 3], np.int8)).tolist() == [3, 3]


def test_permute_concat_slice_by_explicit_indexing():
    x = np.arange(24, dtype=np.int32).reshape(2, 3, 4)
    y = P.permute(x, (2, 0, 1))
    assert y.shape == (4, 2, 3)
    for c in range(4):
        for a in range(2):
            for b in range(3):
                assert y[c, a, b] == x[a, b, c]
    parts = [x[:, :1, :], x[:, 1:, :]]
    assert np.array_equal(P.concat(parts, 1), x)
    assert P.concat([x, x], 2).shape == (2, 3, 8) and P.concat([x, x], 2)[1, 2, 5] == x[1, 2, 1]
    s = P.slice_(x, 2, 1, 2)
    assert s.shape == (2, 3, 2) and s[1, 0, 0] == x[1, 0, 1] and s[0, 2, 1] == x[0, 2, 2]


def test_matmul_is_k_ascending_with_separate_rounding():
    # (1e8 * 1 + 1 * 1) - 1e8 * 1 in float32, k ascending: 0; any other order or a fused
    # multiply-add over the whole row gives 1
    a = np.array([[1e8, 1.0, -1e8]], np.float32)
    b = np.ones((3, 1), np.float32)
    assert P.binary(P.BIN_MATMUL, a, b)[0, 0] == 0.0


@pytest.mark.parametrize("kind", ["e4m3", "e5m2"])
def test_float8_restatement_against_what_the_format_fixes(kind):
    """The checker's Float8 conversions (DType.h:148-229) against facts that do not come from its own
    formula: the value of every code written out from the format's definition, codes surviving a
    round trip, and, for inputs with few mantissa bits, the code chosen being the nearest value in
    the table of all codes with ties going to the larger magnitude (the reference adds one half
    and truncates)."""
    ebits, mbits, bias = P.F8_LAYOUTS[kind]
    codes = np.arange(256, dtype=np.uint8)
    table = P.f8_bits_to_f32(codes, kind)
    top = (1 << ebits) - 1
    for c in range(256):
        e, m = (c >> mbits) & top, c & ((1 << mbits) - 1)
        sign = -1.0 if c & 0x80 else 1.0
        if e == top:
            assert (np.isinf(table[c]) and np.sign(table[c]) == sign) if m == 0 else np.isnan(table[c])
        elif e == 0:
            assert table[c] == np.float32(sign * m * 2.0 ** (1 - bias - mbits)) and np.signbit(table[c]) == (sign < 0)
        else:
            assert table[c] == np.float32(sign * (1 + m / 2.0 ** mbits) * 2.0 ** (e - bias))
    finite = np.isfinite(table) | np.isinf(table)
    assert np.array_equal(P.f32_to_f8_bits(table[finite], kind), codes[finite])
    # landmarks
    one = P.f32_to_f8_bits(np.float32(1.0), kind)
    assert int(one) == (bias << mbits)
    largest = table[(top << mbits) - 1]
    step = largest - table[(top << mbits) - 2]
    got = P.f32_to_f8_bits(np.array([largest, largest + step / 2 * 0.999, largest + step / 2, np.nan, -np.inf,
                                     -0.0, table[1] / 2, table[1] / 2 * 0.99], np.float32), kind)
    assert got.tolist() == [(top << mbits) - 1, (top << mbits) - 1, top << mbits, top << mbits,
                            0x80 | (top << mbits), 0x80, 1, 0]
    # nearest-value property by brute force over the table
    rng = np.random.default_rng(5)
    pos = table[:top << mbits].astype(np.float64)  # the non-negative finite values, ascending
    assert np.all(np.diff(pos) > 0)
    x = (rng.integers(0, 1 << 14, 4000) * 2.0 ** -14 * rng.choice(2.0 ** np.arange(-bias - mbits, top - bias), 4000))
    x = x[x <= largest].astype(np.float32)
    got = P.f32_to_f8_bits(x, kind)
    for xv, c in zip(x.astype(np.float64), got.tolist()):
        dist = np.abs(pos - xv)
        best = np.flatnonzero(dist == dist.min()).max()  # a tie goes to the larger value
        if xv < pos[1 << mbits] and best == (1 << mbits):
            best -= 1  # below the smallest normal the mantissa is clamped to its field (DType.h:184-185)
        assert c == best, (xv, c, best)
    assert np.array_equal(P.f32_to_f8_bits(-x, kind), got | 0x80)
