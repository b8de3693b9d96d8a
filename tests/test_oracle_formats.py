"""Pins of the CPU checker's scalar types and block decoders (no GPU)."""
import numpy as np
import pytest

import np_decoders
from litenn_amd import synth
from litenn_amd.formats import Q2_K, Q3_K, Q4_0, Q4_1, Q4_K, Q5_0, Q5_1, Q5_K, Q6_K, Q8_0, FORMAT_NAMES

FORMATS = [Q4_0, Q4_1, Q5_0, Q5_1, Q8_0, Q2_K, Q3_K, Q4_K, Q5_K, Q6_K]


def test_block_layouts_match_reference_table(oracle, golden):
    table = golden["block_layouts"]
    for fmt in FORMATS:
        name = FORMAT_NAMES[fmt]
        assert list(oracle.block_layout(fmt)) == table[name]
        assert oracle.row_bytes(fmt, 4096) == 4096 // table[name][0] * table[name][1]
    assert oracle.block_layout(6) == (0, 0) and oracle.block_layout(12) == (0, 0)  # Q8_1, Q8_K: no dequantizer
    assert oracle.row_bytes(Q4_K, 4096 + 32) == 0  # not a whole number of super-blocks


def test_f16_to_f32_exhaustive(oracle):
    """All 65536 bit patterns against numpy's IEEE binary16 (DType.h:112-134 is exact)."""
    bits = np.arange(65536, dtype=np.uint16)
    got = oracle.f16_to_f32(bits)
    want = bits.view(np.float16).astype(np.float32)
    nan = np.isnan(want)
    assert np.array_equal(np.isnan(got), nan)
    assert np.array_equal(got[~nan].view(np.uint32), want[~nan].view(np.uint32))


def litenn_f16_expected(x: np.ndarray) -> np.ndarray:
    """Independent statement of DType.h:63-110 in real arithmetic: |x| is rounded to the binary16
    grid with floor(|x| / ulp + 1/2) (ties up in magnitude), values below 2^-24 vanish (the
    reference returns a signed zero for every exponent < -24, even above the half-way point
    2^-25), and anything that reaches 2^16 becomes infinity."""
    x64 = np.abs(x.astype(np.float64))
    is_inf = np.isinf(x64)
    x64 = np.where(is_inf, 1e30, x64)
    with np.errstate(divide="ignore"):
        e = np.floor(np.log2(np.where(x64 > 0, x64, 1.0)))
    e = np.maximum(e, -14.0)
    ulp = np.exp2(e - 10.0)
    q = np.floor(x64 / ulp + 0.5)
    mag = q * ulp
    mag = np.where(x64 < 2.0**-24, 0.0, mag)
    mag = np.where(mag >= 65536.0, np.inf, mag)
    return np.copysign(mag, x.astype(np.float64)).astype(np.float32)


def test_f32_to_f16_rounds_half_up_in_magnitude(oracle):
    """DType.h:63-110 examines only the first dropped bit: round-to-nearest with ties away from
    zero, checked against a real-arithmetic restatement and against IEEE RNE off the ties."""
    rng = np.random.default_rng(0)
    x = np.concatenate([
        rng.standard_normal(200000).astype(np.float32) * np.float32(10.0),
        (rng.standard_normal(50000) * 1e-6).astype(np.float32),  # subnormal halves
        np.array([0.0, -0.0, 65504.0, 65519.9, 65520.0, 1e6, -1e6, np.inf, -np.inf, 5.96e-8, 2.9e-8, 3.1e-8,
                  1.0 + 2.0**-11, 1.0 + 3 * 2.0**-11, -(2.0 + 2.0**-10), 2.0**-24 * 1.5, 2.0**-14 - 2.0**-25],
                 np.float32),
    ])
    got_bits = oracle.f32_to_f16_bits(x)
    got = oracle.f16_to_f32(got_bits)
    want = litenn_f16_expected(x)
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))
    # off the exact ties (and above the flush threshold) it coincides with IEEE round-to-nearest-even
    with np.errstate(over="ignore"):
        rne = x.astype(np.float16).astype(np.float32)
    differs = got.view(np.uint32) != rne.view(np.uint32)
    ax = np.abs(x.astype(np.float64))
    explained = (ax < 2.0**-24) | (np.abs(ax - (np.abs(got.astype(np.float64)) + np.abs(rne.astype(np.float64))) / 2) == 0)
    assert np.all(~differs | explained)
    assert differs.sum() >= 4  # the explicit ties above really do differ
    assert np.array_equal(oracle.f32_to_f16_bits(np.array([np.nan], np.float32)) & 0x7C00, [0x7C00])


def test_q4_0_reference_payload_fixture_closed_form(oracle, golden):
    """The 18-byte block the reference's importer test stores (it asserts bytes 0 and 17 only);
    its values follow in closed form: d = fp16(0x0010) = 2^-20, y[j] = (lo - 8) d, y[j+16] = (hi - 8) d."""
    fx = golden["q4_0_payload_fixture"]
    raw = np.array(fx["bytes"], np.uint8)
    assert raw[0] == fx["asserted"]["byte0"] and raw[17] == fx["asserted"]["byte17"]
    assert raw.size == fx["asserted"]["num_bytes"] == oracle.row_bytes(Q4_0, 32)
    y = oracle.dequantize(Q4_0, raw, 1, 32)[0]
    d = 2.0**-20
    qs = raw[2:]
    want = np.concatenate([(qs & 15).astype(np.int32) - 8, (qs >> 4).astype(np.int32) - 8]) * d
    assert np.array_equal(y, want.astype(np.float32))
    assert y[0] == (0x2 - 8) * d and y[16] == (0x2 - 8) * d and y[15] == (0xF - 8) * d and y[31] == (0x7 - 8) * d


@pytest.mark.parametrize("fmt", FORMATS)
def test_decoders_agree_with_independent_numpy_decoder_bitwise(oracle, fmt):
    """Uniformly random bytes in every field (scales included): two independently written
    decoders must agree bit for bit, NaN/Inf scales included."""
    rng = np.random.default_rng(fmt)
    k = 512
    rows = 64
    raw = rng.integers(0, 256, size=(rows, oracle.row_bytes(fmt, k)), dtype=np.uint8)
    a = oracle.dequantize(fmt, raw, rows, k)
    b = np_decoders.decode(fmt, raw, k).astype(np.float32)
    # random scale bits include NaN patterns: NaNs must coincide, everything else bit for bit
    nan = np.isnan(b)
    assert np.array_equal(np.isnan(a), nan)
    assert np.array_equal(a[~nan].view(np.uint32), b[~nan].view(np.uint32))
    # and on the benchmark's own weight law
    raw = synth.quant_weights(fmt, 16, 1024, 42)
    a = oracle.dequantize(fmt, raw, 16, 1024)
    b = np_decoders.decode(fmt, raw, 1024)
    assert np.array_equal(a.view(np.uint32), b.view(np.uint32))


def _f16_bytes(v):
    return np.array([v], np.float16).view(np.uint8)


def test_q8_0_closed_form(oracle):
    blk = np.zeros(34, np.uint8)
    blk[0:2] = _f16_bytes(0.5)
    q = np.arange(-16, 16, dtype=np.int8)
    blk[2:] = q.view(np.uint8)
    y = oracle.dequantize(Q8_0, blk, 1, 32)[0]
    assert np.array_equal(y, q.astype(np.float32) * 0.5)


def test_q4_k_reduces_to_nibbles_when_scales_are_one(oracle):
    """d = 1, dmin = 0, every 6-bit scale = 1, every min = 0  =>  y = nibble, laid out as
    64-element groups: 32 low nibbles then 32 high nibbles of the same 32 bytes."""
    blk = np.zeros(144, np.uint8)
    blk[0:2] = _f16_bytes(1.0)
    blk[2:4] = _f16_bytes(0.0)
    blk[4:8] = 1    # scales 0..3 = 1 (bits 6,7 clear => high bits of scales 4..7 are 0)
    blk[8:12] = 0   # mins 0..3 = 0, high bits of mins 4..7 = 0
    blk[12:16] = 1  # low nibble: scale 4..7 = 1; high nibble: min 4..7 = 0
    rng = np.random.default_rng(1)
    qs = rng.integers(0, 256, 128, dtype=np.uint8)
    blk[16:] = qs
    y = oracle.dequantize(Q4_K, blk, 1, 256)[0]
    want = np.concatenate([np.concatenate([g & 15, g >> 4]) for g in qs.reshape(4, 32)]).astype(np.float32)
    assert np.array_equal(y, want)


def test_q4_k_scale_and_min_fields_one_hot(oracle):
    """Each of the 8 (scale, min) pairs is exercised alone with a value that needs its high
    bits (>= 16 for sub-blocks 4..7), pinning the 6-bit packing of get_scale_min_k4."""
    for j in range(8):
        for which, value in (("scale", 37), ("min", 53)):
            s = np.zeros(12, np.int32)
            if j < 4:
                s[j if which == "scale" else j + 4] |= value
            else:
                lo4, hi2 = value & 15, value >> 4
                if which == "scale":
                    s[j + 4] |= lo4
                    s[j - 4] |= hi2 << 6
                else:
                    s[j + 4] |= lo4 << 4
                    s[j] |= hi2 << 6
            blk = np.zeros(144, np.uint8)
            blk[0:2] = _f16_bytes(2.0)
            blk[2:4] = _f16_bytes(0.25)
            blk[4:16] = s.astype(np.uint8)
            blk[16:] = 0x33  # every nibble = 3
            y = oracle.dequantize(Q4_K, blk, 1, 256)[0].reshape(8, 32)
            for sub in range(8):
                if sub != j:
                    assert np.all(y[sub] == 0.0)
                elif which == "scale":
                    assert np.all(y[sub] == 2.0 * value * 3)
                else:
                    assert np.all(y[sub] == -0.25 * value)


def test_q6_k_reduces_to_q_minus_32_when_scales_are_one(oracle):
    blk = np.zeros(210, np.uint8)
    rng = np.random.default_rng(2)
    ql = rng.integers(0, 256, 128, dtype=np.uint8)
    qh = rng.integers(0, 256, 64, dtype=np.uint8)
    blk[0:128], blk[128:192] = ql, qh
    blk[192:208] = 1
    blk[208:210] = _f16_bytes(1.0)
    y = oracle.dequantize(Q6_K, blk, 1, 256)[0]
    # brute force, element by element, straight from the layout description
    want = np.zeros(256, np.float32)
    for e in range(256):
        half, r, l = e // 128, (e % 128) // 32, e % 32
        lo_byte = int(ql[64 * half + l + (32 if r & 1 else 0)])
        low4 = (lo_byte >> 4) if r & 2 else (lo_byte & 15)
        high2 = (int(qh[32 * half + l]) >> (2 * r)) & 3
        want[e] = (low4 | (high2 << 4)) - 32
    assert np.array_equal(y, want)


def test_q6_k_scale_index_one_hot(oracle):
    """Scale s (int8, 16 per super-block) governs elements [16 s, 16 s + 16)."""
    for s in range(16):
        blk = np.zeros(210, np.uint8)
        blk[0:128] = 0x11  # low nibbles 1
        blk[128:192] = 0xAA  # high pairs 2 => q = 1 | (2 << 4) = 33 => q - 32 = 1
        blk[192 + s] = np.array([-7], np.int8).view(np.uint8)[0]
        blk[208:210] = _f16_bytes(0.5)
        y = oracle.dequantize(Q6_K, blk, 1, 256)[0]
        want = np.zeros(256, np.float32)
        want[16 * s:16 * s + 16] = 0.5 * -7 * 1
        assert np.array_equal(y, want)


def test_dequantize_rejects_ragged_rows(oracle):
    with pytest.raises(oracle.OracleError):
        oracle.dequantize(Q4_K, np.zeros(144, np.uint8), 1, 128)
    with pytest.raises(oracle.OracleError):
        oracle.dequantize(6, np.zeros(40, np.uint8), 1, 32)


# ---- the 32-element formats with a fifth bit and / or a minimum, and the remaining K-quants ----------
# Expected values are written element by element straight from the published block definitions, with
# the bit positions spelled out (not through the vectorised decoder above).

def test_q4_1_closed_form(oracle):
    """{fp16 d, fp16 m, 16 bytes}: element j is the low nibble of byte j, element j + 16 its high
    nibble; y = q d + m."""
    blk = np.zeros(20, np.uint8)
    blk[0:2], blk[2:4] = _f16_bytes(0.5), _f16_bytes(-3.0)
    qs = np.random.default_rng(3).integers(0, 256, 16, dtype=np.uint8)
    blk[4:] = qs
    y = oracle.dequantize(Q4_1, blk, 1, 32)[0]
    want = np.array([(int(qs[j % 16]) >> (4 if j >= 16 else 0)) & 15 for j in range(32)], np.float32) * 0.5 - 3.0
    assert np.array_equal(y, want)


@pytest.mark.parametrize("fmt", [Q5_0, Q5_1])
def test_q5_fifth_bit_one_hot(oracle, fmt):
    """Bit j of the 32-bit little-endian qh word is the fifth bit of element j (for the low-nibble
    half and the high-nibble half alike); Q5_0 subtracts 16, Q5_1 adds the minimum."""
    head = 2 if fmt == Q5_0 else 4
    for j in range(32):
        blk = np.zeros(head + 4 + 16, np.uint8)
        blk[0:2] = _f16_bytes(0.25)
        if fmt == Q5_1:
            blk[2:4] = _f16_bytes(1.5)
        blk[head + j // 8] = 1 << (j % 8)
        blk[head + 4:] = 0x21  # low nibbles 1, high nibbles 2
        y = oracle.dequantize(fmt, blk, 1, 32)[0]
        q = np.array([1] * 16 + [2] * 16, np.float32)
        q[j] += 16
        want = (q - 16) * 0.25 if fmt == Q5_0 else q * 0.25 + 1.5
        assert np.array_equal(y, want.astype(np.float32)), j


def test_q2_k_brute_force(oracle):
    """{16 scale bytes, 64 quant bytes, fp16 d, fp16 dmin}: output e sits in half n = e / 128, bit
    plane p = (e % 128) / 32 of byte 32 n + e % 32; scale byte e / 16: low nibble multiplies d, high
    nibble multiplies dmin."""
    rng = np.random.default_rng(4)
    blk = rng.integers(0, 256, 84, dtype=np.uint8)
    blk[80:82], blk[82:84] = _f16_bytes(0.5), _f16_bytes(0.125)
    y = oracle.dequantize(Q2_K, blk, 1, 256)[0]
    want = np.zeros(256, np.float32)
    for e in range(256):
        n, p, l = e // 128, (e % 128) // 32, e % 32
        q = (int(blk[16 + 32 * n + l]) >> (2 * p)) & 3
        sc = int(blk[e // 16])
        want[e] = np.float32(np.float32(0.5 * (sc & 15)) * q) - np.float32(0.125 * (sc >> 4))
    assert np.array_equal(y, want)


def test_q3_k_brute_force_and_scale_packing(oracle):
    """{32 mask bytes, 64 quant bytes, 12 scale bytes, fp16 d}: low two bits as in Q2_K; bit
    e / 32 of mask byte e % 32 set means no -4; scale s = e / 16 is six bits, biased by 32: low
    four from nibble (s / 8) of byte s % 8, top two from bits 2 (s / 4), .. of byte 8 + s % 4."""
    rng = np.random.default_rng(5)
    blk = rng.integers(0, 256, 110, dtype=np.uint8)
    blk[108:110] = _f16_bytes(0.25)
    y = oracle.dequantize(Q3_K, blk, 1, 256)[0]
    want = np.zeros(256, np.float32)
    for e in range(256):
        n, p, l = e // 128, (e % 128) // 32, e % 32
        q = (int(blk[32 + 32 * n + l]) >> (2 * p)) & 3
        if not (int(blk[l]) >> (e // 32)) & 1:
            q -= 4
        s = e // 16
        low4 = (int(blk[96 + s % 8]) >> (4 * (s // 8))) & 15
        top2 = (int(blk[96 + 8 + s % 4]) >> (2 * (s // 4))) & 3
        want[e] = np.float32(0.25 * ((low4 | (top2 << 4)) - 32)) * q
    assert np.array_equal(y, want)
    # one scale alone, with a value that needs its top bits
    for s in range(16):
        blk = np.zeros(110, np.uint8)
        blk[0:32] = 0xFF                      # every mask bit set: no -4
        blk[32:96] = 0x55                     # every 2-bit value 1
        blk[108:110] = _f16_bytes(1.0)
        value = 59                            # 6-bit field; 59 - 32 = 27
        blk[96 + s % 8] |= (value & 15) << (4 * (s // 8))
        blk[96 + 8 + s % 4] |= (value >> 4) << (2 * (s // 4))
        y = oracle.dequantize(Q3_K, blk, 1, 256)[0].reshape(16, 16)
        for t in range(16):
            assert np.all(y[t] == (27.0 if t == s else -32.0)), (s, t)


def test_q5_k_brute_force(oracle):
    """{fp16 d, fp16 dmin, 12 scale bytes (packed as in Q4_K), 32 high-bit bytes, 128 nibble bytes}:
    sub-block s = e / 32 takes the low (s even) or high (s odd) nibbles of bytes 32 (s / 2) + l and
    bit s of high-bit byte l."""
    rng = np.random.default_rng(6)
    blk = rng.integers(0, 256, 176, dtype=np.uint8)
    blk[0:2], blk[2:4] = _f16_bytes(0.5), _f16_bytes(0.25)
    y = oracle.dequantize(Q5_K, blk, 1, 256)[0]
    sc = blk[4:16].astype(np.int32)
    want = np.zeros(256, np.float32)
    for e in range(256):
        s, l = e // 32, e % 32
        byte = int(blk[48 + 32 * (s // 2) + l])
        q = ((byte >> 4) if s & 1 else (byte & 15)) + 16 * ((int(blk[16 + l]) >> s) & 1)
        if s < 4:
            scale, mn = sc[s] & 63, sc[s + 4] & 63
        else:
            scale = (sc[s + 4] & 15) | ((sc[s - 4] >> 6) << 4)
            mn = (sc[s + 4] >> 4) | ((sc[s] >> 6) << 4)
        want[e] = np.float32(np.float32(0.5 * scale) * q) - np.float32(0.25 * mn)
    assert np.array_equal(y, want)
