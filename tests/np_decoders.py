"""Second, independently written decoder of the GGUF block formats (vectorised numpy).

Written from the published ggml block definitions, deliberately in a different style from the C
checker (whole-tensor array slicing instead of per-block loops, integer tables instead of
branches) so that a shared transcription mistake is unlikely.  Used only to cross-check the C
checker bit for bit on random bytes.
"""
from __future__ import annotations

import numpy as np

Q4_0, Q4_1, Q5_0, Q5_1, Q8_0, Q2_K, Q3_K, Q4_K, Q5_K, Q6_K = 1, 2, 3, 4, 5, 7, 8, 9, 10, 11


def _f16(raw_u8_pairs: np.ndarray) -> np.ndarray:
    """[..., 2] uint8 (little endian) -> float32 via IEEE binary16."""
    return np.ascontiguousarray(raw_u8_pairs).view("<f2")[..., 0].astype(np.float32)


def decode_q4_0(raw: np.ndarray, k: int) -> np.ndarray:
    b = raw.reshape(-1, k // 32, 18)
    d = _f16(b[..., 0:2])[..., None]
    qs = b[..., 2:18].astype(np.int32)
    vals = np.concatenate([(qs & 15) - 8, (qs >> 4) - 8], axis=-1).astype(np.float32)
    return (vals * d).reshape(b.shape[0], k)


def decode_q8_0(raw: np.ndarray, k: int) -> np.ndarray:
    b = raw.reshape(-1, k // 32, 34)
    d = _f16(b[..., 0:2])[..., None]
    qs = b[..., 2:34].view(np.int8).astype(np.float32)
    return (qs * d).reshape(b.shape[0], k)


def _q4k_scales_mins(s: np.ndarray):
    """s: [..., 12] uint8 -> (scales [..., 8], mins [..., 8]) as the 6-bit fields."""
    s = s.astype(np.int32)
    sc = np.empty(s.shape[:-1] + (8,), np.int32)
    mn = np.empty_like(sc)
    sc[..., 0:4] = s[..., 0:4] & 63
    mn[..., 0:4] = s[..., 4:8] & 63
    sc[..., 4:8] = (s[..., 8:12] & 15) | ((s[..., 0:4] >> 6) << 4)
    mn[..., 4:8] = (s[..., 8:12] >> 4) | ((s[..., 4:8] >> 6) << 4)
    return sc, mn


def decode_q4_k(raw: np.ndarray, k: int) -> np.ndarray:
    b = raw.reshape(-1, k // 256, 144)
    d = _f16(b[..., 0:2])
    dmin = _f16(b[..., 2:4])
    sc, mn = _q4k_scales_mins(b[..., 4:16])
    q = b[..., 16:144].reshape(b.shape[0], b.shape[1], 4, 32).astype(np.int32)
    # group g of 64 outputs: 32 low nibbles (sub-block 2g) then 32 high nibbles (sub-block 2g+1)
    nib = np.stack([q & 15, q >> 4], axis=3)  # [rows, nb, 4, 2, 32]
    nib = nib.reshape(b.shape[0], b.shape[1], 8, 32).astype(np.float32)
    d1 = (d[..., None] * sc.astype(np.float32))[..., None]
    m1 = (dmin[..., None] * mn.astype(np.float32))[..., None]
    return (d1 * nib - m1).reshape(b.shape[0], k)


def decode_q6_k(raw: np.ndarray, k: int) -> np.ndarray:
    b = raw.reshape(-1, k // 256, 210)
    rows, nb = b.shape[0], b.shape[1]
    ql = b[..., 0:128].reshape(rows, nb, 2, 64).astype(np.int32)
    qh = b[..., 128:192].reshape(rows, nb, 2, 32).astype(np.int32)
    sc = b[..., 192:208].view(np.int8).reshape(rows, nb, 2, 8).astype(np.float32)
    d = _f16(b[..., 208:210])
    # within each 128-half: output 32*r + l, r = 0..3, l = 0..31
    lo = np.stack([ql[..., 0:32] & 15, ql[..., 32:64] & 15, ql[..., 0:32] >> 4, ql[..., 32:64] >> 4], axis=3)
    hi = np.stack([(qh >> (2 * r)) & 3 for r in range(4)], axis=3)
    q = ((lo | (hi << 4)) - 32).astype(np.float32)  # [rows, nb, 2, 4, 32]
    # scale index for (r, l) is l // 16 + 2 r
    idx = (np.arange(32)[None, :] // 16 + 2 * np.arange(4)[:, None])  # [4, 32]
    scale = sc[..., idx]  # [rows, nb, 2, 4, 32]
    out = d[..., None, None, None] * scale * q
    return out.reshape(rows, k)


def _fifth_bits(qh_bytes: np.ndarray) -> np.ndarray:
    """[..., 4] uint8 -> [..., 32] 0/1: bit j of the little-endian word belongs to element j."""
    return np.unpackbits(np.ascontiguousarray(qh_bytes), axis=-1, bitorder="little").astype(np.int32)


def decode_q4_1(raw: np.ndarray, k: int) -> np.ndarray:
    b = raw.reshape(-1, k // 32, 20)
    d, m = _f16(b[..., 0:2])[..., None], _f16(b[..., 2:4])[..., None]
    qs = b[..., 4:20].astype(np.int32)
    vals = np.concatenate([qs & 15, qs >> 4], axis=-1).astype(np.float32)
    return (vals * d + m).reshape(b.shape[0], k)


def decode_q5_0(raw: np.ndarray, k: int) -> np.ndarray:
    b = raw.reshape(-1, k // 32, 22)
    d = _f16(b[..., 0:2])[..., None]
    high = _fifth_bits(b[..., 2:6])
    qs = b[..., 6:22].astype(np.int32)
    vals = (np.concatenate([qs & 15, qs >> 4], axis=-1) + 16 * high - 16).astype(np.float32)
    return (vals * d).reshape(b.shape[0], k)


def decode_q5_1(raw: np.ndarray, k: int) -> np.ndarray:
    b = raw.reshape(-1, k // 32, 24)
    d, m = _f16(b[..., 0:2])[..., None], _f16(b[..., 2:4])[..., None]
    high = _fifth_bits(b[..., 4:8])
    qs = b[..., 8:24].astype(np.int32)
    vals = (np.concatenate([qs & 15, qs >> 4], axis=-1) + 16 * high).astype(np.float32)
    return (vals * d + m).reshape(b.shape[0], k)


def _two_bit_planes(qs: np.ndarray) -> np.ndarray:
    """[..., 64] bytes -> [..., 256] 2-bit values in output order: per 32-byte half, plane p
    (bits 2p, 2p+1) of its 32 bytes gives outputs 32 p .. 32 p + 31 of that half."""
    rows_nb = qs.shape[:-1]
    h = qs.reshape(rows_nb + (2, 1, 32)).astype(np.int32)
    planes = (h >> (2 * np.arange(4))[:, None]) & 3  # [..., 2, 4, 32]
    return planes.reshape(rows_nb + (256,))


def decode_q2_k(raw: np.ndarray, k: int) -> np.ndarray:
    b = raw.reshape(-1, k // 256, 84)
    sc = b[..., 0:16].astype(np.int32)
    q = _two_bit_planes(b[..., 16:80]).astype(np.float32)
    d, dmin = _f16(b[..., 80:82])[..., None], _f16(b[..., 82:84])[..., None]
    dl = np.repeat(d * (sc & 15).astype(np.float32), 16, axis=-1)   # scale s governs outputs 16 s ..
    ml = np.repeat(dmin * (sc >> 4).astype(np.float32), 16, axis=-1)
    return (dl * q - ml).reshape(b.shape[0], k)


def decode_q3_k(raw: np.ndarray, k: int) -> np.ndarray:
    b = raw.reshape(-1, k // 256, 110)
    rows, nb = b.shape[0], b.shape[1]
    low2 = _two_bit_planes(b[..., 32:96])
    # bit t of hmask byte l belongs to output 32 t + l (t = 0..7), and SET means "no -4"
    hm = b[..., 0:32].astype(np.int32)
    high = ((hm[..., None, :] >> np.arange(8)[:, None]) & 1).reshape(rows, nb, 256)
    s = b[..., 96:108].astype(np.int32)
    low4 = np.concatenate([s[..., 0:4] & 15, s[..., 4:8] & 15, s[..., 0:4] >> 4, s[..., 4:8] >> 4], axis=-1)
    top2 = np.concatenate([(s[..., 8:12] >> sh) & 3 for sh in (0, 2, 4, 6)], axis=-1)
    scale = ((low4 | (top2 << 4)) - 32).astype(np.float32)           # 16 six-bit scales, biased by 32
    d = _f16(b[..., 108:110])[..., None]
    dl = np.repeat(d * scale, 16, axis=-1)
    return (dl * (low2 - 4 * (1 - high)).astype(np.float32)).reshape(rows, k)


def decode_q5_k(raw: np.ndarray, k: int) -> np.ndarray:
    b = raw.reshape(-1, k // 256, 176)
    rows, nb = b.shape[0], b.shape[1]
    d, dmin = _f16(b[..., 0:2]), _f16(b[..., 2:4])
    sc, mn = _q4k_scales_mins(b[..., 4:16])
    qh = b[..., 16:48].astype(np.int32)
    q = b[..., 48:176].reshape(rows, nb, 4, 32).astype(np.int32)
    nib = np.stack([q & 15, q >> 4], axis=3).reshape(rows, nb, 8, 32)
    high = (qh[..., None, :] >> np.arange(8)[:, None]) & 1           # bit s of qh[l] -> sub-block s, element l
    vals = (nib + 16 * high).astype(np.float32)
    d1 = (d[..., None] * sc.astype(np.float32))[..., None]
    m1 = (dmin[..., None] * mn.astype(np.float32))[..., None]
    return (d1 * vals - m1).reshape(rows, k)


DECODERS = {Q4_0: decode_q4_0, Q4_1: decode_q4_1, Q5_0: decode_q5_0, Q5_1: decode_q5_1, Q8_0: decode_q8_0,
            Q2_K: decode_q2_k, Q3_K: decode_q3_k, Q4_K: decode_q4_k, Q5_K: decode_q5_k, Q6_K: decode_q6_k}


def decode(fmt: int, raw: np.ndarray, k: int) -> np.ndarray:
    return DECODERS[fmt](np.ascontiguousarray(raw, np.uint8), k)
