"""Second, independently written decoder of the four GGUF block formats (vectorised numpy).

Written from the published ggml block definitions, deliberately in a different style from the C
checker (whole-tensor array slicing instead of per-block loops, integer tables instead of
branches) so that a shared transcription mistake is unlikely.  Used only to cross-check the C
checker bit for bit on random bytes.
"""
from __future__ import annotations

import numpy as np

Q4_0, Q8_0, Q4_K, Q6_K = 1, 5, 9, 11


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


DECODERS = {Q4_0: decode_q4_0, Q8_0: decode_q8_0, Q4_K: decode_q4_k, Q6_K: decode_q6_k}


def decode(fmt: int, raw: np.ndarray, k: int) -> np.ndarray:
    return DECODERS[fmt](np.ascontiguousarray(raw, np.uint8), k)
