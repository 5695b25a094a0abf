"""Independent NumPy decoders / encoders of the GGML block formats the kernels read.

Written from the element's point of view (which byte and which bits hold
element e), not as the grouped loops the C oracle uses, so an indexing mistake
in one is unlikely to be repeated in the other.  float16 -> float32 goes
through numpy's own IEEE conversion.  All arithmetic is float32, one rounding
per operation, in the order of the block definitions.
"""
from __future__ import annotations

import numpy as np

F32 = np.float32


def _f16(b: np.ndarray, off: int) -> np.float32:
    return np.frombuffer(bytes(b[off:off + 2]), dtype="<f2")[0].astype(F32)


# ------------------------------------------------------------------ decode

def decode_q8_0(blk: np.ndarray) -> np.ndarray:
    d = _f16(blk, 0)
    q = blk[2:34].view(np.int8).astype(F32)
    return (d * q).astype(F32)


def decode_q8_1(blk: np.ndarray) -> np.ndarray:
    """{ f16 d; f16 s; i8 qs[32] }: the values are d * qs; the second half word (d * sum of qs) is not part of them."""
    d = _f16(blk, 0)
    q = blk[4:36].view(np.int8)
    return np.array([F32(d * F32(int(v))) for v in q], dtype=np.float32)


def decode_q4_0(blk: np.ndarray) -> np.ndarray:
    d = _f16(blk, 0)
    out = np.empty(32, dtype=F32)
    for e in range(32):
        byte = int(blk[2 + (e % 16)])
        nib = (byte >> 4) if e >= 16 else (byte & 15)
        out[e] = F32(nib - 8) * d
    return out


def _legacy5(blk: np.ndarray, qh_off: int, qs_off: int, e: int) -> int:
    """Stored value of element e of a 32-element block: nibble (low for e < 16) plus, with qh_off >= 0, bit e of the
    little-endian 32-bit word at qh_off as the fifth bit."""
    byte = int(blk[qs_off + (e % 16)])
    q = (byte >> 4) if e >= 16 else (byte & 15)
    if qh_off >= 0:
        word = int.from_bytes(bytes(blk[qh_off:qh_off + 4]), "little")
        q |= ((word >> e) & 1) << 4
    return q


def decode_q4_1(blk: np.ndarray) -> np.ndarray:
    d, m = _f16(blk, 0), _f16(blk, 2)
    return np.array([F32(F32(F32(_legacy5(blk, -1, 4, e)) * d) + m) for e in range(32)], dtype=F32)


def decode_q5_0(blk: np.ndarray) -> np.ndarray:
    d = _f16(blk, 0)
    return np.array([F32(F32(_legacy5(blk, 2, 6, e) - 16) * d) for e in range(32)], dtype=F32)


def decode_q5_1(blk: np.ndarray) -> np.ndarray:
    d, m = _f16(blk, 0), _f16(blk, 2)
    return np.array([F32(F32(F32(_legacy5(blk, 4, 8, e)) * d) + m) for e in range(32)], dtype=F32)


def decode_q2_k(blk: np.ndarray) -> np.ndarray:
    scales, qs, d, dmin = blk[0:16], blk[16:80], _f16(blk, 80), _f16(blk, 82)
    out = np.empty(256, dtype=F32)
    for e in range(256):
        half, run, pos = e // 128, (e % 128) // 32, e % 32
        field = (int(qs[32 * half + pos]) >> (2 * run)) & 3
        s = int(scales[e // 16])
        out[e] = F32(F32(F32(d * F32(s & 15)) * F32(field)) - F32(dmin * F32(s >> 4)))
    return out


def encode_q2_k(d, dmin, sc, mn, q) -> np.ndarray:
    """sc, mn: 16 four-bit scales and minima; q: 256 values in 0..3; the element is d * sc * q - dmin * mn."""
    blk = np.zeros(84, dtype=np.uint8)
    sc = np.asarray(sc, dtype=np.uint8); mn = np.asarray(mn, dtype=np.uint8); q = np.asarray(q, dtype=np.uint8)
    blk[0:16] = (sc & 15) | ((mn & 15) << 4)
    for e in range(256):
        half, run, pos = e // 128, (e % 128) // 32, e % 32
        blk[16 + 32 * half + pos] |= (int(q[e]) & 3) << (2 * run)
    _put_f16(blk, 80, d); _put_f16(blk, 82, dmin)
    return blk


def q3k_scale(scales: np.ndarray, k: int) -> int:
    """Stored 6-bit scale k (0..15) of a Q3_K super-block from its 12 scale bytes."""
    lo = (int(scales[k]) & 15) if k < 8 else (int(scales[k - 8]) >> 4)
    hi = (int(scales[8 + k % 4]) >> (2 * (k // 4))) & 3
    return lo | (hi << 4)


def decode_q3_k(blk: np.ndarray) -> np.ndarray:
    hmask, qs, scales, d = blk[0:32], blk[32:96], blk[96:108], _f16(blk, 108)
    out = np.empty(256, dtype=F32)
    for e in range(256):
        half, run, pos = e // 128, (e % 128) // 32, e % 32
        field = (int(qs[32 * half + pos]) >> (2 * run)) & 3
        third = (int(hmask[pos]) >> (4 * half + run)) & 1
        k = e // 16
        out[e] = F32(F32(d * F32(q3k_scale(scales, k) - 32)) * F32(field - (0 if third else 4)))
    return out


def q4k_scale_min(scales: np.ndarray, j: int):
    s = [int(v) for v in scales]
    if j < 4:
        return s[j] & 63, s[j + 4] & 63
    return (s[j + 4] & 15) | ((s[j - 4] >> 6) << 4), (s[j + 4] >> 4) | ((s[j] >> 6) << 4)


def decode_q4_k(blk: np.ndarray) -> np.ndarray:
    d, dmin = _f16(blk, 0), _f16(blk, 2)
    out = np.empty(256, dtype=F32)
    for e in range(256):
        j = e // 32
        sc, mn = q4k_scale_min(blk[4:16], j)
        byte = int(blk[16 + 32 * (j // 2) + e % 32])
        nib = (byte >> 4) if (j % 2) else (byte & 15)
        dd = F32(d * F32(sc))
        mm = F32(dmin * F32(mn))
        out[e] = F32(F32(dd * F32(nib)) - mm)
    return out


def decode_q5_k(blk: np.ndarray) -> np.ndarray:
    """{ f16 d; f16 dmin; u8 scales[12]; u8 qh[32]; u8 qs[128] }: element e of sub-block j = e // 32 is the nibble of
    Q4_K plus 16 when bit j of qh[e % 32] is set."""
    d, dmin = _f16(blk, 0), _f16(blk, 2)
    out = np.empty(256, dtype=F32)
    for e in range(256):
        j = e // 32
        sc, mn = q4k_scale_min(blk[4:16], j)
        byte = int(blk[48 + 32 * (j // 2) + e % 32])
        nib = (byte >> 4) if (j % 2) else (byte & 15)
        q = nib + (16 if (int(blk[16 + e % 32]) >> j) & 1 else 0)
        dd = F32(d * F32(sc))
        mm = F32(dmin * F32(mn))
        out[e] = F32(F32(dd * F32(q)) - mm)
    return out


def decode_q6_k(blk: np.ndarray) -> np.ndarray:
    d = _f16(blk, 208)
    sc = blk[192:208].view(np.int8)
    out = np.empty(256, dtype=F32)
    for e in range(256):
        half, rem = divmod(e, 128)
        run, l = divmod(rem, 32)          # run 0..3 of 32 elements inside the half
        lo_byte = int(blk[64 * half + l + 32 * (run % 2)])
        nib = (lo_byte >> 4) if run >= 2 else (lo_byte & 15)
        hi2 = (int(blk[128 + 32 * half + l]) >> (2 * run)) & 3
        q = (nib | (hi2 << 4)) - 32
        s = int(sc[8 * half + 2 * run + l // 16])
        out[e] = F32(F32(d * F32(s)) * F32(q))
    return out


DECODERS = {8: (34, 32, decode_q8_0), 2: (18, 32, decode_q4_0), 12: (144, 256, decode_q4_k), 14: (210, 256, decode_q6_k),
            13: (176, 256, decode_q5_k), 3: (20, 32, decode_q4_1), 6: (22, 32, decode_q5_0), 7: (24, 32, decode_q5_1),
            11: (110, 256, decode_q3_k), 10: (84, 256, decode_q2_k), 9: (36, 32, decode_q8_1)}


def decode(ggml_type: int, raw: np.ndarray) -> np.ndarray:
    bb, be, fn = DECODERS[int(ggml_type)]
    raw = np.ascontiguousarray(raw).view(np.uint8).reshape(-1, bb)
    return np.concatenate([fn(b) for b in raw])


# ------------------------------------------------------------------ encode

def _put_f16(blk: np.ndarray, off: int, v) -> None:
    blk[off:off + 2] = np.frombuffer(np.float16(v).tobytes(), dtype=np.uint8)


def encode_q8_0(d, q) -> np.ndarray:
    blk = np.zeros(34, dtype=np.uint8)
    _put_f16(blk, 0, d)
    blk[2:] = np.asarray(q, dtype=np.int8).view(np.uint8)
    return blk


def encode_q8_1(d, q, s=None) -> np.ndarray:
    blk = np.zeros(36, dtype=np.uint8)
    _put_f16(blk, 0, d)
    q = np.asarray(q, dtype=np.int8)
    _put_f16(blk, 2, np.float32(np.float16(d)) * np.float32(int(q.astype(np.int64).sum())) if s is None else s)
    blk[4:] = q.view(np.uint8)
    return blk


def encode_q4_0(d, q) -> np.ndarray:
    """q: 32 values in 0..15 (stored value; the decoded element is (q - 8) * d)."""
    blk = np.zeros(18, dtype=np.uint8)
    _put_f16(blk, 0, d)
    q = np.asarray(q, dtype=np.uint8)
    blk[2:] = q[:16] | (q[16:] << 4)
    return blk


def _legacy5_fields(q):
    """32 stored values (0..31) -> the 16 nibble bytes and the word of fifth bits."""
    q = np.asarray(q, dtype=np.uint8)
    qs = (q[:16] & 15) | ((q[16:] & 15) << 4)
    word = 0
    for e in range(32):
        word |= ((int(q[e]) >> 4) & 1) << e
    return qs, np.frombuffer(word.to_bytes(4, "little"), dtype=np.uint8)


def encode_q4_1(d, m, q) -> np.ndarray:
    """q: 32 values in 0..15; the decoded element is q * d + m."""
    blk = np.zeros(20, dtype=np.uint8)
    _put_f16(blk, 0, d); _put_f16(blk, 2, m)
    blk[4:], _ = _legacy5_fields(q)
    return blk


def encode_q5_0(d, q) -> np.ndarray:
    """q: 32 values in 0..31; the decoded element is (q - 16) * d."""
    blk = np.zeros(22, dtype=np.uint8)
    _put_f16(blk, 0, d)
    blk[6:], blk[2:6] = _legacy5_fields(q)
    return blk


def encode_q5_1(d, m, q) -> np.ndarray:
    """q: 32 values in 0..31; the decoded element is q * d + m."""
    blk = np.zeros(24, dtype=np.uint8)
    _put_f16(blk, 0, d); _put_f16(blk, 2, m)
    blk[8:], blk[4:8] = _legacy5_fields(q)
    return blk


def encode_q3_k(d, sc, q) -> np.ndarray:
    """sc: 16 stored scales in 0..63 (the scale is sc - 32); q: 256 stored values in 0..7 (the element is q - 4)."""
    blk = np.zeros(110, dtype=np.uint8)
    q = np.asarray(q, dtype=np.uint8); sc = np.asarray(sc, dtype=np.uint8)
    for e in range(256):
        half, run, pos = e // 128, (e % 128) // 32, e % 32
        blk[32 + 32 * half + pos] |= (int(q[e]) & 3) << (2 * run)
        blk[pos] |= ((int(q[e]) >> 2) & 1) << (4 * half + run)
    for k in range(16):
        if k < 8:
            blk[96 + k] |= int(sc[k]) & 15
        else:
            blk[96 + k - 8] |= (int(sc[k]) & 15) << 4
        blk[96 + 8 + k % 4] |= ((int(sc[k]) >> 4) & 3) << (2 * (k // 4))
    _put_f16(blk, 108, d)
    return blk


def pack_q4k_scales(sc, mn) -> np.ndarray:
    """8 six-bit scales and 8 six-bit mins into 12 bytes."""
    out = np.zeros(12, dtype=np.uint8)
    for j in range(8):
        s, m = int(sc[j]), int(mn[j])
        if j < 4:
            out[j] |= s
            out[j + 4] |= m
        else:
            out[j + 4] |= (s & 15) | ((m & 15) << 4)
            out[j - 4] |= (s >> 4) << 6
            out[j] |= (m >> 4) << 6
    return out


def encode_q4_k(d, dmin, sc, mn, q) -> np.ndarray:
    """q: 256 values in 0..15."""
    blk = np.zeros(144, dtype=np.uint8)
    _put_f16(blk, 0, d)
    _put_f16(blk, 2, dmin)
    blk[4:16] = pack_q4k_scales(sc, mn)
    q = np.asarray(q, dtype=np.uint8).reshape(4, 2, 32)
    blk[16:] = (q[:, 0, :] | (q[:, 1, :] << 4)).reshape(-1)
    return blk


def encode_q5_k(d, dmin, sc, mn, q) -> np.ndarray:
    """q: 256 values in 0..31."""
    blk = np.zeros(176, dtype=np.uint8)
    _put_f16(blk, 0, d)
    _put_f16(blk, 2, dmin)
    blk[4:16] = pack_q4k_scales(sc, mn)
    q = np.asarray(q, dtype=np.uint8).reshape(8, 32)
    for j in range(8):
        blk[16:48] |= ((q[j] >> 4) & 1) << j
    lo = (q & 15).reshape(4, 2, 32)
    blk[48:] = (lo[:, 0, :] | (lo[:, 1, :] << 4)).reshape(-1)
    return blk


def encode_q6_k(d, sc, q) -> np.ndarray:
    """q: 256 stored values in 0..63 (decoded element is d * sc * (q - 32)); sc: 16 int8."""
    blk = np.zeros(210, dtype=np.uint8)
    q = np.asarray(q, dtype=np.uint8)
    for e in range(256):
        half, rem = divmod(e, 128)
        run, l = divmod(rem, 32)
        v = int(q[e])
        lo_i = 64 * half + l + 32 * (run % 2)
        blk[lo_i] |= ((v & 15) << 4) if run >= 2 else (v & 15)
        blk[128 + 32 * half + l] |= (v >> 4) << (2 * run)
    blk[192:208] = np.asarray(sc, dtype=np.int8).view(np.uint8)
    _put_f16(blk, 208, d)
    return blk
