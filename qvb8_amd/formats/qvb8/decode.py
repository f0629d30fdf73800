"""QVB8 byte layout: constants, bit packing, and the legacy standalone blob.

Host-side only (numpy).  The dense restore is NOT here: restoring weights is the
HIP library's job (qvb8_decode), and a CPU restore exists only as test
infrastructure outside the package.

Layout facts follow the reference reader (formats/qvb8/decode.py:30-43, 70-74,
286-314, 368-430).  A blob written here is read by that reader unchanged.

Standalone blob, version 11, little-endian:
    0   u32 magic 'QVB8' | u32 Q | u32 P | u32 version
    16  f64 tau | u64 n_esc | u32 esc_mode | u64 n_fp8 | 20 zero bytes
    64  f32 min_s[Q] | f32 tau_s[Q] | u8 nbits[Q] | u64 bit_off[Q]
        esc_mode 0: i64 esc_idx[n_esc] | f32 esc_vals[n_esc]
        esc_mode 1: i64 e32_idx | f32 e32_vals | i64 e8_idx | u8 e8_codes | f32 s8[Q]
        u8 ids[]  (everything that remains: payload + 8 pad bytes)
"""
from __future__ import annotations

import struct

import numpy as np

from ...common.errors import Qvb8Error

MAGIC = 0x38425651            # 'QVB8'
VERSION = 11
HEADER_BYTES = 64
_HEADER_FMT = "<IIIIdQIQ20x"
_HEADER_FMT_V10 = "<IIIIdQIB27x"
_HEADER_FMT_V9 = "<IIIIdQ32x"
MAX_NBITS = 32
MAX_CERTIFIED_NBITS = 14
FP16_MANTISSA_BITS = 10
IDS_PAD_BYTES = 8             # a reader lifts a whole word near the end of the payload


def _nbits_for(n_buckets) -> np.ndarray:
    """Bits needed to address n_buckets ids, at least 1 (reference decode.py:138-141).
    Integer arithmetic, so exact powers of two cannot round the wrong way."""
    n = np.maximum(np.asarray(n_buckets, np.int64), 1)
    nb = np.zeros(n.shape, np.int64)
    v = n - 1
    while np.any(v > 0):
        nb += (v > 0)
        v = v >> 1
    return np.maximum(nb, 1)


def _row_bit_offsets(nbits, P: int) -> np.ndarray:
    """Rows are packed back to back: exclusive prefix sum of nbits*P."""
    nb = np.asarray(nbits, np.int64)
    off = np.zeros(len(nb), np.int64)
    if len(nb) > 1:
        np.cumsum(nb[:-1] * P, out=off[1:])
    return off


def payload_bytes(nbits, P: int) -> int:
    return (int(np.asarray(nbits, np.int64).sum()) * P + 7) // 8


def pack_bits_rows(ids: np.ndarray, nbits: np.ndarray):
    """Bit-pack each row at its own width, rows back to back, LSB first.

    Returns (buf uint8 with 8 trailing zero bytes, bit_off uint64[Q]).  Rows whose
    length is a whole number of bytes (P % 8 == 0) are packed eight fields at a time;
    anything else goes bit by bit.
    """
    ids = np.ascontiguousarray(ids, np.uint64)
    Q, P = ids.shape
    nb = np.asarray(nbits, np.int64)
    off = _row_bit_offsets(nb, P)
    total = int((nb * P).sum())
    nbytes = (total + 7) // 8
    buf = np.zeros(nbytes + IDS_PAD_BYTES, np.uint8)
    if Q == 0 or P == 0:
        return buf, off.astype(np.uint64)
    if P % 8 == 0 and int(nb.max()) <= 8:
        g = P // 8
        shifts = np.arange(8, dtype=np.uint64)
        for w in np.unique(nb):
            w = int(w)
            rows = np.nonzero(nb == w)[0]
            f = ids[rows].reshape(len(rows), g, 8)
            word = np.zeros((len(rows), g), np.uint64)
            for j in range(8):
                word |= f[:, :, j] << np.uint64(w * j)
            by = ((word[:, :, None] >> (shifts[None, None, :w] * np.uint64(8)))
                  & np.uint64(0xFF)).astype(np.uint8).reshape(len(rows), g * w)
            dst = (off[rows] >> 3)[:, None] + np.arange(g * w)[None, :]
            buf[dst] = by
        return buf, off.astype(np.uint64)
    bits = np.zeros(nbytes * 8, np.uint8)
    for r in range(Q):
        w = int(nb[r])
        k = np.arange(w, dtype=np.uint64)
        rb = ((ids[r][:, None] >> k[None, :]) & np.uint64(1)).astype(np.uint8)
        bits[int(off[r]):int(off[r]) + w * P] = rb.reshape(-1)
    buf[:nbytes] = np.packbits(bits, bitorder="little")
    return buf, off.astype(np.uint64)


# -- FP8 (E4M3FN) escape pool: read side only --------------------------------------
def _e4m3_lut() -> np.ndarray:
    code = np.arange(256)
    s = np.where(code & 0x80, -1.0, 1.0)
    e = (code >> 3) & 0xF
    m = code & 0x7
    v = np.where(e == 0, s * m * 2.0 ** -9, s * (1.0 + m / 8.0) * np.exp2(e - 7.0))
    v = np.where((e == 15) & (m == 7), np.nan, v)
    return v.astype(np.float32)


def _combine_escapes(e32_idx, e32_vals, e8_idx, e8_codes, s8, P: int):
    """Merge the fp32 pool and the FP8 pool into one list ascending by flat index.
    An FP8 escape's value is fp16(lut[code] * s8[row]) (reference decode.py:127-161)."""
    if len(e8_idx) == 0:
        return e32_idx, e32_vals
    with np.errstate(over="ignore", invalid="ignore"):
        prod = (_e4m3_lut()[e8_codes] * s8[e8_idx // P]).astype(np.float32)
        e8_vals = prod.astype(np.float16).astype(np.float32)
    idx = np.concatenate([e32_idx, e8_idx])
    val = np.concatenate([e32_vals, e8_vals])
    o = np.argsort(idx, kind="stable")
    return idx[o], val[o]


# -- standalone blob ---------------------------------------------------------------
def read_header(blob: bytes):
    """(Q, P, tau, n_esc) from the 64-byte header alone."""
    magic, Q, P, version, tau, n_esc = struct.unpack(_HEADER_FMT_V9, blob[:HEADER_BYTES])
    if magic != MAGIC:
        raise Qvb8Error(f"not a QVB8 blob (magic {magic:#x})")
    if version not in (9, VERSION):
        raise Qvb8Error(f"QVB8 version {version}, expected {VERSION} (or 9)")
    return Q, P, tau, n_esc


def pack_tensor(min_s, tau_s, nbits, bit_off, buf, Q: int, P: int, tau: float,
                esc_idx=None, esc_vals=None) -> bytes:
    """Write a version-11 standalone blob, every escape verbatim (esc_mode 0)."""
    esc_idx = np.zeros(0, np.int64) if esc_idx is None else np.asarray(esc_idx, np.int64)
    esc_vals = np.zeros(0, np.float32) if esc_vals is None else np.asarray(esc_vals, np.float32)
    if len(esc_idx) != len(esc_vals):
        raise Qvb8Error("escape index and value lists differ in length")
    if int(np.max(nbits, initial=1)) > MAX_CERTIFIED_NBITS:
        raise Qvb8Error(f"a row needs more than {MAX_CERTIFIED_NBITS} bits")
    hdr = struct.pack(_HEADER_FMT, MAGIC, int(Q), int(P), VERSION, float(tau), len(esc_idx), 0, 0)
    parts = [hdr,
             np.asarray(min_s, "<f4").tobytes(), np.asarray(tau_s, "<f4").tobytes(),
             np.asarray(nbits, np.uint8).tobytes(), np.asarray(bit_off, "<u8").tobytes(),
             esc_idx.astype("<i8").tobytes(), esc_vals.astype("<f4").tobytes(),
             np.asarray(buf, np.uint8).tobytes()]
    return b"".join(parts)


def unpack_tensor(blob: bytes):
    """Inverse of pack_tensor; also reads versions 9 and 10 and split escape pools.
    Returns (min_s, tau_s, nbits, bit_off, buf, Q, P, tau, esc_idx, esc_vals)."""
    if len(blob) < HEADER_BYTES:
        raise Qvb8Error("QVB8 blob shorter than its header")
    magic, _, _, version = struct.unpack_from("<IIII", blob, 0)
    if magic != MAGIC:
        raise Qvb8Error(f"not a QVB8 blob (magic {magic:#x})")
    if version not in (9, 10, VERSION):
        raise Qvb8Error(f"QVB8 version {version}, expected {VERSION} (or 9, 10)")
    fmt = _HEADER_FMT_V10 if version == 10 else _HEADER_FMT
    magic, Q, P, version, tau, n_esc, esc_mode, n_fp8 = struct.unpack(fmt, blob[:HEADER_BYTES])
    pos = [HEADER_BYTES]

    def take(dt, n):
        a = np.frombuffer(blob, dt, count=n, offset=pos[0]).copy()
        pos[0] += a.nbytes
        return a

    min_s = take("<f4", Q)
    tau_s = take("<f4", Q)
    nbits = take(np.uint8, Q).astype(np.int64)
    bit_off = take("<u8", Q).astype(np.int64)
    if version == 9 or esc_mode == 0:
        esc_idx = take("<i8", n_esc)
        esc_vals = take("<f4", n_esc)
    else:
        if n_fp8 > n_esc:
            raise Qvb8Error(f"header says {n_fp8} FP8 escapes of {n_esc} total")
        n32 = n_esc - n_fp8
        e32_idx, e32_vals = take("<i8", n32), take("<f4", n32)
        e8_idx, e8_codes = take("<i8", n_fp8), take(np.uint8, n_fp8)
        s8 = take("<f4", Q)
        esc_idx, esc_vals = _combine_escapes(e32_idx, e32_vals, e8_idx, e8_codes, s8, P)
    buf = np.frombuffer(blob, np.uint8, offset=pos[0]).copy()
    return (min_s, tau_s, nbits, bit_off, buf, Q, P, tau, esc_idx, esc_vals)
