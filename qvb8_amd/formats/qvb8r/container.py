"""The .qvb8r file: one tensor per file (reference: src/qv_band/formats/qvb8r/container.py).

    b'QVBR' | u32 version (2) | u32 header_len | header JSON | zero pad to 64 | arrays, each 64-byte aligned | u32 crc32

The JSON header holds Q, P, T (most rows in a tile), K (classes), N (symbols), PB (12), the certification record of the
QVB8 pack the tensor came from, and every array as name -> [offset, dtype, shape]; the crc32 covers every byte before
it.  Arrays: perm i32[Q] (sorted row -> original row), freq u16[K, N], tiles i32[nt, 3] (class, first sorted row, rows),
tile_off u32[nt + 1] (in words), states u64[nt, 32], words u32[], drow i16[Q], min_s f32[Q], tau_s f32[Q],
esc_idx i64[E] (flat q * P + c), esc_val f32[E] (exact value), esc_delta f32[E] (exact - fp32 band value).
Slot tables, the block schedule and the read-ahead pad are derived at load (runtime_tables).
"""
from __future__ import annotations

import json
import zlib

import numpy as np

from qvb8_amd.common.errors import QVB8RFormatError
from .codec import PB, slot_tables

MAGIC, VERSION = b"QVBR", 2
PAD_WORDS = 2048          # zero words after the stream: a walker may read this far ahead of its cursor
ARRAYS = ("perm", "freq", "tiles", "tile_off", "states", "words", "drow", "min_s", "tau_s", "esc_idx", "esc_val", "esc_delta")
_DTYPES = dict(perm="<i4", freq="<u2", tiles="<i4", tile_off="<u4", states="<u8", words="<u4", drow="<i2",
               min_s="<f4", tau_s="<f4", esc_idx="<i8", esc_val="<f4", esc_delta="<f4")


def to_bytes(enc: dict, Q: int, P: int, min_s, tau_s, esc_idx, esc_val, esc_delta, cert: dict) -> bytes:
    """The file's bytes (container.py:30-49): `enc` is what codec.encode_ids returns."""
    src = dict(enc, min_s=min_s, tau_s=tau_s, esc_idx=esc_idx, esc_val=esc_val, esc_delta=esc_delta)
    arrs = {k: np.ascontiguousarray(np.asarray(src[k]).astype(_DTYPES[k])) for k in ARRAYS}
    hdr = dict(Q=int(Q), P=int(P), T=int(enc["T"]), K=int(enc["K"]), N=int(enc["N"]), PB=PB, cert=cert, arrays={})
    while True:                                            # offsets depend on the header's own length: until stable
        hj = json.dumps(hdr).encode()
        pos = (12 + len(hj) + 63) // 64 * 64
        for k, a in arrs.items():
            hdr["arrays"][k] = [pos, a.dtype.str, list(a.shape)]
            pos = (pos + a.nbytes + 63) // 64 * 64
        if json.dumps(hdr).encode() == hj:
            break
    buf = bytearray(MAGIC + np.uint32(VERSION).tobytes() + np.uint32(len(hj)).tobytes() + hj)
    for k, a in arrs.items():
        off = hdr["arrays"][k][0]
        buf += b"\0" * (off - len(buf))
        buf += a.tobytes()
    buf += b"\0" * ((len(buf) + 63) // 64 * 64 - len(buf))
    buf += np.uint32(zlib.crc32(buf)).tobytes()
    return bytes(buf)


def write(path: str, enc: dict, Q: int, P: int, min_s, tau_s, esc_idx, esc_val, esc_delta, cert: dict) -> int:
    blob = to_bytes(enc, Q, P, min_s, tau_s, esc_idx, esc_val, esc_delta, cert)
    with open(path, "wb") as fh:
        fh.write(blob)
    return len(blob)


def read(path: str | None = None, blob: bytes | None = None) -> dict:
    """Header fields + arrays (numpy views into the file bytes); QVB8RFormatError on a bad file (container.py:52-71)."""
    raw = blob if blob is not None else open(path, "rb").read()
    where = path or "<blob>"
    if len(raw) < 16 or raw[:4] != MAGIC:
        raise QVB8RFormatError(f"{where}: not a .qvb8r file")
    ver = int(np.frombuffer(raw, "<u4", 1, 4)[0])
    if ver != VERSION:
        raise QVB8RFormatError(f"{where}: .qvb8r version {ver}, this reader knows {VERSION}"
                               + (" (re-transcode the pack from its QVB8 form)" if ver < VERSION else ""))
    if zlib.crc32(memoryview(raw)[:-4]) != int(np.frombuffer(raw, "<u4", 1, len(raw) - 4)[0]):
        raise QVB8RFormatError(f"{where}: crc32 mismatch (truncated or corrupt file)")
    hl = int(np.frombuffer(raw, "<u4", 1, 8)[0])
    try:
        hdr = json.loads(bytes(raw[12:12 + hl]))
    except ValueError as ex:
        raise QVB8RFormatError(f"{where}: unreadable header ({ex})") from None
    if hdr.get("PB") != PB:
        raise QVB8RFormatError(f"{where}: PB {hdr.get('PB')} != {PB}")
    out = dict(hdr)
    for k, (off, dt, shape) in hdr["arrays"].items():
        n = int(np.prod(shape)) if shape else 1
        if off < 0 or off + n * np.dtype(dt).itemsize > len(raw) - 4:
            raise QVB8RFormatError(f"{where}: array {k} lies outside the file")
        out[k] = np.frombuffer(raw, np.dtype(dt), n, off).reshape(shape)
    missing = [k for k in ARRAYS if k not in out]
    if missing:
        raise QVB8RFormatError(f"{where}: arrays missing: {missing}")
    return out


def blocks_for(tiles: np.ndarray, tiles_per_block: int) -> np.ndarray:
    """Block schedule: runs of <= tiles_per_block consecutive tiles of one class -> (class, first tile, tiles)
    (container.py:74-82)."""
    t = np.asarray(tiles)
    n = len(t)
    if n == 0:
        return np.zeros((0, 3), np.int32)
    cls = t[:, 0]
    starts = np.flatnonzero(np.concatenate([[True], cls[1:] != cls[:-1]]))
    ends = np.concatenate([starts[1:], [n]])
    b = []
    for s, e in zip(starts, ends):
        for i in range(int(s), int(e), tiles_per_block):
            b.append((int(cls[s]), i, min(tiles_per_block, int(e) - i)))
    return np.array(b, np.int32).reshape(-1, 3)


def runtime_tables(d: dict):
    """(slot tables u32 (K, 4096), tiles i64, padded words u32, tile offsets i64): what a reader builds once at load
    (container.py:85-89)."""
    tab = slot_tables(d["freq"])
    words = np.concatenate([np.asarray(d["words"], np.uint32), np.zeros(PAD_WORDS, np.uint32)])
    return tab, np.asarray(d["tiles"]).astype(np.int64), words, np.asarray(d["tile_off"]).astype(np.int64)
