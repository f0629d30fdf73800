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
import struct
import zlib

import numpy as np

from qvb8_amd.common.errors import QVB8RFormatError
from .codec import PB, slot_tables

MAGIC, VERSION = b"QVBR", 2
PAD_WORDS = 2048          # zero words after the stream: a walker may read this far ahead of its cursor
ARRAYS = ("perm", "freq", "tiles", "tile_off", "states", "words", "drow", "min_s", "tau_s", "esc_idx", "esc_val", "esc_delta")
_DTYPES = dict(perm="<i4", freq="<u2", tiles="<i4", tile_off="<u4", states="<u8", words="<u4", drow="<i2",
               min_s="<f4", tau_s="<f4", esc_idx="<i8", esc_val="<f4", esc_delta="<f4")


_PREFIX = struct.Struct("<4sII")          # magic, version, length of the header text


def _up64(n: int) -> int:
    return (n + 63) & ~63


def _place(meta: dict, arrays: list) -> tuple[bytes, dict]:
    """Where every array goes.  The table of offsets is part of the header text, and the first array starts behind that
    text: the table is recomputed from the text's length until it no longer changes (the file format's own rule)."""
    table: dict = {}
    while True:
        text = json.dumps(dict(meta, arrays=table)).encode()
        cursor, proposal = _up64(_PREFIX.size + len(text)), {}
        for name, a in arrays:
            proposal[name] = [cursor, a.dtype.str, list(a.shape)]
            cursor = _up64(cursor + a.nbytes)
        if proposal == table:
            return text, table
        table = proposal


def to_bytes(enc: dict, Q: int, P: int, min_s, tau_s, esc_idx, esc_val, esc_delta, cert: dict) -> bytes:
    """The bytes of a .qvb8r file for the arrays codec.encode_ids returned plus the row metadata and escapes of the QVB8
    pack (the reference's writer: container.py:30-49; the same bytes for the same input)."""
    given = dict(enc, min_s=min_s, tau_s=tau_s, esc_idx=esc_idx, esc_val=esc_val, esc_delta=esc_delta)
    arrays = [(name, np.ascontiguousarray(np.asarray(given[name]).astype(_DTYPES[name]))) for name in ARRAYS]
    meta = dict(Q=int(Q), P=int(P), T=int(enc["T"]), K=int(enc["K"]), N=int(enc["N"]), PB=PB, cert=cert)
    text, table = _place(meta, arrays)
    last_name, last = arrays[-1]
    body_end = _up64(table[last_name][0] + last.nbytes)
    out = bytearray(body_end + 4)                                     # zero-filled: every gap is padding already
    _PREFIX.pack_into(out, 0, MAGIC, VERSION, len(text))
    out[_PREFIX.size:_PREFIX.size + len(text)] = text
    view = memoryview(out)
    for name, a in arrays:
        at = table[name][0]
        view[at:at + a.nbytes] = a.reshape(-1).view(np.uint8).data
    struct.pack_into("<I", out, body_end, zlib.crc32(view[:body_end]))
    return bytes(out)


def write(path: str, enc: dict, Q: int, P: int, min_s, tau_s, esc_idx, esc_val, esc_delta, cert: dict) -> int:
    blob = to_bytes(enc, Q, P, min_s, tau_s, esc_idx, esc_val, esc_delta, cert)
    with open(path, "wb") as fh:
        fh.write(blob)
    return len(blob)


def read(path: str | None = None, blob: bytes | None = None) -> dict:
    """The header's fields and every array (numpy views of the file's bytes) as one dict; QVB8RFormatError names what is
    wrong with a file that cannot be used (reference reader: container.py:52-71)."""
    if blob is None:
        with open(path, "rb") as fh:
            blob = fh.read()
    name = path if path else "<bytes>"
    data = memoryview(blob)
    if len(data) < _PREFIX.size + 4:
        raise QVB8RFormatError(f"{name}: {len(data)} bytes is too short for a .qvb8r file")
    magic, version, text_len = _PREFIX.unpack_from(data, 0)
    if magic != MAGIC:
        raise QVB8RFormatError(f"{name}: starts with {bytes(magic)!r}, a .qvb8r file starts with {MAGIC!r}")
    if version != VERSION:
        hint = "; older files must be transcoded again from the QVB8 pack" if version < VERSION else ""
        raise QVB8RFormatError(f"{name}: file format version {version}, supported is {VERSION}{hint}")
    body = len(data) - 4
    (stored_crc,) = struct.unpack_from("<I", data, body)
    if zlib.crc32(data[:body]) != stored_crc:
        raise QVB8RFormatError(f"{name}: checksum does not match the contents (file damaged or cut short)")
    if _PREFIX.size + text_len > body:
        raise QVB8RFormatError(f"{name}: header of {text_len} bytes does not fit the file")
    try:
        fields = json.loads(bytes(data[_PREFIX.size:_PREFIX.size + text_len]))
        table = fields["arrays"]
    except (ValueError, KeyError, TypeError) as why:
        raise QVB8RFormatError(f"{name}: header cannot be parsed ({why})") from None
    if fields.get("PB") != PB:
        raise QVB8RFormatError(f"{name}: coded with {fields.get('PB')}-bit probabilities, this reader handles {PB}")
    absent = [k for k in ARRAYS if k not in table]
    if absent:
        raise QVB8RFormatError(f"{name}: header lists no {', '.join(absent)}")
    result = dict(fields)
    for key, (start, type_str, shape) in table.items():
        dt = np.dtype(type_str)
        count = int(np.prod(shape)) if shape else 1
        if start < 0 or start + count * dt.itemsize > body:
            raise QVB8RFormatError(f"{name}: '{key}' ({count} x {dt}) at byte {start} runs past the end of the file")
        result[key] = np.frombuffer(blob, dt, count, start).reshape(shape)
    return result


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
