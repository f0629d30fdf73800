"""QVBD container ('.qvband' files): reader and writer for formula packs.

Layout (reference formats/qvb8/pack_container.py:8-22, 33-41, 48-106), little-endian:
    0   4s 'QVBD' | u8 version=1 | u32 Q | u32 P | f32 tau | f32 max_err
        | u8 source (0 bf16, 1 fp8_block, 2 q4_block, 3 fp32)
        | u8 calc_method (0 formula; 1 = table, refused)
        | u8 restore (0 fp16, 3 fp16+bf16) | 8 pad bytes            -> 32 bytes
    32  f32 min_s[Q] | f32 tau_s[Q] | u8 nbits[Q]
        u8 ids[payload + 8]            bit_off is not stored: prefix sum of nbits*P
        u64 n_esc_total | u64 n8
        i64 esc32_idx[n32] | esc32 values: u16 bf16 bits, or u32 for an fp32 source
        i64 esc8_idx[n8] | u8 esc8_codes[n8] | f32 s8[Q]
For restore 'fp16+bf16' the stored list holds every escape (the bf16 table); the
fp16 table is the subset named by escape_tables.json next to the pack.
"""
from __future__ import annotations

import struct

import numpy as np

from ...common.errors import Qvb8Error
from .decode import (IDS_PAD_BYTES, _combine_escapes, _row_bit_offsets, payload_bytes)

_MAGIC = b"QVBD"
_VERSION = 1
_CALC_FORMULA = 0
_CALC_TABLE = 1
CALC_FORMULA, CALC_TABLE = _CALC_FORMULA, _CALC_TABLE
_SOURCE_CODES = {"bf16": 0, "fp8_block": 1, "q4_block": 2, "fp32": 3}
_SOURCE_NAMES = {v: k for k, v in _SOURCE_CODES.items()}
_ESC32_WIDTH = {"bf16": 2, "fp8_block": 2, "q4_block": 2, "fp32": 4}
_RESTORE_FP16 = 0
_RESTORE_FP16_BF16 = 3
_RESTORE_NAMES = {_RESTORE_FP16: "fp16", _RESTORE_FP16_BF16: "fp16+bf16"}
_RESTORE_CODES = {v: k for k, v in _RESTORE_NAMES.items()}
_HEADER_FMT = "<4sBIIffBBB8x"
_HEADER_BYTES = struct.calcsize(_HEADER_FMT)
assert _HEADER_BYTES == 32


def _unpack_header(blob: bytes) -> tuple:
    if len(blob) < _HEADER_BYTES:
        raise Qvb8Error("qvband blob shorter than its header")
    magic, ver, Q, P, tau, max_err, src, calc, rcode = struct.unpack(_HEADER_FMT, blob[:_HEADER_BYTES])
    if magic != _MAGIC:
        raise Qvb8Error(f"not a qvband blob (magic {magic!r})")
    if ver != _VERSION:
        raise Qvb8Error(f"qvband version {ver}, reader supports {_VERSION}")
    if rcode not in _RESTORE_NAMES:
        raise Qvb8Error(f"pack has restore code {rcode}: only fp16 (0) and fp16+bf16 (3) are "
                        f"restore precisions; re-pack this tensor")
    if src not in _SOURCE_NAMES:
        raise Qvb8Error(f"unknown source code {src}")
    return (int(Q), int(P), float(tau), float(max_err), _SOURCE_NAMES[src], int(calc),
            _RESTORE_NAMES[rcode])


def calc_method_of(blob: bytes) -> int:
    return _unpack_header(blob)[5]


def pack_formula(*, Q: int, P: int, tau: float, max_err: float, min_s, tau_s, nbits, buf,
                 esc_idx=None, esc_vals=None, source: str = "bf16", restore: str = "fp16") -> bytes:
    """Write a QVBD formula pack.  Every escape goes to the esc32 pool; for a bf16-like
    source its value is stored as the upper 16 bits and must therefore be a bf16 number."""
    esc_idx = np.zeros(0, np.int64) if esc_idx is None else np.asarray(esc_idx, np.int64)
    esc_vals = np.zeros(0, np.float32) if esc_vals is None else np.asarray(esc_vals, np.float32)
    if len(esc_idx) != len(esc_vals):
        raise Qvb8Error("escape index and value lists differ in length")
    nbits = np.asarray(nbits, np.uint8)
    buf = np.asarray(buf, np.uint8)
    want = payload_bytes(nbits, P) + IDS_PAD_BYTES
    if buf.size != want:
        raise Qvb8Error(f"ids payload is {buf.size} bytes, the row widths need {want}")
    hdr = struct.pack(_HEADER_FMT, _MAGIC, _VERSION, int(Q), int(P), float(tau), float(max_err),
                      _SOURCE_CODES[source], _CALC_FORMULA, _RESTORE_CODES[restore])
    if _ESC32_WIDTH[source] == 4:
        raw = esc_vals.astype("<f4").tobytes()
    else:
        bits = np.ascontiguousarray(esc_vals, np.float32).view(np.uint32)
        if np.any(bits & 0xFFFF):
            raise Qvb8Error(f"a {source} pack stores escapes as bf16 bits; got a value that is not a bf16 number")
        raw = (bits >> 16).astype("<u2").tobytes()
    return b"".join([hdr, np.asarray(min_s, "<f4").tobytes(), np.asarray(tau_s, "<f4").tobytes(),
                     nbits.tobytes(), buf.tobytes(), struct.pack("<QQ", len(esc_idx), 0),
                     esc_idx.astype("<i8").tobytes(), raw,
                     np.zeros(int(Q), "<f4").tobytes()])


def unpack_formula(blob: bytes, *, skip_bit_decode: bool = True, fp16_list=None, where: str = "") -> dict:
    """Parse a QVBD formula pack.  The ids stay packed (`buf`): they are decoded on the
    GPU, whatever `skip_bit_decode` says (accepted for call-site compatibility; `codes` is always None).  esc_idx/esc_vals merge both pools ascending by flat index; esc_idx_fp16 /
    esc_vals_fp16 is the fp16 table (the same list for an fp16 pack, a subset chosen
    by `fp16_list` for an fp16+bf16 pack, None when that list is missing)."""
    Q, P, tau, max_err, source, calc, restore = _unpack_header(blob)
    if calc != _CALC_FORMULA:
        raise Qvb8Error(f"unpack_formula got calc_method={calc}, expected {_CALC_FORMULA}")
    pos = [_HEADER_BYTES]

    def take(dt, n):
        a = np.frombuffer(blob, dt, count=n, offset=pos[0]).copy()
        pos[0] += a.nbytes
        return a

    min_s = take("<f4", Q)
    tau_s = take("<f4", Q)
    nbits = take(np.uint8, Q)
    bit_off = _row_bit_offsets(nbits, P)
    buf = take(np.uint8, payload_bytes(nbits, P) + IDS_PAD_BYTES)
    n_total, n8 = struct.unpack_from("<QQ", blob, pos[0])
    pos[0] += 16
    n32 = int(n_total) - int(n8)
    if n32 < 0:
        raise Qvb8Error(f"header says {n8} FP8 escapes of {n_total} total")
    e32_idx = take("<i8", n32)
    if _ESC32_WIDTH[source] == 4:
        e32_vals = take("<u4", n32).view(np.float32)
    else:
        e32_vals = (take("<u2", n32).astype(np.uint32) << np.uint32(16)).view(np.float32)
    e8_idx = take("<i8", int(n8))
    e8_codes = take(np.uint8, int(n8))
    s8 = take("<f4", Q)
    esc_idx, esc_vals = _combine_escapes(e32_idx, e32_vals, e8_idx, e8_codes, s8, P)
    if restore == "fp16+bf16":
        if fp16_list is None:
            ei16 = ev16 = None
        else:
            from .escape_split import select_fp16
            keep = select_fp16(esc_idx, fp16_list, where)
            ei16, ev16 = esc_idx[keep], esc_vals[keep]
    else:
        ei16, ev16 = esc_idx, esc_vals
    return dict(Q=Q, P=P, tau=tau, max_err=max_err, source=source, restore=restore,
                min_s=min_s, tau_s=tau_s, codes=None, esc_idx=esc_idx, esc_vals=esc_vals,
                esc_idx_fp16=ei16, esc_vals_fp16=ev16, nbits=nbits, bit_off=bit_off, buf=buf)
