"""CPU oracle of the QVB8R (rANS-coded band ids) path.  TEST INFRASTRUCTURE: only tests/, the smoke check and the
CPU-baseline leg of bench.py may import this; the product never does.

Restates, with the reference lines each part follows:
  slot_tables      src/qv_band/formats/qvb8r/codec.py:10-20
  read_container   src/qv_band/formats/qvb8r/container.py:52-71  (layout :1-12, writer :30-49)
  blocks_for       container.py:74-82
  runtime_tables   container.py:85-89
  walk / encode    oracle/qvb8r_walk.c (qvb8r_cpu.cpp:35-47 and :76-96), loaded with ctypes
  ids / restore    id = symbol + drow[row]; value = fmaf(id, tau_s, min_s) (qvb8r_cuda.cu:113-115, 302); escapes overwrite
Pinning: slot_tables and blocks_for against the reference's own outputs (tests/golden/ref_qvb8r_tables.npz); the walk by
round trip, a closed-form single-lane rANS and, where oracle/_ref builds, by the reference's compiled encoder and row
decoder; restore by the invariant "QVB8R restore == QVB8 restore of the same ids".  read_container and runtime_tables
by what the reference's own reader returned for a file of this build and by a file the reference's writer made
(tests/golden/ref_qvb8r_file.npz); parity of the writer POLICY is unpinned by construction (the reference ships none).
"""
from __future__ import annotations

import ctypes
import json
import os
import subprocess
import zlib

import numpy as np

from oracle import qvb8_oracle as O

PB, MQ, MAX_ID, MAX_FREQ, CENTRE, PAD_WORDS = 12, 4096, 2048, 1024, 256, 2048
HERE = os.path.dirname(os.path.abspath(__file__))
_LIB = None


class OracleQVB8RError(ValueError):
    pass


def _lib():
    global _LIB
    if _LIB is None:
        path = os.path.join(HERE, "_build", "libqvb8r_oracle.so")
        if not os.path.exists(path):
            subprocess.run(["make", "-C", HERE, "walk"], check=True, stdout=subprocess.DEVNULL)
        lib = ctypes.CDLL(path)
        vp, i64 = ctypes.c_void_p, ctypes.c_int64
        lib.qvb8r_walk.argtypes = [vp, i64, vp, vp, vp, i64, vp, i64, vp]
        lib.qvb8r_walk.restype = i64
        lib.qvb8r_encode_tile.argtypes = [vp, i64, i64, vp, vp, vp, i64, vp]
        lib.qvb8r_encode_tile.restype = i64
        _LIB = lib
    return _LIB


def reference_module():
    """The reference's compiled CPU codec (oracle/_ref/qvb8r_ref.so) or None where it was not built."""
    path = os.path.join(HERE, "_ref", "qvb8r_ref.so")
    if not os.path.exists(path):
        return None
    import importlib.util
    import torch  # noqa: F401  (the extension links against torch)
    spec = importlib.util.spec_from_file_location("qvb8r_ref", path)
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    return mod


def slot_tables(F) -> np.ndarray:
    F = np.asarray(F).astype(np.int64)
    K, N = F.shape
    tab = np.zeros((K, MQ), np.uint32)
    for k in range(K):
        slot = 0
        for s in range(N):
            for d in range(int(F[k, s])):
                tab[k, slot] = s | (d << 11) | ((int(F[k, s]) - 1) << 22)
                slot += 1
        if slot != MQ:
            raise OracleQVB8RError(f"class {k}: frequencies sum to {slot}, not {MQ}")
    return tab


def read_container(blob: bytes) -> dict:
    if blob[:4] != b"QVBR":
        raise OracleQVB8RError("not a .qvb8r file")
    ver, hl = np.frombuffer(blob, "<u4", 2, 4)
    if int(ver) != 2:
        raise OracleQVB8RError(f".qvb8r version {int(ver)}")
    if zlib.crc32(blob[:-4]) != int(np.frombuffer(blob, "<u4", 1, len(blob) - 4)[0]):
        raise OracleQVB8RError("crc32 mismatch")
    hdr = json.loads(blob[12:12 + int(hl)])
    if hdr.get("PB") != PB:
        raise OracleQVB8RError("PB")
    out = dict(hdr)
    for k, (off, dt, shape) in hdr["arrays"].items():
        n = int(np.prod(shape)) if shape else 1
        out[k] = np.frombuffer(blob, np.dtype(dt), n, off).reshape(shape)
    return out


def blocks_for(tiles, tiles_per_block: int) -> np.ndarray:
    b, i, n = [], 0, len(tiles)
    while i < n:
        j = i
        while j < n and j - i < tiles_per_block and tiles[j][0] == tiles[i][0]:
            j += 1
        b.append((tiles[i][0], i, j - i))
        i = j
    return np.array(b, np.int32).reshape(-1, 3)


def runtime_tables(d: dict):
    return (slot_tables(d["freq"]), np.asarray(d["tiles"]).astype(np.int64),
            np.concatenate([np.asarray(d["words"], np.uint32), np.zeros(PAD_WORDS, np.uint32)]),
            np.asarray(d["tile_off"]).astype(np.int64))


def walk(d: dict) -> np.ndarray:
    """Symbols (rows in SORTED order, P) of every tile of the tensor."""
    tab = np.ascontiguousarray(slot_tables(d["freq"]))
    tiles = np.ascontiguousarray(np.asarray(d["tiles"]).astype(np.int64))
    words = np.ascontiguousarray(np.asarray(d["words"], np.uint32))
    off = np.ascontiguousarray(np.asarray(d["tile_off"]).astype(np.int64))
    states = np.ascontiguousarray(np.asarray(d["states"], np.uint64))
    P = int(d["P"])
    R = int(tiles[:, 2].sum()) if len(tiles) else 0
    out = np.zeros((R, P), np.int16)
    rc = _lib().qvb8r_walk(words.ctypes.data, len(words), off.ctypes.data, states.ctypes.data, tiles.ctypes.data,
                           len(tiles), tab.ctypes.data, P, out.ctypes.data)
    if rc != 0:
        raise OracleQVB8RError(f"tile {-rc - 1}: the walk does not consume its stream exactly")
    return out


def encode_tile(sym, f, c):
    """(words, states) of one tile: sym (nr, P) int16, f / c the class's frequencies and exclusive cumulative sums."""
    sym = np.ascontiguousarray(sym, np.int16)
    nr, P = sym.shape
    f = np.ascontiguousarray(f, np.int64)
    c = np.ascontiguousarray(c, np.int64)
    cap = nr * P * PB // 32 + 80
    w = np.zeros(cap, np.uint32)
    st = np.zeros(32, np.uint64)
    n = _lib().qvb8r_encode_tile(sym.ctypes.data, nr, P, f.ctypes.data, c.ctypes.data, w.ctypes.data, cap, st.ctypes.data)
    if n < 0:
        raise OracleQVB8RError("encode_tile failed")
    return w[:n].copy(), st


def ids(d: dict) -> np.ndarray:
    """Band ids (Q, P) in ORIGINAL row order: id = symbol + drow[row]."""
    sym = walk(d).astype(np.int64)
    perm = np.asarray(d["perm"]).astype(np.int64)
    out = np.zeros_like(sym)
    out[perm] = sym + np.asarray(d["drow"]).astype(np.int64)[perm][:, None]
    return out


def reconstruct(d: dict, esc_idx=None, esc_vals=None) -> np.ndarray:
    """fp32 band values, escapes (default: the file's full list) overwritten: the QVB8 restore of the same ids."""
    ei = np.asarray(d["esc_idx"] if esc_idx is None else esc_idx, np.int64)
    ev = np.asarray(d["esc_val"] if esc_vals is None else esc_vals, np.float32)
    return O.reconstruct(np.asarray(d["min_s"], np.float32), np.asarray(d["tau_s"], np.float32), ids(d), ei, ev)
