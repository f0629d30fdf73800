"""QVBandLinearV8R: y = x @ W^T (+ bias) with W resident only as rANS-coded band ids (a .qvb8r tensor).

Same constructor `(d, bias=None, device="cuda", path=None)` over the dict container.read returns, same buffer names and
`from_packfile` / `dense` / `forward` as the reference's module (src/qv_band/formats/qvb8r/module.py:57-325).  Dispatch:

    M <= 48        one fused walk + product (ext.gemv / ext.multi; from two rows on the matrix cores), fp32 band value,
                   escapes corrected after it (esc_delta); the reference splits 17..48 rows into passes of <= 16
                   (module.py:297-305), here one walk serves them all
    more           dense restore in chunks of whole blocks (<= CHUNK_BYTES of fp16 / bf16 weight each) + library GEMMs
"""
from __future__ import annotations

import numpy as np
import torch
import torch.nn as nn

from qvb8_amd import ext_qvb8r as ext
from qvb8_amd.formats.qvb8.module import activation_rows, apply_keeping_fp32_metadata  # noqa: F401  (same metadata rule)
from . import container as QF

WPB = 8                    # tiles per block of the schedule the kernels use
FP32_METADATA = ("min_s", "tau_s", "esc_val", "esc_val_bf16", "esc_delta")


def _t(a, dev):
    a = np.ascontiguousarray(a)
    return torch.from_numpy(a if a.flags.writeable else a.copy()).to(dev)


def _apply_keeping_fp32(module: nn.Module, fn, recurse=True):
    """nn.Module._apply that moves the fp32 decode metadata with the module but never casts it: `.to(bfloat16)` must not
    round min_s / tau_s / escape values (module.py:162-175 of the reference)."""
    keep = {n: module._buffers[n] for n in FP32_METADATA if module._buffers.get(n) is not None}
    for n in keep:
        module._buffers[n] = None
    try:
        out = nn.Module._apply(module, fn, recurse)
    finally:
        dev = module._buffers["words"].device
        for n, b in keep.items():
            module._buffers[n] = b.to(dev)
    return out


def _register_walk_operands(module: nn.Module, d: dict, dev) -> tuple:
    """Registers what every QVB8R kernel walks -- coded words and tile offsets, initial states, tile and block tables, slot
    tables, row order, row constants -- as buffers of `module` (names of the reference's modules); returns (tiles, blocks)
    as host arrays for the caller's own planning."""
    tab, tiles, words, off = QF.runtime_tables(d)
    blocks = QF.blocks_for(tiles, WPB)
    operands = {
        "words": words.view(np.int32), "off": off, "states": np.asarray(d["states"], np.uint64).view(np.int64), "tiles": tiles,
        "drow": np.asarray(d["drow"]).astype(np.int32), "tab": tab.view(np.int32), "perm": np.asarray(d["perm"], np.int32),
        "blocks8": blocks, "min_s": np.asarray(d["min_s"], np.float32), "tau_s": np.asarray(d["tau_s"], np.float32),
    }
    for name, array in operands.items():
        module.register_buffer(name, _t(array, dev), persistent=False)
    return tiles, blocks


def _fp16_subset(positions: np.ndarray, path, certified_bf16: bool):
    """Which entries of the file's (full, bf16) escape list also belong to the fp16 table: all of them for a one-table pack;
    for an fp16+bf16 pack those that escape_tables.json names -- None when that file is not there."""
    if not certified_bf16:
        return np.ones(len(positions), bool)
    from qvb8_amd.formats.qvb8.escape_split import fp16_list_for, select_fp16
    listed = fp16_list_for(path)
    return None if listed is None else select_fp16(positions, listed, str(path))


def _plan_chunks(tiles, blocks, budget_rows: int) -> list:
    """Runs of whole blocks with at most `budget_rows` rows each (a single block may exceed it): (first block, blocks, first
    sorted row, rows)."""
    plan, start = [], 0
    while start < len(blocks):
        stop, rows = start, 0
        while stop < len(blocks):
            block_rows = int(tiles[blocks[stop][1]:blocks[stop][1] + blocks[stop][2], 2].sum())
            if rows and rows + block_rows > budget_rows:
                break
            rows += block_rows
            stop += 1
        plan.append((start, stop - start, int(tiles[blocks[start][1], 1]), rows))
        start = stop
    return plan


class QVBandLinearV8R(nn.Module):
    CHUNK_BYTES = 512 << 20
    bf16_gemm = False
    _TC_SPLIT_MAX = 48

    def __init__(self, d: dict, bias=None, device="cuda", path: str | None = None):
        super().__init__()
        self.path, self._where = path, str(path)
        self._arrays = None if path else d               # built from arrays, not from a file: kept for host_arrays()
        dev = torch.device(device)
        self.out_features, self.in_features, self.T = int(d["Q"]), int(d["P"]), int(d["T"])
        P = self.in_features
        tiles, blocks = _register_walk_operands(self, d, dev)
        self.cert = d.get("cert", {}) or {}
        self.bf16_certified = self.cert.get("restore") == "fp16+bf16"
        # Two escape tables (module.py:100-118): the file holds the full list, which is the bf16 table; the fp16 table is the
        # subset escape_tables.json names.  Without that file an fp16+bf16 pack has one table, and fp16 forwards refuse.
        full_pos = np.asarray(d["esc_idx"]).astype(np.int64)
        full_val = np.asarray(d["esc_val"], np.float32)
        subset = _fp16_subset(full_pos, path, self.bf16_certified)
        self.fp16_table_missing = subset is None
        if subset is None:
            subset = np.ones(len(full_pos), bool)
        pos, val, delta = full_pos[subset], full_val[subset], np.asarray(d["esc_delta"], np.float32)[subset]
        # the correction after a fused product runs per output row: escapes grouped by row, columns ascending inside a row
        # (one thread per (m, q) adds its group in that order -- reproducible)
        by_row = np.argsort(pos, kind="stable")
        rows_hit, per_row = np.unique(pos[by_row] // P, return_counts=True) if len(pos) else (np.zeros(0, np.int64), np.zeros(0, np.int64))
        tables = {"esc_uq": rows_hit.astype(np.int64), "esc_ptr": np.concatenate([[0], np.cumsum(per_row)]).astype(np.int64),
                  "esc_c": (pos[by_row] % P).astype(np.int64), "esc_delta": delta[by_row].astype(np.float32),
                  "esc_flat": pos, "esc_val": val, "esc_flat_bf16": full_pos, "esc_val_bf16": full_val}
        for name, array in tables.items():
            self.register_buffer(name, _t(array, dev), persistent=False)
        self.bias = nn.Parameter(bias.detach().to(dev), requires_grad=False) if bias is not None else None
        # beyond 48 rows of X: dense restore of about CHUNK_BYTES of 16-bit weight at a time
        self.chunks = _plan_chunks(tiles, blocks, max(1, self.CHUNK_BYTES // (2 * P)))

    @classmethod
    def from_packfile(cls, path: str, *, bias=None, tau: float | None = None, device: str = "cuda", blob: bytes | None = None):
        del tau
        d = QF.read(path, blob=blob)
        b = None
        if bias is not None:
            b = bias.detach() if isinstance(bias, torch.Tensor) else torch.tensor(bias)
        return cls(d, bias=b, device=device, path=path)

    def has_host_arrays(self) -> bool:
        return bool(self.path) or self._arrays is not None

    def host_arrays(self) -> dict:
        """The tensor as container.read returns it (host memory): read again from the file the module came from, or the
        arrays it was built from.  What joining members into one fused tensor starts from."""
        if self.path:
            return QF.read(self.path)
        if self._arrays is None:
            raise RuntimeError("QVBandLinearV8R: neither a file nor the source arrays are known for this module")
        return self._arrays

    def _apply(self, fn, recurse=True):
        return _apply_keeping_fp32(self, fn, recurse)

    def extra_repr(self):
        return f"in_features={self.in_features}, out_features={self.out_features}, bias={self.bias is not None}"

    # ---- kernel paths ----------------------------------------------------------------------------------------------
    def _core(self):
        return (self.words, self.off, self.states, self.tiles, self.blocks8, self.tab, self.perm, self.min_s, self.tau_s,
                self.drow)

    def _small(self, x2):
        xk = x2.contiguous()
        y = ext.multi(xk, *self._core(), T=self.T)
        return ext.fix_escapes(xk, self.esc_uq, self.esc_ptr, self.esc_c, self.esc_delta, y)

    def _chunked(self, x2, bf16: bool):
        dt = torch.bfloat16 if bf16 else torch.float16
        xk = x2 if bf16 else x2.float().clamp(-65504, 65504).half()          # saturating fp16, as the small-M paths of QVB8
        ef, ev = (self.esc_flat_bf16, self.esc_val_bf16) if bf16 else (self.esc_flat, self.esc_val)
        P = self.in_features
        y = torch.empty(x2.shape[0], self.out_features, device=x2.device, dtype=torch.float32)
        code = 1 if bf16 else 0
        for b0, nb, base, rows in self.chunks:
            W = ext.decode(*self._core(), P, code, b0, nb, base, rows, T=self.T)
            orows = self.perm[base:base + rows].long()
            if ef.numel():
                # escapes whose row falls in this chunk, at their compact position
                inv = torch.full((self.out_features,), -1, dtype=torch.long, device=W.device)
                inv[orows] = torch.arange(rows, device=W.device)
                pos = inv[ef // P]
                keep = pos >= 0
                W.view(-1)[pos[keep] * P + ef[keep] % P] = ev[keep].to(dt)
            y[:, orows] = torch.mm(xk, W.t(), out_dtype=torch.float32)       # 16-bit operands, fp32 accumulate and result
        return y

    def forward(self, x):
        lead = tuple(x.shape[:-1])
        rows, out_dtype = activation_rows(x, self.words.device)
        M = rows.shape[0]
        if M == 0:
            return rows.new_empty(*lead, self.out_features, dtype=out_dtype)
        dense_bf16 = bool(self.bf16_gemm and rows.dtype == torch.bfloat16 and M > self._TC_SPLIT_MAX)
        if self.fp16_table_missing and not dense_bf16:
            from qvb8_amd.formats.qvb8.escape_split import fp16_missing_error
            raise fp16_missing_error(self._where)
        if M <= self._TC_SPLIT_MAX:
            # one fused walk per call of at most ext.MAX_M rows; more rows are split evenly
            calls = -(-M // ext.MAX_M)
            per_call = -(-M // calls)
            parts = [self._small(rows[at:at + per_call]) for at in range(0, M, per_call)]
            y = parts[0] if len(parts) == 1 else torch.cat(parts)
        else:
            y = self._chunked(rows, bf16=dense_bf16 and bool(self.bf16_certified))
        if self.bias is not None:
            y = y + self.bias.to(y.dtype)
        return y.reshape(*lead, self.out_features).to(out_dtype)

    def dense(self, dtype=torch.bfloat16):
        """The exact weight (Q, P) in `dtype` (escapes applied): for audits and re-packing, never on the hot path
        (module.py:313-325)."""
        if dtype == torch.float16 and self.fp16_table_missing:
            from qvb8_amd.formats.qvb8.escape_split import fp16_missing_error
            raise fp16_missing_error(self._where)
        restore_code = 0 if dtype == torch.float16 else 1 if dtype == torch.bfloat16 else 2
        W = ext.decode(*self._core(), self.in_features, restore_code, 0, self.blocks8.shape[0], -1, 0, T=self.T)
        positions, values = (self.esc_flat_bf16, self.esc_val_bf16) if dtype == torch.bfloat16 else (self.esc_flat, self.esc_val)
        if positions.numel():
            W.view(-1).index_copy_(0, positions, values.to(W.dtype))
        return W.to(dtype)


class QVBandEmbeddingV8R(nn.Module):
    """nn.Embedding over a QVB8R tensor.  A lookup walks only the blocks (up to 8 tiles) that hold looked-up rows, on the GPU,
    and gathers the rows from them: the table stays coded in memory.  The reference decodes the rows on the CPU, one tile
    prefix per row, and keeps the table out of VRAM (src/qv_band/formats/qvb8r/module.py:339-395, qvb8r_cpu.cpp:13-51).
    Value of a row: `min_s + float(id) * tau_s` as an fp32 multiply followed by an fp32 add (two roundings, as that CPU
    code and the QVB8 embedding compute it), the row's escapes written over it, then rounded once to the output dtype."""

    def __init__(self, d: dict, out_dtype=torch.bfloat16, device="cuda", path: str | None = None):
        super().__init__()
        self.path = path
        Q, P = int(d["Q"]), int(d["P"])
        self.num_embeddings, self.embedding_dim, self._out_dtype, self.T = Q, P, out_dtype, int(d["T"])
        dev = torch.device(device)
        tiles, blocks8 = _register_walk_operands(self, d, dev)
        buf = lambda name, a: self.register_buffer(name, _t(a, dev), persistent=False)
        # original row -> slot of its decoded copy inside its block: block number and (tile in block) * T + row in tile
        perm = np.asarray(d["perm"]).astype(np.int64)
        sorted_pos = np.empty(Q, np.int64)
        sorted_pos[perm] = np.arange(Q)
        tile_of_sorted = np.repeat(np.arange(len(tiles)), tiles[:, 2])
        block_of_tile = np.repeat(np.arange(len(blocks8)), blocks8[:, 2])
        tile = tile_of_sorted[sorted_pos]
        buf("row_block", block_of_tile[tile].astype(np.int32))
        buf("row_slot", ((tile - blocks8[block_of_tile[tile], 1]) * self.T + (sorted_pos - tiles[tile, 1])).astype(np.int64))
        # one escape table, chosen by the output dtype (module.py:356-363): the fp16 subset for fp16 output of an fp16+bf16
        # pack (named by escape_tables.json), the file's full list otherwise; grouped by row
        ei = np.asarray(d["esc_idx"]).astype(np.int64)
        ev = np.asarray(d["esc_val"], np.float32)
        two_tables = (d.get("cert", {}) or {}).get("restore") == "fp16+bf16"
        if out_dtype == torch.float16 and two_tables:
            subset = _fp16_subset(ei, path, True)
            if subset is None:
                from qvb8_amd.formats.qvb8.escape_split import fp16_missing_error
                raise fp16_missing_error(str(path))
            ei, ev = ei[subset], ev[subset]
        order = np.argsort(ei, kind="stable")
        ei, ev = ei[order], ev[order]
        counts = np.bincount(ei // P, minlength=Q) if len(ei) else np.zeros(Q, np.int64)
        buf("esc_ptr", np.concatenate([[0], np.cumsum(counts)]).astype(np.int64))
        buf("esc_col", (ei % P).astype(np.int64)); buf("esc_val", ev)

    @classmethod
    def from_packfile(cls, path: str, *, out_dtype=torch.bfloat16, tau: float | None = None, device: str = "cuda",
                      blob: bytes | None = None):
        del tau
        return cls(QF.read(path, blob=blob), out_dtype=out_dtype, device=device, path=path)

    def _apply(self, fn, recurse=True):
        return _apply_keeping_fp32(self, fn, recurse)

    def extra_repr(self):
        return f"{self.num_embeddings}, {self.embedding_dim}, out_dtype={self._out_dtype}, rows walked on the GPU"

    def _core(self):
        return (self.words, self.off, self.states, self.tiles, self.blocks8, self.tab, self.perm, self.min_s, self.tau_s,
                self.drow)

    def _rows(self, rows: torch.Tensor, with_escapes: bool) -> torch.Tensor:
        """(n, P) fp32 values of the given original rows."""
        dev = self.words.device
        rows = rows.reshape(-1).to(device=dev, dtype=torch.int64)
        n, P = rows.numel(), self.embedding_dim
        if n == 0:
            return torch.empty((0, P), dtype=torch.float32, device=dev)
        if bool(((rows < 0) | (rows >= self.num_embeddings)).any()):
            raise IndexError("qvb8r embedding: row id out of range")
        wanted, which = torch.unique(self.row_block[rows], return_inverse=True)
        ids = ext.decode_blocks(wanted.to(torch.int32).contiguous(), *self._core(), P, 3, T=self.T)
        picked = ids[which * (WPB * self.T) + self.row_slot[rows]]
        out = self.min_s[rows, None] + picked.to(torch.float32) * self.tau_s[rows, None]      # multiply, then add: two roundings
        if with_escapes and self.esc_col.numel():
            first, count = self.esc_ptr[rows], self.esc_ptr[rows + 1] - self.esc_ptr[rows]
            total = int(count.sum())
            if total:
                owner = torch.repeat_interleave(torch.arange(n, device=dev), count)
                within = torch.arange(total, device=dev) - torch.repeat_interleave(torch.cumsum(count, 0) - count, count)
                e = first[owner] + within
                out[owner, self.esc_col[e]] = self.esc_val[e]
        return out

    def forward(self, input: torch.Tensor) -> torch.Tensor:
        out = self._rows(input, True).to(self._out_dtype)
        return out.reshape(*input.shape, self.embedding_dim).to(input.device if input.device.type != "cpu" else self.words.device)

    @property
    def weight(self):
        """Dense (Q, P) table in the output dtype, escapes applied, restored in slices of rows."""
        out = torch.empty(self.num_embeddings, self.embedding_dim, dtype=self._out_dtype, device=self.words.device)
        step = max(1, (64 << 20) // (4 * self.embedding_dim))
        for r0 in range(0, self.num_embeddings, step):
            rows = torch.arange(r0, min(r0 + step, self.num_embeddings), device=self.words.device)
            out[r0:r0 + rows.numel()] = self._rows(rows, True).to(self._out_dtype)
        return out
