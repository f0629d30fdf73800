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
from qvb8_amd.formats.qvb8.module import apply_keeping_fp32_metadata  # noqa: F401  (same metadata rule)
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


class QVBandLinearV8R(nn.Module):
    CHUNK_BYTES = 512 << 20
    bf16_gemm = False
    _TC_SPLIT_MAX = 48

    def __init__(self, d: dict, bias=None, device="cuda", path: str | None = None):
        super().__init__()
        self.path = path
        self._arrays = None if path else d               # built from arrays, not from a file: kept for host_arrays()
        tab, tiles, words, off = QF.runtime_tables(d)
        Q, P = int(d["Q"]), int(d["P"])
        self.out_features, self.in_features, self.T = Q, P, int(d["T"])
        dev = torch.device(device)
        buf = lambda name, a: self.register_buffer(name, _t(a, dev), persistent=False)
        buf("words", words.view(np.int32)); buf("off", off)
        buf("states", np.asarray(d["states"], np.uint64).view(np.int64)); buf("tiles", tiles)
        buf("drow", np.asarray(d["drow"]).astype(np.int32))
        buf("tab", tab.view(np.int32)); buf("perm", np.asarray(d["perm"], np.int32))
        blocks8 = QF.blocks_for(tiles, WPB)
        buf("blocks8", blocks8)
        buf("min_s", np.asarray(d["min_s"], np.float32)); buf("tau_s", np.asarray(d["tau_s"], np.float32))
        self.cert = d.get("cert", {}) or {}
        self.bf16_certified = self.cert.get("restore") == "fp16+bf16"
        # two escape tables (module.py:100-118): the file holds the full (bf16) list; the fp16 table comes only from
        # escape_tables.json.  No file on an fp16+bf16 pack: one table, and fp16 forwards refuse.
        ei_b = np.asarray(d["esc_idx"]).astype(np.int64)
        ev_b = np.asarray(d["esc_val"], np.float32)
        ed_b = np.asarray(d["esc_delta"], np.float32)
        need = np.ones(len(ei_b), bool)
        self.fp16_table_missing = False
        self._where = str(path)
        if self.bf16_certified:
            from qvb8_amd.formats.qvb8.escape_split import fp16_list_for, select_fp16
            lst = fp16_list_for(path)
            if lst is None:
                self.fp16_table_missing = True
            else:
                need = select_fp16(ei_b, lst, str(path))
        ei, ev, ed = ei_b[need], ev_b[need], ed_b[need]
        # correction tables grouped by output row (CSR, sorted by row then column): one thread per (m, q) adds its
        # group in this order -- reproducible
        o = np.argsort(ei, kind="stable")
        es = ei[o]
        uq, cnt = np.unique(es // P, return_counts=True) if len(es) else (np.zeros(0, np.int64), np.zeros(0, np.int64))
        buf("esc_uq", uq.astype(np.int64)); buf("esc_ptr", np.concatenate([[0], np.cumsum(cnt)]).astype(np.int64))
        buf("esc_c", (es % P).astype(np.int64)); buf("esc_delta", ed[o].astype(np.float32))
        buf("esc_flat", ei); buf("esc_val", ev)
        buf("esc_flat_bf16", ei_b); buf("esc_val_bf16", ev_b)
        self.bias = None if bias is None else nn.Parameter(bias.detach().to(dev), requires_grad=False)
        # M > 48: chunks of whole blocks, about CHUNK_BYTES of decoded 16-bit weight each:
        # (first block, blocks, first sorted row, rows)
        rows_per_block = [int(tiles[t0:t0 + n, 2].sum()) for _, t0, n in blocks8]
        first_row = [int(tiles[t0, 1]) for _, t0, n in blocks8]
        budget = max(1, self.CHUNK_BYTES // (2 * P))
        self.chunks, b = [], 0
        while b < len(blocks8):
            b1, rows = b, 0
            while b1 < len(blocks8) and (rows == 0 or rows + rows_per_block[b1] <= budget):
                rows += rows_per_block[b1]
                b1 += 1
            self.chunks.append((b, b1 - b, first_row[b], rows))
            b = b1

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
        shp = x.shape
        x2 = x.reshape(-1, shp[-1])
        if x2.device != self.words.device:
            x2 = x2.to(self.words.device)
        out_dtype = x.dtype
        if x2.dtype == torch.float32 and torch.is_autocast_enabled(x2.device.type):
            ad = torch.get_autocast_dtype(x2.device.type)
            if ad in (torch.bfloat16, torch.float16):
                x2, out_dtype = x2.to(ad), ad
        M = x2.shape[0]
        if M == 0:
            return x2.new_empty(*shp[:-1], self.out_features, dtype=out_dtype)
        if self.fp16_table_missing and not (x2.dtype == torch.bfloat16 and self.bf16_gemm and M > self._TC_SPLIT_MAX):
            from qvb8_amd.formats.qvb8.escape_split import fp16_missing_error
            raise fp16_missing_error(self._where)
        if M <= ext.MAX_M:
            y = self._small(x2)
        elif M <= self._TC_SPLIT_MAX:
            n = -(-M // ext.MAX_M)
            step = -(-M // n)
            y = torch.cat([self._small(x2[i:i + step]) for i in range(0, M, step)])
        else:
            y = self._chunked(x2, bf16=bool(self.bf16_gemm and self.bf16_certified and x2.dtype == torch.bfloat16))
        if self.bias is not None:
            y = y + self.bias.to(y.dtype)
        return y.to(out_dtype).reshape(*shp[:-1], self.out_features)

    def dense(self, dtype=torch.bfloat16):
        """The exact weight (Q, P) in `dtype` (escapes applied): for audits and re-packing, never on the hot path
        (module.py:313-325)."""
        code = {torch.float16: 0, torch.bfloat16: 1}.get(dtype, 2)
        if dtype == torch.float16 and self.fp16_table_missing:
            from qvb8_amd.formats.qvb8.escape_split import fp16_missing_error
            raise fp16_missing_error(self._where)
        W = ext.decode(*self._core(), self.in_features, code, 0, self.blocks8.shape[0], -1, 0, T=self.T)
        ef, ev = (self.esc_flat_bf16, self.esc_val_bf16) if dtype == torch.bfloat16 else (self.esc_flat, self.esc_val)
        if ef.numel():
            W.view(-1)[ef] = ev.to(W.dtype)
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
        tab, tiles, words, off = QF.runtime_tables(d)
        Q, P = int(d["Q"]), int(d["P"])
        self.num_embeddings, self.embedding_dim, self._out_dtype, self.T = Q, P, out_dtype, int(d["T"])
        dev = torch.device(device)
        buf = lambda name, a: self.register_buffer(name, _t(a, dev), persistent=False)
        buf("words", words.view(np.int32)); buf("off", off)
        buf("states", np.asarray(d["states"], np.uint64).view(np.int64)); buf("tiles", tiles)
        buf("drow", np.asarray(d["drow"]).astype(np.int32))
        buf("tab", tab.view(np.int32)); buf("perm", np.asarray(d["perm"], np.int32))
        blocks8 = QF.blocks_for(tiles, WPB)
        buf("blocks8", blocks8)
        buf("min_s", np.asarray(d["min_s"], np.float32)); buf("tau_s", np.asarray(d["tau_s"], np.float32))
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
        cert = d.get("cert", {}) or {}
        if out_dtype == torch.float16 and cert.get("restore") == "fp16+bf16":
            from qvb8_amd.formats.qvb8.escape_split import fp16_list_for, fp16_missing_error, select_fp16
            lst = fp16_list_for(path)
            if lst is None:
                raise fp16_missing_error(str(path))
            need = select_fp16(ei, lst, str(path))
            ei, ev = ei[need], ev[need]
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
