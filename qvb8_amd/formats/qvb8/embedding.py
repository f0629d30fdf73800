"""nn.Embedding over a QVB8 pack: rows are restored on demand, on the GPU, by one launch of qvb8_lookup_rows
(reference: src/qv_band/formats/qvb8/embedding.py:21-164, which gathers bytes with torch indexing and loops over the
looked-up rows on the host for escapes).

A lookup has no reduction: row r of the table is `min_s[r] + id[r][c] * tau_s[r]` for its P columns, computed as an fp32
multiply followed by an fp32 add (two roundings, as the reference's torch expression does -- the linear layers use one
fused multiply-add instead), escapes written over it, then rounded once to the output dtype.
"""
from __future__ import annotations

import numpy as np
import torch
import torch.nn as nn

from qvb8_amd import ext_qvb8 as ext
from qvb8_amd.formats.qvb8.module import apply_keeping_fp32_metadata


class QVBandEmbeddingV8(nn.Module):
    """Embedding whose rows are decoded on demand from a QVB8 pack.  Buffers as the reference's (embedding.py:29-44):
    tau_s, min_s, nbits, bit_off, ids, esc_idx, esc_vals -- nbits is kept as uint8 (what the kernels read) where the
    reference widens it to int64 for its torch arithmetic."""

    def __init__(self, *, min_s, nbits, bit_off, ids, Q, P, tau_s, esc_idx, esc_vals, out_dtype=torch.bfloat16):
        super().__init__()
        self.num_embeddings = int(Q)
        self.embedding_dim = int(P)
        self._out_dtype = out_dtype
        self.register_buffer("tau_s", tau_s.to(torch.float32), persistent=False)
        self.register_buffer("min_s", min_s.to(torch.float32), persistent=False)
        self.register_buffer("nbits", nbits.to(torch.uint8), persistent=False)
        self.register_buffer("bit_off", bit_off.to(torch.int64), persistent=False)
        self.register_buffer("ids", ids, persistent=False)
        order = torch.argsort(esc_idx.to(torch.int64), stable=True) if esc_idx.numel() else None
        ei = esc_idx.to(torch.int64)
        ev = esc_vals.to(torch.float32)
        if order is not None:                     # the kernel searches the positions: they must ascend
            ei, ev = ei[order], ev[order]
        self.register_buffer("esc_idx", ei, persistent=False)
        self.register_buffer("esc_vals", ev, persistent=False)

    def _apply(self, fn, recurse=True):
        # model.to(torch.bfloat16) must not round min_s / tau_s / esc_vals (embedding.py:24-27)
        return apply_keeping_fp32_metadata(self, fn, recurse)

    @classmethod
    def from_packfile(cls, path: str, *, out_dtype=torch.bfloat16, tau: float | None = None, device: str = "cuda",
                      blob: bytes | None = None):
        """Reads a `.qvband` / legacy QVB8 pack (embedding.py:46-95).  One escape table is kept, chosen by the output
        dtype: the fp16 table for fp16 output (an fp16+bf16 pack without its escape_tables.json refuses), the full list
        otherwise.  `tau` is ignored (the pack carries its own)."""
        del tau
        if blob is None:
            with open(path, "rb") as fh:
                blob = fh.read()
        if blob[:4] == b"QVBD":
            from qvb8_amd.formats.qvb8.pack_container import CALC_TABLE, calc_method_of, unpack_formula
            if calc_method_of(blob) == CALC_TABLE:
                raise NotImplementedError("qvb8 embedding pack is a table (calc_method=1) pack -- only the formula has "
                                          "an embedding reader; stream this tensor dense instead.")
            from qvb8_amd.formats.qvb8.escape_split import fp16_list_for, fp16_missing_error
            d = unpack_formula(blob, skip_bit_decode=True, fp16_list=fp16_list_for(path), where=str(path))
            min_s, tau_s, nb, bit_off, buf, Q, P = d["min_s"], d["tau_s"], d["nbits"], d["bit_off"], d["buf"], d["Q"], d["P"]
            if out_dtype == torch.float16:
                if d["esc_idx_fp16"] is None:
                    raise fp16_missing_error(str(path))
                esc_idx, esc_vals = d["esc_idx_fp16"], d["esc_vals_fp16"]
            else:
                esc_idx, esc_vals = d["esc_idx"], d["esc_vals"]
        else:
            from qvb8_amd.formats.qvb8.decode import unpack_tensor
            (min_s, tau_s, nb, bit_off, buf, Q, P, _tau, esc_idx, esc_vals) = unpack_tensor(blob)
        dev = torch.device(device)
        return cls(min_s=torch.from_numpy(np.ascontiguousarray(min_s, np.float32)).to(dev),
                   nbits=torch.from_numpy(np.ascontiguousarray(nb, np.uint8)).to(dev),
                   bit_off=torch.from_numpy(np.ascontiguousarray(bit_off, np.int64)).to(dev),
                   ids=torch.from_numpy(np.ascontiguousarray(buf)).to(dev), Q=Q, P=P,
                   tau_s=torch.from_numpy(np.ascontiguousarray(tau_s, np.float32)).to(dev),
                   esc_idx=torch.from_numpy(np.ascontiguousarray(esc_idx, np.int64)).to(dev),
                   esc_vals=torch.from_numpy(np.ascontiguousarray(esc_vals, np.float32)).to(dev), out_dtype=out_dtype)

    def _lookup(self, rows: torch.Tensor, dtype, with_escapes: bool) -> torch.Tensor:
        rows = rows.reshape(-1).to(device=self.ids.device, dtype=torch.int64)
        return ext.lookup_rows(rows, self.ids, self.min_s, self.nbits, self.bit_off, self.embedding_dim, self.tau_s,
                               self.esc_idx if with_escapes else None, self.esc_vals if with_escapes else None, dtype)

    def _decode_rows(self, rows: torch.Tensor) -> torch.Tensor:
        """The given rows as (n, P) fp32 band values, escapes NOT applied (embedding.py:97-124)."""
        return self._lookup(rows, torch.float32, False)

    # An index outside 0..num_embeddings-1: the reference's gathers fail on it (IndexError on the CPU, a device-side
    # assertion on the GPU).  Here the kernel writes a row of NaN and the call stays free of host reads, so that it can be
    # captured in a graph; set check_indices = True to get the IndexError instead (one host read per call).
    check_indices = False

    def forward(self, input: torch.Tensor) -> torch.Tensor:
        """(*input.shape, P) in the output dtype, on the device `input` came from (embedding.py:126-158)."""
        if self.check_indices and input.numel():
            lo, hi = int(input.min()), int(input.max())
            if lo < 0 or hi >= self.num_embeddings:
                raise IndexError(f"embedding index {lo if lo < 0 else hi} outside 0..{self.num_embeddings - 1}")
        out = self._lookup(input, self._out_dtype, True)
        return out.reshape(*input.shape, self.embedding_dim).to(input.device)

    @property
    def weight(self):
        """Dense (Q, P) table in the output dtype -- like the reference's (embedding.py:160-164), the band values of
        every row WITHOUT the escapes."""
        rows = torch.arange(self.num_embeddings, device=self.ids.device)
        return self._lookup(rows, self._out_dtype, False)

    def extra_repr(self):
        return f"{self.num_embeddings}, {self.embedding_dim}, out_dtype={self._out_dtype}"
