"""QVBandLinearV8: y = x @ W^T (+ bias) with W resident in HBM only as bit-packed band ids.

Same class name, constructor, buffers, attributes and `from_packfile` as the reference's compressed-linear operator
(src/qv_band/formats/qvb8/module.py:59-464), so model adapters that swap nn.Linear for it keep working.  The work is
done by libqvb8_amd.so through qvb8_amd.ext_qvb8; there is no dense cache and no CPU path: without the HIP library
every forward raises.

Dispatch on the row count M of the flattened input (the reference's: module.py:379-457):

    M <= 48, P % 128 == 0   matrix-core tile kernel (ext.mma_tiles): ids decoded once for all rows.  fp16 x is used
                            as it is; bf16 / fp32 x is narrowed like saturating_half (the value every fp16 path of the
                            reference multiplies) -- in registers for bf16, so decode (M = 1) is ONE launch;
                            a bf16-certified pack with bf16 x multiplies bf16 operands (the reference's bf16 mode).
                            The band value is the un-narrowed fp32 one, as in the reference's GEMV.
    49 .. 256 rows          the workgroup-tiled decode + GEMM kernel (same entry point) when the rows were copied into
                            width order and all widths are 4..8 (4..7 in bf16 mode): X staged in LDS, ids decoded in
                            registers, no dense weight written
    49 .. 96 rows otherwise equal passes of <= 48 rows (module.py:393-400)
    M <= 8 otherwise        GEMV (ext.gemv_multi)
    else                    dense restore (fp16, or bf16 when bf16_gemm and certified) + one library GEMM
"""
from __future__ import annotations

import numpy as np
import torch
import torch.nn as nn
import torch.nn.functional as F

from qvb8_amd import ext_qvb8 as ext

FP32_METADATA = ("min_s", "tau_s", "esc_vals", "esc_vals_bf16")

_MMA_MAX_M = ext.MMA_MAX_M
_MMA_SPLIT_MAX = 2 * _MMA_MAX_M


def apply_keeping_fp32_metadata(module: nn.Module, fn, recurse=True):
    """nn.Module._apply with the fp32 decode metadata protected from dtype casts: a `.to(bfloat16)` must not round
    min_s / tau_s / escape values (that would move weights by up to ~tau); only the device follows
    (reference: module.py:43-56)."""
    held = {}
    for name in FP32_METADATA:
        buf = module._buffers.get(name)
        if buf is not None:
            held[name] = buf
            module._buffers[name] = None              # nn.Module._apply skips absent buffers
    try:
        result = nn.Module._apply(module, fn, recurse)
    finally:
        anchor = module._buffers.get("ids")           # the metadata lives where the packed ids went
        for name, buf in held.items():
            module._buffers[name] = buf if anchor is None else buf.to(anchor.device)
    return result


class QVBandLinearV8(nn.Module):
    # The first call of the matrix-core path copies the rows once into width-sorted order (same total size; `ids` and
    # `bit_off` are replaced, every kernel keeps working through bit_off), so that calls compute row addresses instead of
    # reading them.  Set False to keep the file's row order in memory.
    sort_rows = True
    bf16_gemm = False             # opt-in: M > 96 bf16 callers decode to bf16 and run one bf16 GEMM (module.py:60-65)
    bf16_certified = False        # the pack certifies |orig - bf16(band)| <= tau (container restore code 3)
    fp16_table_missing = False    # fp16+bf16 pack loaded without escape_tables.json: fp16 forwards refuse

    def __init__(self, *, min_s, nbits, bit_off, ids, Q, P, tau_s, esc_idx, esc_vals, bias=None,
                 esc_idx_bf16=None, esc_vals_bf16=None):
        super().__init__()
        self.in_features = int(P)
        self.out_features = int(Q)
        self.register_buffer("tau_s", tau_s, persistent=False)
        self.register_buffer("min_s", min_s, persistent=False)
        self.register_buffer("nbits", nbits, persistent=False)
        self.register_buffer("bit_off", bit_off, persistent=False)
        self.register_buffer("ids", ids, persistent=False)

        def _sorted(ei, ev):
            # the correction kernels add a row's escapes in list order: ascending positions make results reproducible
            if ei.numel() > 1 and not bool((ei[1:] >= ei[:-1]).all()):
                o = torch.argsort(ei, stable=True)
                ei, ev = ei[o].contiguous(), ev[o].contiguous()
            return ei, ev
        esc_idx, esc_vals = _sorted(esc_idx, esc_vals)
        if esc_idx_bf16 is None:
            esc_idx_bf16, esc_vals_bf16 = esc_idx, esc_vals
        else:
            esc_idx_bf16, esc_vals_bf16 = _sorted(esc_idx_bf16, esc_vals_bf16)
        self.register_buffer("esc_idx", esc_idx, persistent=False)
        self.register_buffer("esc_vals", esc_vals, persistent=False)
        self.register_buffer("esc_idx_bf16", esc_idx_bf16, persistent=False)
        self.register_buffer("esc_vals_bf16", esc_vals_bf16, persistent=False)
        self.bias = None if bias is None else nn.Parameter(bias, requires_grad=False)

    # ---- construction ------------------------------------------------------------------------------------------

    @classmethod
    def from_encoded(cls, enc: dict, *, bias=None, device=None):
        """From the dict qvb8_amd.formats.qvb8.pack.encode_tensor returns (synthetic packs, tests, benchmarks)."""
        dev = torch.device(device) if device is not None else enc["ids"].device
        two = enc.get("restore") == "fp16+bf16"
        m = cls(min_s=enc["min_s"].to(dev), nbits=enc["nbits"].to(dev), bit_off=enc["bit_off"].to(dev),
                ids=enc["ids"].to(dev), Q=enc["Q"], P=enc["P"], tau_s=enc["tau_s"].to(dev),
                esc_idx=enc["esc_idx"].to(dev), esc_vals=enc["esc_vals"].to(dev),
                bias=None if bias is None else bias.to(dev),
                esc_idx_bf16=enc["esc_idx_bf16"].to(dev) if two else None,
                esc_vals_bf16=enc["esc_vals_bf16"].to(dev) if two else None)
        m.bf16_certified = two
        return m

    @classmethod
    def from_packfile(cls, path: str, *, bias=None, tau: float | None = None, device: str = "cuda",
                      blob: bytes | None = None):
        """Reads a `.qvband` / legacy QVB8 pack (module.py:162-218).  `tau` is accepted for call-site compatibility
        and ignored: every pack carries its own certified tau."""
        del tau
        if blob is None:
            with open(path, "rb") as fh:
                blob = fh.read()
        dev = torch.device(device)
        b = None
        if bias is not None:
            b = (bias.detach() if isinstance(bias, torch.Tensor) else torch.tensor(bias)).to(dev)
        esc_bf16 = (None, None)
        fp16_missing = False
        certified = False
        if blob[:4] != b"QVBD":
            from qvb8_amd.formats.qvb8.decode import unpack_tensor
            (min_s, tau_s, nb, bit_off, buf, Q, P, _tau, esc_idx, esc_vals) = unpack_tensor(blob)
        else:
            from qvb8_amd.formats.qvb8.pack_container import calc_method_of, unpack_formula, CALC_TABLE
            if calc_method_of(blob) == CALC_TABLE:
                raise NotImplementedError("qvb8 table (calc_method=1) packs are not read by QVBandLinearV8; "
                                          "this is a pre-unification file, re-pack it.")
            from qvb8_amd.formats.qvb8.escape_split import fp16_list_for
            d = unpack_formula(blob, skip_bit_decode=True, fp16_list=fp16_list_for(path), where=str(path))
            min_s, tau_s, nb, bit_off, buf = d["min_s"], d["tau_s"], d["nbits"], d["bit_off"], d["buf"]
            Q, P = d["Q"], d["P"]
            certified = d.get("restore") == "fp16+bf16"
            if d["esc_idx_fp16"] is None:
                esc_idx, esc_vals = d["esc_idx"], d["esc_vals"]
                fp16_missing = True
            else:
                esc_idx, esc_vals = d["esc_idx_fp16"], d["esc_vals_fp16"]
                if d["esc_idx_fp16"] is not d["esc_idx"]:
                    esc_bf16 = (torch.from_numpy(d["esc_idx"].astype(np.int64)).to(dev),
                                torch.from_numpy(d["esc_vals"].astype(np.float32)).to(dev))
        mod = cls(min_s=torch.from_numpy(np.ascontiguousarray(min_s, np.float32)).to(dev),
                  nbits=torch.from_numpy(np.ascontiguousarray(nb, np.uint8)).to(dev),
                  bit_off=torch.from_numpy(np.ascontiguousarray(bit_off, np.int64)).to(dev),
                  ids=torch.from_numpy(np.ascontiguousarray(buf)).to(dev),
                  Q=Q, P=P, tau_s=torch.from_numpy(np.ascontiguousarray(tau_s, np.float32)).to(dev),
                  esc_idx=torch.from_numpy(np.ascontiguousarray(esc_idx, np.int64)).to(dev),
                  esc_vals=torch.from_numpy(np.ascontiguousarray(esc_vals, np.float32)).to(dev),
                  bias=b, esc_idx_bf16=esc_bf16[0], esc_vals_bf16=esc_bf16[1])
        mod.bf16_certified = certified
        mod.fp16_table_missing = fp16_missing
        mod._where = str(path)
        return mod

    def escapes(self, dtype=torch.float16):
        """(esc_idx, esc_vals) for a decode that rounds the weight to `dtype` (module.py:116-124)."""
        if dtype == torch.bfloat16:
            return self.esc_idx_bf16, self.esc_vals_bf16
        if dtype == torch.float16 and self.fp16_table_missing:
            from qvb8_amd.formats.qvb8.escape_split import fp16_missing_error
            raise fp16_missing_error(getattr(self, "_where", "QVBandLinearV8"))
        return self.esc_idx, self.esc_vals

    def row_subset(self, rows: torch.Tensor) -> "QVBandLinearV8":
        """A linear over output rows `rows` only, sharing this module's `ids` buffer: rows of a pack are independent
        (own min_s, tau_s, width, offset), so a subset costs no weight memory (module.py:126-160)."""
        rows = rows.to(self.min_s.device).long()
        P = self.in_features
        remap = torch.full((self.out_features,), -1, dtype=torch.long, device=rows.device)
        remap[rows] = torch.arange(rows.numel(), device=rows.device)

        def sub(esc_idx, esc_vals):
            if not esc_idx.numel():
                return esc_idx, esc_vals
            q = esc_idx // P
            keep = remap[q] >= 0
            return remap[q[keep]] * P + esc_idx[keep] % P, esc_vals[keep]
        esc_idx, esc_vals = sub(self.esc_idx, self.esc_vals)
        same = self.esc_idx_bf16 is self.esc_idx
        ei_b, ev_b = (None, None) if same else sub(self.esc_idx_bf16, self.esc_vals_bf16)
        m = type(self)(min_s=self.min_s[rows], nbits=self.nbits[rows], bit_off=self.bit_off[rows], ids=self.ids,
                       Q=int(rows.numel()), P=P, tau_s=self.tau_s[rows], esc_idx=esc_idx, esc_vals=esc_vals,
                       bias=None, esc_idx_bf16=ei_b, esc_vals_bf16=ev_b)
        m.bf16_certified = self.bf16_certified
        m.fp16_table_missing = self.fp16_table_missing
        return m

    def _apply(self, fn, recurse=True):
        out = apply_keeping_fp32_metadata(self, fn, recurse)
        self.__dict__.pop("_mma_cache", None)           # the row records follow the buffers: rebuild after a move
        return out

    # ---- launch metadata ---------------------------------------------------------------------------------------

    def _mma_order(self):
        """(perm, rowinfo, layout) for ext.mma_tiles, or None when the tile kernel cannot read this weight.  Rows are sorted by
        width so that a 16-row tile shares one width (one decode pass); the row records hold, in that order, where each
        row's ids start, its width, tau_s, min_s and its output row.  Built once per weight, like the reference's
        perm / tile_nb (module.py:230-277); never built inside a graph capture (the width check reads the device)."""
        cached = self.__dict__.get("_mma_cache", False)
        if cached is not False:
            return cached
        if torch.cuda.is_current_stream_capturing():
            return None
        order = None
        if self.ids.is_cuda and self.in_features % 128 == 0 and self.ids.data_ptr() % 4 == 0 and self.out_features > 0:
            nb = self.nbits.to(torch.int16)
            if 1 <= int(nb.min()) and int(nb.max()) <= 14:
                perm = torch.argsort(nb, stable=True).to(torch.int32).contiguous()
                layout = None
                row_bytes = int((self.nbits.to(torch.int64) * self.in_features).sum().item()) // 8
                if self.sort_rows and 2 * row_bytes >= self.ids.numel():      # not for a small view into a shared stack
                    srt = ext.sort_rows_by_width(self.ids, self.nbits, self.bit_off, self.in_features, perm)
                    if srt is not None:
                        self.ids, self.bit_off, layout = srt
                rowinfo = ext.mma_prepare(self.nbits, self.bit_off, self.tau_s, self.min_s, self.in_features,
                                          self.ids.numel(), perm)
                order = (perm, rowinfo, layout)
        self._mma_cache = order
        return order

    def _gemm_ok(self, layout, bf16_mode: bool) -> bool:
        """Whether the workgroup-tiled kernel (49..256 rows) can read this weight: rows stored in width order, every
        width one the sliced decode handles, whole 256-column groups."""
        if layout is None or self.in_features % 256 != 0:
            return False
        top = 7 if bf16_mode else 8
        return all(4 <= int(layout.nbits[c]) <= top for c in range(int(layout.n_classes)))

    # ---- forward -----------------------------------------------------------------------------------------------

    def _finish(self, y, orig, out_dtype):
        y = y.reshape(*orig[:-1], self.out_features)
        if self.bias is not None:
            y = y + self.bias.to(y.dtype)
        return y.to(out_dtype)

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        orig = x.shape
        x2d = x.reshape(-1, orig[-1])
        if x2d.device != self.min_s.device:
            x2d = x2d.to(self.min_s.device)
        out_dtype = x.dtype
        if x2d.dtype == torch.float32 and torch.is_autocast_enabled(x2d.device.type):
            ad = torch.get_autocast_dtype(x2d.device.type)          # honour autocast like nn.Linear (module.py:336-344)
            if ad in (torch.bfloat16, torch.float16):
                x2d = x2d.to(ad)
                out_dtype = ad
        M = x2d.shape[0]
        if self.fp16_table_missing and x2d.dtype == torch.float16:
            from qvb8_amd.formats.qvb8.escape_split import fp16_missing_error
            raise fp16_missing_error(getattr(self, "_where", "QVBandLinearV8"))
        if M == 0:
            return x2d.new_zeros((*orig[:-1], self.out_features), dtype=out_dtype)
        xk = x2d.contiguous()
        bf16_mode = bool(self.bf16_certified) and xk.dtype == torch.bfloat16
        if self.fp16_table_missing and not bf16_mode:
            from qvb8_amd.formats.qvb8.escape_split import fp16_missing_error
            raise fp16_missing_error(getattr(self, "_where", "QVBandLinearV8"))
        ei, ev = (self.esc_idx_bf16, self.esc_vals_bf16) if bf16_mode else (self.esc_idx, self.esc_vals)

        order = self._mma_order() if M <= max(_MMA_SPLIT_MAX, ext.MMA_GEMM_MAX_M) else None
        if order is not None and M > _MMA_MAX_M and not self._gemm_ok(order[2], bf16_mode):
            if M > _MMA_SPLIT_MAX:
                order = None                                        # dense restore + library GEMM below
            else:
                n = -(-M // _MMA_MAX_M)
                step = -(-M // n)
                return torch.cat([self.forward(xk[i:i + step]) for i in range(0, M, step)]) \
                    .reshape(*orig[:-1], self.out_features).to(out_dtype)
        if order is not None:
            perm, rowinfo, layout = order
            xm = xk if xk.dtype in (torch.float16, torch.bfloat16) else ext.saturating_half(xk)
            y = ext.mma_tiles(xm, self.ids, self.min_s, self.nbits, self.bit_off, self.in_features, self.tau_s,
                              ei, ev, perm=perm, saturate=not bf16_mode, rowinfo=rowinfo, layout=layout)
            return self._finish(y, orig, out_dtype)
        if M <= 8:
            y = ext.gemv_multi(xk, self.ids, self.min_s, self.nbits, self.bit_off, self.in_features, self.tau_s,
                               self.esc_idx, self.esc_vals)
            return self._finish(y, orig, out_dtype)
        if xk.dtype == torch.bfloat16 and self.bf16_gemm and self.bf16_certified:
            W = ext.decode_bf16(self.ids, self.min_s, self.nbits, self.bit_off, self.in_features, self.tau_s,
                                self.esc_idx_bf16, self.esc_vals_bf16)
            b = None if self.bias is None else self.bias.to(torch.bfloat16)
            return F.linear(xk, W, b).reshape(*orig[:-1], self.out_features)
        if xk.dtype == torch.float16:
            W = ext.decode(self.ids, self.min_s, self.nbits, self.bit_off, self.in_features, self.tau_s,
                           self.esc_idx, self.esc_vals)
            b16 = None if self.bias is None else self.bias.to(torch.float16)
            return F.linear(xk, W, b16).reshape(*orig[:-1], self.out_features)
        y = ext.forward(xk, self.ids, self.min_s, self.nbits, self.bit_off, self.in_features, self.tau_s,
                        self.esc_idx, self.esc_vals)
        return self._finish(y, orig, out_dtype)


def enable_bf16_gemm(model: nn.Module) -> tuple[int, int]:
    """Put every bf16-certified QVBandLinearV8 in `model` on the bf16 GEMM for large M; returns
    (switched, packed_linears) (module.py:506-524)."""
    n = tot = 0
    for m in model.modules():
        if isinstance(m, QVBandLinearV8):
            tot += 1
            if m.bf16_certified:
                m.bf16_gemm = True
                n += 1
    return n, tot


def footprint_report(module) -> dict:
    """Resident bytes of the packed linears under `module`: ids, escapes (12 bytes each), row metadata, and the
    bytes-per-parameter figure a caller compares with dense fp16's 2.0 (module.py:527-587)."""
    ids = escapes = meta = 0
    n_esc = n_params = n_lin = 0
    for _, m in module.named_modules():
        if not isinstance(m, QVBandLinearV8):
            continue
        n_lin += 1
        n_params += m.out_features * m.in_features
        ids += m.ids.numel() * m.ids.element_size()
        tabs = [m.esc_idx, m.esc_vals]
        if m.esc_idx_bf16.data_ptr() != m.esc_idx.data_ptr():
            tabs += [m.esc_idx_bf16, m.esc_vals_bf16]
        for t in tabs:
            n_esc += t.numel()
            escapes += t.numel() * t.element_size()
        for t in (m.min_s, m.tau_s, m.nbits, m.bit_off):
            meta += t.numel() * t.element_size()
    total = ids + escapes + meta
    return {"linears": n_lin, "params": n_params, "escape_count": n_esc, "ids_bytes": ids, "escape_bytes": escapes,
            "meta_bytes": meta, "total_bytes": total,
            "bytes_per_param": (total / n_params) if n_params else 0.0,
            "escape_ratio": (n_esc / n_params) if n_params else 0.0}
