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

import os

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


def _ascending(positions, values):
    """An escape list in ascending flat positions (the correction kernels add a row's escapes in list order, so a sorted
    list makes results reproducible); returned as it is when it already is."""
    if positions.numel() < 2 or bool((positions[1:] >= positions[:-1]).all()):
        return positions, values
    order = torch.argsort(positions, stable=True)
    return positions[order].contiguous(), values[order].contiguous()


def activation_rows(x: torch.Tensor, device):
    """x as contiguous (M, P) rows on `device`, and the type results go back in.  Under autocast an fp32 input is computed
    and returned in the autocast type, as nn.Linear does (module.py:336-344)."""
    rows = x.reshape(-1, x.shape[-1]).to(device)
    result_dtype = x.dtype
    if rows.dtype == torch.float32 and torch.is_autocast_enabled(rows.device.type):
        low = torch.get_autocast_dtype(rows.device.type)
        if low in (torch.float16, torch.bfloat16):
            rows, result_dtype = rows.to(low), low
    return rows.contiguous(), result_dtype


def _on(dev, array, dtype):
    return torch.from_numpy(np.ascontiguousarray(array, dtype)).to(dev)


class QVBandLinearV8(nn.Module):
    # The first call of the matrix-core path copies the rows once into width-sorted order (same total size; `ids` and
    # `bit_off` are replaced, every kernel keeps working through bit_off), so that calls compute row addresses instead of
    # reading them.  Set False to keep the file's row order in memory.
    sort_rows = True
    # With the sort, every whole 16-row tile of one width 4..8 is stored in planes: the same bytes, permuted inside the tile
    # so that each request of a wave of the matrix-core kernels is one contiguous run (measured on the 9B decode step:
    # 7 % faster than rows back to back).  QVB8_PLANES=0 in the environment or False here keeps the rows back to back.
    plane_tiles = True
    bf16_gemm = False             # opt-in: M > 96 bf16 callers decode to bf16 and run one bf16 GEMM (module.py:60-65)
    bf16_certified = False        # the pack certifies |orig - bf16(band)| <= tau (container restore code 3)
    fp16_table_missing = False    # fp16+bf16 pack loaded without escape_tables.json: fp16 forwards refuse
    _planes = False               # some rows are stored in planes (set with the launch data)

    def __init__(self, *, min_s, nbits, bit_off, ids, Q, P, tau_s, esc_idx, esc_vals, bias=None,
                 esc_idx_bf16=None, esc_vals_bf16=None):
        super().__init__()
        self.out_features, self.in_features = int(Q), int(P)
        fp16_table = _ascending(esc_idx, esc_vals)
        # one table serves both modes unless the pack certifies bf16 separately (then the bf16 list is the full one)
        bf16_table = fp16_table if esc_idx_bf16 is None else _ascending(esc_idx_bf16, esc_vals_bf16)
        held = dict(tau_s=tau_s, min_s=min_s, nbits=nbits, bit_off=bit_off, ids=ids,
                    esc_idx=fp16_table[0], esc_vals=fp16_table[1], esc_idx_bf16=bf16_table[0], esc_vals_bf16=bf16_table[1])
        for name, tensor in held.items():               # none of them is saved with a state dict: the pack file is the source
            self.register_buffer(name, tensor, persistent=False)
        self.bias = nn.Parameter(bias, requires_grad=False) if bias is not None else None

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
        dev = torch.device(device)
        raw = blob if blob is not None else open(path, "rb").read()
        tables = dict(fp16=None, bf16=None)             # (positions, values) per mode; bf16 stays None when one table serves both
        flags = dict(bf16_certified=False, fp16_table_missing=False)
        if raw[:4] == b"QVBD":
            from qvb8_amd.formats.qvb8.escape_split import fp16_list_for
            from qvb8_amd.formats.qvb8.pack_container import CALC_TABLE, calc_method_of, unpack_formula
            if calc_method_of(raw) == CALC_TABLE:
                raise NotImplementedError("QVBandLinearV8 reads formula packs only: this file keeps a value table per row "
                                          "(calc_method = 1, written before the formats were unified) and has to be packed again")
            rec = unpack_formula(raw, skip_bit_decode=True, fp16_list=fp16_list_for(path), where=str(path))
            flags["bf16_certified"] = rec.get("restore") == "fp16+bf16"
            full = (rec["esc_idx"], rec["esc_vals"])
            if rec["esc_idx_fp16"] is None:             # a two-table pack whose fp16 list is not at hand: bf16 callers only
                tables["fp16"], flags["fp16_table_missing"] = full, True
            else:
                tables["fp16"] = (rec["esc_idx_fp16"], rec["esc_vals_fp16"])
                if rec["esc_idx_fp16"] is not rec["esc_idx"]:
                    tables["bf16"] = full
        else:
            from qvb8_amd.formats.qvb8.decode import unpack_tensor
            names = ("min_s", "tau_s", "nbits", "bit_off", "buf", "Q", "P", "tau", "esc_idx", "esc_vals")
            rec = dict(zip(names, unpack_tensor(raw)))
            tables["fp16"] = (rec["esc_idx"], rec["esc_vals"])
        if isinstance(bias, torch.Tensor):
            bias = bias.detach().to(dev)
        elif bias is not None:
            bias = torch.tensor(bias).to(dev)
        second = tables["bf16"]
        mod = cls(min_s=_on(dev, rec["min_s"], np.float32), tau_s=_on(dev, rec["tau_s"], np.float32),
                  nbits=_on(dev, rec["nbits"], np.uint8), bit_off=_on(dev, rec["bit_off"], np.int64),
                  ids=_on(dev, rec["buf"], None), Q=rec["Q"], P=rec["P"], bias=bias,
                  esc_idx=_on(dev, tables["fp16"][0], np.int64), esc_vals=_on(dev, tables["fp16"][1], np.float32),
                  esc_idx_bf16=None if second is None else _on(dev, second[0], np.int64),
                  esc_vals_bf16=None if second is None else _on(dev, second[1], np.float32))
        mod.bf16_certified, mod.fp16_table_missing = flags["bf16_certified"], flags["fp16_table_missing"]
        mod._where = str(path)
        return mod

    def escapes(self, dtype=torch.float16):
        """The escape table that goes with a weight rounded to `dtype`: the full list for bf16, the fp16 table otherwise
        (reference: module.py:116-124).  An fp16+bf16 pack whose fp16 table could not be determined refuses fp16."""
        wants_bf16 = dtype == torch.bfloat16
        if not wants_bf16:
            self._need_fp16_table(dtype == torch.float16)
        return (self.esc_idx_bf16, self.esc_vals_bf16) if wants_bf16 else (self.esc_idx, self.esc_vals)

    def _need_fp16_table(self, asked: bool = True):
        """Raises when an fp16 result is asked of a two-table pack whose fp16 escape list could not be determined."""
        if asked and self.fp16_table_missing:
            from qvb8_amd.formats.qvb8.escape_split import fp16_missing_error
            raise fp16_missing_error(getattr(self, "_where", type(self).__name__))

    def row_subset(self, rows: torch.Tensor) -> "QVBandLinearV8":
        """The linear restricted to output rows `rows` (in that order).  A pack's rows are independent -- each has its own
        min_s, tau_s, width and bit offset -- so the subset only selects row metadata and keeps pointing into THIS
        module's `ids`: no weight bytes are copied (what the reference does for a restricted vocabulary head,
        module.py:126-160).  Escapes of other rows are dropped, the kept ones renumbered to the new row order."""
        rows = rows.to(device=self.min_s.device, dtype=torch.long)
        P, n = self.in_features, int(rows.numel())
        new_row_of = torch.full((self.out_features,), -1, dtype=torch.long, device=rows.device)
        new_row_of[rows] = torch.arange(n, device=rows.device)

        def restrict(table):
            idx, vals = table
            if idx.numel() == 0:
                return idx, vals
            target = new_row_of[torch.div(idx, P, rounding_mode="floor")]
            kept = target >= 0
            return target[kept] * P + torch.remainder(idx[kept], P), vals[kept]

        fp16_tab = restrict((self.esc_idx, self.esc_vals))
        one_table = self.esc_idx_bf16 is self.esc_idx
        bf16_tab = (None, None) if one_table else restrict((self.esc_idx_bf16, self.esc_vals_bf16))
        picked = {name: getattr(self, name)[rows] for name in ("min_s", "tau_s", "nbits", "bit_off")}
        sub = type(self)(ids=self.ids, Q=n, P=P, esc_idx=fp16_tab[0], esc_vals=fp16_tab[1], bias=None,
                         esc_idx_bf16=bf16_tab[0], esc_vals_bf16=bf16_tab[1], **picked)
        sub.bf16_certified, sub.fp16_table_missing = self.bf16_certified, self.fp16_table_missing
        return sub

    def _apply(self, fn, recurse=True):
        out = apply_keeping_fp32_metadata(self, fn, recurse)
        self.__dict__.pop("_mma_cache", None)           # the row records follow the buffers: rebuild after a move
        return out

    # ---- launch metadata ---------------------------------------------------------------------------------------

    def _mma_order(self):
        """(perm, rowinfo, layout) for ext.mma_tiles, or None when the tile kernel cannot read this weight.  Rows are sorted by
        width so that a 16-row tile shares one width (one decode pass); the row records hold, in that order, where each
        row's ids start, its width, tau_s, min_s and its output row.  Built once per weight, like the reference's
        perm / tile_nb (module.py:230-277).  Inside a graph capture only an earlier result can be used: a first call there
        raises."""
        cached = self.__dict__.get("_mma_cache", False)
        if cached is not False:
            return cached
        if torch.cuda.is_current_stream_capturing():
            # building them reads the device (width range) and may re-order `ids`: not inside a capture, and falling
            # back to another kernel here would make a captured graph compute something else than eager calls do
            raise RuntimeError("QVBandLinearV8: first call inside a graph capture -- call the module once (or prepare()) "
                               "before capturing")
        order = None
        if self.ids.is_cuda and self.in_features % 128 == 0 and self.ids.data_ptr() % 4 == 0 and self.out_features > 0:
            nb = self.nbits.to(torch.int16)
            if 1 <= int(nb.min()) and int(nb.max()) <= 14:
                layout = self.__dict__.get("_sorted_layout")                  # sorted before (the buffers have moved since)
                stored = self.__dict__.get("_stored_perm") if layout is not None else None
                # the order the rows were stored in, when a caller chose it (store_in_order); else by width
                perm = stored.to(self.ids.device) if stored is not None else torch.argsort(nb, stable=True).to(torch.int32).contiguous()
                row_bytes = int((self.nbits.to(torch.int64) * self.in_features).sum().item()) // 8
                if layout is None and self.sort_rows and 2 * row_bytes >= self.ids.numel():   # not for a small view into a shared stack
                    planes = self.plane_tiles and os.environ.get("QVB8_PLANES", "1") != "0"
                    ids, nbits, bit_off, order = self.ids, self.nbits, self.bit_off, perm
                    # whole tiles only: a tile across two widths is read row by row, and a launch waits for its slowest
                    # workgroup -- so up to 15 rows per width are stored one width up (their values do not change)
                    wide = ext.widen_rows_to_whole_tiles(ids, nbits, bit_off, self.in_features) if planes else None
                    if wide is not None:
                        ids, nbits, bit_off = wide
                        order = torch.argsort(nbits.to(torch.int16), stable=True).to(torch.int32).contiguous()
                    srt = ext.sort_rows_by_width(ids, nbits, bit_off, self.in_features, order, planes=planes)
                    if srt is not None:
                        self.ids, self.bit_off, layout = srt
                        self.nbits, perm = nbits, order
                        self._sorted_layout = layout
                self._planes = ext.rows_in_planes(self.bit_off)               # also a subset of, or a copy of, such a weight
                rowinfo = ext.mma_prepare(self.nbits, self.bit_off, self.tau_s, self.min_s, self.in_features,
                                          self.ids.numel(), perm)
                order = (perm, rowinfo, layout)
        self._mma_cache = order
        return order

    def store_in_order(self, perm: torch.Tensor, new_nbits: torch.Tensor | None = None) -> bool:
        """Stores the rows once more, in the position order `perm` (int32, position -> row) instead of sorted by width,
        row q in fields of new_nbits[q] >= nbits[q] bits (its ids, and so every value, unchanged), whole tiles in planes;
        along `perm` the widths must not decrease and take at most three values.  For callers whose kernel wants rows that
        belong together side by side (the MLP's gate and up rows of the same outputs).  Every other path of this module
        keeps working on the new bytes.  False, and nothing changed, when the pack cannot be stored that way."""
        if torch.cuda.is_current_stream_capturing():
            raise RuntimeError("QVBandLinearV8.store_in_order: not inside a graph capture")
        P = self.in_features
        if not self.ids.is_cuda or P % 128 != 0 or self.esc_idx.numel() or self.esc_idx_bf16.numel():
            return False
        ids, bit_off, nbits = self.ids, self.bit_off, self.nbits
        if new_nbits is not None and not bool((new_nbits == nbits).all()):
            packed = ext.repack_rows(ids, nbits, bit_off, P, new_nbits)
            if packed is None:
                return False
            ids, bit_off = packed
            nbits = new_nbits.to(torch.uint8)
        perm = perm.to(device=ids.device, dtype=torch.int32).contiguous()
        srt = ext.sort_rows_by_width(ids, nbits, bit_off, P, perm, planes=True)
        if srt is None:
            return False
        self.ids, self.bit_off, layout = srt
        self.nbits = nbits
        self._sorted_layout, self._stored_perm = layout, perm
        self._planes = ext.rows_in_planes(self.bit_off)
        rowinfo = ext.mma_prepare(self.nbits, self.bit_off, self.tau_s, self.min_s, P, self.ids.numel(), perm)
        self._mma_cache = (perm, rowinfo, layout)
        return True

    def prepare(self) -> "QVBandLinearV8":
        """Builds the per-weight launch data now (load time) instead of on the first forward; returns self."""
        self._mma_order()
        return self

    def _gemm_ok(self, layout, bf16_mode: bool) -> bool:
        """Whether the workgroup-tiled kernel (49..256 rows) can read this weight: rows stored in width order, every
        width one the sliced decode handles, whole 256-column groups."""
        if layout is None or self.in_features % 256 != 0:
            return False
        top = 7 if bf16_mode else 8
        return all(4 <= int(layout.nbits[c]) <= top for c in range(int(layout.n_classes)))

    # ---- forward -----------------------------------------------------------------------------------------------

    def _finish(self, y, orig, out_dtype):
        """(M, Q) results of a kernel -> the caller's leading dimensions, bias added, in the caller's type."""
        lead = tuple(orig[:-1])
        if self.bias is not None:
            y = y + self.bias.to(y.dtype)
        return y.reshape(*lead, self.out_features).to(out_dtype)

    def _rows_of(self, x: torch.Tensor):
        return activation_rows(x, self.min_s.device)

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        orig = x.shape
        xk, out_dtype = self._rows_of(x)
        M = xk.shape[0]
        # the mode decides the escape table: bf16 rows of a pack that certifies bf16 separately take the full list, every other
        # call the fp16 table -- which a two-table pack may lack
        bf16_mode = bool(self.bf16_certified) and xk.dtype == torch.bfloat16
        self._need_fp16_table(xk.dtype == torch.float16)
        if M == 0:
            return xk.new_zeros((*orig[:-1], self.out_features), dtype=out_dtype)
        self._need_fp16_table(not bf16_mode)
        ei, ev = self.escapes(torch.bfloat16 if bf16_mode else torch.float32)

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
            # without escapes and bias the kernels round the results to the caller's type themselves: no cast pass over Y
            direct = out_dtype if (ei.numel() == 0 and self.bias is None and out_dtype in (torch.float16, torch.bfloat16)) else None
            y = ext.mma_tiles(xm, self.ids, self.min_s, self.nbits, self.bit_off, self.in_features, self.tau_s,
                              ei, ev, perm=perm, saturate=not bf16_mode, rowinfo=rowinfo, layout=layout, out_dtype=direct,
                              planes=self._planes)
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
    packed = [m for m in model.modules() if isinstance(m, QVBandLinearV8)]
    certified = [m for m in packed if m.bf16_certified]
    for m in certified:
        m.bf16_gemm = True
    return len(certified), len(packed)


def footprint_report(module) -> dict:
    """What the packed linears under `module` keep resident, by kind: packed ids, escape tables (each table counted once;
    an fp16+bf16 pack holds two), per-row metadata; and the bytes per weight that a caller compares with the 2.0 of a
    dense 16-bit copy (the reference reports the same figures, module.py:527-587)."""
    def nbytes(*tensors):
        return sum(t.numel() * t.element_size() for t in tensors)

    report = dict(linears=0, params=0, escape_count=0, ids_bytes=0, escape_bytes=0, meta_bytes=0)
    for m in module.modules():
        if not isinstance(m, QVBandLinearV8):
            continue
        tables = [(m.esc_idx, m.esc_vals)]
        if m.esc_idx_bf16.data_ptr() != m.esc_idx.data_ptr():
            tables.append((m.esc_idx_bf16, m.esc_vals_bf16))
        report["linears"] += 1
        report["params"] += m.out_features * m.in_features
        report["ids_bytes"] += nbytes(m.ids)
        report["meta_bytes"] += nbytes(m.min_s, m.tau_s, m.nbits, m.bit_off)
        for idx, vals in tables:
            report["escape_count"] += idx.numel() + vals.numel()
            report["escape_bytes"] += nbytes(idx, vals)
    report["total_bytes"] = report["ids_bytes"] + report["escape_bytes"] + report["meta_bytes"]
    n = report["params"]
    report["bytes_per_param"] = report["total_bytes"] / n if n else 0.0
    report["escape_ratio"] = report["escape_count"] / n if n else 0.0
    return report
