"""The MLP of a decoder layer as ONE launch at decode: down(silu(gate(x)) * up(x)) for 1..4 rows (ext.mlp_fused).

Run as separate products, gate+up and down each pay a launch's fixed cost -- on MI355X several microseconds in which no
weight byte moves, about as long as the down product's bytes take.  The reference takes the launch cost off the HOST by
replaying each MLP as a captured graph (src/qv_band/formats/qvb8/moe_graph.py:145-178, install_mlp_graphs); a graph node
still is a launch, so here the block is one kernel: the gate+up product, the activation and the down product run in one
resident grid and hand H over inside it.

`QVBandMLPV8` stands where a model's `mlp` module stood (gate_proj / up_proj / down_proj of QVBandLinearV8, SiLU): for
1..4 rows it can make the one launch (`one_launch`, off by default: see there), for anything else -- more rows, fp32
activations, a pack the kernel cannot read -- it computes the same chain with the separate products on the SAME stored
bytes (nothing is held twice).  Values: gate and
up results rounded to the activations' type, SiLU in fp32 rounded to it, the product rounded to it, the down product's
input narrowed like every fp16-path activation -- what the separate modules and torch's elementwise kernels produce.
"""
from __future__ import annotations

import os

import torch
import torch.nn as nn
import torch.nn.functional as F

from qvb8_amd import ext_qvb8 as ext
from .fuse import concat_linears
from .module import QVBandLinearV8, activation_rows

UNIT = 16                      # outputs per unit: 16 gate rows and the 16 matching up rows lie side by side


def unit_order(nbits: torch.Tensor, inter: int):
    """(perm, new_nbits) that store a gate+up pack (rows 0..inter-1 gate, the rest up) unit by unit, or None.

    Outputs are sorted by width (an output's width = the wider of its gate and its up row, at least 4), cut into units of
    16, and every row of a unit is stored in the unit's widest width, so that both tiles of a unit are whole tiles of one
    width and the units form at most three runs of one width each.  Position 32 u + r is the gate row of the unit's r-th
    output, 32 u + 16 + r its up row."""
    if inter % UNIT != 0 or nbits.numel() != 2 * inter:
        return None
    nb = nbits.to(torch.int64)
    per_output = torch.maximum(nb[:inter], nb[inter:]).clamp_(min=4)
    if int(per_output.max()) > 8:
        return None
    outputs = torch.argsort(per_output, stable=True)
    unit_width = per_output[outputs].view(-1, UNIT).amax(1)                 # ascending: the outputs were sorted
    if int(torch.unique(unit_width).numel()) > 3:
        return None
    width_of = torch.empty_like(per_output)
    width_of[outputs] = unit_width.repeat_interleave(UNIT)
    new_nbits = torch.cat([width_of, width_of]).to(torch.uint8)
    by_unit = outputs.view(-1, UNIT)
    perm = torch.stack([by_unit, by_unit + inter], 1).reshape(-1).to(torch.int32)
    return perm, new_nbits


def _whole_tiles(layout, rows: int) -> bool:
    return all(int(layout.first_pos[c]) % rows == 0 for c in range(int(layout.n_classes) + 1)) and \
        all(4 <= int(layout.nbits[c]) <= 8 for c in range(int(layout.n_classes)))


class QVBandMLPV8(nn.Module):
    """gate_proj / up_proj / down_proj (QVBandLinearV8, no bias, no escapes) with gated SiLU between them."""

    max_rows = ext.MLP_MAX_ROWS
    # Whether 1..4 rows take the one-launch kernel.  Off by default: measured on the 9B shapes (hidden 4096, inter 12288) the
    # one launch takes 29.6 us against 30.0 us for the two separate launches -- the hand-over inside the grid costs what the
    # launch it saves costs (see the kernel's source) --, so the separate products, which every other row count uses anyway,
    # stay the default.  QVB8_MLP_FUSED=1 in the environment (or True here) switches it on.
    one_launch = False

    def __init__(self, gate: QVBandLinearV8, up: QVBandLinearV8, down: QVBandLinearV8):
        super().__init__()
        if gate.in_features != up.in_features or gate.out_features != up.out_features or down.in_features != gate.out_features:
            raise ValueError("QVBandMLPV8: gate and up must be (inter, hidden), down (out, inter)")
        self.hidden, self.inter, self.out_features = gate.in_features, gate.out_features, down.out_features
        self.in_features = self.hidden
        self.gate_up = concat_linears([gate, up])[0]
        self.down = down
        self.fused_ready = False
        self._ws = self._plan = None
        self._prepare_fused()

    def _prepare_fused(self):
        """Stores gate+up unit by unit and down in width order, both in planes; fused_ready says whether the one-launch
        kernel can read them (no bias, no escapes, widths 4..8, at most three widths each, whole tiles)."""
        gu, dn = self.gate_up, self.down
        ok = (gu.ids.is_cuda and gu.bias is None and dn.bias is None and not gu.esc_idx.numel() and not dn.esc_idx.numel()
              and not gu.esc_idx_bf16.numel() and not dn.esc_idx_bf16.numel() and not gu.fp16_table_missing and not dn.fp16_table_missing
              and self.hidden % 128 == 0 and self.inter % 128 == 0 and self.out_features % 16 == 0
              and os.environ.get("QVB8_PLANES", "1") != "0")
        if ok:
            order = unit_order(gu.nbits, self.inter)
            ok = order is not None and gu.store_in_order(*order)
        if ok:
            d = dn._mma_order()
            ok = d is not None and d[2] is not None and dn._planes and _whole_tiles(d[2], 16)
        if ok:
            ok = _whole_tiles(gu._mma_cache[2], 32)
        self.fused_ready = bool(ok)
        self._ws = self._plan = None
        if ok:
            self._ws, self._plan = ext.mlp_init(gu.ids, gu._mma_cache[1], gu._mma_cache[2], dn.ids, d[1], d[2],
                                                self.hidden, self.inter, self.out_features)

    def _apply(self, fn, recurse=True):
        out = super()._apply(fn, recurse)
        if self._ws is not None and self._ws.device != self.gate_up.ids.device:      # the weights moved: describe them anew
            self._prepare_fused()
        return out

    def error_raised(self) -> bool:
        """Whether a one-launch call on this module ever gave up its wait for H (its result then was NaN); one host read."""
        return self._ws is not None and bool(self._ws[:8].view(torch.int32)[1].item())

    def separate(self, rows: torch.Tensor) -> torch.Tensor:
        """The same chain with the two products launched separately (any row count and type)."""
        gu = self.gate_up(rows)
        g, u = gu[..., :self.inter], gu[..., self.inter:]
        return self.down(F.silu(g) * u)

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        rows, out_dtype = activation_rows(x, self.gate_up.min_s.device)
        M = rows.shape[0]
        if (self.fused_ready and 1 <= M <= self.max_rows and rows.dtype in (torch.float16, torch.bfloat16)
                and os.environ.get("QVB8_MLP_FUSED", "1" if self.one_launch else "0") != "0"):
            y = ext.mlp_fused(rows, self._ws, self._plan, mid_dtype=rows.dtype, out_dtype=rows.dtype)
            return y.reshape(*x.shape[:-1], self.out_features).to(out_dtype)
        return self.separate(rows).reshape(*x.shape[:-1], self.out_features).to(out_dtype)

    def extra_repr(self):
        return f"hidden={self.hidden}, inter={self.inter}, out_features={self.out_features}, one_launch={self.fused_ready}"


def _is_silu(fn) -> bool:
    return isinstance(fn, nn.SiLU) or fn is F.silu or "silu" in type(fn).__name__.lower() or "silu" in getattr(fn, "__name__", "").lower()


def install_fused_mlps(model: nn.Module, names=("mlp",)) -> int:
    """Replaces every submodule called `mlp` (or any of `names`) that is gate_proj / up_proj / down_proj of QVBandLinearV8
    with a SiLU `act_fn` by a QVBandMLPV8; returns how many.  Run it BEFORE same-input fusion (which would turn gate_proj
    and up_proj into members of a fused group).  Counterpart of install_mlp_graphs (moe_graph.py:145-178)."""
    n = 0
    for parent in list(model.modules()):
        for name in names:
            child = getattr(parent, name, None)
            if not isinstance(child, nn.Module) or isinstance(child, QVBandMLPV8):
                continue
            parts = [getattr(child, a, None) for a in ("gate_proj", "up_proj", "down_proj")]
            if not all(isinstance(p, QVBandLinearV8) for p in parts) or not _is_silu(getattr(child, "act_fn", None)):
                continue
            if any(p.bias is not None for p in parts):
                continue
            for a in ("gate_proj", "up_proj", "down_proj"):       # the separate copies go before the fused one is built
                setattr(child, a, None)
            setattr(parent, name, QVBandMLPV8(*parts))
            del parts
            n += 1
    if n and torch.cuda.is_available():
        torch.cuda.empty_cache()
    return n
