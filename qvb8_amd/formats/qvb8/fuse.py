"""Same-input fusion: sibling packed linears that read the same activation (q/k/v, gate/up) run as ONE launch.

Rows of a QVB8 pack are independent (own min_s, tau_s, width, bit offset), so packs with the same P concatenate into one
virtual tensor: ids buffers back to back (each part 16-byte aligned), bit offsets and escape positions shifted.  Every
kernel runs unchanged on it and each row's result is computed exactly as before, so outputs are bit-identical to the
separate launches; the output is split back per member as views.  On MI355X a launch costs several microseconds before
the first packed byte arrives, which at M = 1 is as long as streaming a whole 4096 x 4096 weight: fewer, larger
launches are the point.  Counterpart of the reference's fusion for its entropy-coded format
(src/qv_band/formats/qvb8r/fuse.py:25-119); here it applies to QVBandLinearV8.
"""
from __future__ import annotations

import torch
import torch.nn as nn

from qvb8_amd.common.fusion import SAME_INPUT_GROUPS, FusedGroup as _FusedGroup, FusedMember, fuse_groups  # noqa: F401
from .module import QVBandLinearV8

_ALIGN = 16


def concat_linears(mods: list[QVBandLinearV8]) -> tuple[QVBandLinearV8, list[int]]:
    """One QVBandLinearV8 holding the rows of `mods` in order (same P, same device), and the row split points."""
    if not mods:
        raise ValueError("qvb8 concat: no members")
    P = mods[0].in_features
    dev = mods[0].ids.device
    if any(m.in_features != P for m in mods):
        raise ValueError("qvb8 concat: members must share P")
    if any(m.ids.device != dev for m in mods):
        raise ValueError("qvb8 concat: members must be on one device")
    if any(m.fp16_table_missing for m in mods):
        raise ValueError("qvb8 concat: a member has no fp16 escape table")
    parts, offs, total = [], [], 0
    for m in mods:
        offs.append(total)
        n = m.ids.numel()
        total += (n + _ALIGN - 1) // _ALIGN * _ALIGN
    ids = torch.zeros(total + 8, dtype=torch.uint8, device=dev)
    bit_off, esc = [], {False: ([], []), True: ([], [])}
    rq = 0
    two_tables = any(m.esc_idx_bf16 is not m.esc_idx for m in mods)
    for m, o in zip(mods, offs):
        ids[o:o + m.ids.numel()] = m.ids
        bit_off.append(m.bit_off + 8 * o)
        for bf in (False, True):
            ei, ev = (m.esc_idx_bf16, m.esc_vals_bf16) if bf else (m.esc_idx, m.esc_vals)
            esc[bf][0].append(ei + rq * P)
            esc[bf][1].append(ev)
        rq += m.out_features
    bias = None
    if any(m.bias is not None for m in mods):
        bias = torch.cat([m.bias.detach().float() if m.bias is not None
                          else torch.zeros(m.out_features, device=dev) for m in mods])
    fused = QVBandLinearV8(
        min_s=torch.cat([m.min_s for m in mods]), nbits=torch.cat([m.nbits for m in mods]),
        bit_off=torch.cat(bit_off), ids=ids, Q=rq, P=P, tau_s=torch.cat([m.tau_s for m in mods]),
        esc_idx=torch.cat(esc[False][0]), esc_vals=torch.cat(esc[False][1]), bias=bias,
        esc_idx_bf16=torch.cat(esc[True][0]) if two_tables else None,
        esc_vals_bf16=torch.cat(esc[True][1]) if two_tables else None)
    fused.bf16_certified = all(m.bf16_certified for m in mods)
    fused.bf16_gemm = all(m.bf16_gemm for m in mods)
    splits, acc = [], 0
    for m in mods[:-1]:
        acc += m.out_features
        splits.append(acc)
    return fused, splits


class FusedGroup(_FusedGroup):
    """The fused launch of a group of QVBandLinearV8 (members in the order given)."""

    def __init__(self, mods: list[QVBandLinearV8]):
        lin, splits = concat_linears(mods)
        super().__init__(lin, splits)


def _all_packed(owner, names) -> bool:
    mods = [getattr(owner, a, None) for a in names]
    return (all(isinstance(m, QVBandLinearV8) for m in mods) and len({m.in_features for m in mods}) == 1
            and not any(m.fp16_table_missing for m in mods))


def fuse_same_input(model: nn.Module) -> int:
    """Replace every same-input group of QVBandLinearV8 siblings by members of one fused launch; returns the number of
    groups fused.  The fused linear adds the members' biases itself."""
    return fuse_groups(model, _all_packed, concat_linears, "_qvb8_fused")
