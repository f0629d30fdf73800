"""Same-input fusion for QVB8R: sibling linears fed the same activation (q/k/v, gate/up, qkv/z) run as ONE walk.

QVB8R tensors with the same row length join into one virtual tensor: every tile stays a stream of its own, so joining
is bookkeeping -- sorted rows, classes and word offsets of a later member are shifted behind those of the members before
it -- and every kernel runs unchanged on the result.  Each row's sum is computed exactly as in the member's own launch,
so outputs are bit-identical; they are split back per member as views.
Counterpart of the reference's src/qv_band/formats/qvb8r/fuse.py:25-119 (`concat`, `fuse_same_input`); the loader calls
fuse_same_input once after swapping (the format's `finalize` hook in the registry).
"""
from __future__ import annotations

import numpy as np
import torch
import torch.nn as nn

from qvb8_amd.common.fusion import SAME_INPUT_GROUPS, FusedGroup, FusedMember, fuse_groups  # noqa: F401
from .module import QVBandLinearV8R

# how a member's arrays enter the joined tensor: which running total is added to which column (None = the whole array)
_SHIFTED = {"perm": (None, "rows"), "esc_idx": (None, "flat")}
_PLAIN = ("states", "words", "drow", "min_s", "tau_s", "esc_val", "esc_delta")


def concat(ds: list[dict]) -> tuple[dict, list[int]]:
    """Joins QVB8R tensors (dicts as container.read returns them) with one row length into one; the rows of ds[0] come
    first.  Returns the joined dict and the row numbers at which the members' outputs are split."""
    if not ds:
        raise ValueError("qvb8r concat: no members")
    P = int(ds[0]["P"])
    if any(int(d["P"]) != P for d in ds):
        raise ValueError("qvb8r concat: members must share P")
    n_sym = max(int(d["N"]) for d in ds)
    rows = np.cumsum([0] + [int(d["Q"]) for d in ds])                 # first row of each member (sorted and original alike)
    classes = np.cumsum([0] + [int(d["K"]) for d in ds])
    words_at = np.cumsum([0] + [len(d["words"]) for d in ds])
    parts: dict = {k: [] for k in ("perm", "freq", "tiles", "tile_off", "esc_idx") + _PLAIN}
    for d, r0, k0, w0 in zip(ds, rows, classes, words_at):
        parts["perm"].append(np.asarray(d["perm"]).astype(np.int64) + r0)
        table = np.zeros((int(d["K"]), n_sym), np.uint16)            # frequency tables widened to the largest alphabet
        table[:, :np.asarray(d["freq"]).shape[1]] = d["freq"]
        parts["freq"].append(table)
        parts["tiles"].append(np.asarray(d["tiles"]).astype(np.int64) + np.array([k0, r0, 0]))
        parts["tile_off"].append(np.asarray(d["tile_off"]).astype(np.int64)[:-1] + w0)
        parts["esc_idx"].append(np.asarray(d["esc_idx"]).astype(np.int64) + r0 * P)
        for name in _PLAIN:
            parts[name].append(np.asarray(d[name]))
    parts["tile_off"].append(np.array([words_at[-1]], np.int64))      # one past the last tile's words
    joined = {k: np.concatenate(v) for k, v in parts.items()}
    joined["perm"] = joined["perm"].astype(np.int32)
    joined["tiles"] = joined["tiles"].astype(np.int32)
    joined.update(P=P, N=n_sym, Q=int(rows[-1]), K=int(classes[-1]), T=max(int(d["T"]) for d in ds))
    return joined, [int(r) for r in rows[1:-1]]


def concat_linears(mods: list[QVBandLinearV8R]) -> tuple[QVBandLinearV8R, list[int]]:
    """One QVBandLinearV8R over the members' rows (read again from their files, or from the arrays they were built from),
    on the members' device."""
    dev = mods[0].words.device
    joined, splits = concat([m.host_arrays() for m in mods])
    bias = None
    if any(m.bias is not None for m in mods):              # added by the fused linear in fp32, before the one rounding to
        bias = torch.cat([m.bias.detach().float() if m.bias is not None     # the caller's dtype: as each member does alone
                          else torch.zeros(m.out_features, device=dev) for m in mods])
    return QVBandLinearV8R(joined, bias=bias, device=dev), splits


def _all_coded(owner, names) -> bool:
    mods = [getattr(owner, a, None) for a in names]
    return (all(isinstance(m, QVBandLinearV8R) and m.has_host_arrays() for m in mods)
            and len({m.in_features for m in mods}) == 1)


def fuse_same_input(model: nn.Module) -> int:
    """Replace every same-input group of QVBandLinearV8R siblings by members of one fused walk; returns the number of
    groups fused.  The fused linear adds the members' biases itself (the reference adds a member's bias to its slice
    after the result was rounded to the caller's dtype; adding it before keeps the fused output equal to the member's
    own, bit for bit)."""
    return fuse_groups(model, _all_coded, concat_linears, "_qvb8r_fused")
