"""escape_tables.json: which escapes of an fp16+bf16 pack belong to the fp16 table.

An fp16+bf16 pack stores ONE escape list (every escape: the bf16 table).  Decodes
that round the weight to fp16, or keep it in fp32, use a subset of it, named per pack
file in `escape_tables.json` (version 2) in the pack folder: either the subset itself
("fp16") or its complement ("bf16_only"), plus the two counts for validation.
Reader behaviour follows the reference (formats/qvb8/escape_split.py:12-56).
"""
from __future__ import annotations

import json
import os

import numpy as np

from ...common.errors import EscapeTableError

TABLES_FILE = "escape_tables.json"
_CACHE: dict = {}


def _hint(where: str) -> str:
    return f"put the {TABLES_FILE} that was written with this pack into {where}"


def fp16_list_for(path: str | None):
    """(kind, positions, n_bf16, n_fp16) for pack file `path`, or None when the folder
    has no table file or no fp16+bf16 entry for it."""
    if not path:
        return None
    folder = os.path.abspath(os.path.dirname(path))
    if folder not in _CACHE:
        f = os.path.join(folder, TABLES_FILE)
        if not os.path.exists(f):
            _CACHE[folder] = {}
        else:
            try:
                with open(f) as fh:
                    data = json.load(fh)
                if data.get("version") != 2:
                    raise EscapeTableError(f"{f}: version {data.get('version')}, this reader knows 2; {_hint(folder)}")
                _CACHE[folder] = data["tensors"]
            except (OSError, ValueError, KeyError) as ex:
                raise EscapeTableError(f"{f}: unreadable ({ex}); {_hint(folder)}") from None
    e = _CACHE[folder].get(os.path.basename(path))
    if e is None or e.get("restore") != "fp16+bf16":
        return None
    kind = "fp16" if "fp16" in e else "bf16_only"
    return (kind, np.asarray(e[kind], np.int64), int(e["n_bf16"]), int(e["n_fp16"]))


def select_fp16(full_idx, fp16_list, where: str = "") -> np.ndarray:
    """Keep-mask over the pack's full escape list.  Validates only: the file must match
    the pack (same count, every listed position an escape of the pack)."""
    kind, lst, n_bf16, n_fp16 = fp16_list
    full_idx = np.asarray(full_idx, np.int64)
    if n_bf16 != len(full_idx):
        raise EscapeTableError(f"{where}: {TABLES_FILE} says {n_bf16} escapes, the pack has "
                               f"{len(full_idx)}: the file belongs to another pack")
    hit = np.isin(full_idx, lst)
    if int(hit.sum()) != len(lst):
        raise EscapeTableError(f"{where}: {TABLES_FILE} lists {len(lst) - int(hit.sum())} positions "
                               f"that are not escapes of this pack")
    keep = hit if kind == "fp16" else ~hit
    if int(keep.sum()) != n_fp16:
        raise EscapeTableError(f"{where}: {TABLES_FILE} fp16 table has {int(keep.sum())} entries, "
                               f"n_fp16 says {n_fp16}")
    return keep


def fp16_missing_error(where: str) -> EscapeTableError:
    return EscapeTableError(f"{where}: fp16 run on an fp16+bf16 pack without {TABLES_FILE} "
                            f"(the fp16 escape table)")


def update_tables(folder: str, name: str, all_idx, fp16_idx) -> str:
    """Add or replace the entry of pack file `name` in the folder's escape_tables.json.
    all_idx: every escape position of the pack; fp16_idx: those of the fp16 table.  The
    shorter of the subset and its complement is stored."""
    f = os.path.join(folder, TABLES_FILE)
    tensors = {}
    if os.path.exists(f):
        with open(f) as fh:
            tensors = json.load(fh).get("tensors", {})
    all_idx = np.asarray(all_idx, np.int64)
    fp16_idx = np.asarray(fp16_idx, np.int64)
    only = np.setdiff1d(all_idx, fp16_idx)
    ent = dict(restore="fp16+bf16", n_bf16=int(len(all_idx)), n_fp16=int(len(fp16_idx)))
    if len(fp16_idx) <= len(only):
        ent["fp16"] = fp16_idx.tolist()
    else:
        ent["bf16_only"] = only.tolist()
    tensors[name] = ent
    with open(f, "w") as fh:
        json.dump(dict(version=2, tensors=tensors), fh)
    _CACHE.pop(os.path.abspath(folder), None)
    return f
