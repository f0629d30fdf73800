"""A pack directory: `manifest.json` plus one pack file per tensor, and the step that swaps a model's modules for the
operators that read them.

The manifest is the reference's (run/run_inference.py:553-563 reads it): `format` names the registry entry
(common/formats.py), `tau` the certified bound, `tensors` maps a checkpoint tensor key to {"pack": file name, ...},
`failed` lists tensors that could not be packed (they stay dense), `hf_model` the source checkpoint.  One slice of a
routed-expert stack has the key "<base tensor>#expert<e>" (common/expert_key.py:18); the slices of one block are read
together into one expert-stack operator.

`swap_modules` is the part of the reference's loader (run/run_inference.py:545-800) that concerns the operators: it does
not build, download or place models -- it takes any nn.Module whose submodule paths match the manifest's keys.
"""
from __future__ import annotations

import json
import os

import torch.nn as nn

from qvb8_amd.common.formats import FormatSpec, get_format

EXPERT_KEY_SEP = "#expert"
MANIFEST = "manifest.json"


def parse_expert_key(key: str):
    """"<base>#expert<e>" -> (base, e); any other key -> (key, None)  (run_inference.py:48-53)."""
    base, sep, idx = key.partition(EXPERT_KEY_SEP)
    return (base, int(idx)) if sep else (key, None)


def tensor_key_to_module(key: str) -> str:
    """Checkpoint tensor key -> module path of the text model: drops a trailing ".weight" and maps the multimodal
    wrappers' prefixes onto the text model's (run/common.py:12-31)."""
    if key.endswith(".weight"):
        key = key[:-len(".weight")]
    for prefix, repl in (("language_model.backbone.", "model."), ("model.language_model.", "model."), ("language_model.", "")):
        if key.startswith(prefix):
            return repl + key[len(prefix):]
    return key


class PackDir:
    """The manifest of a pack directory and the paths it names."""

    def __init__(self, path: str):
        self.path = str(path)
        with open(os.path.join(self.path, MANIFEST)) as fh:
            self.manifest = json.load(fh)
        if not isinstance(self.manifest.get("tensors"), dict):
            raise ValueError(f"{self.path}/{MANIFEST}: no `tensors` table")
        self.tensors: dict = self.manifest["tensors"]
        self.tau = self.manifest.get("tau")
        self.failed: dict = self.manifest.get("failed") or {}
        self.hf_model = self.manifest.get("hf_model")
        self.spec: FormatSpec = get_format(self.manifest.get("format"))

    def packfile(self, key: str) -> str:
        return os.path.join(self.path, self.tensors[key]["pack"])

    def spec_of(self, key: str) -> FormatSpec:
        """A tensor's own file extension chooses its reader, not the directory-wide format (run_inference.py:699-708)."""
        ext = os.path.splitext(self.tensors[key]["pack"])[1].lstrip(".")
        return self.spec if ext == self.spec.name or not ext else get_format(ext)

    def expert_stacks(self) -> dict:
        """{block module path: {projection name: {expert index: pack path}}} of every "#expert" key."""
        out: dict = {}
        for key in self.tensors:
            base, e = parse_expert_key(key)
            if e is None:
                continue
            block, _, proj = tensor_key_to_module(base).rpartition(".")
            out.setdefault(block, {}).setdefault(proj, {})[e] = self.packfile(key)
        return out


def write_manifest(path: str, tensors: dict, *, tau: float, fmt: str = "qvband", hf_model: str | None = None,
                   failed: dict | None = None) -> str:
    """Writes `manifest.json` for pack files already in `path`; `tensors` maps tensor key -> pack file name (or a dict
    with at least "pack")."""
    table = {k: (dict(v) if isinstance(v, dict) else {"pack": v}) for k, v in tensors.items()}
    out = os.path.join(path, MANIFEST)
    with open(out, "w") as fh:
        json.dump({"format": fmt, "tau": tau, "hf_model": hf_model, "failed": failed or {}, "tensors": table}, fh, indent=1)
    return out


def _resolve(model: nn.Module, path: str):
    """(module path that exists, module): the path as given, else with the "model." prefix some checkpoints' keys omit
    (run_inference.py:672-695).  AttributeError when neither exists."""
    for cand in ((path,) if path.startswith("model.") else (path, "model." + path)):
        try:
            return cand, model.get_submodule(cand)
        except AttributeError:
            continue
    raise AttributeError(path)


def _set(model: nn.Module, path: str, new: nn.Module) -> None:
    parent, _, leaf = path.rpartition(".")
    setattr(model.get_submodule(parent) if parent else model, leaf, new)


def swap_modules(model: nn.Module, pack_dir, *, device: str = "cuda", out_dtype=None, finalize: bool = True) -> dict:
    """Replaces, in place, every module of `model` that the pack directory covers:

      * complete routed-expert stacks (module with `num_experts`, every expert of gate_up_proj and down_proj packed)
        -> `spec.experts.from_packfiles`
      * nn.Embedding -> the embedding reader of the tensor's format (`out_dtype`: the model's dtype, bf16 if not given)
      * nn.Linear    -> `spec.linear.from_packfile`, keeping the module's bias

    then runs the format's `finalize` (same-input fusion).  Anything else is left as it is and reported: a key whose
    module is absent (vision tower of a text-only skeleton), a partly packed stack, a format without the needed reader.
    Returns {"linear": [...], "embedding": [...], "experts": [...], "skipped": {path: reason}, "fused": n}."""
    import torch
    pd = pack_dir if isinstance(pack_dir, PackDir) else PackDir(pack_dir)
    out_dtype = torch.bfloat16 if out_dtype is None else out_dtype
    report = {"linear": [], "embedding": [], "experts": [], "skipped": {}, "fused": 0}

    for block, projs in pd.expert_stacks().items():
        try:
            block, owner = _resolve(model, block)
        except AttributeError:
            report["skipped"][block] = "module not present in this model"
            continue
        n = getattr(owner, "num_experts", None)
        gu, dn = projs.get("gate_up_proj", {}), projs.get("down_proj", {})
        if n is None:
            report["skipped"][block] = "no num_experts attribute"
        elif len(gu) != n or len(dn) != n:
            report["skipped"][block] = f"only {len(gu)}/{n} gate_up and {len(dn)}/{n} down slices packed"
        elif pd.spec.experts is None:
            report["skipped"][block] = f"format {pd.spec.name} has no expert reader"
        else:
            stack = pd.spec.experts.from_packfiles(gu, dn, num_experts=n, act_fn=getattr(owner, "act_fn", None),
                                                   device=device, tau=pd.tau)
            if hasattr(stack, "prepare"):
                stack.prepare()                  # the stacks' rows are re-stored now, not on the first routed call
            _set(model, block, stack)
            report["experts"].append(block)

    for key in pd.tensors:
        if parse_expert_key(key)[1] is not None:
            continue
        try:
            path, owner = _resolve(model, tensor_key_to_module(key))
        except AttributeError:
            report["skipped"][tensor_key_to_module(key)] = "module not present in this model"
            continue
        spec = pd.spec_of(key)
        if isinstance(owner, nn.Embedding):
            if spec.embedding is None:
                report["skipped"][path] = f"format {spec.name} has no embedding reader"
                continue
            _set(model, path, spec.embedding.from_packfile(pd.packfile(key), out_dtype=out_dtype, device=device, tau=pd.tau))
            report["embedding"].append(path)
        elif isinstance(owner, nn.Linear):
            _set(model, path, spec.linear.from_packfile(pd.packfile(key), bias=owner.bias, device=device, tau=pd.tau))
            report["linear"].append(path)
        else:
            report["skipped"][path] = f"{type(owner).__name__} is neither nn.Linear nor nn.Embedding"
    if finalize and pd.spec.finalize is not None:
        report["fused"] = int(pd.spec.finalize(model) or 0)
    return report
