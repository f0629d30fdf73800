"""Pack-format registry: a pack directory's manifest names its format; loaders look the classes up here
(reference: src/qv_band/common/formats.py:16-48, 51-104).

    spec = get_format(manifest["format"])
    lin  = spec.linear.from_packfile(path, device=dev)

Entries: "qvb8" / "qvband" (the container's file extension) and "qvb8r", each with its linear and embedding class and
its `finalize` hook (same-input fusion).  There is no CPU reader in this build (`cpu_linear` is None): a caller that
needs one gets a clear error from `require`, never another format's class.
"""
from __future__ import annotations

import dataclasses
import re


@dataclasses.dataclass(frozen=True)
class FormatSpec:
    name: str
    linear: type
    embedding: type | None
    experts: type | None
    cpu_linear: type | None = None
    cpu_embedding: type | None = None
    decoder: object | None = None            # Callable(linear) -> dense (Q, P) tensor
    finalize: object | None = None           # Callable(model), run once after every module is swapped

    def filename(self, tensor_name: str) -> str:
        """Pack filename for a tensor, in this format's extension."""
        return re.sub(r"[^A-Za-z0-9]", "_", tensor_name) + "." + self.name


_REGISTRY: dict = {}


def _build_registry() -> None:
    if _REGISTRY:
        return
    import torch
    from qvb8_amd import ext_qvb8 as ext
    from qvb8_amd.formats.qvb8.backends_experts import QVBandExpertsV8
    from qvb8_amd.formats.qvb8.embedding import QVBandEmbeddingV8
    from qvb8_amd.formats.qvb8.fuse import fuse_same_input
    from qvb8_amd.formats.qvb8.module import QVBandLinearV8
    from qvb8_amd.formats.qvb8r.fuse import fuse_same_input as fuse_same_input_r
    from qvb8_amd.formats.qvb8r.module import QVBandEmbeddingV8R, QVBandLinearV8R

    def _decode_v8(lin):
        return ext.decode(lin.ids, lin.min_s, lin.nbits, lin.bit_off, lin.in_features, lin.tau_s, lin.esc_idx, lin.esc_vals)

    _REGISTRY["qvb8"] = FormatSpec("qvb8", QVBandLinearV8, QVBandEmbeddingV8, QVBandExpertsV8, decoder=_decode_v8, finalize=fuse_same_input)
    _REGISTRY["qvband"] = dataclasses.replace(_REGISTRY["qvb8"], name="qvband")
    # no expert reader for qvb8r: expert stacks of such a pack directory stay dense (as in the reference's registry)
    _REGISTRY["qvb8r"] = FormatSpec("qvb8r", QVBandLinearV8R, QVBandEmbeddingV8R, None, decoder=lambda lin: lin.dense(torch.float32),
                                    finalize=fuse_same_input_r)


def get_format(name: str | None) -> FormatSpec:
    _build_registry()
    spec = _REGISTRY.get(name)
    if spec is None:
        raise ValueError(f"pack format {name!r} is not supported -- known formats: {', '.join(sorted(_REGISTRY))}")
    return spec


def require(spec: FormatSpec, backend: str):
    """The class `spec` provides for `backend`, or a clear error (formats.py:113-126)."""
    cls = getattr(spec, backend, None)
    if cls is None:
        raise NotImplementedError(f"pack format {spec.name!r} has no {backend} reader -- this path needs one, and reading "
                                  f"the packs with another format's class would return silent garbage.")
    return cls


def decode_pack(path: str, spec: FormatSpec | None = None, device: str = "cuda", dtype=None):
    """Dense (Q, P) weights of a pack file (bf16 unless `dtype`), decoded on the GPU: for audits and re-packing, never
    on the inference path (formats.py:129-160)."""
    import torch
    dtype = torch.bfloat16 if dtype is None else dtype
    if spec is None:
        spec = get_format(path.rsplit(".", 1)[-1])
    if str(device).startswith("cpu"):
        raise NotImplementedError("decode_pack: packs are decoded by GPU kernels only in this build")
    lin = spec.linear.from_packfile(path, device=device)
    try:
        return require(spec, "decoder")(lin).to(dtype)
    finally:
        del lin


def known_formats() -> tuple:
    _build_registry()
    return tuple(sorted(_REGISTRY))
