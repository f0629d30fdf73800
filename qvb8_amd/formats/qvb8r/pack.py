"""QVB8 -> QVB8R transcode: the same band ids, rANS-coded.  The restore of the result equals the QVB8 restore of the
source bit for bit (same ids, same min_s / tau_s, same escapes), so the certificate carries over unchanged."""
from __future__ import annotations

import numpy as np

from . import codec, container


def transcode(enc: dict, *, n_classes: int | None = None, rows_per_tile: int | None = None) -> dict:
    """`enc` = qvb8_amd.formats.qvb8.pack.encode_tensor(..., keep_ids=True).  Returns the dict container.read would
    return for the written file (header fields + arrays): what QVBandLinearV8R is built from."""
    if "ids_dense" not in enc:
        raise ValueError("transcode needs the unpacked ids: encode_tensor(..., keep_ids=True)")
    Q, P = int(enc["Q"]), int(enc["P"])
    ids = enc["ids_dense"].cpu().numpy()
    r = codec.encode_ids(ids, n_classes=n_classes, rows_per_tile=rows_per_tile)
    min_s = enc["min_s"].cpu().numpy().astype(np.float32)
    tau_s = enc["tau_s"].cpu().numpy().astype(np.float32)
    esc_idx = enc["esc_idx_bf16"].cpu().numpy().astype(np.int64)          # the file holds the full list
    esc_val = enc["esc_vals_bf16"].cpu().numpy().astype(np.float32)
    q, c = esc_idx // P, esc_idx % P
    # exact - fp32 band value, the band value with ONE rounding (fused multiply-add), via float64: id * tau_s is exact there
    band = (ids[q, c].astype(np.int64).astype(np.float64) * tau_s[q].astype(np.float64) + min_s[q].astype(np.float64)).astype(np.float32)
    esc_delta = (esc_val - band).astype(np.float32)
    cert = dict(tau=float(enc["tau"]), max_err=float(enc["max_err"]), restore=enc["restore"], source=enc["source"])
    d = dict(r, Q=Q, P=P, PB=codec.PB, cert=cert, min_s=min_s, tau_s=tau_s, esc_idx=esc_idx, esc_val=esc_val, esc_delta=esc_delta)
    return d


def to_bytes(d: dict) -> bytes:
    return container.to_bytes(d, d["Q"], d["P"], d["min_s"], d["tau_s"], d["esc_idx"], d["esc_val"], d["esc_delta"], d["cert"])


def write_pack(path: str, d: dict, fp16_idx=None) -> int:
    """Write the .qvb8r file; for an fp16+bf16 pack also record which escapes form the fp16 table (escape_tables.json)."""
    import os
    n = container.write(path, d, d["Q"], d["P"], d["min_s"], d["tau_s"], d["esc_idx"], d["esc_val"], d["esc_delta"], d["cert"])
    if d["cert"].get("restore") == "fp16+bf16" and fp16_idx is not None:
        from qvb8_amd.formats.qvb8.escape_split import update_tables
        update_tables(os.path.dirname(os.path.abspath(path)), os.path.basename(path), d["esc_idx"], np.asarray(fp16_idx, np.int64))
    return n
