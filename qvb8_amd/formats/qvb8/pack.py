"""Synthetic QVB8 pack writer.

The reference ships readers only; its calibration / pack writer is not published.
This writer produces packs the readers accept and whose restore meets the
certificate, which is all the format asks of a writer (reference
formats/qvb8/decode.py:14-43 for the codebook, module.py:66-78 for what is certified).
It is written with torch tensor operations only, so it runs on whatever device the
weight lives on (a 9B-shape layer set is encoded on the GPU in seconds).

Per row:
    step   tau_s = 2*(tau - h)*(1 - 2^-12), h = half an ULP of the coarsest restore
           dtype at the row's peak magnitude: the certificate is on the NARROWED value
           fp16(band) (and bf16(band) for an fp16+bf16 pack), so the bucket must leave
           room for that rounding
    origin min_s = row_min + tau_s/2 (bucket centre), id = nearest bucket, clamped
    width  nbits = max(1, ceil(log2(buckets))), capped at `max_nbits` (window centred on
           the row median; whatever falls outside becomes an escape)
Every element is then checked: |narrow(fma(id, tau_s, min_s)) - w| < tau, strictly; an
element that fails is stored exactly as an escape.
"""
from __future__ import annotations

import numpy as np
import torch

from ...common.errors import Qvb8Error
from . import decode as L
from . import pack_container as C


def _half_ulp(mag: torch.Tensor, mant_bits: int, min_exp: int) -> torch.Tensor:
    """Half an ULP of a float format with `mant_bits` explicit mantissa bits and
    smallest normal exponent `min_exp`, at magnitude `mag` (float64 tensor)."""
    _, e = torch.frexp(mag.clamp_min(2.0 ** (min_exp - 1)))     # mag = m * 2^e, m in [0.5, 1)
    e = (e - 1).clamp_min(min_exp)
    return torch.pow(torch.tensor(2.0, dtype=torch.float64, device=mag.device),
                     (e - mant_bits - 1).double())


def band_fp32(ids: torch.Tensor, tau_s: torch.Tensor, min_s: torch.Tensor) -> torch.Tensor:
    """fma(float(id), tau_s[row], min_s[row]) rounded once to fp32, computed in float64:
    id < 2^14 and tau_s has 24 significant bits, so the product is exact in float64 and
    the sum is exact too for the exponent gaps that occur here; one rounding follows."""
    return (ids.double() * tau_s.double()[:, None] + min_s.double()[:, None]).float()


def _pack_rows(ids: torch.Tensor, nb: torch.Tensor, P: int):
    """ids (Q,P) int64, nb (Q,) int64 -> (payload uint8 with 8 pad bytes, bit_off int64)."""
    Q = ids.shape[0]
    dev = ids.device
    row_bits = nb * P
    bit_off = torch.zeros(Q, dtype=torch.int64, device=dev)
    if Q > 1:
        bit_off[1:] = torch.cumsum(row_bits[:-1], 0)
    total_bits = int(row_bits.sum())
    nbytes = (total_bits + 7) // 8
    if Q == 0 or P == 0:
        return torch.zeros(nbytes + L.IDS_PAD_BYTES, dtype=torch.uint8, device=dev), bit_off
    if P % 8 != 0 or int(nb.max()) > 8:
        buf, _ = L.pack_bits_rows(ids.cpu().numpy(), nb.cpu().numpy())
        return torch.from_numpy(buf).to(dev), bit_off
    buf = torch.zeros(nbytes + L.IDS_PAD_BYTES, dtype=torch.uint8, device=dev)
    g = P // 8
    widths = torch.unique(nb).tolist()
    for w in widths:
        rows = torch.nonzero(nb == w).view(-1) if len(widths) > 1 else None
        f = (ids if rows is None else ids[rows]).view(-1, g, 8)
        word = f[:, :, 0].clone()
        for j in range(1, 8):
            word |= f[:, :, j] << (w * j)
        sh = torch.arange(w, device=dev, dtype=torch.int64) * 8
        by = ((word.unsqueeze(-1) >> sh) & 0xFF).to(torch.uint8).view(f.shape[0], g * w)
        if rows is None:
            buf[:nbytes] = by.reshape(-1)
        else:
            L_row = g * w
            step = max(1, (32 << 20) // L_row)
            base = bit_off[rows] >> 3
            ar = torch.arange(L_row, device=dev, dtype=torch.int64)
            for i in range(0, len(rows), step):
                dst = base[i:i + step, None] + ar[None, :]
                buf[dst.reshape(-1)] = by[i:i + step].reshape(-1)
    return buf, bit_off


@torch.no_grad()
def encode_tensor(W: torch.Tensor, tau: float, *, restore: str = "fp16", source: str | None = None,
                  max_nbits: int = L.MAX_CERTIFIED_NBITS, force_escapes=None, keep_ids: bool = False) -> dict:
    """Encode a (Q, P) weight.  Returns torch tensors on W's device:
    min_s, tau_s (f32), nbits (u8), bit_off (i64), ids (u8 payload + 8 pad bytes),
    esc_idx/esc_vals (the fp16 table: every decode that keeps fp32 or rounds to fp16),
    esc_idx_bf16/esc_vals_bf16 (all escapes: decodes that round to bf16), plus Q, P, tau,
    max_err (over both restore precisions the pack certifies), restore, source.
    `force_escapes`: flat positions stored as escapes whatever the band says.  `keep_ids`: also return the unpacked
    ids as `ids_dense` (Q, P) int16 (what the entropy coder of the QVB8R format starts from)."""
    if restore not in ("fp16", "fp16+bf16"):
        raise Qvb8Error(f"restore must be 'fp16' or 'fp16+bf16', not {restore!r}")
    if W.dim() != 2:
        raise Qvb8Error("encode_tensor wants a (Q, P) matrix")
    if not 1 <= max_nbits <= L.MAX_CERTIFIED_NBITS:
        raise Qvb8Error(f"max_nbits must be in 1..{L.MAX_CERTIFIED_NBITS}")
    if source is None:
        source = "bf16" if W.dtype == torch.bfloat16 else "fp32"
    Q, P = W.shape
    dev = W.device
    Wf = W.float().contiguous()
    if not bool(torch.isfinite(Wf).all()):
        raise Qvb8Error("weight has non-finite values")
    Wd = Wf.double()
    if Q == 0 or P == 0:
        z32 = torch.zeros(Q, dtype=torch.float32, device=dev)
        e = torch.zeros(0, dtype=torch.int64, device=dev)
        v = torch.zeros(0, dtype=torch.float32, device=dev)
        return dict(Q=Q, P=P, tau=float(tau), max_err=0.0, restore=restore, source=source, min_s=z32,
                    tau_s=z32.clone(), nbits=torch.ones(Q, dtype=torch.uint8, device=dev),
                    bit_off=torch.arange(Q, device=dev, dtype=torch.int64) * P,
                    ids=torch.zeros((Q * P + 7) // 8 + L.IDS_PAD_BYTES, dtype=torch.uint8, device=dev),
                    esc_idx=e, esc_vals=v, esc_idx_bf16=e, esc_vals_bf16=v)
    lo, hi = Wd.amin(1), Wd.amax(1)
    peak = torch.maximum(lo.abs(), hi.abs()) + tau
    h = _half_ulp(peak, 10, -14)
    if restore == "fp16+bf16":
        h = torch.maximum(h, _half_ulp(peak, 7, -126))
    slack = tau - h
    ts = torch.where(slack > 0.125 * tau, 2.0 * slack * (1.0 - 2.0 ** -12), torch.full_like(slack, tau))
    ts32 = ts.float()
    ts = ts32.double()
    n_buckets = torch.floor((hi - lo) / ts).long() + 1
    nb = torch.from_numpy(L._nbits_for(n_buckets.cpu().numpy())).to(dev)
    row_min = lo.clone()
    over = nb > max_nbits
    if bool(over.any()):
        # window of 2^max_nbits buckets centred on the row median; the rest escapes
        med = Wd[over].median(1).values
        span = (2.0 ** max_nbits) * ts[over]
        start = torch.minimum(torch.maximum(med - 0.5 * span, lo[over]), hi[over] - span + ts[over])
        row_min[over] = start
        nb = nb.clamp_max(max_nbits)
    min_s32 = (row_min + 0.5 * ts).float()
    top = (torch.ones_like(nb) << nb) - 1
    ids = torch.round((Wd - min_s32.double()[:, None]) / ts[:, None]).long()
    ids = torch.minimum(ids.clamp_min_(0), top[:, None])
    band = band_fp32(ids, ts32, min_s32)
    err16 = (band.half().double() - Wd).abs()
    bad16 = ~(err16 < tau)
    if restore == "fp16+bf16":
        errb = (band.bfloat16().double() - Wd).abs()
        bad_all = bad16 | ~(errb < tau)
    else:
        errb = None
        bad_all = bad16
    if force_escapes is not None:
        fe = torch.as_tensor(force_escapes, dtype=torch.int64, device=dev)
        bad16.view(-1)[fe] = True
        bad_all.view(-1)[fe] = True
    esc_all = torch.nonzero(bad_all.view(-1)).view(-1)
    esc_16 = torch.nonzero(bad16.view(-1)).view(-1)
    vals_all = Wf.view(-1)[esc_all]
    vals_16 = Wf.view(-1)[esc_16]
    # certificate over what a reader restores: narrowed band where not escaped, narrowed exact value where escaped
    e16 = torch.where(bad16, (Wf.half().double() - Wd).abs(), err16)
    max_err = float(e16.max())
    if errb is not None:
        eb = torch.where(bad_all, (Wf.bfloat16().double() - Wd).abs(), errb)
        max_err = max(max_err, float(eb.max()))
    buf, bit_off = _pack_rows(ids, nb, P)
    same = esc_all.numel() == esc_16.numel()
    extra = dict(ids_dense=ids.to(torch.int16)) if keep_ids else {}
    return dict(**extra, Q=Q, P=P, tau=float(tau), max_err=max_err, restore=restore, source=source,
                min_s=min_s32, tau_s=ts32, nbits=nb.to(torch.uint8), bit_off=bit_off, ids=buf,
                esc_idx=esc_16, esc_vals=vals_16,
                esc_idx_bf16=esc_16 if same else esc_all, esc_vals_bf16=vals_16 if same else vals_all)


def _np(t):
    return t.detach().cpu().numpy()


def to_qvbd_blob(enc: dict) -> bytes:
    """QVBD ('.qvband') bytes of an encoded tensor.  The stored escape list is the full
    one; an fp16+bf16 pack whose fp16 table is shorter also needs escape_tables.json."""
    return C.pack_formula(Q=enc["Q"], P=enc["P"], tau=enc["tau"], max_err=enc["max_err"],
                          min_s=_np(enc["min_s"]), tau_s=_np(enc["tau_s"]), nbits=_np(enc["nbits"]),
                          buf=_np(enc["ids"]), esc_idx=_np(enc["esc_idx_bf16"]),
                          esc_vals=_np(enc["esc_vals_bf16"]), source=enc["source"], restore=enc["restore"])


def to_qvb8_blob(enc: dict) -> bytes:
    """Legacy standalone '.qvb8' bytes (fp16 escape table, verbatim fp32 values)."""
    return L.pack_tensor(_np(enc["min_s"]), _np(enc["tau_s"]), _np(enc["nbits"]), _np(enc["bit_off"]),
                         _np(enc["ids"]), enc["Q"], enc["P"], enc["tau"],
                         _np(enc["esc_idx"]), _np(enc["esc_vals"]))


def write_pack(path: str, enc: dict) -> None:
    """Write `enc` to `path` ('.qvb8' -> standalone blob, anything else -> QVBD) and, for
    an fp16+bf16 QVBD pack, add its entry to the folder's escape_tables.json."""
    import os
    legacy = path.endswith(".qvb8")
    with open(path, "wb") as fh:
        fh.write(to_qvb8_blob(enc) if legacy else to_qvbd_blob(enc))
    if not legacy and enc["restore"] == "fp16+bf16":
        from .escape_split import update_tables
        update_tables(os.path.dirname(os.path.abspath(path)), os.path.basename(path),
                      _np(enc["esc_idx_bf16"]), _np(enc["esc_idx"]))
