"""Per-channel affine KV codec (reference: src/qv_band/kv/codec.py): fixed bits per element of a (seq, head_dim)
segment of one kv head, one (min_s, tau_s) per channel,

    id = round((x - min_c) / step_c),  step_c = (max_c - min_c) / (2^B - 1),  recon = min_c + id * step_c,

no escapes (minimum and maximum cover every value).  The encoder runs as torch ops on the tensor's device; the ids are
kept bit-packed, LSB first, row-major (codec.py:53-82), as the cache stores them between attention calls.
"""
from __future__ import annotations

import math
from dataclasses import dataclass

import torch

STEP_FLOOR = 1e-12
MAX_BITS = 16


class KVCertificateError(ValueError):
    """tau is below what 16 bits per element can certify for a head (codec.py:171-172)."""


def pack_ids(ids: torch.Tensor, bits: int) -> torch.Tensor:
    """Flat ids (< 2^bits) -> uint8, fields LSB first and bit-contiguous (codec.py:53-68)."""
    n = ids.numel()
    shifts = torch.arange(bits, device=ids.device, dtype=torch.int64)
    stream = ((ids.reshape(-1, 1).to(torch.int64) >> shifts) & 1).to(torch.uint8).reshape(-1)
    pad = (-stream.numel()) % 8
    if pad:
        stream = torch.cat([stream, stream.new_zeros(pad)])
    weights = (1 << torch.arange(8, device=ids.device, dtype=torch.int64)).to(torch.uint8)
    out = (stream.reshape(-1, 8) * weights).sum(dim=1, dtype=torch.int64).to(torch.uint8)
    assert out.numel() == (n * bits + 7) // 8
    return out


def unpack_ids(packed: torch.Tensor, bits: int, n: int) -> torch.Tensor:
    """Inverse of pack_ids: int64[n] (codec.py:71-82)."""
    shifts = torch.arange(8, device=packed.device, dtype=torch.int64)
    stream = ((packed.reshape(-1, 1).to(torch.int64) >> shifts) & 1).reshape(-1)[: n * bits].reshape(n, bits)
    return (stream << torch.arange(bits, device=packed.device, dtype=torch.int64)).sum(dim=1)


@dataclass(eq=False)
class BandedKV:
    """One kv head of one segment (codec.py:99-166)."""
    packed: torch.Tensor            # uint8, bits * seq * head_dim bits, row-major
    min_s: torch.Tensor             # (head_dim,) fp32
    tau_s: torch.Tensor             # (head_dim,) fp32 step per channel
    bits: int
    orig_shape: tuple               # (seq, head_dim)
    orig_dtype: torch.dtype
    tau: float

    def nbytes(self) -> int:
        return int(self.packed.numel() + 4 * (self.min_s.numel() + self.tau_s.numel()))

    @property
    def max_error(self) -> float:
        return float(self.tau_s.max()) * 0.5

    def ids(self) -> torch.Tensor:
        seq, hd = self.orig_shape
        return unpack_ids(self.packed, self.bits, seq * hd).reshape(seq, hd)

    def decode_all_torch(self, device=None, dtype=torch.float32) -> torch.Tensor:
        """min_s + id * tau_s in fp32, rounded once to `dtype` (codec.py:117-118)."""
        dev = self.packed.device if device is None else torch.device(device)
        ids = self.ids().to(dev)
        return (self.min_s.to(dev) + ids.to(torch.float32) * self.tau_s.to(dev)).to(dtype)

    def truncate(self, n_rows: int) -> "BandedKV":
        """The first n_rows tokens, not re-quantised: a byte prefix of `packed` (codec.py:120-139)."""
        seq, hd = self.orig_shape
        if not 0 < n_rows <= seq:
            raise ValueError(f"truncate({n_rows}) outside 1..{seq}")
        if n_rows == seq:
            return self
        nbytes = (n_rows * hd * self.bits + 7) // 8
        return BandedKV(self.packed[:nbytes].clone(), self.min_s, self.tau_s, self.bits, (n_rows, hd), self.orig_dtype, self.tau)


    def take_rows(self, rows: torch.Tensor) -> "BandedKV":
        """Only the given token rows (indices inside 0..seq-1), not re-quantised: the ids are unpacked, selected and
        packed again at the same width with the same constants (codec.py:141-158)."""
        seq, hd = self.orig_shape
        rows = rows.to(torch.int64)
        if rows.numel() == 0 or int(rows.min()) < 0 or int(rows.max()) >= seq:
            raise ValueError(f"take_rows indices must lie in 0..{seq - 1} and be non-empty")
        if rows.numel() == seq and bool((rows == torch.arange(seq, device=rows.device)).all()):
            return self
        kept = self.ids()[rows.to(self.packed.device)]
        return BandedKV(pack_ids(kept.reshape(-1), self.bits), self.min_s, self.tau_s, self.bits, (int(rows.numel()), hd),
                        self.orig_dtype, self.tau)

    def decode_all(self) -> torch.Tensor:
        return self.decode_all_torch("cpu", torch.float32)

    def decode_row(self, row_idx: int) -> torch.Tensor:
        return self.decode_all()[row_idx]

    outlier_count = property(lambda s: 0)           # minimum and maximum cover every value: there are no escapes
    outlier_ratio = property(lambda s: 0.0)


def unband_kv_4d(banded: list, batch: int, heads: int, device="cpu") -> torch.Tensor:
    """(batch, heads, seq, head_dim) in the cache's dtype from one BandedKV per head (codec.py:252-262)."""
    if not banded:
        return torch.empty(batch, heads, 0, 0, device=device)
    seq, dim = banded[0].orig_shape
    mats = [bk.decode_all_torch(device, banded[0].orig_dtype) for bk in banded]
    return torch.stack(mats, dim=0).reshape(batch, heads, seq, dim)


def _channel_grid(x, lo, span, widths):
    """Nearest point of each channel's grid of 2^w - 1 intervals over [lo, lo + span] (w per head): (ids, step)."""
    levels = torch.tensor([float((1 << w) - 1) for w in widths], device=x.device).view(-1, 1, 1)
    step = (span / levels).clamp_min(STEP_FLOOR)
    return torch.minimum(torch.round((x - lo) / step).clamp_(min=0), levels), step


def band_kv_heads(t: torch.Tensor, orig_dtype: torch.dtype, bits: int, tau: float = 0.0, certify: bool = True) -> list:
    """(heads, seq, head_dim) -> one BandedKV per head (codec.py:175-241).  With certify and tau > 0, `bits` is a floor:
    a head's width rises (to 16 at most) until the decoder's own expression, rounded to `orig_dtype`, is within tau of
    every element; KVCertificateError when 16 bits do not reach it.  Heads are independent: only the heads that still
    miss tau are quantised again, one host read per round."""
    heads, seq, dim = t.shape
    x = torch.nan_to_num(t.detach().to(torch.float32), nan=0.0, posinf=0.0, neginf=0.0)
    lo = x.amin(1, keepdim=True)
    span = x.amax(1, keepdim=True) - lo
    widths = [bits] * heads
    open_heads = []
    if certify and tau > 0:
        open_heads = list(range(heads))
        for i, widest in enumerate(span.amax((1, 2)).cpu().tolist()):     # first guess: half a step within tau
            if widest > 0:
                widths[i] = min(MAX_BITS, max(bits, math.ceil(math.log2(widest / (2.0 * tau) + 1.0))))
    ids, step = _channel_grid(x, lo, span, widths)
    while open_heads:
        sel = torch.tensor(open_heads, device=x.device)
        shown = (lo[sel] + ids[sel] * step[sel]).to(orig_dtype).to(torch.float32)      # what the decoder will hand out
        miss = (shown - x[sel]).abs().amax((1, 2)).cpu().tolist()
        open_heads = [i for i, e in zip(open_heads, miss) if e > tau]
        if not open_heads:
            break
        worst = dict(zip(sel.tolist(), miss))
        for i in open_heads:
            if widths[i] >= MAX_BITS:
                raise KVCertificateError(f"head {i}: at {MAX_BITS} bits the per-channel grid is still {worst[i]:.4g} off, "
                                         f"tau = {tau:g} cannot be certified for values stored as {orig_dtype}")
            widths[i] += 1
        sel = torch.tensor(open_heads, device=x.device)
        ids[sel], step[sel] = _channel_grid(x[sel], lo[sel], span[sel], [widths[i] for i in open_heads])
    return [BandedKV(pack_ids(ids[i].to(torch.int64).reshape(-1), widths[i]), lo[i, 0].contiguous(), step[i, 0].contiguous(),
                     widths[i], (seq, dim), orig_dtype, tau) for i in range(heads)]
