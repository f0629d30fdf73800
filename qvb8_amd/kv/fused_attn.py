"""Attention straight over the banded KV cache's ids (reference: src/qv_band/kv/fused_attn.py:155-316): the ids of all
segments of a layer lie in one (capacity, kv heads, head_dim) buffer, the affine constants per segment / head / channel
beside them, and the kernel restores keys and values tile by tile -- nothing of the context's size is ever built.

`attend` is the reference's call: it folds the softmax scale into the queries, launches qvb8_attn_fwd through the C ABI
and combines the splits.  There is no other backend: without the HIP library it raises.
"""
from __future__ import annotations

import math
import os

import torch

from qvb8_amd import _lib

BLOCK_N = 32          # keys per tile of the table; the kernel takes tiles of at most 32 keys


class QVLayout:
    """The id buffers, constants and tile table of one layer (fused_attn.py:155-186).  ki / vi: (capacity, Hkv, D)
    uint8, or int16 holding 16-bit patterns; kmin / vmin hold the range CENTRE when kc / vc are given."""

    def __init__(self, ki, vi, kmin, kstep, vmin, vstep, seg_len, device, block_n=BLOCK_N, kc=None, vc=None,
                 hk=None, hv=None, hrow=None):
        if hk is not None or hv is not None or hrow is not None:
            raise NotImplementedError("the high-byte pool of 9..16-bit heads is not read: store such layers' ids in 16 bits "
                                      "(layout_from_segments(..., allow_wide=True))")
        if block_n > BLOCK_N:
            raise ValueError(f"tiles of {block_n} keys: the kernel takes at most {BLOCK_N}")
        self.block_n = block_n
        n_seg = len(seg_len)
        zeros = lambda: torch.zeros(n_seg, kmin.shape[1], dtype=torch.float32, device=device)     # noqa: E731
        self.kc = kc if kc is not None else zeros()
        self.vc = vc if vc is not None else zeros()
        self.ki, self.vi = ki, vi
        self.kmin, self.kstep, self.vmin, self.vstep = kmin, kstep, vmin, vstep
        self.n = int(sum(seg_len))
        starts, lens, segs, pos = [], [], [], 0
        for si, sl in enumerate(seg_len):
            for a in range(0, sl, block_n):
                starts.append(pos + a)
                lens.append(min(block_n, sl - a))
                segs.append(si)
            pos += sl
        table = torch.tensor([starts, lens, segs], dtype=torch.int32).reshape(3, -1).to(device)
        self.t_start, self.t_len, self.t_seg = table[0].contiguous(), table[1].contiguous(), table[2].contiguous()
        self.n_tiles = len(starts)


def layout_from_segments(segs_k, segs_v, seg_len, device, allow_wide: bool = False):
    """segs_*: per segment a list with one BandedKV per kv head (fused_attn.py:189-216).  Returns None when a head uses
    more than 8 bits -- unless allow_wide, which stores every id in 16 bits instead (the kernel reads either)."""
    nseg, h = len(segs_k), len(segs_k[0])
    n = sum(seg_len)
    d = segs_k[0][0].orig_shape[1]
    wide = any(bk.bits > 8 for store in (segs_k, segs_v) for seg in store for bk in seg)
    if wide and not allow_wide:
        return None
    dt = torch.int16 if wide else torch.uint8
    ki = torch.empty(n, h, d, dtype=dt, device=device)
    vi = torch.empty_like(ki)
    P = [torch.empty(nseg, h, d, dtype=torch.float32, device=device) for _ in range(4)]
    KC = torch.zeros(nseg, h, dtype=torch.float32, device=device)
    VC = torch.zeros_like(KC)
    pos = 0
    for si in range(nseg):
        sl = seg_len[si]
        for hi in range(h):
            for store, ids_t, mid, st, C in ((segs_k, ki, P[0], P[1], KC), (segs_v, vi, P[2], P[3], VC)):
                bk = store[si][hi]
                ids = bk.ids().to(device)
                ids_t[pos:pos + sl, hi] = (ids.to(torch.int32) - ((ids > 32767).to(torch.int32) << 16)).to(dt) if wide else ids.to(dt)
                c = ((1 << bk.bits) - 1) / 2.0
                mid[si, hi] = (bk.min_s + bk.tau_s * c).to(device)      # range centre
                st[si, hi] = bk.tau_s.to(device)
                C[si, hi] = c
        pos += sl
    return QVLayout(ki, vi, P[0], P[1], P[2], P[3], list(seg_len), device, kc=KC, vc=VC)


def fwd(q, ki, vi, kmid, kstep, vmid, vstep, kc, vc, ts, tl, tseg, o, m, l, q_pos0: int, tps: int, scale: float, G: int) -> None:
    """The compiled kernel's call (ext.fwd, kv/cuda_attn/qvattn_cuda.cu:262-287): fills o (S, Hkv, R, D), m, l (S, Hkv, R)."""
    if q.dtype != torch.float16 or q.stride(2) != 1:
        raise RuntimeError("q must be fp16, contiguous in D")
    wide = ki.dtype == torch.int16
    if not (wide or ki.dtype == torch.uint8) or vi.dtype != ki.dtype or ki.stride(2) != 1 or ki.stride() != vi.stride():
        raise RuntimeError("ids layout")
    for p in (kmid, kstep, vmid, vstep, kc, vc, ts, tl, tseg, o, m, l):
        if not p.is_contiguous() or p.device != q.device:
            raise RuntimeError("constants, tile table and outputs must be contiguous and on q's device")
    if ts.dtype != torch.int32 or tl.dtype != torch.int32 or tseg.dtype != torch.int32 or o.dtype != torch.float32:
        raise RuntimeError("tile table must be int32, outputs fp32")
    lib = _lib.load()
    with torch.cuda.device(q.device):
        rc = lib.qvb8_attn_fwd(q.data_ptr(), q.stride(0), q.stride(1), ki.data_ptr(), vi.data_ptr(), 2 if wide else 1,
                               ki.stride(0), ki.stride(1), kmid.data_ptr(), kstep.data_ptr(), vmid.data_ptr(), vstep.data_ptr(),
                               kc.data_ptr(), vc.data_ptr(), ts.data_ptr(), tl.data_ptr(), tseg.data_ptr(), ts.numel(),
                               o.data_ptr(), m.data_ptr(), l.data_ptr(), o.shape[0], o.shape[2], ki.shape[1], q.shape[2],
                               int(q_pos0), int(tps), float(scale), int(G), torch.cuda.current_stream().cuda_stream)
    _lib._check(rc, lib)


def rows_per_workgroup(rows: int, d: int) -> int:
    """Query rows one workgroup of the kernel serves from a restored tile: 16, 32 from 17 rows on, 64 from 33 rows on
    when the heads have 128 channels (qvb8_attn.hip, launch_attn)."""
    return 16 if rows <= 16 else 32 if (rows <= 32 or d == 256) else 64


def plan_splits(n_tiles: int, hkv: int, rows: int, device, per_cu: int | None = None, d: int = 256, wide: bool = False) -> tuple:
    """(tiles per split, splits): as many workgroups as the card holds at once -- three per compute unit (four with byte ids and
    128 channels), two when a workgroup serves more than 16 rows or reads 16-bit ids with 256 channels (the kernel's
    registers) -- and fewer
    splits for long query blocks (fused_attn.py:259-264, 271-275).  Measured over 32768 / 131072 keys with three
    resident workgroups of 16 rows: 768 workgroups 27.2 / 74.9 us, 512 27.7 / 86.1, 1024 28.5 / 81.8, 1536 29.5 / 76.5."""
    block = rows_per_workgroup(rows, d)
    if per_cu is None:
        per_cu = 2 if (block > 16 or (wide and d == 256)) else 4 if (d == 128 and not wide) else 3
    per_cu = int(os.environ.get("QVB8_ATTN_WG_PER_CU", per_cu))          # a knob for measurements
    n_rb = -(-rows // block)
    want = per_cu * torch.cuda.get_device_properties(device).multi_processor_count
    n_splits = max(1, min(n_tiles, want // max(1, hkv * n_rb)))
    tps = max(1, math.ceil(n_tiles / n_splits))
    return tps, max(1, math.ceil(n_tiles / tps))


def combine_splits(o, m, l, G: int):
    """Per-split (unnormalised o, running max m, running sum l) of `fwd` -> (out (MQ, Hq, D), lse (MQ, Hq)), one launch
    of qvb8_attn_combine: every split is weighted by exp(m - max over splits); a row no split saw a key for gives 0
    and -inf (fused_attn.py:302-316)."""
    S, hkv, rows, d = o.shape
    mq = rows // G
    out = torch.empty(mq, hkv * G, d, dtype=torch.float32, device=o.device)
    lse = torch.empty(mq, hkv * G, dtype=torch.float32, device=o.device)
    lib = _lib.load()
    with torch.cuda.device(o.device):
        rc = lib.qvb8_attn_combine(o.data_ptr(), m.data_ptr(), l.data_ptr(), S, hkv, rows, d, int(G), out.data_ptr(), lse.data_ptr(),
                                   torch.cuda.current_stream().cuda_stream)
    _lib._check(rc, lib)
    return out, lse


def merge_lse_all(o, lse):
    """n normalised partial results o (n, ..., D) with their log-sum-exps lse (n, ...) -> (merged result, merged lse), one
    launch (fused_attn.py:769-778: the banded part and the dense residual of a layer, the blocks of a tiered cache)."""
    n, d = o.shape[0], o.shape[-1]
    rows = lse[0].numel()
    oc = o.to(torch.float32).contiguous()
    mc = lse.to(torch.float32).contiguous()
    out = torch.empty(o.shape[1:], dtype=torch.float32, device=o.device)
    lse_out = torch.empty(lse.shape[1:], dtype=torch.float32, device=o.device)
    lib = _lib.load()
    with torch.cuda.device(o.device):
        rc = lib.qvb8_attn_combine(oc.data_ptr(), mc.data_ptr(), None, n, 1, rows, d, max(rows, 1), out.data_ptr(), lse_out.data_ptr(),
                                   torch.cuda.current_stream().cuda_stream)
    _lib._check(rc, lib)
    return out, lse_out


def merge_lse(o1, lse1, o2, lse2):
    """Two partial results (fused_attn.py:781-788)."""
    return merge_lse_all(torch.stack([o1, o2]), torch.stack([lse1, lse2]))


def attend(q, lay: QVLayout, q_pos0: int, scale: float, n_splits: int | None = None,
           num_warps: int = 4, num_stages: int = 1, block_m: int | None = None):
    """q: (MQ, Hq, D) bf16 / fp16 queries at positions q_pos0 .. q_pos0 + MQ - 1.  Returns (o (MQ, Hq, D) fp32, lse
    (MQ, Hq) fp32) over the banded keys with position <= the query's; rows without a visible key get lse = -inf
    (fused_attn.py:246-316).  num_warps / num_stages / block_m are the reference's tuning knobs of its other kernel;
    they are accepted and have no meaning here."""
    del num_warps, num_stages, block_m
    mq, hq, d = q.shape
    hkv = lay.ki.shape[1]
    g = hq // hkv
    rows = mq * g
    if n_splits is None:
        tps, n_splits = plan_splits(lay.n_tiles, hkv, rows, q.device, d=d, wide=lay.ki.dtype == torch.int16)
    else:
        tps = max(1, math.ceil(lay.n_tiles / max(1, n_splits)))
        n_splits = max(1, math.ceil(lay.n_tiles / tps))
    # fp16 queries: the softmax scale goes in first (|q| shrinks), then they saturate, so that an outlier channel cannot
    # turn into inf and a row into NaN (fused_attn.py:276-279)
    qc = q.contiguous()
    if qc.dtype not in (torch.float32, torch.float16, torch.bfloat16):
        qc = qc.float()
    q16 = torch.empty(qc.shape, dtype=torch.float16, device=qc.device)
    lib = _lib.load()
    with torch.cuda.device(qc.device):
        _lib._check(lib.qvb8_scale_sat_half(qc.data_ptr(), _lib.dtype_code(qc.dtype), qc.numel(), float(scale), q16.data_ptr(),
                                            torch.cuda.current_stream().cuda_stream), lib)
    o = torch.empty(n_splits, hkv, rows, d, dtype=torch.float32, device=q.device)
    m = torch.empty(n_splits, hkv, rows, dtype=torch.float32, device=q.device)
    l = torch.empty_like(m)
    fwd(q16, lay.ki, lay.vi, lay.kmin, lay.kstep, lay.vmin, lay.vstep, lay.kc.contiguous(), lay.vc.contiguous(),
        lay.t_start, lay.t_len, lay.t_seg, o, m, l, q_pos0, tps, 1.0, g)
    return combine_splits(o, m, l, g)
