"""The QVB8 operator functions, with the names and positional argument orders of the
reference's `qvb8_cuda` extension module (qvb8_cuda.cu:2673-2691), implemented by
libqvb8_amd.so.  torch is used for device memory (outputs come from torch's caching
allocator, like the reference's torch::empty) and for the current stream only.

    forward(X, ids, min_s, row_nbits, row_bit_off, P, tau_s, esc_idx, esc_vals)   any M
    gemv(...)            M = 1, X fp16        gemv_multi(...)   M = 1..8
    decode(ids, min_s, row_nbits, row_bit_off, P, tau_s, esc_idx, esc_vals)       (Q, P) fp16
    decode_bf16(...)     (Q, P) bf16
Additions without a counterpart there: decode_f32 (the fp32 band value), certify,
saturating_half, lookup_rows (the embedding read, which the reference does in torch).
"""
from __future__ import annotations

import ctypes

import torch

from . import _lib


def _check_pack(ids, min_s, row_nbits, row_bit_off, tau_s):
    _lib.require_cuda(ids, min_s, row_nbits, row_bit_off, tau_s)
    if ids.dtype != torch.uint8:
        raise RuntimeError("ids must be uint8")
    if min_s.dtype != torch.float32 or tau_s.dtype != torch.float32:
        raise RuntimeError("min_s and tau_s must be fp32")
    if row_nbits.dtype != torch.uint8:
        raise RuntimeError("row_nbits must be uint8")
    if row_bit_off.dtype != torch.int64:
        raise RuntimeError("row_bit_off must be int64")
    Q = min_s.numel()
    if tau_s.numel() != Q or row_nbits.numel() != Q or row_bit_off.numel() != Q:
        raise RuntimeError("per-row metadata lengths differ")
    return Q


def _check_escapes(esc_idx, esc_vals):
    n = 0 if esc_idx is None else esc_idx.numel()
    if n:
        _lib.require_cuda(esc_idx, esc_vals)
        if esc_idx.dtype != torch.int64 or esc_vals.dtype != torch.float32 or esc_vals.numel() != n:
            raise RuntimeError("escapes must be int64 positions and float32 values of equal length")
    return n


def _decode_to(code, dtype, ids, min_s, row_nbits, row_bit_off, P, tau_s, esc_idx, esc_vals):
    lib = _lib.load()
    Q = _check_pack(ids, min_s, row_nbits, row_bit_off, tau_s)
    n_esc = _check_escapes(esc_idx, esc_vals)
    ids, min_s, tau_s = ids.contiguous(), min_s.contiguous(), tau_s.contiguous()
    row_nbits, row_bit_off = row_nbits.contiguous(), row_bit_off.contiguous()
    with torch.cuda.device(ids.device):
        out = torch.empty((Q, int(P)), dtype=dtype, device=ids.device)
        st = _lib.stream_of(ids)
        _lib._check(lib.qvb8_decode(_lib.ptr(ids), ids.numel(), _lib.ptr(min_s), _lib.ptr(tau_s), _lib.ptr(row_nbits),
                                    _lib.ptr(row_bit_off), Q, int(P), code, _lib.ptr(out), st), lib)
        if n_esc:
            ei, ev = esc_idx.contiguous(), esc_vals.contiguous()
            _lib._check(lib.qvb8_scatter_escapes(_lib.ptr(out), code, out.numel(), _lib.ptr(ei), _lib.ptr(ev), n_esc, st), lib)
    return out


def decode(ids, min_s, row_nbits, row_bit_off, P, tau_s, esc_idx, esc_vals):
    """Dense (Q, P) fp16 weight: fp16(fma(id, tau_s, min_s)), escapes written over it."""
    return _decode_to(_lib.F16, torch.float16, ids, min_s, row_nbits, row_bit_off, P, tau_s, esc_idx, esc_vals)


def decode_bf16(ids, min_s, row_nbits, row_bit_off, P, tau_s, esc_idx, esc_vals):
    """Dense (Q, P) bf16 weight, the band value rounded once to bf16."""
    return _decode_to(_lib.BF16, torch.bfloat16, ids, min_s, row_nbits, row_bit_off, P, tau_s, esc_idx, esc_vals)


def decode_f32(ids, min_s, row_nbits, row_bit_off, P, tau_s, esc_idx, esc_vals):
    """Dense (Q, P) fp32 band values (what the GEMV multiplies), escapes exact."""
    return _decode_to(_lib.F32, torch.float32, ids, min_s, row_nbits, row_bit_off, P, tau_s, esc_idx, esc_vals)


def lookup_rows(rows, ids, min_s, row_nbits, row_bit_off, P, tau_s, esc_idx, esc_vals, out_dtype=torch.float32):
    """(n, P) rows `rows` of the table in `out_dtype`: min_s + id * tau_s in two fp32 roundings, then the rows'
    escapes written over it -- QVBandEmbeddingV8._decode_rows plus the escape loop of its forward
    (formats/qvb8/embedding.py:92-152) as one launch.  A row number outside the table gives a row of NaN."""
    lib = _lib.load()
    Q = _check_pack(ids, min_s, row_nbits, row_bit_off, tau_s)
    n_esc = _check_escapes(esc_idx, esc_vals)
    _lib.require_cuda(rows)
    if rows.dtype != torch.int64:
        raise RuntimeError("rows must be int64")
    rows = rows.reshape(-1).contiguous()
    ids, min_s, tau_s = ids.contiguous(), min_s.contiguous(), tau_s.contiguous()
    row_nbits, row_bit_off = row_nbits.contiguous(), row_bit_off.contiguous()
    code = _lib.dtype_code(out_dtype)
    with torch.cuda.device(ids.device):
        out = torch.empty((rows.numel(), int(P)), dtype=out_dtype, device=ids.device)
        ei = esc_idx.contiguous() if n_esc else None
        ev = esc_vals.contiguous() if n_esc else None
        _lib._check(lib.qvb8_lookup_rows(_lib.ptr(rows), rows.numel(), _lib.ptr(ids), ids.numel(), _lib.ptr(min_s),
                                         _lib.ptr(tau_s), _lib.ptr(row_nbits), _lib.ptr(row_bit_off), Q, int(P),
                                         _lib.ptr(ei), _lib.ptr(ev), n_esc, code, _lib.ptr(out), _lib.stream_of(ids)), lib)
    return out


def certify(restored: torch.Tensor, original: torch.Tensor, tau: float):
    """(max |restored - original|, number of elements not strictly under tau), computed
    on the GPU.  One host read of 8 bytes."""
    lib = _lib.load()
    _lib.require_cuda(restored, original)
    if restored.numel() != original.numel():
        raise RuntimeError("certify: tensors differ in size")
    a, b = restored.contiguous(), original.contiguous()
    with torch.cuda.device(a.device):
        res = torch.empty(2, dtype=torch.int32, device=a.device)
        _lib._check(lib.qvb8_certify(_lib.ptr(a), _lib.dtype_code(a.dtype), _lib.ptr(b), _lib.dtype_code(b.dtype),
                                     a.numel(), float(tau), res.data_ptr(), _lib.stream_of(a)), lib)
    host = res.cpu()
    return float(host[:1].view(torch.float32)[0]), int(host[1]) & 0xFFFFFFFF


def saturating_half(X: torch.Tensor) -> torch.Tensor:
    """Activations as fp16, clamped to +-65504 (NaN kept).  fp16 input is returned as is."""
    if X.dtype == torch.float16:
        return X.contiguous()
    lib = _lib.load()
    _lib.require_cuda(X)
    Xc = X.contiguous()
    if Xc.dtype not in (torch.float32, torch.bfloat16):
        Xc = Xc.float()
    with torch.cuda.device(Xc.device):
        out = torch.empty(Xc.shape, dtype=torch.float16, device=Xc.device)
        _lib._check(lib.qvb8_sat_half(_lib.ptr(Xc), _lib.dtype_code(Xc.dtype), Xc.numel(), _lib.ptr(out),
                                      _lib.stream_of(Xc)), lib)
    return out


def gemv_multi(X, ids, min_s, row_nbits, row_bit_off, P, tau_s, esc_idx, esc_vals):
    """(M, P) x packed (Q, P) -> fp32 (M, Q), 1 <= M <= 8: one pass over the packed ids."""
    lib = _lib.load()
    Q = _check_pack(ids, min_s, row_nbits, row_bit_off, tau_s)
    n_esc = _check_escapes(esc_idx, esc_vals)
    _lib.require_cuda(X)
    if X.dim() != 2 or X.shape[1] != int(P):
        raise RuntimeError(f"X must be (M, {int(P)})")
    M = X.shape[0]
    if not 1 <= M <= 8:
        raise RuntimeError(f"qvb8 GEMV-multi: M={M} is outside the instantiated range 1..8; callers above "
                           f"this (forward) route M>8 to the small-M GEMM")
    Xc = X.contiguous()
    if Xc.dtype not in (torch.float32, torch.float16, torch.bfloat16):
        Xc = Xc.float()
    ids, min_s, tau_s = ids.contiguous(), min_s.contiguous(), tau_s.contiguous()
    row_nbits, row_bit_off = row_nbits.contiguous(), row_bit_off.contiguous()
    with torch.cuda.device(Xc.device):
        Y = torch.empty((M, Q), dtype=torch.float32, device=Xc.device)
        ei = esc_idx.contiguous() if n_esc else None
        ev = esc_vals.contiguous() if n_esc else None
        _lib._check(lib.qvb8_gemv(_lib.ptr(Xc), _lib.dtype_code(Xc.dtype), M, _lib.ptr(ids), ids.numel(),
                                  _lib.ptr(min_s), _lib.ptr(tau_s), _lib.ptr(row_nbits), _lib.ptr(row_bit_off),
                                  Q, int(P), _lib.ptr(ei), _lib.ptr(ev), n_esc, _lib.ptr(Y), None, 0,
                                  _lib.stream_of(Xc)), lib)
    return Y


def gemv(X, ids, min_s, row_nbits, row_bit_off, P, tau_s, esc_idx, esc_vals):
    """M = 1 entry: X holds P fp16 values; returns fp32 (1, Q)."""
    if X.dtype != torch.float16:
        raise RuntimeError("X must be fp16")
    if X.numel() != int(P):
        raise RuntimeError("X length must equal P")
    return gemv_multi(X.reshape(1, int(P)), ids, min_s, row_nbits, row_bit_off, P, tau_s, esc_idx, esc_vals)


MMA_MAX_M = 48
MMA_GEMM_MAX_M = 256          # with a row layout (rows stored in width order, widths 4..8): the workgroup-tiled kernel
MMA_SATURATE_X = 1
MMA_Y_F16, MMA_Y_BF16 = 2, 4                      # qvb8_mma_flags: results stored as fp16 / bf16
MMA_PLANES = 8                                    # qvb8_mma_flags: the pack has rows stored in planes


def mma_prepare(row_nbits, row_bit_off, tau_s, min_s, P, ids_bytes, perm=None):
    """Row records (int64 tensor of qvb8_mma_rowinfo_bytes(Q) bytes) for mma_tiles: built once per weight."""
    lib = _lib.load()
    _lib.require_cuda(row_nbits, row_bit_off, tau_s, min_s)
    Q = row_nbits.numel()
    row_nbits, row_bit_off = row_nbits.contiguous(), row_bit_off.contiguous()
    tau_s, min_s = tau_s.contiguous(), min_s.contiguous()
    if perm is not None and perm.numel():
        if perm.dtype != torch.int32 or perm.numel() != Q or not perm.is_cuda:
            raise RuntimeError("qvb8 mma-multi: perm must be an int32 GPU tensor of length Q (or empty)")
        perm = perm.contiguous()
    else:
        perm = None
    with torch.cuda.device(row_nbits.device):
        out = torch.empty(lib.qvb8_mma_rowinfo_bytes(Q) // 8, dtype=torch.int64, device=row_nbits.device)
        _lib._check(lib.qvb8_mma_prepare(_lib.ptr(row_nbits), _lib.ptr(row_bit_off), _lib.ptr(tau_s), _lib.ptr(min_s),
                                         _lib.ptr(perm), Q, int(P),
                                         int(ids_bytes), _lib.ptr(out), _lib.stream_of(row_nbits)), lib)
    return out


PLANE_FLAG = 1 << 62          # bit offset words: the row is stored in planes (bits 0..47 its tile, bits 48..51 its row there)


def rows_in_planes(row_bit_off) -> bool:
    """Whether any row of the pack is stored in planes (one host read)."""
    return bool(((row_bit_off >> 62) & 1).any()) if row_bit_off.numel() else False


def _plane_index(P: int, w: int, device):
    """For one 16-row tile of width w: (dword index in planes, dword index with the rows back to back) of every dword."""
    rows = torch.arange(16, device=device).view(16, 1, 1)
    cg = torch.arange(P // 32, device=device).view(1, -1, 1)
    d = torch.arange(w, device=device).view(1, 1, -1)
    native = rows * (P // 32 * w) + cg * w + d
    lane = rows + 16 * (cg % 4)
    step_dw = (cg // 4) * (64 * w)
    planes = torch.where(d < 4, step_dw + lane * 4 + d, step_dw + 256 + lane * (w - 4) + (d - 4))
    return planes.reshape(-1), native.reshape(-1)


def rows_back_to_back(ids, row_nbits, row_bit_off, P):
    """Undoes the planes: (ids, row_bit_off) with every row of the pack stored back to back again (the bytes of each
    tile permuted back in place, plain bit offsets).  The arguments themselves when no row is stored in planes."""
    if not rows_in_planes(row_bit_off):
        return ids, row_bit_off
    P = int(P)
    flagged = (row_bit_off >> 62) & 1 == 1
    tile_bit = row_bit_off & ((1 << 48) - 1)
    r_in_tile = (row_bit_off >> 48) & 15
    nb = row_nbits.to(torch.int64)
    new_off = torch.where(flagged, tile_bit + r_in_tile * P * nb, row_bit_off)
    out = ids.clone()
    src32, dst32 = ids[: ids.numel() // 4 * 4].view(torch.int32), out[: ids.numel() // 4 * 4].view(torch.int32)
    for w in torch.unique(nb[flagged]).tolist():
        to_planes, to_native = _plane_index(P, int(w), ids.device)
        tile_dw0 = torch.unique(tile_bit[flagged & (nb == w)]) // 32       # a subset of the rows may not hold a tile's first
        for k in range(0, tile_dw0.numel(), 256):                          # bounded index tensors
            base = tile_dw0[k:k + 256, None]
            dst32[(base + to_native[None, :]).reshape(-1)] = src32[(base + to_planes[None, :]).reshape(-1)]
    return out, new_off


def tile_uniform_widths(row_nbits, tile_rows=16, lo=4, hi=8):
    """Per-row widths that make every tile of `tile_rows` consecutive rows (in row order) one width: each row of a tile
    whose widths all lie in lo..hi gets the tile's largest width; other rows keep theirs.  None when nothing changes."""
    Q = row_nbits.numel()
    whole = Q // tile_rows * tile_rows
    if whole == 0:
        return None
    nb = row_nbits[:whole].to(torch.int64).view(-1, tile_rows)
    top, low = nb.amax(1, keepdim=True), nb.amin(1, keepdim=True)
    target = torch.where((low >= lo) & (top <= hi), top.expand_as(nb), nb).reshape(-1)
    if bool((target == row_nbits[:whole]).all()):
        return None
    out = row_nbits.clone()
    out[:whole] = target.to(row_nbits.dtype)
    return out


def repack_rows(ids, row_nbits, row_bit_off, P, new_nbits, chunk_rows=256):
    """The rows stored again back to back, in row order from byte 0, row q in fields of new_nbits[q] >= row_nbits[q] bits:
    the ids, and with them every value of the weight, are unchanged.  Returns (ids, row_bit_off); None when P % 8 != 0."""
    P = int(P)
    if P % 8 != 0:
        return None
    ids, row_bit_off = rows_back_to_back(ids, row_nbits, row_bit_off, P)
    old, new = row_nbits.to(torch.int64), new_nbits.to(torch.int64)
    if bool((new < old).any()):
        raise RuntimeError("repack_rows: a row cannot be stored in fewer bits than it has")
    row_bits = new * P
    new_off = torch.cumsum(row_bits, 0) - row_bits
    total = int(row_bits.sum().item()) // 8
    out = torch.zeros(total + 8, dtype=torch.uint8, device=ids.device)
    dev = ids.device
    cols = torch.arange(P, device=dev, dtype=torch.int64)
    for w0, w1 in torch.unique(torch.stack([old, new], 1), dim=0).tolist():          # one host read, at load
        rows = torch.nonzero((old == w0) & (new == w1)).reshape(-1)
        nbytes = P * w1 // 8
        span = torch.arange(nbytes, device=dev, dtype=torch.int64)
        for k in range(0, rows.numel(), chunk_rows):
            r = rows[k:k + chunk_rows]
            src, dst = row_bit_off[r], new_off[r] >> 3
            if w0 == w1 and bool((src % 8 == 0).all()):
                out[(dst[:, None] + span[None, :]).reshape(-1)] = ids[((src >> 3)[:, None] + span[None, :]).reshape(-1)]
                continue
            pos = src[:, None] + cols[None, :] * w0
            byte, sh = pos >> 3, pos & 7
            word = ids[byte].to(torch.int64) | (ids[byte + 1].to(torch.int64) << 8) | (ids[byte + 2].to(torch.int64) << 16)
            val = ((word >> sh) & ((1 << w0) - 1)).to(torch.int32)
            bits = ((val[:, :, None] >> torch.arange(w1, device=dev, dtype=torch.int32)) & 1).reshape(r.numel(), -1, 8)
            packed = (bits << torch.arange(8, device=dev, dtype=torch.int32)).sum(2).to(torch.uint8)
            out[(dst[:, None] + span[None, :]).reshape(-1)] = packed.reshape(-1)
    return out, new_off


def widen_rows_to_whole_tiles(ids, row_nbits, row_bit_off, P, tile_rows=16, top=8):
    """Stores a few rows with more bits than they need so that, sorted by width, every run of one width is a whole number
    of 16-row tiles: of each width (ascending) the last `count % 16` rows move up to the next width present (up to
    `top`).  A row's ids, tau_s and min_s stay what they are -- only the field its ids are stored in gets wider, so
    every value of the weight is unchanged -- and at most 15 rows per width grow by a bit or two each.  Returns
    (ids, row_nbits, row_bit_off) with the widened rows appended to a copy of `ids`, or None when nothing moves."""
    P = int(P)
    ids, row_bit_off = rows_back_to_back(ids, row_nbits, row_bit_off, P)
    nb = row_nbits.to(torch.int64)
    widths, counts = torch.unique(nb, return_counts=True)
    widths, counts = widths.tolist(), counts.tolist()                      # one host read, at load
    moves = []                                                             # (rows, from width, to width)
    carried = None                                                         # rows moved up into the class at hand
    for k, (w, n) in enumerate(zip(widths, counts)):
        rows = torch.nonzero(nb == w).reshape(-1)
        members = [(rows, w)] if carried is None else [(rows, w)] + carried
        total = n + (0 if carried is None else sum(int(r.numel()) for r, _ in carried))
        carried = None
        spill = total % tile_rows
        if k + 1 == len(widths) or widths[k + 1] > top or spill == 0:
            continue
        up, out = widths[k + 1], []
        for r, w0 in reversed(members):                                    # rows that came from below move on first
            take = min(spill, int(r.numel()))
            if take:
                out.append((r[int(r.numel()) - take:], w0))
                spill -= take
        carried = out
        for r, w0 in out:
            moves.append((r, w0, up))
    # a row moved twice is listed twice: its last move counts
    final = {}
    for r, w0, up in moves:
        for q in r.tolist():
            final[q] = (final[q][0] if q in final else w0, up)
    if not final:
        return None
    new_nb, new_off = row_nbits.clone(), row_bit_off.clone()
    base = (ids.numel() - 8 + 15) // 16 * 16                               # the pad bytes of the old end are reused
    parts, at = [], base
    cols = torch.arange(P, device=ids.device, dtype=torch.int64)
    for q, (w0, up) in sorted(final.items()):
        pos = row_bit_off[q] + cols * w0
        byte, sh = pos >> 3, pos & 7
        word = ids[byte].to(torch.int64) | (ids[byte + 1].to(torch.int64) << 8) | (ids[byte + 2].to(torch.int64) << 16)
        val = (word >> sh) & ((1 << w0) - 1)
        bits = ((val[:, None] >> torch.arange(up, device=ids.device)) & 1).reshape(-1, 8)
        parts.append((bits << torch.arange(8, device=ids.device)).sum(1).to(torch.uint8))
        new_nb[q], new_off[q] = up, at * 8
        at += P * up // 8
    out_ids = torch.zeros(at + 8, dtype=torch.uint8, device=ids.device)
    out_ids[: ids.numel() - 8] = ids[: ids.numel() - 8]
    out_ids[base:at] = torch.cat(parts)
    return out_ids, new_nb, new_off


def sort_rows_by_width(ids, row_nbits, row_bit_off, P, perm, planes=False):
    """Copies the rows of a pack into `perm` order (rows of one width back to back, from byte 0), once, at load: returns
    (ids_sorted, row_bit_off_sorted, layout) -- the new ids buffer, the new per-row bit offsets (still indexed by row) and
    the _lib.MmaLayout that lets mma_tiles compute row addresses instead of reading them.  None when the pack cannot be
    laid out that way (P % 128 != 0, rows that do not start on 16-byte boundaries, more than 3 distinct widths).
    `planes`: every whole 16-row tile (positions 16 t .. 16 t + 15) that lies inside one run of a width 4..8 is stored in
    planes -- the same bytes, permuted inside the tile so that each request of the matrix-core kernels is one contiguous
    run -- and its rows' offsets carry PLANE_FLAG (every kernel of the library reads such rows; callers pass
    mma_tiles(planes=True)).  A pack that already has rows in planes is read as if they were back to back."""
    _lib.require_cuda(ids, row_nbits, row_bit_off, perm)
    Q, P = row_nbits.numel(), int(P)
    if Q == 0 or P % 128 != 0:
        return None
    ids, row_bit_off = rows_back_to_back(ids, row_nbits, row_bit_off, P)
    if bool((row_bit_off % 128 != 0).any()):
        return None
    nb_sorted = row_nbits[perm.long()].to(torch.int64)
    widths, counts = torch.unique_consecutive(nb_sorted, return_counts=True)
    widths, counts = widths.tolist(), counts.tolist()                      # one host read, at load
    if len(widths) > _lib.MMA_MAX_CLASSES or sorted(set(widths)) != widths:
        return None
    row_bits = nb_sorted * P
    new_off_sorted = torch.cumsum(row_bits, 0) - row_bits                  # rows back to back in the new order
    total_bytes = int(row_bits.sum().item()) // 8
    out = torch.zeros(total_bytes + 8, dtype=torch.uint8, device=ids.device)
    src16 = ids[: (ids.numel() // 16) * 16].view(-1, 16)
    dst16 = out[:total_bytes].view(-1, 16)
    src_off = row_bit_off[perm.long()]
    layout = _lib.MmaLayout()
    layout.n_classes = len(widths)
    pos = 0
    for c, (w, n) in enumerate(zip(widths, counts)):
        layout.first_pos[c], layout.nbits[c] = pos, int(w)
        blocks = P * w // 128                                              # 16-byte blocks per row
        ar = torch.arange(blocks, device=ids.device)
        for r0 in range(pos, pos + n, 4096):                               # bounded index tensors
            r1 = min(pos + n, r0 + 4096)
            s_idx = (src_off[r0:r1, None] // 128 + ar[None, :]).reshape(-1)
            d_idx = (new_off_sorted[r0:r1, None] // 128 + ar[None, :]).reshape(-1)
            if int(s_idx.max().item()) >= src16.shape[0]:
                return None
            dst16[d_idx] = src16[s_idx]
        pos += n
    layout.first_pos[len(widths)] = Q
    if planes:
        src32 = out[:total_bytes].view(torch.int32)
        dst = out.clone()
        dst32 = dst[:total_bytes].view(torch.int32)
        pos = 0
        for w, n in zip(widths, counts):
            t_first, t_end = -(-pos // 16) * 16, (pos + n) // 16 * 16
            if 4 <= w <= 8 and t_end > t_first:
                to_planes, to_native = _plane_index(P, w, ids.device)
                tile_dw0 = new_off_sorted[t_first:t_end:16] // 32          # first dword of each whole tile
                for k in range(0, tile_dw0.numel(), 256):                  # bounded index tensors
                    base = tile_dw0[k:k + 256, None]
                    dst32[(base + to_planes[None, :]).reshape(-1)] = src32[(base + to_native[None, :]).reshape(-1)]
                inside = torch.arange(t_first, t_end, device=ids.device)
                new_off_sorted[inside] = (new_off_sorted[inside - inside % 16]) | ((inside % 16) << 48) | PLANE_FLAG
            pos += n
        out = dst
    new_off = torch.empty_like(row_bit_off)
    new_off[perm.long()] = new_off_sorted
    return out, new_off, layout


def mma_tiles(X, ids, min_s, row_nbits, row_bit_off, P, tau_s, esc_idx, esc_vals, perm=None, saturate=True,
              rowinfo=None, layout=None, out_dtype=None, planes=False):
    """Matrix-core path for P % 128 == 0: X (fp16 or bf16) times the fp32 band value, fp32 (M, Q).  1 <= M <= 48 always;
    49 <= M <= 256 (the workgroup-tiled decode + GEMM kernel) when `layout` is given and its widths are 4..8.
    `perm` (int32, position -> row) groups rows of equal width into tiles; `rowinfo` = mma_prepare(...) for the
    same perm (built on the fly when absent); `layout` = the third result of sort_rows_by_width for a pack whose rows were
    copied into that order (needs `rowinfo`).  `saturate` (bf16 X only): X is narrowed like saturating_half while it
    is loaded and the product runs on fp16 operands, as every fp16 path of the reference does; without it bf16 X is
    multiplied as it is on bf16 operands.  `out_dtype` torch.float16 / torch.bfloat16: the kernels store the results
    rounded to that type (the same values as casting the fp32 result; only for a weight without escapes).  `planes`:
    the pack has rows stored in planes (sort_rows_by_width(planes=True))."""
    lib = _lib.load()
    Q = _check_pack(ids, min_s, row_nbits, row_bit_off, tau_s)
    n_esc = _check_escapes(esc_idx, esc_vals)
    _lib.require_cuda(X)
    if X.dim() != 2 or X.shape[1] != int(P):
        raise RuntimeError(f"X must be (M, {int(P)})")
    M = X.shape[0]
    if not 1 <= M <= (MMA_GEMM_MAX_M if layout is not None else MMA_MAX_M):
        raise RuntimeError(f"qvb8 mma-multi: M={M} outside 1..{MMA_GEMM_MAX_M if layout is not None else MMA_MAX_M}")
    if int(P) % 128 != 0 or ids.data_ptr() % 4 != 0:
        raise RuntimeError("qvb8 mma-multi: needs P%128==0 and 4-byte-aligned ids")
    if X.dtype not in (torch.float16, torch.bfloat16):
        raise RuntimeError("qvb8 mma-multi: X must be fp16 or bf16")
    if perm is not None and perm.numel():
        if perm.dtype != torch.int32 or perm.numel() != Q or not perm.is_cuda:
            raise RuntimeError("qvb8 mma-multi: perm must be an int32 GPU tensor of length Q (or empty)")
        perm = perm.contiguous()
    else:
        perm = None
    if rowinfo is not None and (rowinfo.dtype != torch.int64 or rowinfo.numel() * 8 != lib.qvb8_mma_rowinfo_bytes(Q)
                                or not rowinfo.is_cuda):
        raise RuntimeError("qvb8 mma-multi: rowinfo must be the int64 GPU tensor mma_prepare returned")
    Xc = X.contiguous()
    ids, min_s, tau_s = ids.contiguous(), min_s.contiguous(), tau_s.contiguous()
    row_nbits, row_bit_off = row_nbits.contiguous(), row_bit_off.contiguous()
    with torch.cuda.device(Xc.device):
        if out_dtype in (torch.float16, torch.bfloat16):
            if n_esc:
                raise RuntimeError("qvb8 mma-multi: fp16 / bf16 results need a weight without escapes")
            y_flag = MMA_Y_F16 if out_dtype == torch.float16 else MMA_Y_BF16
        elif out_dtype in (None, torch.float32):
            out_dtype, y_flag = torch.float32, 0
        else:
            raise RuntimeError("qvb8 mma-multi: results are fp32, fp16 or bf16")
        Y = torch.empty((M, Q), dtype=out_dtype, device=Xc.device)
        ei = esc_idx.contiguous() if n_esc else None
        ev = esc_vals.contiguous() if n_esc else None
        need = lib.qvb8_mma_workspace_bytes(M, Q, int(P))          # row records when none are passed; more for the tiled kernel
        ws = None if (rowinfo is not None and need <= lib.qvb8_mma_rowinfo_bytes(Q)) else \
            torch.empty((need + 7) // 8, dtype=torch.int64, device=Xc.device)
        _lib._check(lib.qvb8_mma(_lib.ptr(Xc), _lib.dtype_code(Xc.dtype), M, _lib.ptr(ids), ids.numel(),
                                 _lib.ptr(min_s), _lib.ptr(tau_s), _lib.ptr(row_nbits), _lib.ptr(row_bit_off),
                                 Q, int(P), _lib.ptr(ei), _lib.ptr(ev), n_esc, _lib.ptr(perm),
                                 None if rowinfo is None else rowinfo.contiguous().data_ptr(),
                                 None if layout is None else ctypes.addressof(layout),
                                 (MMA_SATURATE_X if saturate else 0) | y_flag | (MMA_PLANES if planes else 0), _lib.ptr(Y),
                                 None if ws is None else ws.data_ptr(), 0 if ws is None else ws.numel() * 8,
                                 _lib.stream_of(Xc)), lib)
    return Y


MLP_MAX_ROWS = 4                                  # QVB8_MLP_MAX_ROWS
MLP_SILU_GATED, MLP_TEST_STALE_TAG = 0, 0x100     # qvb8_mlp_act


MLP_H_AT = 128                                    # byte of the workspace at which H starts (state words and description before it)


def mlp_init(gu_ids, gu_rowinfo, gu_layout, dn_ids, dn_rowinfo, dn_layout, hidden, inter, out_features):
    """(workspace, plan) of mlp_fused for one MLP (qvb8_mlp_init): the gate+up pack in unit order and the down pack, both
    stored in planes with a row layout (formats/qvb8/mlp.py builds them).  The workspace is the library's from here on -- it
    carries the block's description and the hand-over's state from call to call, so calls that share it must not overlap;
    word 1 (int32 view) is the sticky error word.  Raises RuntimeError for packs the kernel cannot read."""
    lib = _lib.load()
    _lib.require_cuda(gu_ids, gu_rowinfo, dn_ids, dn_rowinfo)
    plan = _lib.MlpPlan()
    with torch.cuda.device(gu_ids.device):
        ws = torch.empty(int(lib.qvb8_mlp_workspace_bytes(int(inter))), dtype=torch.uint8, device=gu_ids.device)
        _lib._check(lib.qvb8_mlp_init(int(hidden), int(inter), int(out_features),
                                      gu_ids.data_ptr(), gu_ids.numel(), gu_rowinfo.data_ptr(), ctypes.addressof(gu_layout),
                                      dn_ids.data_ptr(), dn_ids.numel(), dn_rowinfo.data_ptr(), ctypes.addressof(dn_layout),
                                      ws.data_ptr(), ws.numel(), ctypes.addressof(plan), _lib.stream_of(gu_ids)), lib)
    return ws, plan


def mlp_fused(X, workspace, plan, mid_dtype=None, out_dtype=None, act=MLP_SILU_GATED):
    """down(silu(gate(x)) * up(x)) for 1..4 rows of X as ONE launch (qvb8_mlp), on the (workspace, plan) of mlp_init.
    `mid_dtype`: the type the values between the products are rounded to (X's by default), `out_dtype` the result's (X's by
    default).  Raises RuntimeError for what the kernel does not cover: callers fall back to the separate products."""
    lib = _lib.load()
    _lib.require_cuda(X, workspace)
    if X.dim() != 2 or X.shape[1] != int(plan.hidden):
        raise RuntimeError(f"X must be (M, {int(plan.hidden)})")
    if X.dtype not in (torch.float16, torch.bfloat16):
        raise RuntimeError("qvb8 mlp: X must be fp16 or bf16")
    M = X.shape[0]
    mid_dtype = X.dtype if mid_dtype is None else mid_dtype
    out_dtype = X.dtype if out_dtype is None else out_dtype
    Xc = X.contiguous()
    with torch.cuda.device(Xc.device):
        Y = torch.empty((M, int(plan.out_features)), dtype=out_dtype, device=Xc.device)
        _lib._check(lib.qvb8_mlp(ctypes.addressof(plan), _lib.ptr(Xc), _lib.dtype_code(Xc.dtype), M, int(act), _lib.dtype_code(mid_dtype),
                                 Y.data_ptr(), _lib.dtype_code(out_dtype), workspace.data_ptr(), _lib.stream_of(Xc)), lib)
    return Y


def mma_multi(X, ids, min_s, row_nbits, row_bit_off, P, tau_s, esc_idx, esc_vals, perm, tile_nb,
              bf16=False, esc_starts=None, general=-1):
    """QVB8 tensor-core multi-row product (M <= 48), bf16.  fp16 mode (bf16=False): X saturated to fp16;
    bf16 mode: X as bf16, not saturated.  `tile_nb`, `esc_starts` and `general` are launch hints of the
    reference's kernels and are not needed here."""
    del tile_nb, esc_starts, general
    if bf16:
        Xk = X if X.dtype == torch.bfloat16 else X.to(torch.bfloat16)
        return mma_tiles(Xk, ids, min_s, row_nbits, row_bit_off, P, tau_s, esc_idx, esc_vals, perm, saturate=False)
    Xk = X if X.dtype in (torch.float16, torch.bfloat16) else saturating_half(X)
    return mma_tiles(Xk, ids, min_s, row_nbits, row_bit_off, P, tau_s, esc_idx, esc_vals, perm, saturate=True)


def _forward(X, ids, min_s, row_nbits, row_bit_off, P, tau_s, esc_idx, esc_vals, out_half):
    M = 1 if X.dim() == 1 else X.shape[0]
    if M <= 8:
        return gemv_multi(X.reshape(M, int(P)), ids, min_s, row_nbits, row_bit_off, P, tau_s, esc_idx, esc_vals)
    # M > 8: certified fp16 weight once, then a library GEMM with fp32 accumulate
    W = decode(ids, min_s, row_nbits, row_bit_off, P, tau_s, esc_idx, esc_vals)
    Xh = saturating_half(X)
    if out_half:
        return torch.mm(Xh, W.t())
    return torch.mm(Xh, W.t(), out_dtype=torch.float32)


def forward(X, ids, min_s, row_nbits, row_bit_off, P, tau_s, esc_idx, esc_vals):
    """Any M.  M <= 8: fused GEMV, fp32 (M, Q).  M > 8: fp16 restore + GEMM, fp32 result."""
    return _forward(X, ids, min_s, row_nbits, row_bit_off, P, tau_s, esc_idx, esc_vals, False)


def forward_half(X, ids, min_s, row_nbits, row_bit_off, P, tau_s, esc_idx, esc_vals):
    """As forward, but the M > 8 GEMM stores fp16."""
    return _forward(X, ids, min_s, row_nbits, row_bit_off, P, tau_s, esc_idx, esc_vals, True)


def _moe(act, X, idx, w, up_ids, up_min, up_tau, up_nb, up_off, Qup, Pup, dn_ids, dn_min, dn_tau, dn_nb, dn_off, Qdn, Pdn):
    lib = _lib.load()
    _lib.require_cuda(X, idx, w, up_ids, up_min, up_tau, up_nb, up_off, dn_ids, dn_min, dn_tau, dn_nb, dn_off)
    if X.dim() != 2 or X.shape[1] != int(Pup):
        raise RuntimeError("moe: bad X")
    if idx.dtype != torch.int64 or w.dtype != torch.float32 or idx.dim() != 2 or tuple(w.shape) != tuple(idx.shape):
        raise RuntimeError("moe: idx must be int64 and w float32, both (tokens, topk)")
    if idx.shape[0] != X.shape[0]:
        raise RuntimeError("moe: one routing row per token")
    if up_min.dim() != 2 or up_min.shape[1] != int(Qup) or dn_min.dim() != 2 or dn_min.shape[1] != int(Qdn) \
            or dn_min.shape[0] != up_min.shape[0]:
        raise RuntimeError("moe: row metadata must be (experts, Q)")
    for t, dt in ((up_ids, torch.uint8), (up_nb, torch.uint8), (up_off, torch.int64), (up_min, torch.float32),
                  (up_tau, torch.float32), (dn_ids, torch.uint8), (dn_nb, torch.uint8), (dn_off, torch.int64),
                  (dn_min, torch.float32), (dn_tau, torch.float32)):
        if t.dtype != dt:
            raise RuntimeError(f"moe: expected {dt}, got {t.dtype}")
    T, k, E = X.shape[0], idx.shape[1], up_min.shape[0]
    Xc, idxc, wc = X.contiguous(), idx.contiguous(), w.contiguous()
    tens = [t.contiguous() for t in (up_ids, up_min, up_tau, up_nb, up_off, dn_ids, dn_min, dn_tau, dn_nb, dn_off)]
    with torch.cuda.device(Xc.device):
        out = torch.empty((T, int(Qdn)), dtype=Xc.dtype, device=Xc.device)
        if T == 0:
            return out
        nws = lib.qvb8_moe_workspace_bytes(T, k, E, int(Qup), int(Pdn), int(Qdn))
        ws = torch.empty(max(nws, 16), dtype=torch.uint8, device=Xc.device)
        u, d = tens[:5], tens[5:]
        _lib._check(lib.qvb8_moe_experts(
            _lib.ptr(Xc), _lib.dtype_code(Xc.dtype), T, _lib.ptr(idxc), _lib.ptr(wc), k, E,
            _lib.ptr(u[0]), u[0].numel(), _lib.ptr(u[1]), _lib.ptr(u[2]), _lib.ptr(u[3]), _lib.ptr(u[4]), int(Qup), int(Pup),
            _lib.ptr(d[0]), d[0].numel(), _lib.ptr(d[1]), _lib.ptr(d[2]), _lib.ptr(d[3]), _lib.ptr(d[4]), int(Qdn), int(Pdn),
            act, _lib.ptr(out), _lib.dtype_code(out.dtype), _lib.ptr(ws), ws.numel(), _lib.stream_of(Xc)), lib)
    return out


MOE_UP_REGULAR, MOE_DOWN_REGULAR = 0x100, 0x200      # qvb8_moe_act flags: one width per stack, rows at regular places


def stack_is_regular(nbits, bit_off, P) -> bool:
    """Whether a stack's (experts, Q) tables are what QVB8_MOE_*_REGULAR states: one width, row q of expert e at
    bit_off[0, 0] + e * (bit_off[1, 0] - bit_off[0, 0]) + q * P * width (one host read)."""
    E, Q = nbits.shape
    w = nbits.reshape(-1)[0].to(torch.int64)
    base = bit_off.reshape(-1)[0]
    stride = bit_off[1, 0] - base if E > 1 else torch.zeros((), dtype=torch.int64, device=bit_off.device)
    want = base + torch.arange(E, device=bit_off.device).view(E, 1) * stride + torch.arange(Q, device=bit_off.device).view(1, Q) * (int(P) * w)
    return bool((nbits == nbits.reshape(-1)[0]).all() & (bit_off == want).all())


def moe_experts(X, idx, w, gu_ids, gu_min, gu_tau, gu_nb, gu_off, Qgu, Pgu, dn_ids, dn_min, dn_tau, dn_nb, dn_off, Qdn, Pdn,
                regular=(False, False)):
    """Routed gated-SiLU expert stack on the stacked layout (reference: qvb8_cuda.cu:937-992); returns (tokens, Qdn)
    in X's dtype.  `regular` = (up, down): the caller states that the stack is regular (stack_is_regular)."""
    act = 0 | (MOE_UP_REGULAR if regular[0] else 0) | (MOE_DOWN_REGULAR if regular[1] else 0)
    return _moe(act, X, idx, w, gu_ids, gu_min, gu_tau, gu_nb, gu_off, Qgu, Pgu, dn_ids, dn_min, dn_tau, dn_nb, dn_off, Qdn, Pdn)


def moe_experts_relu2(X, idx, w, up_ids, up_min, up_tau, up_nb, up_off, Qup, Pup, dn_ids, dn_min, dn_tau, dn_nb, dn_off, Qdn, Pdn,
                      regular=(False, False)):
    """Non-gated expert stack with H = relu(up(x))^2 (reference: qvb8_cuda.cu:1002-1055)."""
    return _moe(1 | (MOE_UP_REGULAR if regular[0] else 0) | (MOE_DOWN_REGULAR if regular[1] else 0), X, idx, w, up_ids, up_min, up_tau, up_nb, up_off, Qup, Pup, dn_ids, dn_min, dn_tau, dn_nb, dn_off, Qdn, Pdn)
