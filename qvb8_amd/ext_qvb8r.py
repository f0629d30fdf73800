"""QVB8R kernels behind the names and positional argument orders of the reference's `qvb8r_cuda` extension
(src/qv_band/formats/qvb8r/backends/cuda_qvb8r/qvb8r_cuda.cu:446-456), on libqvb8_amd.so.

"core" = (words, off, states, tiles, blocks, tab, perm, mn, ts, drow): words u32 (an int32 view is fine) WITH the
2048-word zero pad, off i64 [nt + 1], states u64 (or an int64 view) [nt, 32], tiles i64 [nt, 3], blocks i32 [nb, 3] (runs
of <= 8 tiles of one class), tab u32 [K, 4096], perm i32 [Q], mn / ts f32 [Q], drow i32 [Q] -- all on one GPU.
`T` (most rows in any tile, the file's header field) may be passed to avoid a host read of `tiles`.
"""
from __future__ import annotations

import ctypes

import torch

from . import _lib

MAX_M = 48
_OUT = {0: torch.float16, 1: torch.bfloat16, 2: torch.float32}        # the reference's out_dtype codes of decode()
_ABI_DT = {torch.float32: 0, torch.float16: 1, torch.bfloat16: 2, torch.int16: 3}


def _core(words, off, states, tiles, blocks, tab, perm, mn, ts, drow, P):
    ts_ = (words, off, states, tiles, blocks, tab, perm, mn, ts, drow)
    _lib.require_cuda(*ts_)
    for t in ts_:
        if not t.is_contiguous():
            raise RuntimeError("qvb8r: inputs must be contiguous GPU tensors")
    want = ((words, 4), (off, 8), (states, 8), (tiles, 8), (blocks, 4), (tab, 4), (perm, 4), (mn, 4), (ts, 4), (drow, 4))
    for t, size in want:
        if t.element_size() != size:
            raise RuntimeError("qvb8r: a core tensor has the wrong element size")
    Q = mn.numel()
    nt = tiles.shape[0] if tiles.dim() == 2 else tiles.numel() // 3
    if off.numel() != nt + 1 or states.numel() != nt * 32 or perm.numel() != Q or ts.numel() != Q or drow.numel() != Q \
            or tab.numel() % 4096 != 0 or blocks.numel() % 3 != 0:
        raise RuntimeError("qvb8r: core tensors disagree in size")
    c = _lib.RCore(words.data_ptr(), words.numel(), off.data_ptr(), states.data_ptr(), tiles.data_ptr(), nt,
                   blocks.data_ptr(), blocks.numel() // 3, tab.data_ptr(), tab.numel() // 4096, perm.data_ptr(),
                   mn.data_ptr(), ts.data_ptr(), drow.data_ptr(), Q, int(P))
    return c, Q, nt


def _rows_bound(tiles, T):
    if T is not None:
        return int(T)
    return int(tiles.reshape(-1, 3)[:, 2].max()) if tiles.numel() else 1


def _product(X, core, T):
    lib = _lib.load()
    _lib.require_cuda(X)
    if X.dim() == 1:
        X = X.reshape(1, -1)
    M, P = X.shape
    if not 1 <= M <= MAX_M:
        raise RuntimeError(f"qvb8r: M={M} outside 1..{MAX_M}")
    if X.dtype not in (torch.float32, torch.float16, torch.bfloat16):
        raise RuntimeError("qvb8r: X must be fp32, fp16 or bf16")
    c, Q, _ = _core(*core, P)
    Xc = X.contiguous()
    with torch.cuda.device(Xc.device):
        Y = torch.empty((M, Q), dtype=torch.float32, device=Xc.device)
        ws = torch.empty(max(16, lib.qvb8r_gemv_workspace_bytes(M, P)), dtype=torch.uint8, device=Xc.device)
        _lib._check(lib.qvb8r_gemv(Xc.data_ptr(), _lib.dtype_code(Xc.dtype), M, ctypes.byref(c), _rows_bound(core[3], T),
                                   Y.data_ptr(), ws.data_ptr(), ws.numel(), _lib.stream_of(Xc)), lib)
    return Y


def gemv(X, words, off, states, tiles, blocks, tab, perm, mn, ts, drow, T=None):
    """M = 1: X (P,) -> Y (Q,) fp32 (qvb8r_cuda.cu:346-357)."""
    return _product(X.reshape(1, -1), (words, off, states, tiles, blocks, tab, perm, mn, ts, drow), T).reshape(-1)


def multi(X, words, off, states, tiles, blocks, tab, perm, mn, ts, drow, T=None):
    """M = 2..8 (here up to 48): X (M, P) fp32, fp16 or bf16 -> Y (M, Q) fp32 (qvb8r_cuda.cu:359-383)."""
    return _product(X, (words, off, states, tiles, blocks, tab, perm, mn, ts, drow), T)


def tc(X, words, off, states, tiles, blocks, tab, perm, mn, ts, drow, T):
    """M = 9..16 (here up to 48; qvb8r_cuda.cu:385-396).  The same kernel as multi: the fp32 band value is multiplied, not its fp16
    rounding, so the escape correction that goes with it is the fp32 one (esc_delta)."""
    return _product(X, (words, off, states, tiles, blocks, tab, perm, mn, ts, drow), T)


def decode(words, off, states, tiles, blocks, tab, perm, mn, ts, drow, P, out_dtype, b0, nb, row_base, nrows, T=None):
    """Dense rows of blocks [b0, b0 + nb): out_dtype 0 fp16 / 1 bf16 / 2 fp32 (the reference's codes).  row_base < 0:
    the whole (Q, P) weight in original row order; else a compact (nrows, P) chunk of sorted rows from row_base on
    (qvb8r_cuda.cu:398-424).  Escapes are not applied."""
    lib = _lib.load()
    c, Q, _ = _core(words, off, states, tiles, blocks, tab, perm, mn, ts, drow, P)
    dt = _OUT[int(out_dtype)]
    rows = Q if row_base < 0 else int(nrows)
    with torch.cuda.device(mn.device):
        W = torch.empty((rows, int(P)), dtype=dt, device=mn.device)
        _lib._check(lib.qvb8r_decode(ctypes.byref(c), _rows_bound(tiles, T), _ABI_DT[dt], int(b0), int(nb), int(row_base),
                                     W.data_ptr(), rows, _lib.stream_of(mn)), lib)
    return W


def decode_blocks(block_list, words, off, states, tiles, blocks, tab, perm, mn, ts, drow, P, out_dtype=3, T=None):
    """Rows of the listed blocks (int32 GPU tensor of block numbers) in fixed slots: row r of tile h of list entry j at
    row (j * 8 + h) * T + r of the result, (len(list) * 8 * T, P).  out_dtype 0 fp16 / 1 bf16 / 2 fp32 band values (escapes
    not applied), 3 the ids as int16.  Slots without a row are left as allocated (not initialised)."""
    lib = _lib.load()
    _lib.require_cuda(block_list)
    if block_list.dtype != torch.int32 or not block_list.is_contiguous():
        raise RuntimeError("qvb8r: block_list must be a contiguous int32 GPU tensor")
    c, Q, _ = _core(words, off, states, tiles, blocks, tab, perm, mn, ts, drow, P)
    Tb = _rows_bound(tiles, T)
    dt = torch.int16 if int(out_dtype) == 3 else _OUT[int(out_dtype)]
    n = block_list.numel()
    with torch.cuda.device(mn.device):
        W = torch.empty((n * 8 * Tb, int(P)), dtype=dt, device=mn.device)
        _lib._check(lib.qvb8r_decode_blocks(ctypes.byref(c), Tb, _ABI_DT[dt], block_list.data_ptr(), n, W.data_ptr(), W.shape[0],
                                            _lib.stream_of(mn)), lib)
    return W


def ids(P, words, off, states, tiles, blocks, tab, perm, mn, ts, drow, T=None):
    """The band ids (Q, P) int16 in original row order (qvb8r_cuda.cu:426-444)."""
    lib = _lib.load()
    c, Q, _ = _core(words, off, states, tiles, blocks, tab, perm, mn, ts, drow, P)
    with torch.cuda.device(mn.device):
        W = torch.empty((Q, int(P)), dtype=torch.int16, device=mn.device)
        _lib._check(lib.qvb8r_decode(ctypes.byref(c), _rows_bound(tiles, T), 3, 0, c.n_blocks, -1, W.data_ptr(), Q,
                                     _lib.stream_of(mn)), lib)
    return W


def fix_escapes(X, uq, ptr, ec, ed, Y):
    """Y[m, uq[u]] += sum of X[m, ec[e]] * ed[e] over the escapes of output uq[u]; mutates Y (qvb8r_cuda.cu:311-331)."""
    lib = _lib.load()
    _lib.require_cuda(X, uq, ptr, ec, ed, Y)
    if Y.dtype != torch.float32 or not Y.is_contiguous() or Y.dim() != 2:
        raise RuntimeError("qvb8r fix_escapes: Y must be a contiguous fp32 (M, Q) tensor")
    Xc = X.contiguous()
    if Xc.dim() != 2 or Xc.shape[0] != Y.shape[0]:
        raise RuntimeError("qvb8r fix_escapes: X must be (M, P) with Y's M")
    U = uq.numel()
    if ptr.numel() != U + 1 or ec.numel() != ed.numel() or uq.dtype != torch.int64 or ptr.dtype != torch.int64 \
            or ec.dtype != torch.int64 or ed.dtype != torch.float32:
        raise RuntimeError("qvb8r fix_escapes: bad escape tables")
    if U:
        _lib._check(lib.qvb8r_fix_escapes(Xc.data_ptr(), _lib.dtype_code(Xc.dtype), Xc.shape[0], uq.contiguous().data_ptr(),
                                          ptr.contiguous().data_ptr(), ec.contiguous().data_ptr(), ed.contiguous().data_ptr(),
                                          U, Y.data_ptr(), Y.shape[1], Xc.shape[1], _lib.stream_of(Xc)), lib)
    return Y
