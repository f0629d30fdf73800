"""QVB8R codec, host side: slot tables (what a reader derives at load) and the writer that turns band ids into the
rANS streams the kernels walk.

Stream format (reference: src/qv_band/formats/qvb8r/codec.py:4-21, backends/cuda_qvb8r/qvb8r_cpu.cpp:53-100 and the
walk in qvb8r_cuda.cu:51-75): rows are sorted by class; a tile is a run of consecutive sorted rows of one class and
carries 32 interleaved rANS states (lane j codes the columns congruent to j mod 32, row-major, 32 columns per step).
States are 64-bit in [2^32, 2^64), probabilities 12-bit (a class's frequencies sum to 4096, each <= 1024), the stream is
32-bit words.  The decoder takes two symbols per lane, then every lane whose state fell below 2^32 takes the next
word of the tile's stream, in lane order.  symbol = id - drow[row] (rows are coded centred on one symbol).

The reference ships no writer policy (which rows share a class, how frequencies are quantised, how many rows make a
tile): those choices here are this build's own; any stream the walk decodes back to the ids conforms.
"""
from __future__ import annotations

import numpy as np

from qvb8_amd.common.errors import QVB8RFormatError

PB = 12
MQ = 1 << PB
MAX_ID = 2048
MAX_FREQ = 1024
CENTRE = 256
ROWS_PER_TILE_DIV = 4096
LANES = 32


def slot_tables(F: np.ndarray) -> np.ndarray:
    """(K, N) frequencies -> (K, 4096) packed slot entries: symbol | (slot - cum[symbol]) << 11 | (freq - 1) << 22
    (codec.py:10-20)."""
    F = np.asarray(F).astype(np.int64)
    K, N = F.shape
    if np.any(F.sum(1) != MQ) or np.any(F < 0) or np.any(F > MAX_FREQ) or N > MAX_ID:
        raise QVB8RFormatError("qvb8r: each class needs frequencies in 0..1024 that sum to 4096 over at most 2048 symbols")
    C = np.concatenate([np.zeros((K, 1), np.int64), np.cumsum(F, 1)[:, :-1]], 1)
    tab = np.zeros((K, MQ), np.uint32)
    for k in range(K):
        s = np.repeat(np.arange(N), F[k])
        d = np.arange(MQ) - C[k][s]
        tab[k] = (s | (d << 11) | ((F[k][s] - 1) << 22)).astype(np.uint32)
    return tab


def quantise_frequencies(counts: np.ndarray) -> np.ndarray:
    """Histogram (N,) -> frequencies (N,) int64 that sum to 4096, every occurring symbol >= 1, none above 1024."""
    c = np.asarray(counts, np.float64)
    N = len(c)
    tot = c.sum()
    if tot <= 0:
        c = np.ones(N)
        tot = float(N)
    f = np.floor(c * MQ / tot).astype(np.int64)
    f[(c > 0) & (f == 0)] = 1
    f = np.minimum(f, MAX_FREQ)
    diff = MQ - int(f.sum())
    order = np.argsort(-c, kind="stable")
    while diff != 0:
        moved = False
        for i in order:
            if diff > 0 and f[i] < MAX_FREQ:
                f[i] += 1; diff -= 1; moved = True
            elif diff < 0 and f[i] > 1:
                f[i] -= 1; diff += 1; moved = True
            if diff == 0:
                break
        if not moved:
            raise QVB8RFormatError("qvb8r: cannot fit the frequencies (too many distinct symbols for 4096 slots)")
    return f


def _encode_group(sym: np.ndarray, r0: np.ndarray, nr: int, f: np.ndarray, c: np.ndarray):
    """rANS-encode tiles that all have `nr` rows.  sym (R, P) int16 symbols in sorted row order, r0 (n,) first rows,
    f / c (n, N) the tiles' class frequencies and exclusive cumulative sums.  Returns (list of word arrays, states (n, 32))."""
    n = len(r0)
    P = sym.shape[1]
    S = P // LANES
    x = np.full((n, LANES), 1 << 32, np.uint64)
    cap = nr * P * PB // 32 + 2 * LANES + 8
    buf = np.zeros((n, cap), np.uint32)
    cur = np.full(n, cap, np.int64)                      # words are written from the end: the decoder reads them in reverse
    rows = np.arange(n)[:, None]
    lane_rank_above = np.arange(LANES - 1, -1, -1)        # lane l is pushed after the lanes above it
    for p in range(nr * S // 2 - 1, -1, -1):
        a, b = 2 * p, 2 * p + 1
        s1 = sym[r0 + a // S, (a % S) * LANES:(a % S) * LANES + LANES].astype(np.int64)     # (n, 32)
        s2 = sym[r0 + b // S, (b % S) * LANES:(b % S) * LANES + LANES].astype(np.int64)
        f1 = np.take_along_axis(f, s1, 1).astype(np.uint64); c1 = np.take_along_axis(c, s1, 1).astype(np.uint64)
        f2 = np.take_along_axis(f, s2, 1).astype(np.uint64); c2 = np.take_along_axis(c, s2, 1).astype(np.uint64)
        if np.any(f1 == 0) or np.any(f2 == 0):
            raise QVB8RFormatError("qvb8r: a symbol with zero frequency occurs in its class")
        emit = x >= ((f1 * f2) << np.uint64(40))
        if emit.any():
            # push order inside a pair: lane 31 first ... lane 0 last; the finished buffer is reversed, so the word
            # pushed first sits at the highest address of the pair's run
            er = emit[:, ::-1]                                        # column k <-> lane 31 - k
            rank = np.cumsum(er, 1) - 1                               # push index within the pair
            cnt = er.sum(1)
            pos = (cur[:, None] - 1 - rank)[:, ::-1]                  # back to lane order
            tt, ll = np.nonzero(emit)
            buf[tt, pos[tt, ll]] = (x[tt, ll] & np.uint64(0xFFFFFFFF)).astype(np.uint32)
            cur -= cnt
            x = np.where(emit, x >> np.uint64(32), x)
        x = ((x // f2) << np.uint64(PB)) + x % f2 + c2
        x = ((x // f1) << np.uint64(PB)) + x % f1 + c1
    del rows, lane_rank_above
    return [buf[t, cur[t]:].copy() for t in range(n)], x


def encode_ids(ids: np.ndarray, *, n_classes: int | None = None, rows_per_tile: int | None = None) -> dict:
    """Band ids (Q, P) -> the arrays of a .qvb8r file: perm, freq, tiles, tile_off, states, words, drow, plus T, K, N.
    P must be a multiple of 128 (a symbol pair never straddles a row)."""
    ids = np.asarray(ids)
    if ids.ndim != 2 or ids.shape[1] % 128 != 0 or ids.shape[0] == 0:
        raise QVB8RFormatError("qvb8r: ids must be (Q, P) with P % 128 == 0 and Q > 0")
    Q, P = ids.shape
    # row statistics and the symbols, a block of rows at a time (the temporaries of a whole 200-million-id tensor at once
    # would be gigabytes)
    RB = max(1, (1 << 22) // P)
    lo, hi, med = np.zeros(Q, np.int64), np.zeros(Q, np.int64), np.zeros(Q, np.int64)
    for r in range(0, Q, RB):
        blk = ids[r:r + RB].astype(np.int32)
        lo[r:r + RB], hi[r:r + RB] = blk.min(1), blk.max(1)
        med[r:r + RB] = np.median(blk, 1).astype(np.int64)
    drow = med - CENTRE
    drow = np.where(lo - drow < 0, lo, drow)              # symbols must not be negative
    if np.any(hi - drow >= MAX_ID) or np.any(np.abs(drow) > 32767):
        raise QVB8RFormatError("qvb8r: a row's ids span more than 2048 symbols: keep this tensor as QVB8")
    sym_orig = np.empty((Q, P), np.int16)
    spread = np.zeros(Q, np.float64)
    for r in range(0, Q, RB):
        blk = ids[r:r + RB].astype(np.int32) - drow[r:r + RB, None].astype(np.int32)
        sym_orig[r:r + RB] = blk
        spread[r:r + RB] = blk.astype(np.float64).std(1)
    N = int((hi - drow).max()) + 1
    # classes: rows of similar spread share a frequency table
    K = n_classes if n_classes is not None else (1 if Q < 64 else min(8, max(1, Q // 256)))
    K = max(1, min(K, Q))
    order = np.argsort(spread, kind="stable")
    cls_of_sorted = (np.arange(Q) * K) // Q               # equal-size groups along the sorted spread
    perm = order.astype(np.int32)                         # sorted row -> original row
    sym = sym_orig[order]
    del sym_orig
    F = np.zeros((K, N), np.int64)
    for k in range(K):
        rows_k = np.nonzero(cls_of_sorted == k)[0]
        hist = np.zeros(N, np.int64)
        for r in range(0, len(rows_k), RB):
            hist += np.bincount(sym[rows_k[r]:rows_k[min(r + RB, len(rows_k)) - 1] + 1].reshape(-1), minlength=N)
        F[k] = quantise_frequencies(hist)
    C = np.concatenate([np.zeros((K, 1), np.int64), np.cumsum(F, 1)[:, :-1]], 1)
    T = rows_per_tile if rows_per_tile is not None else max(1, ROWS_PER_TILE_DIV // P)
    tiles = []
    for k in range(K):
        idx = np.nonzero(cls_of_sorted == k)[0]
        for r in range(int(idx[0]), int(idx[-1]) + 1, T):
            tiles.append((k, r, min(T, int(idx[-1]) + 1 - r)))
    tiles = np.array(tiles, np.int32).reshape(-1, 3)
    nt = len(tiles)
    words_of = [None] * nt
    states = np.zeros((nt, LANES), np.uint64)
    for nr in np.unique(tiles[:, 2]):
        sel = np.nonzero(tiles[:, 2] == nr)[0]
        for i0 in range(0, len(sel), 1024):               # bounded scratch: 1024 tiles at a time
            part = sel[i0:i0 + 1024]
            w, x = _encode_group(sym, tiles[part, 1].astype(np.int64), int(nr), F[tiles[part, 0]], C[tiles[part, 0]])
            for t, ww in zip(part, w):
                words_of[t] = ww
            states[part] = x
    tile_off = np.zeros(nt + 1, np.int64)
    tile_off[1:] = np.cumsum([len(w) for w in words_of])
    if tile_off[-1] >= 1 << 32:
        raise QVB8RFormatError("qvb8r: stream longer than 2^32 words")
    words = np.concatenate(words_of).astype(np.uint32) if nt else np.zeros(0, np.uint32)
    return dict(perm=perm, freq=F.astype(np.uint16), tiles=tiles, tile_off=tile_off.astype(np.uint32), states=states,
                words=words, drow=drow.astype(np.int16), T=int(tiles[:, 2].max()), K=int(K), N=int(N))
