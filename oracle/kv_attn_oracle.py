"""CPU oracle for attention over the banded KV cache.  TEST INFRASTRUCTURE ONLY.

Plain numpy restatement of what the reference's kernel and its caller compute; nothing in the shipped package may
import it (only tests/, the smoke check and the CPU-baseline leg of the benchmark do).  Paths are relative to the
reference tree, src/qv_band/...

Pinning status (what fixes each function besides this file's own text; the reference holds no test or vector for it):
  band_kv / decode_kv      closed forms: the ids are the nearest grid points (|x - recon| <= step / 2 in float64),
                           the certificate |dtype(recon) - x| <= tau is re-measured, constant channels give id 0
  restore_tile             float64 closed form of mid + step * (id - c), rounded once to fp32 (libm fmaf via the
                           QVB8 oracle's fma32) and once to fp16 (numpy.float16); equals the codec's
                           min_s + id * tau_s to fp32 rounding
  fwd_split                a two-key known answer by hand; the textbook softmax(q k^T) v in float64 over the same
                           restored K / V (causal mask included) agrees with the combined splits within the fp16
                           rounding of the probabilities; m is the exact row maximum; a different split of the
                           tiles changes the result only by rounding; rows that see no key give m = -inf, l = 0
  combine                  log-sum-exp identity: any partition of the tiles gives the same normalised result
What no check can pin: whether the reference's binary contracts `mid + step * (id - c)` into one fused multiply-add
(nvcc does by default; assumed here) -- the two readings differ by one fp32 ulp before the rounding to fp16, which is far
inside the tolerance the parity tests state.
"""
from __future__ import annotations

import math

import numpy as np

from oracle.qvb8_oracle import fma32

STEP_FLOOR = 1e-12          # kv/codec.py:41
MAX_BITS = 16               # kv/codec.py:168


def _round_dtype(v: np.ndarray, dtype: str) -> np.ndarray:
    if dtype == "fp16":
        return v.astype(np.float16).astype(np.float32)
    if dtype == "bf16":
        import torch
        return torch.from_numpy(np.ascontiguousarray(v, np.float32)).to(torch.bfloat16).to(torch.float32).numpy()
    return v.astype(np.float32)


def band_kv(x: np.ndarray, bits: int, tau: float = 0.0, dtype: str = "bf16"):
    """(heads, seq, head_dim) -> per head (ids int64 (seq, head_dim), min_s, tau_s, bits)  (kv/codec.py:175-241):
    per-channel minimum and range over the sequence, step = range / (2^B - 1) floored, id = round((x - min) / step)
    clamped; B starts at max(bits, ceil(log2(range / 2 tau + 1))) per head and rises until the decode expression
    min + id * step, rounded to the storage dtype, is within tau of x."""
    x = np.nan_to_num(np.asarray(x, np.float32), nan=0.0, posinf=0.0, neginf=0.0)
    h = x.shape[0]
    mn = x.min(axis=1, keepdims=True)
    rng = x.max(axis=1, keepdims=True) - mn
    certify = tau > 0
    bvec = []
    for i in range(h):
        w = float(rng[i].max())
        need = max(bits, math.ceil(math.log2(w / (2.0 * tau) + 1.0))) if certify and w > 0 else bits
        bvec.append(min(max(need, bits), MAX_BITS))
    out = [None] * h
    for i in range(h):
        while True:
            L = np.float32((1 << bvec[i]) - 1)
            step = np.maximum(rng[i] / L, np.float32(STEP_FLOOR)).astype(np.float32)
            ids = np.minimum(np.maximum(np.rint((x[i] - mn[i]) / step), 0), L)
            if not certify:
                break
            recon = _round_dtype((mn[i] + ids * step).astype(np.float32), dtype)
            if float(np.abs(recon - x[i]).max()) <= tau:
                break
            if bvec[i] >= MAX_BITS:
                raise ValueError(f"head {i}: {MAX_BITS} bits cannot certify tau={tau}")
            bvec[i] += 1
        out[i] = (ids.astype(np.int64), mn[i, 0].copy(), step[0].copy(), bvec[i])
    return out


def decode_kv(ids, min_s, tau_s) -> np.ndarray:
    """min_s + id * tau_s in fp32, product and sum rounded separately (kv/codec.py:117-118)."""
    return (min_s.astype(np.float32) + ids.astype(np.float32) * tau_s.astype(np.float32)).astype(np.float32)


def centre_form(min_s, tau_s, bits: int):
    """(mid, step, c) of the attention layout: c = (2^B - 1) / 2, mid = min_s + tau_s * c  (kv/fused_attn.py:210-214)."""
    c = np.float32(((1 << bits) - 1) / 2.0)
    return (min_s.astype(np.float32) + tau_s.astype(np.float32) * c).astype(np.float32), tau_s.astype(np.float32), c


def restore_tile(ids, mid, step, c) -> np.ndarray:
    """fp16(fma(step, float(id) - c, mid)) widened to fp32  (kv/cuda_attn/qvattn_cuda.cu:46-47, 87-88)."""
    d = (ids.astype(np.float32) - np.float32(c)).astype(np.float32)          # exact: ids < 2^16, c a half-integer
    v = fma32(np.broadcast_to(step, d.shape), d, np.broadcast_to(mid, d.shape))
    return v.astype(np.float16).astype(np.float32)


def tile_table(seg_len, block_n: int = 32):
    """(first key, length, segment) of every tile; a tile never straddles a segment  (kv/fused_attn.py:171-178)."""
    ts, tl, tseg, pos = [], [], [], 0
    for si, sl in enumerate(seg_len):
        for a in range(0, sl, block_n):
            ts.append(pos + a)
            tl.append(min(block_n, sl - a))
            tseg.append(si)
        pos += sl
    return np.array(ts, np.int32), np.array(tl, np.int32), np.array(tseg, np.int32)


def fwd_split(q, ki, vi, kmid, kstep, vmid, vstep, kc, vc, ts, tl, tseg, q_pos0: int, tps: int, scale: float, G: int):
    """The kernel of kv/cuda_attn/qvattn_cuda.cu:97-255 for all kv heads, splits and rows.
    q (MQ, Hq, D) fp16 values; ki / vi (cap, Hkv, D) integer ids; constants (nseg, Hkv, D), kc / vc (nseg, Hkv).
    Returns o (S, Hkv, R, D), m, l (S, Hkv, R) in fp32, R = MQ * G."""
    q = np.asarray(q, np.float16).astype(np.float32)
    MQ, Hq, D = q.shape
    Hkv = ki.shape[1]
    R = MQ * G
    n_tiles = len(ts)
    S = max(1, -(-n_tiles // tps))
    o = np.zeros((S, Hkv, R, D), np.float32)
    m = np.full((S, Hkv, R), -np.inf, np.float32)
    l = np.zeros((S, Hkv, R), np.float32)
    rows = np.arange(R)
    qpos = q_pos0 + rows // G
    sc = np.float32(scale)
    for h in range(Hkv):
        qh = q[rows // G, h * G + rows % G]                              # (R, D)
        for sp in range(S):
            acc = np.zeros((R, D), np.float32)
            m_run = np.full(R, -np.inf, np.float32)
            l_run = np.zeros(R, np.float32)
            for t in range(sp * tps, min((sp + 1) * tps, n_tiles)):
                start, nlen, seg = int(ts[t]), int(tl[t]), int(tseg[t])
                k = restore_tile(ki[start:start + nlen, h], kmid[seg, h], kstep[seg, h], kc[seg, h])
                v = restore_tile(vi[start:start + nlen, h], vmid[seg, h], vstep[seg, h], vc[seg, h])
                s = (qh.astype(np.float64) @ k.astype(np.float64).T).astype(np.float32)      # fp16 operands, wide accumulate
                ok = (start + np.arange(nlen))[None, :] <= qpos[:, None]
                with np.errstate(invalid="ignore", over="ignore"):
                    sv = np.where(ok, s * sc, -np.inf).astype(np.float32)
                    mx = sv.max(axis=1) if nlen else np.full(R, -np.inf, np.float32)
                    m_new = np.maximum(m_run, mx)
                    m_safe = np.where(np.isinf(m_new) & (m_new < 0), np.float32(0), m_new)
                    p = np.where(np.isinf(sv) & (sv < 0), np.float32(0), np.exp(sv - m_safe[:, None], dtype=np.float32))
                    p = p.astype(np.float16).astype(np.float32)                              # rounded before sum and product
                    alpha = np.where(np.isinf(m_run) & (m_run < 0), np.float32(0),
                                     np.where(m_new == m_run, np.float32(1), np.exp(m_run - m_safe, dtype=np.float32)))
                l_run = (l_run * alpha + p.sum(axis=1, dtype=np.float32)).astype(np.float32)
                acc = (acc * alpha[:, None] + (p.astype(np.float64) @ v.astype(np.float64)).astype(np.float32)).astype(np.float32)
                m_run = m_new.astype(np.float32)
            o[sp, h], m[sp, h], l[sp, h] = acc, m_run, l_run
    return o, m, l


def combine(o, m, l, MQ: int, G: int):
    """Splits -> (out (MQ, Hq, D), lse (MQ, Hq))  (kv/fused_attn.py:302-316)."""
    S, Hkv, R, D = o.shape
    with np.errstate(invalid="ignore", divide="ignore"):
        if S == 1:
            lsum, mx_s = l[0], m[0]
            out = o[0] / np.maximum(lsum, np.float32(1e-30))[..., None]
            mx_s = np.where(np.isinf(mx_s), np.float32(0), mx_s)
        else:
            mx = m.max(axis=0)
            mx_s = np.where(np.isinf(mx), np.float32(0), mx)
            w = np.exp(m - mx_s, dtype=np.float32)
            lsum = (l * w).sum(axis=0, dtype=np.float32)
            out = (o * w[..., None]).sum(axis=0, dtype=np.float32) / np.maximum(lsum, np.float32(1e-30))[..., None]
        lse = np.where(lsum > 0, mx_s + np.log(np.maximum(lsum, np.float32(1e-30))), -np.inf).astype(np.float32)
    out = out.reshape(Hkv, MQ, G, D).transpose(1, 0, 2, 3).reshape(MQ, Hkv * G, D).astype(np.float32)
    lse = lse.reshape(Hkv, MQ, G).transpose(1, 0, 2).reshape(MQ, Hkv * G)
    return out, lse


def attend(q, scale: float, lay: dict, q_pos0: int, tps: int):
    """The caller of the kernel (kv/fused_attn.py:246-316, the branch that uses the compiled kernel): the softmax
    scale is folded into q in fp32, q saturates to fp16, the kernel runs with scale 1, the splits are combined."""
    qs = np.clip(np.asarray(q, np.float32) * np.float32(scale), -65504.0, 65504.0).astype(np.float16)
    G = qs.shape[1] // lay["ki"].shape[1]
    o, m, l = fwd_split(qs, lay["ki"], lay["vi"], lay["kmid"], lay["kstep"], lay["vmid"], lay["vstep"], lay["kc"], lay["vc"],
                        lay["ts"], lay["tl"], lay["tseg"], q_pos0, tps, 1.0, G)
    return combine(o, m, l, qs.shape[0], G)


def dense_reference(q, scale: float, lay: dict, q_pos0: int):
    """Textbook softmax(q k^T * scale) v in float64 over the restored (fp16-rounded) keys and values, key position <=
    query position: the referee for fwd_split + combine."""
    q = np.asarray(q, np.float64)
    MQ, Hq, D = q.shape
    Hkv = lay["ki"].shape[1]
    G = Hq // Hkv
    n = int(lay["ts"][-1] + lay["tl"][-1]) if len(lay["ts"]) else 0
    out = np.zeros((MQ, Hq, D))
    lse = np.full((MQ, Hq), -np.inf)
    K = np.zeros((n, Hkv, D))
    V = np.zeros((n, Hkv, D))
    for t in range(len(lay["ts"])):
        a, ln, seg = int(lay["ts"][t]), int(lay["tl"][t]), int(lay["tseg"][t])
        for h in range(Hkv):
            K[a:a + ln, h] = restore_tile(lay["ki"][a:a + ln, h], lay["kmid"][seg, h], lay["kstep"][seg, h], lay["kc"][seg, h])
            V[a:a + ln, h] = restore_tile(lay["vi"][a:a + ln, h], lay["vmid"][seg, h], lay["vstep"][seg, h], lay["vc"][seg, h])
    for tq in range(MQ):
        vis = min(n, q_pos0 + tq + 1)
        if vis <= 0:
            continue
        for hq in range(Hq):
            s = K[:vis, hq // G] @ q[tq, hq] * scale
            mx = s.max()
            p = np.exp(s - mx)
            out[tq, hq] = p @ V[:vis, hq // G] / p.sum()
            lse[tq, hq] = mx + np.log(p.sum())
    return out, lse
