"""The CPU oracle of the banded-KV attention against what the mathematics fixes (the reference holds no vector for it)."""
import numpy as np
import pytest

from oracle import kv_attn_oracle as A
from oracle import qvb8_oracle as O


def make_layout(seed, seg_len, Hkv, D, bits=6, tau=0.0, spread=1.0, block_n=32):
    """Synthetic cache: per segment and head a banded K and V, ids in one (n, Hkv, D) buffer, centre-form constants."""
    rng = np.random.default_rng(seed)
    n, nseg = sum(seg_len), len(seg_len)
    ki = np.zeros((n, Hkv, D), np.int64)
    vi = np.zeros_like(ki)
    P = [np.zeros((nseg, Hkv, D), np.float32) for _ in range(4)]
    kc = np.zeros((nseg, Hkv), np.float32)
    vc = np.zeros_like(kc)
    pos = 0
    for si, sl in enumerate(seg_len):
        for which, ids_t, mid, st, C in (("k", ki, P[0], P[1], kc), ("v", vi, P[2], P[3], vc)):
            x = (rng.normal(0, spread, (Hkv, sl, D)) * rng.uniform(0.2, 3.0, (Hkv, 1, D))).astype(np.float32)
            for h, (ids, mn, step, b) in enumerate(A.band_kv(x, bits, tau)):
                ids_t[pos:pos + sl, h] = ids
                mid[si, h], st[si, h], C[si, h] = A.centre_form(mn, step, b)
        pos += sl
    ts, tl, tseg = A.tile_table(seg_len, block_n)
    return dict(ki=ki, vi=vi, kmid=P[0], kstep=P[1], vmid=P[2], vstep=P[3], kc=kc, vc=vc, ts=ts, tl=tl, tseg=tseg)


def test_band_kv_nearest_grid_point_and_certificate():
    rng = np.random.default_rng(0)
    x = rng.normal(0, 2, (3, 50, 16)).astype(np.float32)
    x[1, :, 3] = 0.75                                      # a constant channel: range 0, every id 0
    for ids, mn, step, b in A.band_kv(x, 6):
        assert b == 6 and ids.min() >= 0 and ids.max() <= 63
    heads = A.band_kv(x, 6)
    for h, (ids, mn, step, b) in enumerate(heads):
        recon = mn.astype(np.float64) + ids * step.astype(np.float64)
        assert np.all(np.abs(recon - x[h]) <= step.astype(np.float64) / 2 * (1 + 1e-5) + 1e-7)
    assert np.all(heads[1][0][:, 3] == 0)
    # certified: the width rises until the rounded decode is within tau
    tau = 0.02
    for h, (ids, mn, step, b) in enumerate(A.band_kv(x, 4, tau, "bf16")):
        assert b > 4
        recon = A._round_dtype(A.decode_kv(ids, mn, step), "bf16")
        assert np.abs(recon - A._round_dtype(x[h], "fp32")).max() <= tau


def test_restore_tile_closed_form_and_codec_agreement():
    rng = np.random.default_rng(1)
    ids = rng.integers(0, 64, (40, 32))
    mn = rng.normal(0, 1, 32).astype(np.float32)
    step = rng.uniform(1e-3, 0.1, 32).astype(np.float32)
    mid, st, c = A.centre_form(mn, step, 6)
    assert c == 31.5
    got = A.restore_tile(ids, mid, st, c)
    exact = mid.astype(np.float64) + st.astype(np.float64) * (ids - 31.5)
    want = exact.astype(np.float32).astype(np.float16).astype(np.float32)    # the sum is exact in float64 here
    assert np.array_equal(got, want)
    # the centre form is the codec's min + id * step up to fp32 rounding of the shifted constant
    assert np.allclose(got, A.decode_kv(ids, mn, step).astype(np.float16).astype(np.float32), rtol=2e-3, atol=1e-6)


def test_two_keys_by_hand():
    """q . k equal for both keys -> p = (1, 1): the result is the mean of the two values, m = the common score, l = 2."""
    D = 128
    ki = np.zeros((2, 1, D), np.int64); ki[:, 0, 0] = 3
    vi = np.zeros((2, 1, D), np.int64); vi[0, 0, :] = 2; vi[1, 0, :] = 6
    one = np.ones((1, 1, D), np.float32)
    lay = dict(ki=ki, vi=vi, kmid=0 * one, kstep=one, vmid=0 * one, vstep=0.5 * one, kc=np.zeros((1, 1), np.float32),
               vc=np.zeros((1, 1), np.float32), ts=np.array([0], np.int32), tl=np.array([2], np.int32), tseg=np.array([0], np.int32))
    q = np.zeros((1, 1, D), np.float16); q[0, 0, 0] = 0.5
    o, m, l = A.fwd_split(q, lay["ki"], lay["vi"], lay["kmid"], lay["kstep"], lay["vmid"], lay["vstep"], lay["kc"], lay["vc"],
                          lay["ts"], lay["tl"], lay["tseg"], q_pos0=5, tps=1, scale=2.0, G=1)
    assert m[0, 0, 0] == 3.0 and l[0, 0, 0] == 2.0 and np.all(o[0, 0, 0] == 4.0)        # 0.5 * 3 * 2; values 1 and 3 summed
    out, lse = A.combine(o, m, l, 1, 1)
    assert np.all(out == 2.0) and abs(lse[0, 0] - (3.0 + np.log(2.0))) < 1e-6
    # causal: a query at position 0 sees the first key only
    o, m, l = A.fwd_split(q, lay["ki"], lay["vi"], lay["kmid"], lay["kstep"], lay["vmid"], lay["vstep"], lay["kc"], lay["vc"],
                          lay["ts"], lay["tl"], lay["tseg"], q_pos0=0, tps=1, scale=2.0, G=1)
    assert l[0, 0, 0] == 1.0 and np.all(o[0, 0, 0] == 1.0)


@pytest.mark.parametrize("D,Hkv,G,MQ,seg_len,q_pos0", [
    (128, 2, 4, 1, [70, 33], 102), (128, 1, 2, 5, [40, 9, 64], 60), (256, 2, 1, 3, [31, 1, 32], 200)])
def test_splits_against_the_textbook(D, Hkv, G, MQ, seg_len, q_pos0):
    lay = make_layout(D + MQ, seg_len, Hkv, D)
    rng = np.random.default_rng(7)
    q = rng.normal(0, 1, (MQ, Hkv * G, D)).astype(np.float32)
    scale = D ** -0.5
    ref, ref_lse = A.dense_reference(np.clip(q * np.float32(scale), -65504, 65504).astype(np.float16).astype(np.float64), 1.0, lay, q_pos0)
    for tps in (1, 2, 100):
        out, lse = A.attend(q, scale, lay, q_pos0, tps)
        assert out.shape == (MQ, Hkv * G, D)
        vis = np.isfinite(ref_lse)
        assert np.array_equal(np.isfinite(lse), vis)
        assert np.allclose(lse[vis], ref_lse[vis], atol=2e-3)
        bound = 1.5e-3 * np.abs(ref).max(axis=-1, keepdims=True) + 1e-6          # p is rounded to fp16: 2^-11 relative
        assert np.all(np.abs(out - ref) <= bound)


def test_row_maximum_is_exact_and_unseen_rows_are_empty():
    lay = make_layout(3, [64], 1, 128)
    rng = np.random.default_rng(2)
    q = rng.normal(0, 1, (4, 2, 128)).astype(np.float16)
    # queries at positions -2 .. 1: the first two see nothing
    o, m, l = A.fwd_split(q, lay["ki"], lay["vi"], lay["kmid"], lay["kstep"], lay["vmid"], lay["vstep"], lay["kc"], lay["vc"],
                          lay["ts"], lay["tl"], lay["tseg"], q_pos0=-2, tps=1, scale=0.25, G=2)
    assert np.all(np.isneginf(m[:, 0, :4])) and np.all(l[:, 0, :4] == 0) and np.all(o[:, 0, :4] == 0)
    assert np.all(np.isneginf(m[1])) and np.all(l[1] == 0)                      # the second tile starts at key 32
    K = A.restore_tile(lay["ki"][:2, 0], lay["kmid"][0, 0], lay["kstep"][0, 0], lay["kc"][0, 0]).astype(np.float64)
    for r in range(4, 8):
        vis = 1 if r < 6 else 2
        s = (K[:vis] @ q[r // 2, r % 2].astype(np.float64)).astype(np.float32) * np.float32(0.25)
        assert m[0, 0, r] == s.max()
    out, lse = A.combine(o, m, l, 4, 2)
    assert np.all(out[:2] == 0) and np.all(np.isneginf(lse[:2])) and np.all(np.isfinite(lse[2:]))
