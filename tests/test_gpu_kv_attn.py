"""GPU parity: attention over the banded KV cache (qvb8_attn_fwd through the C ABI, and `attend` above it) against the
CPU oracle's restatement of the reference's kernel and caller.

Floating point, so a tolerance -- stated where it is used: the kernel and the oracle restore the same fp16 keys and
values bit for bit; what differs is the order of the fp32 sums, the device's exp, and through them now and then the
fp16 rounding of a probability (one fp16 ulp = 2^-10 relative at most).  Bounds: 1e-3 relative on the softmax state,
1e-3 * max|v| on results, and 3e-4 in the relative root-mean-square."""
import numpy as np
import pytest
import torch

from oracle import kv_attn_oracle as A
from qvb8_amd.kv import codec as C
from qvb8_amd.kv import fused_attn as FA
from tests.test_oracle_kv_attn import make_layout

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def to_device(lay, wide=False, slack=0):
    """numpy layout -> device tensors; `slack` > 0 embeds the ids in a larger buffer (more capacity, more heads)."""
    n, hkv, d = lay["ki"].shape
    out = {}
    for name in ("ki", "vi"):
        a = lay[name]
        t = torch.from_numpy(a.astype(np.uint16).view(np.int16) if wide else a.astype(np.uint8))
        if slack:
            big = torch.zeros(n + slack, hkv + 1, d, dtype=t.dtype)
            big[:n, :hkv] = t
            out[name] = big.to(DEV)[:n, :hkv]
        else:
            out[name] = t.to(DEV)
    for name in ("kmid", "kstep", "vmid", "vstep", "kc", "vc", "ts", "tl", "tseg"):
        out[name] = torch.from_numpy(lay[name]).to(DEV)
    return out


def run_fwd(lay, dl, q16, q_pos0, tps, G):
    mq, hq, d = q16.shape
    hkv = lay["ki"].shape[1]
    S = max(1, -(-len(lay["ts"]) // tps))
    o = torch.full((S, hkv, mq * G, d), float("nan"), device=DEV)
    m = torch.full((S, hkv, mq * G), float("nan"), device=DEV)
    l = torch.full_like(m, float("nan"))
    FA.fwd(q16, dl["ki"], dl["vi"], dl["kmid"], dl["kstep"], dl["vmid"], dl["vstep"], dl["kc"], dl["vc"],
           dl["ts"], dl["tl"], dl["tseg"], o, m, l, q_pos0, tps, 1.0, G)
    return o.cpu().numpy(), m.cpu().numpy(), l.cpu().numpy()


def vmax(lay):
    return float(np.abs(lay["vmid"]).max() + (np.abs(lay["vstep"]) * (np.abs(lay["vc"]).max() + 1)).max())


def check_split_outputs(got, want, lay):
    (o, m, l), (o_r, m_r, l_r) = got, want
    assert np.array_equal(np.isneginf(m), np.isneginf(m_r)) and not np.isnan(m).any()
    fin = np.isfinite(m_r)
    assert np.all(np.abs(m[fin] - m_r[fin]) <= 1e-3 * np.abs(m_r[fin]) + 1e-3)
    assert np.all(np.abs(l - l_r) <= 1e-3 * l_r + 1e-6) and np.all(l[~fin] == 0)
    assert np.all(o[~fin] == 0) and not np.isnan(o).any()
    # a different running maximum rescales o and l together: compare the normalised pieces
    with np.errstate(invalid="ignore"):
        w = np.where(fin, np.exp(m_r - m), 1.0)
    assert np.all(np.abs(o * (1 / w)[..., None] - o_r) <= 1e-3 * vmax(lay) * l_r[..., None] + 1e-6)


CASES = [
    # D, Hkv, G, MQ, seg_len, q_pos0, bits, tps
    (128, 2, 4, 1, [70, 33], 102, 6, 2),
    (128, 1, 2, 5, [40, 9, 64], 60, 6, 1),
    (256, 2, 1, 3, [31, 1, 32], 200, 6, 3),
    (256, 4, 6, 1, [300], 299, 6, 4),                 # a decode step of a 24-head model
    (256, 1, 8, 2, [32, 32, 5], 68, 8, 100),
    (128, 2, 3, 12, [100], 50, 5, 2),                 # 36 rows: three row blocks, causal cut inside the tiles
    (128, 1, 1, 3, [64], -2, 6, 1),                   # the first queries see no key at all
    (256, 2, 2, 1, [1], 0, 6, 1),
    (256, 1, 6, 1, [500, 17], 516, 6, 7),             # splits of 7 tiles: both register sets and the odd last piece in use
    (128, 2, 4, 2, [333], 332, 7, 5),
    # more than 16 rows: a workgroup serves two or four blocks of 16 rows from one restored tile
    (256, 1, 6, 4, [90, 40], 126, 6, 2),              # 24 rows: two blocks, the second half empty
    (256, 2, 8, 5, [70], 65, 6, 1),                   # 40 rows: two workgroups of two blocks, causal cut inside
    (128, 1, 8, 3, [64, 3], 64, 6, 2),                # 24 rows, 128 channels
    (128, 2, 6, 11, [100], 95, 6, 3),                 # 66 rows: four blocks + a second workgroup with two rows
]


@pytest.mark.parametrize("D,Hkv,G,MQ,seg_len,q_pos0,bits,tps", CASES)
def test_fwd_matches_the_oracle(D, Hkv, G, MQ, seg_len, q_pos0, bits, tps):
    lay = make_layout(D + MQ + G, seg_len, Hkv, D, bits=bits)
    rng = np.random.default_rng(11)
    q = (rng.normal(0, 1, (MQ, Hkv * G, D)) * D ** -0.5).astype(np.float16)
    want = A.fwd_split(q, lay["ki"], lay["vi"], lay["kmid"], lay["kstep"], lay["vmid"], lay["vstep"], lay["kc"], lay["vc"],
                       lay["ts"], lay["tl"], lay["tseg"], q_pos0, tps, 1.0, G)
    for slack in (0, 7):
        dl = to_device(lay, slack=slack)
        got = run_fwd(lay, dl, torch.from_numpy(q).to(DEV), q_pos0, tps, G)
        check_split_outputs(got, want, lay)
        out, lse = A.combine(*got, MQ, G)
        ref, ref_lse = A.combine(*want, MQ, G)
        assert np.all(np.abs(out - ref) <= 1e-3 * vmax(lay) + 1e-6)
        if np.abs(ref).max() > 0:
            assert np.sqrt(((out - ref) ** 2).mean()) <= 3e-4 * np.sqrt((ref ** 2).mean())


def test_fwd_sixteen_bit_ids_and_strided_queries():
    D, Hkv, G, MQ = 128, 2, 2, 2
    lay = make_layout(5, [50, 20], Hkv, D, bits=11)
    assert lay["ki"].max() > 255
    rng = np.random.default_rng(3)
    qbig = torch.from_numpy((rng.normal(0, 1, (MQ, Hkv * G + 1, 2 * D)) * 0.1).astype(np.float16)).to(DEV)
    q = qbig[:, 1:, D:]                                   # strides of a larger tensor
    want = A.fwd_split(q.cpu().numpy(), lay["ki"], lay["vi"], lay["kmid"], lay["kstep"], lay["vmid"], lay["vstep"], lay["kc"],
                       lay["vc"], lay["ts"], lay["tl"], lay["tseg"], 69, 2, 1.0, G)
    got = run_fwd(lay, to_device(lay, wide=True), q, 69, 2, G)
    check_split_outputs(got, want, lay)
    # D = 256 with wide ids
    lay = make_layout(6, [40], 1, 256, bits=9)
    q = torch.from_numpy((rng.normal(0, 1, (1, 4, 256)) * 0.06).astype(np.float16)).to(DEV)
    want = A.fwd_split(q.cpu().numpy(), lay["ki"], lay["vi"], lay["kmid"], lay["kstep"], lay["vmid"], lay["vstep"], lay["kc"],
                       lay["vc"], lay["ts"], lay["tl"], lay["tseg"], 39, 1, 1.0, 4)
    check_split_outputs(run_fwd(lay, to_device(lay, wide=True), q, 39, 1, 4), want, lay)


def test_scale_argument_and_empty_cache():
    lay = make_layout(9, [45], 1, 128)
    rng = np.random.default_rng(4)
    q = rng.normal(0, 1, (1, 2, 128)).astype(np.float16)
    dl = to_device(lay)
    mq, g = 1, 2
    o = torch.empty(1, 1, 2, 128, device=DEV); m = torch.empty(1, 1, 2, device=DEV); l = torch.empty_like(m)
    FA.fwd(torch.from_numpy(q).to(DEV), dl["ki"], dl["vi"], dl["kmid"], dl["kstep"], dl["vmid"], dl["vstep"], dl["kc"], dl["vc"],
           dl["ts"], dl["tl"], dl["tseg"], o, m, l, 44, 2, 0.125, g)
    want = A.fwd_split(q, lay["ki"], lay["vi"], lay["kmid"], lay["kstep"], lay["vmid"], lay["vstep"], lay["kc"], lay["vc"],
                       lay["ts"], lay["tl"], lay["tseg"], 44, 2, 0.125, g)
    check_split_outputs((o.cpu().numpy(), m.cpu().numpy(), l.cpu().numpy()), want, lay)
    # no tiles at all: one empty split
    empty = torch.zeros(0, dtype=torch.int32, device=DEV)
    FA.fwd(torch.from_numpy(q).to(DEV), dl["ki"], dl["vi"], dl["kmid"], dl["kstep"], dl["vmid"], dl["vstep"], dl["kc"], dl["vc"],
           empty, empty, empty, o, m, l, 44, 1, 1.0, g)
    assert torch.isneginf(m).all() and (l == 0).all() and (o == 0).all()


def test_attend_from_banded_segments():
    """Codec -> layout -> attend, against the oracle's caller and against plain torch attention over the decoded cache."""
    torch.manual_seed(0)
    Hkv, G, D, MQ = 2, 4, 128, 3
    seg_len = [48, 80, 21]
    segs_k, segs_v = [], []
    for sl in seg_len:
        segs_k.append(C.band_kv_heads((torch.randn(Hkv, sl, D, device=DEV) * 2).to(torch.bfloat16), torch.bfloat16, 6, tau=0.1))
        segs_v.append(C.band_kv_heads(torch.randn(Hkv, sl, D, device=DEV).to(torch.bfloat16), torch.bfloat16, 6, tau=0.1))
    lay = FA.layout_from_segments(segs_k, segs_v, seg_len, DEV)
    assert lay is not None and lay.ki.dtype == torch.uint8 and lay.n_tiles == 2 + 3 + 1
    n = sum(seg_len)
    q = torch.randn(MQ, Hkv * G, D, device=DEV).to(torch.bfloat16)
    q_pos0, scale = n - MQ, D ** -0.5
    out, lse = FA.attend(q, lay, q_pos0, scale)
    npl = dict(ki=lay.ki.cpu().numpy().astype(np.int64), vi=lay.vi.cpu().numpy().astype(np.int64), kmid=lay.kmin.cpu().numpy(),
               kstep=lay.kstep.cpu().numpy(), vmid=lay.vmin.cpu().numpy(), vstep=lay.vstep.cpu().numpy(), kc=lay.kc.cpu().numpy(),
               vc=lay.vc.cpu().numpy(), ts=lay.t_start.cpu().numpy(), tl=lay.t_len.cpu().numpy(), tseg=lay.t_seg.cpu().numpy())
    for n_splits in (None, 1, 3):
        out, lse = FA.attend(q, lay, q_pos0, scale, n_splits=n_splits)
        ref, ref_lse = A.attend(q.float().cpu().numpy(), scale, npl, q_pos0, tps=2)
        assert out.shape == (MQ, Hkv * G, D) and lse.shape == (MQ, Hkv * G)
        assert np.all(np.abs(out.cpu().numpy() - ref) <= 1e-3 * vmax(npl) + 1e-6)
        assert np.allclose(lse.cpu().numpy(), ref_lse, atol=2e-3)
    # the cache's certificate carries through: attention over the decoded bf16 cache in fp32
    K = torch.cat([torch.stack([bk.decode_all_torch(DEV) for bk in seg], 1) for seg in segs_k])      # (n, Hkv, D)
    V = torch.cat([torch.stack([bk.decode_all_torch(DEV) for bk in seg], 1) for seg in segs_v])
    qf = q.float().reshape(MQ, Hkv, G, D)
    s = torch.einsum("mhgd,nhd->mhgn", qf, K) * scale
    mask = torch.arange(n, device=DEV)[None, :] <= (q_pos0 + torch.arange(MQ, device=DEV))[:, None]
    s = s.masked_fill(~mask[:, None, None, :], float("-inf"))
    dense = torch.einsum("mhgn,nhd->mhgd", torch.softmax(s, -1), V).reshape(MQ, Hkv * G, D)
    assert float((out - dense).abs().max()) <= 4e-3 * float(V.abs().max())
    # a head that needs more than 8 bits: no byte layout, but a 16-bit one on request
    tight = C.band_kv_heads((torch.randn(Hkv, 16, D, device=DEV) * 4).to(torch.bfloat16), torch.bfloat16, 6, tau=0.004)
    assert max(bk.bits for bk in tight) > 8
    assert FA.layout_from_segments([tight], [tight], [16], DEV) is None
    wide = FA.layout_from_segments([tight], [tight], [16], DEV, allow_wide=True)
    assert wide.ki.dtype == torch.int16
    o2, _ = FA.attend(q[:1], wide, 15, scale)
    K2 = torch.stack([bk.decode_all_torch(DEV) for bk in tight], 1)
    s2 = torch.einsum("hgd,nhd->hgn", q[0].float().reshape(Hkv, G, D), K2) * scale
    d2 = torch.einsum("hgn,nhd->hgd", torch.softmax(s2, -1), K2).reshape(Hkv * G, D)
    assert float((o2[0] - d2).abs().max()) <= 4e-3 * float(K2.abs().max())


def test_codec_on_the_device_matches_the_oracle_codec():
    torch.manual_seed(1)
    x = (torch.randn(3, 40, 64) * torch.rand(3, 1, 64) * 3).to(torch.bfloat16)
    got = C.band_kv_heads(x.to(DEV), torch.bfloat16, 5, tau=0.05)
    want = A.band_kv(x.float().numpy(), 5, 0.05, "bf16")
    for bk, (ids, mn, step, b) in zip(got, want):
        assert bk.bits == b and bk.orig_shape == (40, 64)
        assert np.array_equal(bk.min_s.cpu().numpy(), mn) and np.allclose(bk.tau_s.cpu().numpy(), step, rtol=1e-6)
        mine = bk.ids().cpu().numpy()
        assert np.abs(mine - ids).max() <= 1 and (mine == ids).mean() > 0.999
        assert float((bk.decode_all_torch(DEV, torch.bfloat16).float().cpu() - x[got.index(bk)].float()).abs().max()) <= 0.05
        assert torch.equal(bk.truncate(7).ids(), bk.ids()[:7])


def test_attn_refusals_through_the_c_abi():
    from qvb8_amd import _lib
    lib = _lib.load()
    lay = make_layout(1, [40], 1, 128)
    dl = to_device(lay)
    q = torch.zeros(1, 2, 128, dtype=torch.float16, device=DEV)
    o = torch.empty(2, 1, 2, 128, device=DEV); m = torch.empty(2, 1, 2, device=DEV); l = torch.empty_like(m)
    st = torch.cuda.current_stream().cuda_stream

    def call(**kw):
        a = dict(q=q.data_ptr(), sq_r=q.stride(0), sq_h=q.stride(1), ki=dl["ki"].data_ptr(), idb=1, s_n=dl["ki"].stride(0),
                 n_tiles=2, o=o.data_ptr(), n_splits=2, n_rows=2, hkv=1, D=128, q_pos0=39, tps=1, G=2, kmid=dl["kmid"].data_ptr())
        a.update(kw)
        return lib.qvb8_attn_fwd(a["q"], a["sq_r"], a["sq_h"], a["ki"], dl["vi"].data_ptr(), a["idb"], a["s_n"], dl["ki"].stride(1),
                                 a["kmid"], dl["kstep"].data_ptr(), dl["vmid"].data_ptr(), dl["vstep"].data_ptr(),
                                 dl["kc"].data_ptr(), dl["vc"].data_ptr(), dl["ts"].data_ptr(), dl["tl"].data_ptr(),
                                 dl["tseg"].data_ptr(), a["n_tiles"], a["o"], m.data_ptr(), l.data_ptr(), a["n_splits"],
                                 a["n_rows"], a["hkv"], a["D"], a["q_pos0"], a["tps"], 1.0, a["G"], st)
    assert call() == 0
    assert call(n_rows=0) == 0
    for bad in (dict(D=64), dict(idb=3), dict(q=None), dict(o=None), dict(n_splits=1), dict(tps=0), dict(G=0), dict(n_rows=3),
                dict(q=q.data_ptr() + 2), dict(sq_h=130), dict(ki=dl["ki"].data_ptr() + 1), dict(s_n=130), dict(ki=None),
                dict(kmid=dl["kmid"].data_ptr() + 4), dict(q_pos0=2 ** 31)):
        assert call(**bad) != 0, bad
        assert lib.qvb8_last_error().decode().startswith("qvb8_attn_fwd"), bad


def test_combine_matches_the_oracle():
    """qvb8_attn_combine against the caller's combination: random splits, rows nobody saw, a single split."""
    rng = np.random.default_rng(8)
    for S, hkv, MQ, G, D in ((5, 2, 3, 4, 128), (1, 1, 2, 2, 256), (300, 1, 1, 6, 256)):
        R = MQ * G
        o = rng.normal(0, 1, (S, hkv, R, D)).astype(np.float32)
        m = rng.normal(0, 3, (S, hkv, R)).astype(np.float32)
        l = rng.uniform(0.5, 30, (S, hkv, R)).astype(np.float32)
        m[:, 0, 0] = -np.inf; l[:, 0, 0] = 0; o[:, 0, 0] = 0            # a row without a visible key
        if S > 1:
            m[1, 0, 1] = -np.inf; l[1, 0, 1] = 0; o[1, 0, 1] = 0        # one empty split among full ones
        want, want_lse = A.combine(o, m, l, MQ, G)
        got, lse = FA.combine_splits(torch.from_numpy(o).to(DEV), torch.from_numpy(m).to(DEV), torch.from_numpy(l).to(DEV), G)
        assert got.shape == (MQ, hkv * G, D) and lse.shape == (MQ, hkv * G)
        assert np.allclose(got.cpu().numpy(), want, rtol=1e-5, atol=1e-6)
        assert np.array_equal(np.isneginf(lse.cpu().numpy()), np.isneginf(want_lse))
        fin = np.isfinite(want_lse)
        assert np.allclose(lse.cpu().numpy()[fin], want_lse[fin], rtol=1e-6, atol=1e-5)
        assert np.all(got.cpu().numpy()[0, 0] == 0)


@pytest.mark.parametrize("D,bits,wide,shift", [(128, 6, False, 0.0), (256, 8, False, 0.0), (128, 11, True, 0.0), (256, 9, True, 0.0),
                                               (256, 6, False, 0.3), (128, 5, False, -7.0)])
def test_restored_keys_and_values_are_the_oracles_bits(D, bits, wide, shift):
    """Read the kernel's restored K and V back, bit for bit: every key is a tile and a split of its own, so a split's
    p is exp(0) = 1 and its output row IS the restored V of that key, and with a one-hot query its running maximum IS
    one restored K element (1.0 * k, alone in an fp32 sum)."""
    Hkv, n = 2, 37
    lay = make_layout(D + bits, [20, 17], Hkv, D, bits=bits, spread=3.0)
    lay["ts"] = np.arange(n, dtype=np.int32)
    lay["tl"] = np.ones(n, np.int32)
    lay["tseg"] = (np.arange(n) >= 20).astype(np.int32)
    # id centres other than (2^B - 1) / 2 as well: moved by an integer, moved by 0.3
    lay["kc"] = (lay["kc"] + np.float32(shift)).astype(np.float32)
    lay["vc"] = (lay["vc"] - np.float32(shift)).astype(np.float32)
    dl = to_device(lay, wide=wide)
    G = 16
    K = np.zeros((n, Hkv, D), np.float32)
    V = np.zeros_like(K)
    for c0 in range(0, D, G):
        q = np.zeros((1, Hkv * G, D), np.float16)
        for g in range(G):
            q[0, np.arange(Hkv) * G + g, c0 + g] = 1.0
        o, m, l = run_fwd(lay, dl, torch.from_numpy(q).to(DEV), n - 1, 1, G)        # (n splits, Hkv, G, ...)
        assert np.all(l == 1.0)
        K[:, :, c0:c0 + G] = m
        V = o[:, :, 0, :]
        assert np.array_equal(o, np.broadcast_to(o[:, :, :1, :], o.shape))
    for h in range(Hkv):
        for a, b, seg in ((0, 20, 0), (20, 37, 1)):
            wk = A.restore_tile(lay["ki"][a:b, h], lay["kmid"][seg, h], lay["kstep"][seg, h], lay["kc"][seg, h])
            wv = A.restore_tile(lay["vi"][a:b, h], lay["vmid"][seg, h], lay["vstep"][seg, h], lay["vc"][seg, h])
            assert np.array_equal(K[a:b, h].view(np.uint32), wk.view(np.uint32))
            assert np.array_equal(V[a:b, h].view(np.uint32), wv.view(np.uint32))


@pytest.mark.parametrize("blocks", ["1", "2", "4"])
def test_row_blocks_per_workgroup_do_not_change_the_result(blocks, monkeypatch):
    """The same 36 rows served as three workgroups of one block, two of two, one of four (128 channels)."""
    lay = make_layout(21, [100], 2, 128)
    rng = np.random.default_rng(5)
    q = (rng.normal(0, 1, (12, 6, 128)) * 128 ** -0.5).astype(np.float16)
    want = A.fwd_split(q, lay["ki"], lay["vi"], lay["kmid"], lay["kstep"], lay["vmid"], lay["vstep"], lay["kc"], lay["vc"],
                       lay["ts"], lay["tl"], lay["tseg"], 88, 2, 1.0, 3)
    monkeypatch.setenv("QVB8_ATTN_ROW_BLOCKS", blocks)
    got = run_fwd(lay, to_device(lay), torch.from_numpy(q).to(DEV), 88, 2, 3)
    check_split_outputs(got, want, lay)


def test_random_shapes_match_the_oracle():
    """Sixty seeded random caches and query blocks: head_dim, heads, group size, tokens, ragged segments, id width, the
    first query position (before, inside and behind the cache), tiles per split, embedded buffers."""
    rng = np.random.default_rng(12345)
    for it in range(60):
        D = int(rng.choice([128, 256])); Hkv = int(rng.integers(1, 4)); G = int(rng.choice([1, 2, 3, 4, 6, 8])); MQ = int(rng.integers(1, 14))
        seg_len = [int(rng.integers(1, 120)) for _ in range(int(rng.integers(1, 4)))]
        n = sum(seg_len); bits = int(rng.choice([4, 6, 8, 10]))
        q_pos0 = int(rng.integers(-3, n + 5)); tps = int(rng.choice([1, 2, 3, 5, 8, 1000]))
        lay = make_layout(1000 + it, seg_len, Hkv, D, bits=bits)
        q = (rng.normal(0, 1, (MQ, Hkv * G, D)) * D ** -0.5).astype(np.float16)
        want = A.fwd_split(q, lay["ki"], lay["vi"], lay["kmid"], lay["kstep"], lay["vmid"], lay["vstep"], lay["kc"], lay["vc"],
                           lay["ts"], lay["tl"], lay["tseg"], q_pos0, tps, 1.0, G)
        got = run_fwd(lay, to_device(lay, wide=bits > 8, slack=int(rng.integers(0, 3))), torch.from_numpy(q).to(DEV), q_pos0, tps, G)
        try:
            check_split_outputs(got, want, lay)
        except AssertionError as ex:
            raise AssertionError(f"case {it}: D={D} Hkv={Hkv} G={G} MQ={MQ} seg_len={seg_len} bits={bits} q_pos0={q_pos0} tps={tps}") from ex


def test_query_preparation_is_the_callers_expression():
    """qvb8_scale_sat_half == (q.float() * scale).clamp(-65504, 65504).to(fp16), bit for bit, NaN and overflow included."""
    from qvb8_amd import _lib
    lib = _lib.load()
    g = torch.Generator(device=DEV).manual_seed(3)
    for dt in (torch.bfloat16, torch.float16, torch.float32):
        x = (torch.randn(5, 12, 128, device=DEV, generator=g) * 300).to(dt)
        x.view(-1)[:4] = torch.tensor([float("nan"), float("inf"), -float("inf"), 6e4], device=DEV).to(dt)
        for scale in (128 ** -0.5, 1.0, 40.0):
            out = torch.empty(x.shape, dtype=torch.float16, device=DEV)
            rc = lib.qvb8_scale_sat_half(x.data_ptr(), _lib.dtype_code(dt), x.numel(), scale, out.data_ptr(), torch.cuda.current_stream().cuda_stream)
            assert rc == 0
            want = (x.float() * scale).clamp(-65504.0, 65504.0).to(torch.float16)
            assert torch.equal(out.view(torch.int16)[~torch.isnan(want)], want.view(torch.int16)[~torch.isnan(want)])
            assert torch.equal(torch.isnan(out), torch.isnan(want))
    assert lib.qvb8_scale_sat_half(None, 0, 4, 1.0, None, None) != 0 and lib.qvb8_scale_sat_half(None, 0, 0, 1.0, None, None) == 0


def test_merge_by_log_sum_exp_is_attention_over_the_union():
    """Attention over two halves of a cache, merged by their log-sum-exps, equals attention over the whole; a part that
    saw no key (lse = -inf) drops out; the formulas of the reference's merge give the same numbers."""
    torch.manual_seed(9)
    Hkv, G, D, MQ = 2, 3, 128, 2
    parts = []
    for sl in (70, 45):
        k = C.band_kv_heads((torch.randn(Hkv, sl, D, device=DEV) * 2).to(torch.bfloat16), torch.bfloat16, 6)
        v = C.band_kv_heads(torch.randn(Hkv, sl, D, device=DEV).to(torch.bfloat16), torch.bfloat16, 6)
        parts.append((k, v, sl))
    whole = FA.layout_from_segments([p[0] for p in parts], [p[1] for p in parts], [p[2] for p in parts], DEV)
    first = FA.layout_from_segments([parts[0][0]], [parts[0][1]], [70], DEV)
    second = FA.layout_from_segments([parts[1][0]], [parts[1][1]], [45], DEV)
    q = torch.randn(MQ, Hkv * G, D, device=DEV).to(torch.bfloat16)
    scale = D ** -0.5
    o_all, l_all = FA.attend(q, whole, 115 - MQ, scale)
    o1, l1 = FA.attend(q, first, 115 - MQ, scale)
    o2, l2 = FA.attend(q, second, 45 - MQ, scale)             # positions relative to the second part's first key
    o, l = FA.merge_lse(o1, l1, o2, l2)
    assert o.shape == o_all.shape and l.shape == l_all.shape
    assert float((o - o_all).abs().max()) <= 2e-3 * float(whole.vmin.abs().max() + 32 * whole.vstep.max())
    assert float((l - l_all).abs().max()) <= 2e-3
    # the reference's expressions
    m = torch.maximum(l1, l2)
    w1, w2 = torch.exp(l1 - m), torch.exp(l2 - m)
    assert torch.allclose(o, (o1 * w1[..., None] + o2 * w2[..., None]) / (w1 + w2)[..., None], rtol=1e-5, atol=1e-6)
    assert torch.allclose(l, m + torch.log(w1 + w2), rtol=1e-6, atol=1e-5)
    # a part without a visible key
    o0, l0 = FA.attend(q, second, -5, scale)
    assert torch.isneginf(l0).all()
    o, l = FA.merge_lse_all(torch.stack([o1, o0, o2]), torch.stack([l1, l0, l2]))
    assert float((o - o_all).abs().max()) <= 2e-3 * float(whole.vmin.abs().max() + 32 * whole.vstep.max())
    on, ln = FA.merge_lse(o0, l0, o0, l0)
    assert torch.isneginf(ln).all() and (on == 0).all()
