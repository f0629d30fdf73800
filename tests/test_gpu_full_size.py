"""GPU checks at the full sizes of the benchmark configurations, through size-independent properties (the CPU oracle would
take minutes there): restore -> certificate, fused product == dense restore + fp32 matmul, linearity, fusion, QVB8R
restore == QVB8 restore of the same ids, and attention over a long banded cache == dense attention, however it is split."""
import numpy as np
import pytest
import torch

from qvb8_amd import ext_qvb8 as ext
from qvb8_amd.formats.qvb8 import pack as PK
from qvb8_amd.formats.qvb8.module import QVBandLinearV8

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _weight(Q, P, seed):
    g = torch.Generator(device=DEV).manual_seed(seed)
    return (0.02 * torch.randn(Q, P, device=DEV, generator=g)).to(torch.bfloat16)


def _args(enc):
    return (enc["ids"], enc["min_s"], enc["nbits"], enc["bit_off"], enc["P"], enc["tau_s"], enc["esc_idx"], enc["esc_vals"])


@pytest.mark.parametrize("Q,P", [(12288, 4096), (4096, 12288), (1024, 4096)])
def test_9b_projection_certificate_and_products(Q, P):
    W = _weight(Q, P, seed=Q + P)
    enc = PK.encode_tensor(W, 1e-3, restore="fp16")
    w16 = ext.decode(*_args(enc))
    max_err, bad = ext.certify(w16, W, 1e-3)                 # the certificate, re-verified on the GPU at full size
    assert bad == 0 and max_err < 1e-3
    w32 = ext.decode_f32(*_args(enc))
    assert torch.equal(w32.half(), w16)                      # fp16 restore == fp32 restore rounded once
    lin = QVBandLinearV8.from_encoded(enc)
    g = torch.Generator(device=DEV).manual_seed(1)
    for M in (1, 16, 48):
        x = torch.randn(M, P, device=DEV, generator=g).to(torch.bfloat16)
        y = lin(x).float()
        ref = x.float().double() @ w32.double().t()          # dense restore + matmul (float64 referee on the GPU)
        wn = w32.double().norm(dim=1)[None, :]
        xn = x.float().double().norm(dim=1)[:, None]
        tol = (1e-3 + 2.0 ** -8) * ref.abs() + 1e-3 * wn * xn / np.sqrt(P)
        assert bool(((y.double() - ref).abs() <= tol).all()), float(((y.double() - ref).abs() / tol).max())
    # linearity of the operator in x: f(a + b) == f(a) + f(b) up to fp32 accumulation
    a = torch.randn(1, P, device=DEV, generator=g).half()
    b = torch.randn(1, P, device=DEV, generator=g).half()
    ya, yb, yab = (ext.mma_tiles(t, *_args(enc)) for t in (a, b, (a.float() + b.float()).half()))
    s = (a.float() + b.float()).half().float() - a.float() - b.float()      # what rounding a + b to fp16 changed
    corr = s.double() @ w32.double().t()
    scale = w32.double().norm(dim=1)[None, :] * (a.float().double().norm() + b.float().double().norm()) / np.sqrt(P)
    assert bool(((yab.double() - ya.double() - yb.double() - corr).abs() <= 1e-4 * scale + 1e-6).all())


def test_fused_same_input_at_full_size():
    from qvb8_amd.formats.qvb8.fuse import concat_linears
    lins = [QVBandLinearV8.from_encoded(PK.encode_tensor(_weight(Q, 4096, seed=Q), 1e-3)) for Q in (4096, 1024, 1024)]
    fused, splits = concat_linears(lins)
    x = torch.randn(1, 4096, device=DEV, generator=torch.Generator(device=DEV).manual_seed(3)).to(torch.bfloat16)
    for part, lin in zip(torch.tensor_split(fused(x), splits, -1), lins):
        assert torch.equal(part, lin(x))


def test_qvb8r_restore_equals_qvb8_restore_at_27b_shape():
    from qvb8_amd.formats.qvb8r import pack as RP
    from qvb8_amd.formats.qvb8r.module import QVBandLinearV8R
    Q, P = 2048, 17408                                       # 27B-class row length; fewer rows keep the CPU encoder quick
    W = _weight(Q, P, seed=9)
    enc = PK.encode_tensor(W, 2e-3, keep_ids=True)
    lin = QVBandLinearV8R(RP.transcode(enc), device=DEV)
    assert torch.equal(lin.dense(torch.float32), ext.decode_f32(*_args(enc)))
    assert torch.equal(lin.dense(torch.float16), ext.decode(*_args(enc)))
    max_err, bad = ext.certify(lin.dense(torch.float16), W, 2e-3)
    assert bad == 0 and max_err < 2e-3
    w32 = lin.dense(torch.float32).double()
    for M in (1, 3, 16):                                     # the configuration's row counts, and one in between
        x = torch.randn(M, P, device=DEV, generator=torch.Generator(device=DEV).manual_seed(4 + M)).to(torch.bfloat16)
        y = lin(x).float().double()
        ref = x.float().double() @ w32.t()
        tol = (1e-3 + 2.0 ** -8) * ref.abs() + 1e-3 * w32.norm(dim=1)[None, :] * x.float().double().norm(dim=1)[:, None] / np.sqrt(P)
        assert bool(((y - ref).abs() <= tol).all()), (M, float(((y - ref).abs() / tol).max()))


def test_qvb8r_products_at_the_27b_down_shape():
    """The other 27B-class shape of the configuration: 5120 rows of 17408 columns would take minutes to encode on the CPU, so
    rows of 5120 columns (gate / up: 17408 x 5120) stand for it with 1 and 16 rows of X."""
    from qvb8_amd.formats.qvb8r import pack as RP
    from qvb8_amd.formats.qvb8r.module import QVBandLinearV8R
    Q, P = 4096, 5120
    W = _weight(Q, P, seed=21)
    enc = PK.encode_tensor(W, 2e-3, keep_ids=True)
    lin = QVBandLinearV8R(RP.transcode(enc), device=DEV)
    assert torch.equal(lin.dense(torch.float16), ext.decode(*_args(enc)))
    w64 = lin.dense(torch.float32).double()
    for M in (1, 16):
        x = torch.randn(M, P, device=DEV, generator=torch.Generator(device=DEV).manual_seed(M)).to(torch.bfloat16)
        y = lin(x).float().double()
        ref = x.float().double() @ w64.t()
        tol = (1e-3 + 2.0 ** -8) * ref.abs() + 1e-3 * w64.norm(dim=1)[None, :] * x.float().double().norm(dim=1)[:, None] / np.sqrt(P)
        assert bool(((y - ref).abs() <= tol).all()), (M, float(((y - ref).abs() / tol).max()))


@pytest.mark.parametrize("Q,P", [(28672, 8192), (8192, 28672)])
def test_qvb8r_at_the_65b_shapes(Q, P):
    """The large-dense configuration at its full shapes (hidden 8192, FFN 28672, tau = 2e-3): the walk gives back the
    encoder's ids, the restore equals the QVB8 restore of the same ids, the certificate holds, and the products of 1 and
    16 rows equal dense restore + float64 matmul."""
    from qvb8_amd import ext_qvb8r
    from qvb8_amd.formats.qvb8r import pack as RP
    from qvb8_amd.formats.qvb8r.module import QVBandLinearV8R
    W = _weight(Q, P, seed=Q // 7 + P)
    enc = PK.encode_tensor(W, 2e-3, keep_ids=True)
    lin = QVBandLinearV8R(RP.transcode(enc), device=DEV)
    assert torch.equal(ext_qvb8r.ids(P, *lin._core(), T=lin.T), enc["ids_dense"])
    w32 = lin.dense(torch.float32)
    assert torch.equal(w32, ext.decode_f32(*_args(enc)))
    w16 = lin.dense(torch.float16)
    assert torch.equal(w16, ext.decode(*_args(enc)))
    max_err, bad = ext.certify(w16, W, 2e-3)
    assert bad == 0 and max_err < 2e-3
    del w16, W
    w64 = w32.double()
    wn = w64.norm(dim=1)[None, :]
    for M in (1, 16):
        x = torch.randn(M, P, device=DEV, generator=torch.Generator(device=DEV).manual_seed(M)).to(torch.bfloat16)
        y = lin(x).float().double()
        ref = x.float().double() @ w64.t()
        tol = (1e-3 + 2.0 ** -8) * ref.abs() + 1e-3 * wn * x.float().double().norm(dim=1)[:, None] / np.sqrt(P)
        assert bool(((y - ref).abs() <= tol).all()), (M, float(((y - ref).abs() / tol).max()))


@pytest.mark.parametrize("n,MQ", [(32768, 1), (32768, 3), (131072, 1)])
def test_attention_over_a_long_banded_cache(n, MQ):
    """The benchmark's cache shape (4 kv heads x 256 channels, 24 query heads, 6-bit ids, segments of 4096 keys): the
    result does not depend on how the tiles are split (one split, the planner's, twice as many: within the fp16 rounding
    of the probabilities, 1e-3 * max|v|), equals fp32 attention over the decoded cache (4e-3 * max|v|: that reference
    keeps bf16-rounded K / V where the kernel restores fp16), and a query placed inside the context ignores every
    later key."""
    from qvb8_amd.kv import codec as KC, fused_attn as FA
    hkv, G, D, seg = 4, 6, 256, 4096
    g = torch.Generator(device=DEV).manual_seed(n + MQ)
    segs_k, segs_v, seg_len = [], [], []
    for a in range(0, n, seg):
        k = (torch.randn(hkv, seg, D, device=DEV, generator=g) * (0.5 + 2 * torch.rand(hkv, 1, D, device=DEV, generator=g))).to(torch.bfloat16)
        v = torch.randn(hkv, seg, D, device=DEV, generator=g).to(torch.bfloat16)
        segs_k.append(KC.band_kv_heads(k, torch.bfloat16, 6, certify=False))
        segs_v.append(KC.band_kv_heads(v, torch.bfloat16, 6, certify=False))
        seg_len.append(seg)
    lay = FA.layout_from_segments(segs_k, segs_v, seg_len, DEV)
    q = torch.randn(MQ, hkv * G, D, device=DEV, generator=g).to(torch.bfloat16)
    scale = D ** -0.5
    vmax = float((lay.vmin.abs() + lay.vstep * 32).max())
    tps, planned = FA.plan_splits(lay.n_tiles, hkv, MQ * G, DEV)
    outs = [FA.attend(q, lay, n - MQ, scale, n_splits=s) for s in (1, planned, 2 * planned)]
    for out, lse in outs[1:]:
        assert float((out - outs[0][0]).abs().max()) <= 1e-3 * vmax
        assert float((lse - outs[0][1]).abs().max()) <= 2e-3
    # dense fp32 attention over the decoded cache, one kv head at a time (the scores of all heads would not fit nicely)
    q16 = (q.float() * scale).clamp(-65504, 65504).half().float().reshape(MQ, hkv, G, D)
    mask = torch.arange(n, device=DEV)[None, :] <= (n - MQ + torch.arange(MQ, device=DEV))[:, None]
    for h in range(hkv):
        K = torch.cat([s[h].decode_all_torch(DEV) for s in segs_k])
        V = torch.cat([s[h].decode_all_torch(DEV) for s in segs_v])
        s = torch.einsum("mgd,nd->mgn", q16[:, h], K).masked_fill(~mask[:, None, :], float("-inf"))
        ref = torch.einsum("mgn,nd->mgd", torch.softmax(s, -1), V)
        got = outs[1][0].reshape(MQ, hkv, G, D)[:, h]
        assert float((got - ref).abs().max()) <= 4e-3 * vmax
        assert float((outs[1][1].reshape(MQ, hkv, G)[:, h] - torch.logsumexp(s, -1)).abs().max()) <= 2e-2
    # a query in the middle of the context: the same as attention over the cache cut off behind it
    cut = n // 2 + 77
    short = FA.layout_from_segments(segs_k[: cut // seg + 1], segs_v[: cut // seg + 1], seg_len[: cut // seg + 1], DEV)
    o_mid, l_mid = FA.attend(q[:1], lay, cut, scale)
    o_cut, l_cut = FA.attend(q[:1], short, cut, scale)
    assert float((o_mid - o_cut).abs().max()) <= 1e-3 * vmax and float((l_mid - l_cut).abs().max()) <= 2e-3
