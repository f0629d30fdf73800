"""GPU checks at the full sizes of the benchmark configurations, through size-independent properties (the CPU oracle would
take minutes there): restore -> certificate, fused product == dense restore + fp32 matmul, linearity, fusion and QVB8R
restore == QVB8 restore of the same ids."""
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
    x = torch.randn(3, P, device=DEV, generator=torch.Generator(device=DEV).manual_seed(4)).to(torch.bfloat16)
    y = lin(x).float().double()
    w32 = lin.dense(torch.float32).double()
    ref = x.float().double() @ w32.t()
    tol = (1e-3 + 2.0 ** -8) * ref.abs() + 1e-3 * w32.norm(dim=1)[None, :] * x.float().double().norm(dim=1)[:, None] / np.sqrt(P)
    assert bool(((y - ref).abs() <= tol).all())
