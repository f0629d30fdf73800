"""GPU tests of the one-launch MLP (qvb8_mlp through QVBandMLPV8): against the CPU oracle's chain, against the separate
products on the same bytes, the state it carries from call to call, graph replay, and the bounded wait giving up."""
import os

import numpy as np
import pytest
import torch
import torch.nn as nn

from oracle import qvb8_oracle as O
from qvb8_amd import ext_qvb8 as ext
from qvb8_amd.formats.qvb8 import pack as PK
from qvb8_amd.formats.qvb8.mlp import QVBandMLPV8, install_fused_mlps, unit_order
from qvb8_amd.formats.qvb8.module import QVBandLinearV8
from tests import helpers as H

pytestmark = pytest.mark.gpu


@pytest.fixture(autouse=True)
def _one_launch(monkeypatch):
    monkeypatch.setenv("QVB8_MLP_FUSED", "1")          # the module's default is the separate products
DEV = "cuda:0"
NAME = {torch.bfloat16: "bf16", torch.float16: "fp16"}


def _weight(Q, P, seed, spread):
    """N(0, 0.02) rows; with `spread` every row has its own scale (0.5x .. 2x), so the rows need three different widths."""
    g = torch.Generator().manual_seed(seed)
    W = 0.02 * torch.randn(Q, P, generator=g)
    if spread:
        W = W * torch.exp2(2.0 * torch.rand(Q, 1, generator=g) - 1.0)
    return W.to(torch.bfloat16)


def _restored(enc):
    d = H.oracle_view(enc)
    return O.reconstruct(d["min_s"], d["tau_s"], H.oracle_ids(d), d["esc_idx"], d["esc_vals"])


def _build(hidden, inter, out, seed, spread=False, tau=1e-3):
    encs = [PK.encode_tensor(_weight(q, p, seed + i, spread).to(DEV), tau, restore="fp16")
            for i, (q, p) in enumerate(((inter, hidden), (inter, hidden), (out, inter)))]
    Ws = [_restored(e) for e in encs]                                   # before the modules re-store the bytes
    mlp = QVBandMLPV8(*[QVBandLinearV8.from_encoded(e) for e in encs])
    return mlp, Ws


def _check(y, x, Ws, dtype, M):
    y_ref, h_ref = O.mlp_reference(x.float().cpu().numpy(), *Ws, NAME[dtype])
    # the down product's bound, plus what one rounding step of H (a few of its values may land on the other side of a tie)
    # and the rounding of Y to the caller's type can move a result
    tol = H.gemv_tolerance(y_ref, Ws[2], O.sat_half(h_ref))
    eps = 2.0 ** -8 if dtype == torch.bfloat16 else 2.0 ** -11
    tol = tol + eps * np.abs(y_ref) + 4 * eps * np.abs(Ws[2]).max() * np.abs(h_ref).max()
    diff = np.abs(y.float().cpu().numpy().astype(np.float64).reshape(M, -1) - y_ref)
    assert np.all(diff <= tol), (float(diff.max()), float((diff / tol).max()))
    return h_ref


def _h_of(mlp, M):
    """H as the last call with M rows left it in the workspace: (values as float32, tags)."""
    words = mlp._ws[ext.MLP_H_AT:].view(torch.int32)
    base = mlp.inter * (M * (M - 1) // 2)
    w = words[base: base + M * mlp.inter].cpu().numpy().astype(np.uint32)
    return (w & 0xFFFF).astype(np.uint16).view(np.float16).astype(np.float32).reshape(M, mlp.inter), w >> 16


SHAPES = [  # hidden, inter, out, spread
    (512, 768, 512, False),        # most workgroups without a unit or a tile
    (1024, 2048, 1024, True),      # rows of several widths
    (4096, 12288, 4096, False),    # the 9B layer: three units and one tile per workgroup, two panels of down
    (5120, 2560, 5120, False),     # rows of 40 steps (five per wave), more down tiles than workgroups
    (8192, 1024, 256, False),      # two panels of gate+up
]


@pytest.mark.parametrize("shape", SHAPES)
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_one_launch_against_the_oracle_and_the_separate_products(shape, dtype):
    hidden, inter, out, spread = shape
    mlp, Ws = _build(hidden, inter, out, seed=11 * hidden + inter, spread=spread)
    assert mlp.fused_ready, mlp
    for M in (1, 3, 4, 2, 1):                                           # the call count of a row count goes on across other counts
        if M * hidden > 32768:
            continue
        g = torch.Generator().manual_seed(M)
        x = torch.randn(M, hidden, generator=g).to(dtype).to(DEV)
        print("mlp", shape, dtype, "M", M, flush=True)
        y = mlp(x)
        torch.cuda.synchronize()
        assert y.dtype == dtype and y.shape == (M, out)
        h_ref = _check(y, x, Ws, dtype, M)
        # H as the kernel handed it over: the oracle's, but for a few values a rounding step or two aside
        h, tags = _h_of(mlp, M)
        assert len(np.unique(tags)) == 1 and tags[0] != 0
        step = 2.0 ** -7 if dtype == torch.bfloat16 else 2.0 ** -10
        xs = O.sat_half(x.float().cpu().numpy())
        g_ref, u_ref = O.linear_f64(xs, Ws[0]), O.linear_f64(xs, Ws[1])
        # what the bound of each product, and a rounding step of g, u, silu(g) and h each, can move h by (|silu'| <= 1.1)
        dg = H.gemv_tolerance(g_ref, Ws[0], xs) + step * np.abs(g_ref)
        du = H.gemv_tolerance(u_ref, Ws[1], xs) + step * np.abs(u_ref)
        bound = 1.1 * dg * np.abs(u_ref) + du * np.abs(O.silu(g_ref)) + 2 * step * np.abs(h_ref) + 1e-7
        gap = np.abs(h - O.sat_half(h_ref))
        assert np.all(gap <= bound), (float((gap / bound).max()),)
        # (fp16 steps are eight times finer than bf16 steps: more of the products' last bits show)
        assert (gap > 0).mean() < (3e-2 if dtype == torch.bfloat16 else 0.25), (float((gap > 0).mean()),)
        # the separate products on the same bytes: the same chain, rounded at the same places
        y_sep = mlp.separate(x)
        d = (y.float() - y_sep.float()).abs()
        scale = y_sep.float().abs().max().item()
        assert d.max().item() <= 2e-2 * scale and (d > 0).float().mean().item() < (0.05 if dtype == torch.bfloat16 else 0.5), (d.max().item(), scale)
    assert not mlp.error_raised()


def test_fewer_workgroups_than_cus_and_step_variants(monkeypatch):
    """A grid of 24 workgroups walks several units and tiles each; three and four steps per wave in the down phase."""
    mlp, Ws = _build(1024, 2048, 1024, seed=5, spread=True)
    x = torch.randn(2, 1024, generator=torch.Generator().manual_seed(9)).to(torch.bfloat16).to(DEV)
    ys = []
    for wgs, t2 in ((0, 0), (24, 3), (24, 4), (8, 4)):
        monkeypatch.setenv("QVB8_MLP_WGS", str(wgs))
        monkeypatch.setenv("QVB8_MLP_T2", str(t2))
        print("mlp grid", wgs, t2, flush=True)
        y = mlp(x)
        torch.cuda.synchronize()
        _check(y, x, Ws, torch.bfloat16, 2)
        ys.append(y)
    assert not mlp.error_raised()


def test_unit_order_pairs_gate_and_up_rows():
    nb = torch.tensor([7] * 40 + [6] * 24 + [5] * 64 + [7] * 128, dtype=torch.uint8)        # inter = 128
    perm, new_nb = unit_order(nb, 128)
    perm = perm.view(-1, 2, 16)
    assert bool((perm[:, 1] == perm[:, 0] + 128).all()) and sorted(perm[:, 0].reshape(-1).tolist()) == list(range(128))
    w = new_nb.long()
    assert bool((w >= nb.long()).all()) and bool((w[:128] == w[128:]).all())
    along = w[perm.reshape(-1).long()]
    assert bool((along[1:] >= along[:-1]).all()) and bool((along.view(-1, 32).amin(1) == along.view(-1, 32).amax(1)).all())
    assert unit_order(torch.full((2 * 100,), 7, dtype=torch.uint8), 100) is None          # not whole units
    assert unit_order(torch.tensor([9] * 32, dtype=torch.uint8), 16) is None              # too wide for the sliced decode


def test_graph_replay_follows_its_input():
    mlp, Ws = _build(1024, 2048, 1024, seed=21)
    x = torch.zeros(1, 1024, dtype=torch.bfloat16, device=DEV)
    mlp(x)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        y = mlp(x)
    for i in range(4):
        xi = torch.randn(1, 1024, generator=torch.Generator().manual_seed(40 + i)).to(torch.bfloat16).to(DEV)
        x.copy_(xi)
        graph.replay()
        torch.cuda.synchronize()
        _check(y, xi, Ws, torch.bfloat16, 1)
        assert torch.equal(y, mlp(xi))                                 # eager calls in between share the workspace
    assert not mlp.error_raised()


def test_the_wait_for_h_is_bounded(monkeypatch):
    """H labelled as another call's never arrives: every workgroup gives up after the bound, the results are NaN, the
    error word is raised -- and the next call finds the workspace in order."""
    mlp, Ws = _build(1024, 2048, 1024, seed=33)
    x = torch.randn(1, 1024, generator=torch.Generator().manual_seed(1)).to(torch.bfloat16).to(DEV)
    good = mlp(x)
    torch.cuda.synchronize()
    monkeypatch.setenv("QVB8_MLP_WAIT_US", "200")
    print("mlp stale tag", flush=True)
    y = ext.mlp_fused(x, mlp._ws, mlp._plan, act=ext.MLP_SILU_GATED | ext.MLP_TEST_STALE_TAG)
    torch.cuda.synchronize()
    assert bool(torch.isnan(y.float()).all())
    assert mlp.error_raised()
    state = mlp._ws[:32].view(torch.int32).cpu()
    assert state[0].item() == 0                                        # every workgroup was counted, the count was closed
    monkeypatch.delenv("QVB8_MLP_WAIT_US")
    mlp._ws[4:8].zero_()
    again = mlp(x)
    torch.cuda.synchronize()
    assert torch.equal(again, good) and not mlp.error_raised()


def test_what_the_kernel_does_not_cover_goes_the_separate_way():
    mlp, Ws = _build(512, 768, 512, seed=3)
    for M, dtype in ((6, torch.bfloat16), (2, torch.float32)):
        x = torch.randn(M, 512, generator=torch.Generator().manual_seed(M)).to(dtype).to(DEV)
        y = mlp(x)
        assert y.dtype == dtype and y.shape == (M, 512)
        if dtype == torch.bfloat16:
            _check(y, x, Ws, dtype, M)
    with pytest.raises(RuntimeError):
        ext.mlp_fused(torch.zeros(5, 512, dtype=torch.bfloat16, device=DEV), mlp._ws, mlp._plan)
    with pytest.raises(RuntimeError):                                  # a plan goes with the workspace it was made for
        ext.mlp_fused(torch.zeros(1, 512, dtype=torch.bfloat16, device=DEV), mlp._ws.clone(), mlp._plan)


def test_install_replaces_a_models_mlps():
    class Mlp(nn.Module):
        def __init__(self, seed):
            super().__init__()
            mk = lambda q, p, s: QVBandLinearV8.from_encoded(PK.encode_tensor(_weight(q, p, s, False).to(DEV), 1e-3, restore="fp16"))
            self.gate_proj, self.up_proj, self.down_proj = mk(768, 512, seed), mk(768, 512, seed + 1), mk(512, 768, seed + 2)
            self.act_fn = nn.SiLU()

        def forward(self, x):
            return self.down_proj(self.act_fn(self.gate_proj(x)) * self.up_proj(x))

    class Layer(nn.Module):
        def __init__(self, seed):
            super().__init__()
            self.mlp = Mlp(seed)

    model = nn.ModuleList([Layer(10), Layer(20)])
    x = torch.randn(1, 512, generator=torch.Generator().manual_seed(2)).to(torch.bfloat16).to(DEV)
    before = [l.mlp(x) for l in model]
    assert install_fused_mlps(model) == 2
    assert all(isinstance(l.mlp, QVBandMLPV8) and l.mlp.fused_ready for l in model)
    for l, b in zip(model, before):
        d = (l.mlp(x).float() - b.float()).abs()
        assert d.max().item() <= 2e-2 * b.float().abs().max().item()
