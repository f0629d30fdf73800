"""GPU: graph replay of blocks built on the compressed operators is bit-identical to eager execution, replay after
replay, with the program's own eager work and synchronisations in between."""
import numpy as np
import pytest
import torch
import torch.nn as nn

from oracle import qvb8_oracle as O
from qvb8_amd.formats.qvb8 import pack as PK
from qvb8_amd.formats.qvb8.backends_experts import QVBandExpertsV8
from qvb8_amd.formats.qvb8.fuse import fuse_same_input
from qvb8_amd.formats.qvb8.graph import GraphedBlock, install_block_graphs
from qvb8_amd.formats.qvb8.module import QVBandLinearV8
from tests import helpers as H

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


_RESTORED = {}          # module -> the oracle's restore of its pack (float32), for the float64 referee


def _lin(Q, P, seed):
    enc = PK.encode_tensor(H.synth_weight(Q, P, seed=seed).to(DEV), 1e-3, restore="fp16")
    lin = QVBandLinearV8.from_encoded(enc)
    d = H.oracle_view(enc)
    _RESTORED[lin] = O.reconstruct(d["min_s"], d["tau_s"], H.oracle_ids(d), d["esc_idx"], d["esc_vals"])
    return lin


def _mlp_oracle(mlp, x):
    """gate / up / down through the oracle's restored weights in float64, with the roundings the module chain makes: the
    activations saturated to fp16 on the way into every product, each product's result rounded to bf16."""
    bf = lambda a: O.narrow_bf16(a.astype(np.float32)).astype(np.float64)
    xs = O.sat_half(x.float().cpu().numpy())
    g = bf(O.linear_f64(xs, _RESTORED[mlp.gate_proj]))
    u = bf(O.linear_f64(xs, _RESTORED[mlp.up_proj]))
    h = bf(bf(g / (1.0 + np.exp(-g))) * u)
    return O.linear_f64(O.sat_half(h.astype(np.float32)), _RESTORED[mlp.down_proj])


class _Mlp(nn.Module):
    def __init__(self, h, inter):
        super().__init__()
        self.gate_proj, self.up_proj, self.down_proj = _lin(inter, h, 1), _lin(inter, h, 2), _lin(h, inter, 3)

    def forward(self, x):
        return self.down_proj(torch.nn.functional.silu(self.gate_proj(x)) * self.up_proj(x))


class _Moe(nn.Module):
    def __init__(self, h, inter, E, k):
        super().__init__()
        gu = [_lin(2 * inter, h, 10 + e) for e in range(E)]
        dn = [_lin(h, inter, 40 + e) for e in range(E)]
        self.restored = ([_RESTORED[m] for m in gu], [_RESTORED[m] for m in dn])     # before the stack re-stores the rows
        self.experts = QVBandExpertsV8(gu, dn, num_experts=E)
        self.router = nn.Linear(h, E, bias=False).to(DEV).to(torch.bfloat16)
        self.k = k

    def route(self, x):
        p = torch.softmax(self.router(x).float(), -1)
        w, idx = torch.topk(p, self.k, -1)
        return idx, w / w.sum(-1, keepdim=True)

    def forward(self, x):
        return self.experts(x, *self.route(x))


class _Layer(nn.Module):
    def __init__(self, block):
        super().__init__()
        self.mlp = block


@pytest.mark.parametrize("kind", ["mlp", "moe"])
@torch.no_grad()
def test_graph_replay_is_bit_identical(kind):
    torch.manual_seed(0)
    layer = _Layer(_Mlp(512, 256) if kind == "mlp" else _Moe(256, 128, 6, 2))
    if kind == "mlp":
        unfused = layer.mlp
        x0 = torch.randn(3, 512, device=DEV).to(torch.bfloat16)
        ref = _mlp_oracle(unfused, x0)                              # the referee: oracle restore + float64 arithmetic
        assert fuse_same_input(layer) == 1                          # gate+up as one launch, inside the graph as well
        got = layer.mlp(x0).float().cpu().numpy().astype(np.float64)
        scale = np.sqrt(np.mean(ref ** 2))
        assert np.all(np.abs(got - ref) <= 2.0 ** -6 * np.abs(ref) + 2.0 ** -6 * scale), float(np.abs(got - ref).max() / scale)
    eager = layer.mlp
    assert install_block_graphs(layer) == 1 and isinstance(layer.mlp, GraphedBlock)
    assert install_block_graphs(layer) == 0                         # already wrapped
    h = 512 if kind == "mlp" else 256
    for rows in (1, 4):
        xs = [torch.randn(rows, h, device=DEV).to(torch.bfloat16) for _ in range(5)]
        want = [eager(x).clone() for x in xs]
        for rep in range(5):                                        # call 1 eager, call 2 captures, 3.. replay
            got = layer.mlp(xs[rep])
            torch.cuda.synchronize()
            _ = (xs[rep].float() @ xs[rep].float().T).sum().item()  # the program's own eager work between replays
            assert torch.equal(got, want[rep]), (kind, rows, rep)
            if kind == "moe":                                       # and the replayed result is the oracle's, not just eager's
                idx, w = eager.route(xs[rep])
                ref = O.moe_reference(xs[rep].float().cpu().numpy(), idx.cpu().numpy(), w.float().cpu().numpy(), *eager.restored)
                diff = np.abs(got.float().cpu().numpy().astype(np.float64) - ref)
                tol = (1e-3 + 2.0 ** -8) * np.abs(ref) + 1.5e-3 * np.sqrt(np.mean(ref ** 2))      # the MoE tests' bar
                assert np.all(diff <= tol), (rows, rep, float((diff / tol).max()))
    assert sum(1 for v in layer.mlp._graphs.values() if isinstance(v, tuple)) == 2
    big = torch.randn(64, h, device=DEV).to(torch.bfloat16)         # prefill-sized input: eager, no new graph
    assert torch.equal(layer.mlp(big), eager(big))
    assert sum(1 for v in layer.mlp._graphs.values() if isinstance(v, tuple)) == 2
