"""The pack directory: manifest and key handling on the CPU; on the GPU, a toy model's modules swapped from a directory
written by this build's writers and compared with the dense model."""
import json
import os

import numpy as np
import pytest
import torch
import torch.nn as nn

from qvb8_amd.common import packdir as PD


def test_expert_keys_and_module_paths():
    assert PD.parse_expert_key("model.layers.0.mlp.experts.gate_up_proj#expert003") == ("model.layers.0.mlp.experts.gate_up_proj", 3)
    assert PD.parse_expert_key("model.layers.0.mlp.gate_proj.weight") == ("model.layers.0.mlp.gate_proj.weight", None)
    assert PD.tensor_key_to_module("model.language_model.layers.0.mlp.gate_proj.weight") == "model.layers.0.mlp.gate_proj"
    assert PD.tensor_key_to_module("language_model.backbone.layers.1.mixer.in_proj.weight") == "model.layers.1.mixer.in_proj"
    assert PD.tensor_key_to_module("language_model.lm_head.weight") == "lm_head"
    assert PD.tensor_key_to_module("model.layers.0.mlp.experts.down_proj") == "model.layers.0.mlp.experts.down_proj"


def test_manifest_round_trip_and_expert_grouping(tmp_path):
    tensors = {"model.embed_tokens.weight": "model_embed_tokens_weight.qvband",
               "model.layers.0.mlp.experts.gate_up_proj#expert000": {"pack": "gu0.qvband", "restore": "fp16", "P": 64},
               "model.layers.0.mlp.experts.gate_up_proj#expert001": "gu1.qvband",
               "model.layers.0.mlp.experts.down_proj#expert001": "dn1.qvb8"}
    PD.write_manifest(str(tmp_path), tensors, tau=1e-3, hf_model="nobody/toy", failed={"x.weight": "range"})
    pd = PD.PackDir(str(tmp_path))
    assert pd.tau == 1e-3 and pd.spec.name == "qvband" and pd.hf_model == "nobody/toy" and list(pd.failed) == ["x.weight"]
    assert pd.packfile("model.embed_tokens.weight") == os.path.join(str(tmp_path), "model_embed_tokens_weight.qvband")
    assert pd.spec_of("model.layers.0.mlp.experts.down_proj#expert001").name == "qvb8"
    st = pd.expert_stacks()
    assert list(st) == ["model.layers.0.mlp.experts"]
    assert sorted(st["model.layers.0.mlp.experts"]["gate_up_proj"]) == [0, 1] and list(st["model.layers.0.mlp.experts"]["down_proj"]) == [1]
    with open(os.path.join(tmp_path, "manifest.json"), "w") as fh:
        json.dump({"format": "no-such-format", "tensors": {}}, fh)
    with pytest.raises(ValueError):
        PD.PackDir(str(tmp_path))
    with open(os.path.join(tmp_path, "manifest.json"), "w") as fh:
        json.dump({"format": "qvb8"}, fh)
    with pytest.raises(ValueError):
        PD.PackDir(str(tmp_path))


class _Experts(nn.Module):
    def __init__(self, E, hidden, inter):
        super().__init__()
        self.num_experts = E
        self.gate_up_proj = nn.Parameter(0.02 * torch.randn(E, 2 * inter, hidden))
        self.down_proj = nn.Parameter(0.02 * torch.randn(E, hidden, inter))
        self.act_fn = nn.SiLU()

    def forward(self, x, idx, w):
        out = torch.zeros_like(x)
        for t in range(x.shape[0]):
            for j in range(idx.shape[1]):
                e = int(idx[t, j])
                g, u = (self.gate_up_proj[e] @ x[t]).chunk(2)
                out[t] += w[t, j] * (self.down_proj[e] @ (self.act_fn(g) * u))
        return out


class _Attn(nn.Module):
    def __init__(self, h):
        super().__init__()
        self.q_proj, self.k_proj, self.v_proj = nn.Linear(h, h, bias=True), nn.Linear(h, h // 2, bias=False), nn.Linear(h, h // 2, bias=False)


class _Mlp(nn.Module):
    def __init__(self, h, E, inter):
        super().__init__()
        self.experts = _Experts(E, h, inter)


class _Layer(nn.Module):
    def __init__(self, h, E, inter):
        super().__init__()
        self.self_attn, self.mlp, self.norm = _Attn(h), _Mlp(h, E, inter), nn.LayerNorm(h)


class _Inner(nn.Module):
    def __init__(self, vocab, h, E, inter):
        super().__init__()
        self.embed_tokens = nn.Embedding(vocab, h)
        self.layers = nn.ModuleList([_Layer(h, E, inter)])


class _Toy(nn.Module):
    def __init__(self, vocab=200, h=256, E=4, inter=64):
        super().__init__()
        self.model = _Inner(vocab, h, E, inter)
        self.lm_head = nn.Linear(h, vocab, bias=False)


@pytest.mark.gpu
@torch.no_grad()
def test_swap_modules_of_a_toy_model(tmp_path):
    from qvb8_amd.formats.qvb8 import pack as PK
    from qvb8_amd.formats.qvb8.backends_experts import QVBandExpertsV8
    from qvb8_amd.formats.qvb8.embedding import QVBandEmbeddingV8
    from qvb8_amd.formats.qvb8.fuse import FusedMember
    from qvb8_amd.formats.qvb8.module import QVBandLinearV8
    dev, tau = "cuda:0", 1e-3
    torch.manual_seed(0)
    toy = _Toy()
    with torch.no_grad():
        for p in toy.parameters():
            if p.dim() >= 2:
                p.copy_((0.02 * torch.randn_like(p)).to(torch.bfloat16).float())
    dense = {k: v.detach().clone() for k, v in toy.state_dict().items()}
    tensors = {}

    def pack(key, W, fname):
        PK.write_pack(os.path.join(tmp_path, fname), PK.encode_tensor(W.to(dev).to(torch.bfloat16), tau, restore="fp16"))
        tensors[key] = fname
    # keys as a multimodal checkpoint names them; the head without its "model." prefix; one tensor nobody can place
    pack("model.language_model.embed_tokens.weight", dense["model.embed_tokens.weight"], "embed.qvband")
    for n in ("q_proj", "k_proj", "v_proj"):
        pack(f"model.language_model.layers.0.self_attn.{n}.weight", dense[f"model.layers.0.self_attn.{n}.weight"], f"{n}.qvband")
    pack("lm_head.weight", dense["lm_head.weight"], "head.qvb8")
    pack("model.visual.patch_embed.proj.weight", dense["lm_head.weight"], "vis.qvband")
    pack("model.language_model.layers.0.norm.weight", dense["lm_head.weight"], "norm.qvband")
    for e in range(4):
        pack(f"model.language_model.layers.0.mlp.experts.gate_up_proj#expert{e:03d}", dense["model.layers.0.mlp.experts.gate_up_proj"][e], f"gu{e}.qvband")
        pack(f"model.language_model.layers.0.mlp.experts.down_proj#expert{e:03d}", dense["model.layers.0.mlp.experts.down_proj"][e], f"dn{e}.qvband")
    PD.write_manifest(str(tmp_path), tensors, tau=tau)

    ref = _Toy()
    ref.load_state_dict(dense)
    toy = toy.to(dev)
    rep = PD.swap_modules(toy, str(tmp_path), device=dev, out_dtype=torch.float32)
    assert rep["embedding"] == ["model.embed_tokens"] and rep["experts"] == ["model.layers.0.mlp.experts"]
    assert sorted(rep["linear"]) == ["lm_head", "model.layers.0.self_attn.k_proj", "model.layers.0.self_attn.q_proj", "model.layers.0.self_attn.v_proj"]
    assert rep["fused"] == 1 and set(rep["skipped"]) == {"model.visual.patch_embed.proj", "model.layers.0.norm"}
    assert isinstance(toy.model.embed_tokens, QVBandEmbeddingV8) and isinstance(toy.lm_head, QVBandLinearV8)
    assert isinstance(toy.model.layers[0].mlp.experts, QVBandExpertsV8) and isinstance(toy.model.layers[0].self_attn.q_proj, FusedMember)

    tok = torch.tensor([3, 199, 0, 57])
    x = toy.model.embed_tokens(tok.to(dev))
    x_ref = ref.model.embed_tokens(tok).detach()
    assert float((x.cpu() - x_ref).abs().max()) < tau
    x16 = x_ref.to(torch.float16).to(dev)                          # same activations on both sides from here on
    for n in ("q_proj", "k_proj", "v_proj"):
        y = getattr(toy.model.layers[0].self_attn, n)(x16).float().cpu()
        y_ref = getattr(ref.model.layers[0].self_attn, n)(x16.float().cpu())
        assert torch.allclose(y, y_ref, rtol=2e-3, atol=tau * float(x_ref.abs().sum(-1).max())), n
    idx = torch.tensor([[0, 3], [1, 2], [3, 0], [2, 2]])
    w = torch.full((4, 2), 0.5)
    m = toy.model.layers[0].mlp.experts(x16, idx.to(dev), w.to(dev)).float().cpu()
    m_ref = ref.model.layers[0].mlp.experts(x16.float().cpu(), idx, w)
    assert torch.allclose(m, m_ref, rtol=2e-2, atol=2e-3 * float(m_ref.abs().max()) + 1e-6)
    logits = toy.lm_head(x16).float().cpu()
    assert torch.allclose(logits, ref.lm_head(x16.float().cpu()), rtol=2e-3, atol=tau * float(x_ref.abs().sum(-1).max()))
