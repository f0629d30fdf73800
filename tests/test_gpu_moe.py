"""GPU parity of the routed MoE expert stack (qvb8_moe_experts through ext.moe_experts / QVBandExpertsV8) against the
CPU oracle's per-token loop over restored weights."""
import numpy as np
import pytest
import torch
import torch.nn as nn

from oracle import qvb8_oracle as O
from qvb8_amd import ext_qvb8 as ext
from qvb8_amd.formats.qvb8 import pack as PK
from qvb8_amd.formats.qvb8.backends_experts import QVBandExpertsV8
from qvb8_amd.formats.qvb8.module import QVBandLinearV8
from tests import helpers as H

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _experts(E, hidden, inter, tau, seed, gated=True):
    gu, dn, Wgu, Wdn = [], [], [], []
    for e in range(E):
        for lst, Wl, (Q, P) in ((gu, Wgu, ((2 if gated else 1) * inter, hidden)), (dn, Wdn, (hidden, inter))):
            W = H.synth_weight(Q, P, seed=seed + 2 * e + len(lst)).to(DEV)
            enc = PK.encode_tensor(W, tau, restore="fp16")
            assert enc["esc_idx"].numel() == 0
            lst.append(QVBandLinearV8.from_encoded(enc))
            d = H.oracle_view(enc)
            Wl.append(O.reconstruct(d["min_s"], d["tau_s"], H.oracle_ids(d), d["esc_idx"], d["esc_vals"]))
    return gu, dn, Wgu, Wdn


def _route(T, E, k, seed):
    rng = np.random.default_rng(seed)
    idx, w = O.router_topk(rng.normal(size=(T, E)), k)
    return idx, w


def _check(out, ref, out_dtype, roundings=1):
    """`roundings`: how many times intermediate results pass through out_dtype (the per-expert loop rounds the up
    output, the activation product, the down output and the weighted sum)."""
    eps = {torch.float32: 0.0, torch.float16: 2.0 ** -11, torch.bfloat16: 2.0 ** -8}[out_dtype] * roundings
    got = out.float().cpu().numpy().astype(np.float64)
    scale = np.sqrt(np.mean(ref ** 2)) + 1e-30
    # Relative part: the bar of every product test here (1e-3) plus the roundings to out_dtype.  Absolute part, in units of
    # the output's rms: the two chained products each carry the product tests' error (fp32 accumulation over 768..2048
    # terms), and on the matrix-core paths H goes from the first to the second as fp16 (2^-11 per element, which the down
    # product averages over its terms rather than adds up).  Measured: the worst element of these tests uses about half of
    # 1e-3 rms, the worst of 1500 randomised calls (2..11 experts, 1..16 tokens, hidden 128..2048) 1.25e-3 rms.
    tol = (1e-3 + eps) * np.abs(ref) + (1.5e-3 + eps * (roundings > 1)) * scale
    diff = np.abs(got - ref)
    assert np.all(diff <= tol), (float(diff.max()), float((diff / tol).max()))


@pytest.mark.parametrize("T,k,dtype", [(1, 2, torch.bfloat16), (3, 4, torch.float16), (8, 2, torch.float32), (20, 3, torch.bfloat16)])
def test_moe_small_stack(T, k, dtype):
    E, hidden, inter = 8, 256, 96
    gu, dn, Wgu, Wdn = _experts(E, hidden, inter, 2e-3, seed=100)
    idx, w = _route(T, E, k, seed=T)
    x = torch.randn(T, hidden, generator=torch.Generator().manual_seed(T)).to(dtype)
    mod = QVBandExpertsV8(gu, dn, num_experts=E)
    out = mod(x.to(DEV), torch.from_numpy(idx).to(DEV), torch.from_numpy(w).to(DEV))
    assert mod._stk not in (None, False) and out.dtype == dtype and out.shape == (T, hidden)
    ref = O.moe_reference(x.float().numpy(), idx, w, Wgu, Wdn)
    _check(out, ref, dtype)
    # the per-expert loop over the same (now stacked) modules agrees
    loop = mod._forward_loop(x.to(DEV), torch.from_numpy(idx).to(DEV), torch.from_numpy(w).to(DEV).to(dtype))
    _check(loop, ref, dtype if dtype != torch.float32 else torch.float16, roundings=4)
    # an expert index outside the stack poisons the output instead of reading somewhere else
    bad = torch.from_numpy(idx).to(DEV).clone()
    bad[0, 0] = E
    assert torch.isnan(mod(x.to(DEV), bad, torch.from_numpy(w).to(DEV)).float()).all()


def test_moe_config4_shape():
    """Qwen-35B-A3B-shape layer, fewer experts resident: hidden 2048, gate/up 2048->768, top-8, 1 and 8 tokens."""
    E, hidden, inter = 16, 2048, 768
    gu, dn, Wgu, Wdn = _experts(E, hidden, inter, 2e-3, seed=500)
    mod = QVBandExpertsV8(gu, dn, num_experts=E)
    for T in (1, 8):
        idx, w = _route(T, E, 8, seed=10 + T)
        x = torch.randn(T, hidden, generator=torch.Generator().manual_seed(T)).to(torch.bfloat16)
        out = mod(x.to(DEV), torch.from_numpy(idx).to(DEV), torch.from_numpy(w).to(DEV))
        _check(out, O.moe_reference(x.float().numpy(), idx, w, Wgu, Wdn), torch.bfloat16)
        again = mod(x.to(DEV), torch.from_numpy(idx).to(DEV), torch.from_numpy(w).to(DEV))
        assert torch.equal(out, again)                       # reproducible run to run


def test_moe_relu2_and_odd_widths():
    """Non-gated ReLU^2 stack on hand-made packs whose rows use every width 1..14 (the per-element path included)."""
    E, hidden, inter = 3, 128, 64
    ups, dns, Wup, Wdn = [], [], [], []
    for e in range(E):
        for lst, Wl, (Q, P), widths in ((ups, Wup, (inter, hidden), list(range(1, 15))), (dns, Wdn, (hidden, inter), [4, 5, 6, 7, 8])):
            d = H.mixed_width_pack(Q, P, widths, seed=7 * e + len(lst))
            d["tau_s"] = d["tau_s"] * (1.0 / (1 << 6))            # keep products of wide rows in range
            a = H.to_device_args(d, DEV)
            lst.append(dict(ids=a[0], min_s=a[1], nbits=a[2], bit_off=a[3], tau_s=a[5]))
            Wl.append(O.reconstruct(d["min_s"], d["tau_s"], d["ids_dense"], d["esc_idx"], d["esc_vals"]))

    def stack(lst):
        offs, total = [], 0
        for t in lst:
            offs.append(total)
            total += (t["ids"].numel() + 15) // 16 * 16
        ids = torch.zeros(total + 64, dtype=torch.uint8, device=DEV)
        for o, t in zip(offs, lst):
            ids[o:o + t["ids"].numel()] = t["ids"]
        return (ids, torch.stack([t["min_s"] for t in lst]), torch.stack([t["tau_s"] for t in lst]),
                torch.stack([t["nbits"] for t in lst]), torch.stack([t["bit_off"] + 8 * o for t, o in zip(lst, offs)]))
    T, k = 5, 2
    idx, w = _route(T, E, k, seed=3)
    x = torch.randn(T, hidden, generator=torch.Generator().manual_seed(1)).to(torch.float16)
    out = ext.moe_experts_relu2(x.to(DEV), torch.from_numpy(idx).to(DEV), torch.from_numpy(w).to(DEV),
                                *stack(ups), inter, hidden, *stack(dns), hidden, inter)
    _check(out, O.moe_reference(x.float().numpy(), idx, w, Wup, Wdn, act="relu2"), torch.float16)


def _hand_made_stack(E, Q, P, widths, seed):
    """E hand-made experts of (Q, P) with the given row widths, stacked as QVBandExpertsV8.build_stack lays them out;
    returns the operands after X / idx / w of ext.moe_experts and the restored weights."""
    lst, Ws = [], []
    for e in range(E):
        d = H.mixed_width_pack(Q, P, widths, seed=seed + e)
        d["tau_s"] = d["tau_s"] * (1.0 / (1 << 6))
        a = H.to_device_args(d, DEV)
        lst.append(dict(ids=a[0], min_s=a[1], nbits=a[2], bit_off=a[3], tau_s=a[5]))
        Ws.append(O.reconstruct(d["min_s"], d["tau_s"], d["ids_dense"], d["esc_idx"], d["esc_vals"]))
    offs, total = [], 0
    for t in lst:
        offs.append(total)
        total += (t["ids"].numel() + 15) // 16 * 16
    ids = torch.zeros(total + 64, dtype=torch.uint8, device=DEV)
    for o, t in zip(offs, lst):
        ids[o:o + t["ids"].numel()] = t["ids"]
    ops = (ids, torch.stack([t["min_s"] for t in lst]), torch.stack([t["tau_s"] for t in lst]),
           torch.stack([t["nbits"] for t in lst]), torch.stack([t["bit_off"] + 8 * o for t, o in zip(lst, offs)]))
    return ops, Ws


@pytest.mark.parametrize("gated", [True, False])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_moe_one_token_on_the_matrix_cores(gated, dtype, monkeypatch):
    """One token takes two launches (up with the activation, down with the weighted sum) on MFMA tiles.  Rows of every
    width 1..14 in the up stack (sliced tiles, mixed tiles and element-by-element rows), 4..8 in the down stack; against
    the oracle, against the general path, run to run, and with an expert number outside the stack."""
    E, hidden, inter, k = 5, 256, 128, 3
    Qup = 2 * inter if gated else inter
    up_ops, Wup = _hand_made_stack(E, Qup, hidden, [6, 6, 6, 6, 6, 6, 6, 6, 6, 6, 6, 6, 6, 6, 6, 6, 7, 5] + list(range(1, 15)), seed=40)
    dn_ops, Wdn = _hand_made_stack(E, hidden, inter, [4, 5, 6, 7, 8], seed=80)
    idx, w = _route(1, E, k, seed=11)
    x = torch.randn(1, hidden, generator=torch.Generator().manual_seed(2)).to(dtype)
    fn = ext.moe_experts if gated else ext.moe_experts_relu2
    args = (x.to(DEV), torch.from_numpy(idx).to(DEV), torch.from_numpy(w).to(DEV), *up_ops, Qup, hidden, *dn_ops, hidden, inter)
    monkeypatch.setenv("QVB8_MOE_ONE_TOKEN", "1")
    out = fn(*args)
    assert out.dtype == dtype and out.shape == (1, hidden)
    ref = O.moe_reference(x.float().numpy(), idx, w, Wup, Wdn, act="silu" if gated else "relu2")
    _check(out, ref, dtype)
    assert torch.equal(out, fn(*args))
    monkeypatch.setenv("QVB8_MOE_ONE_TOKEN", "0")
    general = fn(*args)
    _check(general, ref, dtype)
    scale = float(np.sqrt(np.mean(ref ** 2)))
    assert float((out.float() - general.float()).abs().max()) <= 4e-3 * scale + 2.0 ** -7 * float(np.abs(ref).max())
    monkeypatch.setenv("QVB8_MOE_ONE_TOKEN", "1")
    bad = torch.from_numpy(idx).to(DEV).clone()
    bad[0, 1] = E + 3
    assert torch.isnan(fn(args[0], bad, *args[2:]).float()).all()


def test_moe_refusals():
    E, hidden, inter = 2, 128, 32
    gu, dn, _, _ = _experts(E, hidden, inter, 2e-3, seed=900)
    mod = QVBandExpertsV8(gu, dn, num_experts=E, act_fn=nn.GELU())
    assert mod.build_stack() is False                        # unknown activation: the loop path serves it
    x = torch.randn(2, hidden).to(torch.bfloat16).to(DEV)
    idx = torch.tensor([[0, 1], [1, 0]], device=DEV)
    w = torch.full((2, 2), 0.5, device=DEV)
    assert mod(x, idx, w).shape == (2, hidden)
    with pytest.raises(ValueError):
        QVBandExpertsV8(gu[:1], dn, num_experts=E)
    g = QVBandExpertsV8(gu, dn, num_experts=E)
    assert g.build_stack()
    s, d = g._stk
    with pytest.raises(RuntimeError):                        # gate_up / down shapes disagree
        ext.moe_experts(x, idx, w, s["ids"], s["min_s"], s["tau_s"], s["nbits"], s["bit_off"], s["Q"], s["P"],
                        d["ids"], d["min_s"], d["tau_s"], d["nbits"], d["bit_off"], d["Q"], d["P"] + 32)


@pytest.mark.parametrize("T,k,dtype", [(2, 2, torch.bfloat16), (3, 2, torch.bfloat16), (5, 4, torch.float16), (16, 8, torch.bfloat16),
                                       (9, 1, torch.float16)])
@pytest.mark.parametrize("group_from", ["3", None])
def test_moe_few_tokens_share_each_expert(T, k, dtype, group_from, monkeypatch):
    """2..16 tokens on the matrix cores: one grid row per token through the one-token kernels, or (from seven tokens on by
    default, from three with QVB8_MOE_GROUP_FROM=3) the tokens that chose an expert share one walk over it.  Shapes the grouped
    kernels take (row lengths that are multiples of 128), more experts than get selected and experts selected by many
    tokens at once; against the oracle, reproducible, and equal to the per-token result of the same library."""
    E, hidden, inter = 12, 384, 128
    gu, dn, Wgu, Wdn = _experts(E, hidden, inter, 2e-3, seed=900)
    idx, w = _route(T, E, k, seed=50 + T)
    idx[:, 0] = 3                                              # one expert chosen by every token
    if k > 1:
        for t in range(T):                                     # keep a token's choices distinct
            others = [e for e in range(E) if e != 3]
            idx[t, 1:] = np.random.default_rng(t).choice(others, k - 1, replace=False)
    x = torch.randn(T, hidden, generator=torch.Generator().manual_seed(T)).to(dtype)
    if group_from is not None:
        monkeypatch.setenv("QVB8_MOE_GROUP_FROM", group_from)
    mod = QVBandExpertsV8(gu, dn, num_experts=E)
    args = (x.to(DEV), torch.from_numpy(idx).to(DEV), torch.from_numpy(w).to(DEV))
    out = mod(*args)
    _check(out, O.moe_reference(x.float().numpy(), idx, w, Wgu, Wdn), dtype)
    assert torch.equal(out, mod(*args))
    # token by token through the one-token kernels: the same products, H and the weighted sums rounded the same way
    single = torch.cat([mod(args[0][t:t + 1], args[1][t:t + 1], args[2][t:t + 1]) for t in range(T)])
    _check(single, O.moe_reference(x.float().numpy(), idx, w, Wgu, Wdn), dtype)
    bad = args[1].clone()
    bad[T - 1, 0] = E + 5                                      # an expert number outside the stack: NaN for its token at least
    assert torch.isnan(mod(args[0], bad, args[2]).float()[T - 1]).all()


@pytest.mark.parametrize("group_from", ["3", None])
def test_moe_few_tokens_relu2_and_rows_the_slicing_cannot_read(group_from, monkeypatch):
    """The few-token kernels (6 tokens: grouped walk or one grid row per token; 13: grouped walk) on hand-made packs: non-gated ReLU^2, every width 1..14 among the up rows (the element-wise
    path inside the grouped kernel), row lengths of 128 and 256."""
    E, hidden, inter = 4, 256, 128
    ups, dns, Wup, Wdn = [], [], [], []
    for e in range(E):
        for lst, Wl, (Q, P), widths in ((ups, Wup, (inter, hidden), list(range(1, 15))), (dns, Wdn, (hidden, inter), [4, 5, 6, 7, 8, 11])):
            d = H.mixed_width_pack(Q, P, widths, seed=17 * e + len(lst))
            d["tau_s"] = d["tau_s"] * (1.0 / (1 << 7))
            a = H.to_device_args(d, DEV)
            lst.append(dict(ids=a[0], min_s=a[1], nbits=a[2], bit_off=a[3], tau_s=a[5]))
            Wl.append(O.reconstruct(d["min_s"], d["tau_s"], d["ids_dense"], d["esc_idx"], d["esc_vals"]))

    def stack(lst):
        offs, total = [], 0
        for t in lst:
            offs.append(total)
            total += (t["ids"].numel() + 15) // 16 * 16
        ids = torch.zeros(total + 64, dtype=torch.uint8, device=DEV)
        for o, t in zip(offs, lst):
            ids[o:o + t["ids"].numel()] = t["ids"]
        return (ids, torch.stack([t["min_s"] for t in lst]), torch.stack([t["tau_s"] for t in lst]),
                torch.stack([t["nbits"] for t in lst]), torch.stack([t["bit_off"] + 8 * o for t, o in zip(lst, offs)]))
    if group_from is not None:
        monkeypatch.setenv("QVB8_MOE_GROUP_FROM", group_from)
    for T, k in ((6, 2), (13, 3)):
        idx, w = _route(T, E, k, seed=T)
        x = torch.randn(T, hidden, generator=torch.Generator().manual_seed(T)).to(torch.float16)
        out = ext.moe_experts_relu2(x.to(DEV), torch.from_numpy(idx).to(DEV), torch.from_numpy(w).to(DEV),
                                    *stack(ups), inter, hidden, *stack(dns), hidden, inter)
        _check(out, O.moe_reference(x.float().numpy(), idx, w, Wup, Wdn, act="relu2"), torch.float16)


def test_moe_few_tokens_rows_longer_than_2048_columns(monkeypatch):
    """The grouped walk (asked for from three tokens on) with rows of 2304 columns in the up projection (eight steps per wave, one register set) and of
    640 in the down projection; 4 tokens, top-2 of 4 experts."""
    E, hidden, inter = 4, 2304, 640
    gu, dn, Wgu, Wdn = _experts(E, hidden, inter, 2e-3, seed=4100)
    monkeypatch.setenv("QVB8_MOE_GROUP_FROM", "3")
    mod = QVBandExpertsV8(gu, dn, num_experts=E)
    idx, w = _route(4, E, 2, seed=77)
    x = torch.randn(4, hidden, generator=torch.Generator().manual_seed(3)).to(torch.bfloat16)
    out = mod(x.to(DEV), torch.from_numpy(idx).to(DEV), torch.from_numpy(w).to(DEV))
    _check(out, O.moe_reference(x.float().numpy(), idx, w, Wgu, Wdn), torch.bfloat16)


def test_moe_config4_all_128_experts():
    """The 35B-A3B-shape layer with all 128 experts resident (hidden 2048, gate/up 2048->768, top-8): 1, 4 and 6 tokens (one
    grid row per token) and 8 (the grouped walk)."""
    E, hidden, inter = 128, 2048, 768
    gu, dn, Wgu, Wdn = _experts(E, hidden, inter, 2e-3, seed=7000)
    mod = QVBandExpertsV8(gu, dn, num_experts=E)
    for T in (1, 4, 6, 8):
        idx, w = _route(T, E, 8, seed=30 + T)
        x = torch.randn(T, hidden, generator=torch.Generator().manual_seed(T)).to(torch.bfloat16)
        out = mod(x.to(DEV), torch.from_numpy(idx).to(DEV), torch.from_numpy(w).to(DEV))
        _check(out, O.moe_reference(x.float().numpy(), idx, w, Wgu, Wdn), torch.bfloat16)


@pytest.mark.parametrize("T", [1, 2, 5, 16])
def test_moe_regular_stack_changes_no_result(T, monkeypatch):
    """QVBandExpertsV8 stores a stack whose widths lie close together in ONE width, rows in row order at regular places,
    and tells the kernels (QVB8_MOE_*_REGULAR): the results are bit for bit those of the stack as the files have it
    (QVB8_MOE_UNIFORM_TILES=0), and within tolerance of the oracle; a stack that is not regular is never claimed to be."""
    E, hidden, inter, k = 6, 256, 128, 2
    idx, w = _route(T, E, k, seed=T)
    x = torch.randn(T, hidden, generator=torch.Generator().manual_seed(T)).to(torch.bfloat16).to(DEV)
    outs = {}
    monkeypatch.setenv("QVB8_MOE_ONE_WIDTH_GROWTH", "0.25")      # the short rows of this test spread over two widths evenly
    for flag in ("0", "1"):
        monkeypatch.setenv("QVB8_MOE_UNIFORM_TILES", flag)
        gu, dn, Wgu, Wdn = [], [], [], []
        for e in range(E):                              # normal weights: rows of two neighbouring widths, mixed at random
            for lst, Wl, (Q, P) in ((gu, Wgu, (2 * inter, hidden)), (dn, Wdn, (hidden, inter))):
                W = (0.02 * torch.randn(Q, P, generator=torch.Generator().manual_seed(700 + 2 * e + len(lst)))).to(torch.bfloat16).to(DEV)
                enc = PK.encode_tensor(W, 2e-3, restore="fp16")
                assert enc["esc_idx"].numel() == 0 and int(enc["nbits"].min()) < int(enc["nbits"].max())
                lst.append(QVBandLinearV8.from_encoded(enc))
                v = H.oracle_view(enc)
                Wl.append(O.reconstruct(v["min_s"], v["tau_s"], H.oracle_ids(v), v["esc_idx"], v["esc_vals"]))
        mod = QVBandExpertsV8(gu, dn, num_experts=E)
        assert mod.build_stack()
        g, d = mod._stk
        if flag == "1":
            assert g["regular"] and d["regular"] and int(g["nbits"].min()) == int(g["nbits"].max())
            assert ext.stack_is_regular(g["nbits"], g["bit_off"], hidden) and ext.stack_is_regular(d["nbits"], d["bit_off"], inter)
        else:
            assert not g["regular"] and not d["regular"]
        outs[flag] = mod(x, torch.from_numpy(idx).to(DEV), torch.from_numpy(w).to(DEV))
        # the experts' own modules still give what they gave: the stack holds their rows, wider or not
        one = gu[1](x)
        ref1 = x.float().cpu().numpy().astype(np.float64) @ Wgu[1].astype(np.float64).T
        assert float(np.abs(one.float().cpu().numpy() - ref1).max()) <= 2e-2 * float(np.abs(ref1).max())
    assert torch.equal(outs["0"], outs["1"])
    _check(outs["1"], O.moe_reference(x.float().cpu().numpy(), idx, w, Wgu, Wdn), torch.bfloat16)
    # a claim that does not hold is not made for a stack built by hand
    ops, _ = _hand_made_stack(3, 64, 128, [5, 6], seed=5)
    assert not ext.stack_is_regular(ops[3], ops[4], 128)


@pytest.mark.parametrize("T", [1, 8])
def test_moe_regular_stack_off_dword_boundaries(T, monkeypatch):
    """A stack that is regular as the interface defines it -- one width, rows at regular places -- but moved by one byte,
    so that no row starts on a dword boundary: with the statement the kernels give what they give without it."""
    E, hidden, inter, k = 6, 256, 128, 2
    monkeypatch.setenv("QVB8_MOE_ONE_WIDTH_GROWTH", "0.25")
    gu, dn, Wgu, Wdn = [], [], [], []
    for e in range(E):
        for lst, Wl, (Q, P) in ((gu, Wgu, (2 * inter, hidden)), (dn, Wdn, (hidden, inter))):
            W = (0.02 * torch.randn(Q, P, generator=torch.Generator().manual_seed(900 + 2 * e + len(lst)))).to(torch.bfloat16).to(DEV)
            enc = PK.encode_tensor(W, 2e-3, restore="fp16")
            lst.append(QVBandLinearV8.from_encoded(enc))
            v = H.oracle_view(enc)
            Wl.append(O.reconstruct(v["min_s"], v["tau_s"], H.oracle_ids(v), v["esc_idx"], v["esc_vals"]))
    mod = QVBandExpertsV8(gu, dn, num_experts=E)
    assert mod.build_stack()
    g, d = mod._stk
    assert g["regular"] and d["regular"]

    def moved(st):
        ids = torch.cat([torch.zeros(1, dtype=torch.uint8, device=DEV), st["ids"]])
        return ids, st["min_s"], st["tau_s"], st["nbits"], st["bit_off"] + 8

    gm, dm = moved(g), moved(d)
    assert ext.stack_is_regular(gm[3], gm[4], hidden) and ext.stack_is_regular(dm[3], dm[4], inter)
    idx, w = _route(T, E, k, seed=3 + T)
    x = torch.randn(T, hidden, generator=torch.Generator().manual_seed(T)).to(torch.bfloat16).to(DEV)
    args = (x, torch.from_numpy(idx).to(DEV), torch.from_numpy(w).to(DEV), *gm, 2 * inter, hidden, *dm, hidden, inter)
    plain = ext.moe_experts(*args)
    stated = ext.moe_experts(*args, regular=(True, True))
    assert torch.equal(plain, stated)
    _check(stated, O.moe_reference(x.float().cpu().numpy(), idx, w, Wgu, Wdn), torch.bfloat16)


def test_moe_grouped_walk_and_an_expert_listed_twice_for_a_token():
    """Seven to sixteen tokens group the pairs by expert, the pairs of an expert being the rows of ONE operand: as many as
    there are tokens.  A token may list an expert twice as long as that holds (the pairs are rows of their own); an expert
    with more pairs than tokens gives NaN everywhere rather than a sum with pairs missing."""
    E, hidden, inter, k, T = 6, 256, 128, 2, 8
    gu, dn, Wgu, Wdn = _experts(E, hidden, inter, 2e-3, seed=300)
    mod = QVBandExpertsV8(gu, dn, num_experts=E)
    idx, w = _route(T, E, k, seed=5)
    x = torch.randn(T, hidden, generator=torch.Generator().manual_seed(5)).to(torch.bfloat16).to(DEV)
    twice = idx.copy()
    twice[3, 1] = twice[3, 0]
    out = mod(x, torch.from_numpy(twice).to(DEV), torch.from_numpy(w).to(DEV))
    _check(out, O.moe_reference(x.float().cpu().numpy(), twice, w, Wgu, Wdn), torch.bfloat16)
    crowded = idx.copy()
    crowded[:, 0] = 2                                    # every token chooses expert 2 ...
    crowded[:, 1] = np.where(crowded[:, 1] == 2, 3, crowded[:, 1])
    crowded[0, 1] = 2                                    # ... and one of them twice: nine pairs for eight tokens
    out = mod(x, torch.from_numpy(crowded).to(DEV), torch.from_numpy(w).to(DEV))
    assert bool(torch.isnan(out.float()).all())
