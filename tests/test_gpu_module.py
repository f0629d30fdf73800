"""GPU tests of QVBandLinearV8 (the operator the model adapters call): every dispatch branch against the CPU oracle."""
import os

import numpy as np
import pytest
import torch

from oracle import qvb8_oracle as O
from qvb8_amd.formats.qvb8 import pack as PK
from qvb8_amd.formats.qvb8.module import QVBandLinearV8, enable_bf16_gemm, footprint_report
from tests import helpers as H

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _ref(enc, x, saturate, bf16_table=False, narrow=None):
    d = H.oracle_view(enc, bf16_table=bf16_table)
    Wr = O.reconstruct(d["min_s"], d["tau_s"], H.oracle_ids(d), d["esc_idx"], d["esc_vals"])
    if narrow == "fp16":
        Wr = O.narrow_fp16(Wr)
    elif narrow == "bf16":
        Wr = O.narrow_bf16(Wr)
    xs = x.float().cpu().numpy().reshape(-1, x.shape[-1])
    if saturate:
        xs = O.sat_half(xs)
    return O.linear_f64(xs, Wr), Wr, xs


def _close(y, ref, Wr, xs, out_dtype):
    tol = H.gemv_tolerance(ref, Wr, xs)
    if out_dtype != torch.float32:                       # one more rounding, to the caller's 16-bit dtype
        eps = 2.0 ** -8 if out_dtype == torch.bfloat16 else 2.0 ** -11
        tol = tol + eps * np.abs(ref)
    diff = np.abs(y.float().cpu().numpy().astype(np.float64).reshape(ref.shape) - ref)
    assert np.all(diff <= tol), (float(diff.max()), float((diff / tol).max()))


@pytest.mark.parametrize("M", [1, 4, 8, 16, 48, 60, 96])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
def test_linear_small_m(M, dtype):
    W = H.synth_weight(200, 1024, seed=3).to(DEV)
    enc = PK.encode_tensor(W, 1e-3, restore="fp16", force_escapes=[0, 1024 * 7 + 5, 1024 * 199 + 1023])
    bias = torch.linspace(-1, 1, 200, device=DEV)
    lin = QVBandLinearV8.from_encoded(enc, bias=bias)
    g = torch.Generator().manual_seed(M)
    x = torch.randn(2, M // 2, 1024, generator=g).to(dtype).to(DEV) if M % 2 == 0 else torch.randn(M, 1024, generator=g).to(dtype).to(DEV)
    y = lin(x)
    assert y.dtype == dtype and y.shape == (*x.shape[:-1], 200)
    ref, Wr, xs = _ref(enc, x, saturate=True)
    _close(y, ref + bias.double().cpu().numpy(), Wr, xs, dtype)


def test_linear_without_matrix_core_shape_and_large_m():
    """P % 128 != 0: GEMV for M <= 8, dense restore + library GEMM above (fp16 restore for fp16 callers)."""
    W = H.synth_weight(96, 200, seed=5).to(DEV)
    enc = PK.encode_tensor(W, 1e-3, restore="fp16")
    lin = QVBandLinearV8.from_encoded(enc)
    assert lin._mma_order() is None
    for M, dtype in ((3, torch.bfloat16), (20, torch.float32), (20, torch.float16), (150, torch.bfloat16)):
        x = torch.randn(M, 200, generator=torch.Generator().manual_seed(M)).to(dtype).to(DEV)
        y = lin(x)
        narrow = "fp16" if M > 8 else None                 # above 8 rows the weight is restored to fp16 first
        ref, Wr, xs = _ref(enc, x, saturate=True, narrow=narrow)
        _close(y, ref, Wr, xs, dtype)
    W2 = H.synth_weight(64, 1024, seed=6).to(DEV)
    lin2 = QVBandLinearV8.from_encoded(PK.encode_tensor(W2, 1e-3, restore="fp16"))
    x = torch.randn(130, 1024, generator=torch.Generator().manual_seed(1)).to(torch.float16).to(DEV)
    ref, Wr, xs = _ref(PK.encode_tensor(W2, 1e-3, restore="fp16"), x, saturate=True, narrow="fp16")
    _close(lin2(x), ref, Wr, xs, torch.float16)


def test_bf16_certified_pack_modes():
    W = H.synth_weight(128, 1024, seed=9).to(DEV)
    enc = PK.encode_tensor(W, 1e-3, restore="fp16+bf16")
    lin = QVBandLinearV8.from_encoded(enc)
    assert lin.bf16_certified and enable_bf16_gemm(lin) == (1, 1)
    x = torch.randn(16, 1024, generator=torch.Generator().manual_seed(2)).to(torch.bfloat16).to(DEV)
    ref, Wr, xs = _ref(enc, x, saturate=False, bf16_table=True)
    _close(lin(x), ref, Wr, xs, torch.bfloat16)             # bf16 operands, bf16 escape table
    xm = torch.randn(128, 1024, generator=torch.Generator().manual_seed(3)).to(torch.bfloat16).to(DEV)
    ref, Wr, xs = _ref(enc, xm, saturate=False, bf16_table=True)
    _close(lin(xm), ref, Wr, xs, torch.bfloat16)            # 49..256 rows: still the fused path on bf16 operands
    xl = torch.randn(300, 1024, generator=torch.Generator().manual_seed(4)).to(torch.bfloat16).to(DEV)
    ref, Wr, xs = _ref(enc, xl, saturate=False, bf16_table=True, narrow="bf16")
    _close(lin(xl), ref, Wr, xs, torch.bfloat16)            # more rows: bf16 restore + one bf16 GEMM
    rep = footprint_report(lin)
    assert rep["linears"] == 1 and rep["params"] == 128 * 1024 and rep["bytes_per_param"] < 1.2


def test_row_subset_and_dtype_cast_keep_metadata():
    W = H.synth_weight(300, 512, seed=11).to(DEV)
    enc = PK.encode_tensor(W, 1e-3, restore="fp16", force_escapes=[512 * 17 + 3, 512 * 250 + 9])
    lin = QVBandLinearV8.from_encoded(enc)
    rows = torch.tensor([250, 3, 17, 299, 100], device=DEV)
    sub = lin.row_subset(rows)
    assert sub.ids.data_ptr() == lin.ids.data_ptr() and sub.out_features == 5
    x = torch.randn(2, 512, generator=torch.Generator().manual_seed(4)).to(torch.bfloat16).to(DEV)
    assert torch.equal(sub(x), lin(x)[:, rows])
    before = lin.tau_s.clone()
    lin.to(torch.bfloat16)
    assert lin.tau_s.dtype == torch.float32 and torch.equal(lin.tau_s, before) and lin.esc_vals.dtype == torch.float32


def test_from_packfile_roundtrip(tmp_path):
    W = H.synth_weight(64, 256, seed=13).to(DEV)
    for restore, name in (("fp16", "a.qvband"), ("fp16+bf16", "b.qvband"), ("fp16", "c.qvb8")):
        enc = PK.encode_tensor(W, 1e-3, restore=restore, force_escapes=[5, 256 * 63 + 255])
        path = os.path.join(tmp_path, name)
        PK.write_pack(path, enc)
        lin = QVBandLinearV8.from_packfile(path, device=DEV)
        ref = QVBandLinearV8.from_encoded(enc)
        assert lin.bf16_certified == (restore == "fp16+bf16") and not lin.fp16_table_missing
        for k in ("tau_s", "min_s", "nbits", "bit_off", "ids", "esc_idx", "esc_vals", "esc_idx_bf16", "esc_vals_bf16"):
            assert torch.equal(getattr(lin, k), getattr(ref, k)), k
        x = torch.randn(3, 256, generator=torch.Generator().manual_seed(5)).to(torch.float16).to(DEV)
        assert torch.equal(lin(x), ref(x))


def test_same_input_fusion_is_bit_identical():
    import torch.nn as nn
    from qvb8_amd.formats.qvb8.fuse import FusedMember, concat_linears, fuse_same_input
    lins, encs = [], []
    for i, Q in enumerate((96, 40, 33)):
        W = H.synth_weight(Q, 512, seed=20 + i).to(DEV)
        enc = PK.encode_tensor(W, 1e-3, restore="fp16", force_escapes=[3 + i, 512 * (Q - 1) + 500])
        encs.append(enc)
        lins.append(QVBandLinearV8.from_encoded(enc, bias=torch.full((Q,), 0.5 * i, device=DEV) if i != 1 else None))
    fused, splits = concat_linears(lins)
    assert splits == [96, 136] and fused.out_features == 169 and fused.ids.data_ptr() % 16 == 0
    for M, dtype in ((1, torch.bfloat16), (12, torch.float16), (70, torch.bfloat16), (120, torch.float16)):
        x = torch.randn(M, 512, generator=torch.Generator().manual_seed(M)).to(dtype).to(DEV)
        parts = torch.tensor_split(fused(x), splits, -1)
        for part, lin, enc in zip(parts, lins, encs):
            assert torch.equal(part, lin(x)), (M, dtype)
            # and against the oracle, not only against the separate launch
            ref, Wr, xs = _ref(enc, x, saturate=True, narrow="fp16" if M > 256 else None)
            b = lin.bias.double().cpu().numpy() if lin.bias is not None else 0.0
            _close(part, ref + b, Wr, xs, dtype)

    class Attn(nn.Module):
        def __init__(self):
            super().__init__()
            self.q_proj, self.k_proj, self.v_proj = lins
    class Block(nn.Module):
        def __init__(self):
            super().__init__()
            self.self_attn = Attn()
    blk = Block()
    x = torch.randn(2, 512, generator=torch.Generator().manual_seed(9)).to(torch.bfloat16).to(DEV)
    want = [lin(x) for lin in lins]
    assert fuse_same_input(blk) == 1 and isinstance(blk.self_attn.k_proj, FusedMember)
    got = [blk.self_attn.q_proj(x), blk.self_attn.k_proj(x), blk.self_attn.v_proj(x)]
    for a, b in zip(got, want):
        assert torch.equal(a, b)
    assert not blk.self_attn._qvb8_fused.holding()        # every member took its part: nothing is held


@pytest.mark.parametrize("widths,sortable", [([7, 6, 9], True), ([5], True), ([4], True), ([8, 4], True), ([7, 6, 9, 3, 8, 5], False)])
def test_rows_copied_into_width_order(widths, sortable):
    """The module copies its rows once into width-sorted order and then lets the kernel compute row addresses (at most
    three widths; other packs keep the row records).  Either way results match the oracle and the dense restore is
    unchanged by the copy."""
    d = H.mixed_width_pack(70, 256, widths, seed=21)
    d["tau_s"] = d["tau_s"] * (1.0 / 64)
    a = H.to_device_args(d, DEV)
    lin = QVBandLinearV8(min_s=a[1], nbits=a[2], bit_off=a[3], ids=a[0], Q=70, P=256, tau_s=a[5], esc_idx=a[6], esc_vals=a[7])
    from qvb8_amd import ext_qvb8 as ext
    before = ext.decode_f32(lin.ids, lin.min_s, lin.nbits, lin.bit_off, 256, lin.tau_s, lin.esc_idx, lin.esc_vals)
    old_ptr = lin.ids.data_ptr()
    Wr = O.reconstruct(d["min_s"], d["tau_s"], d["ids_dense"], d["esc_idx"], d["esc_vals"])
    for M, dtype in ((1, torch.bfloat16), (20, torch.float16)):
        x = torch.randn(M, 256, generator=torch.Generator().manual_seed(M)).to(dtype).to(DEV)
        y = lin(x)
        xs = O.sat_half(x.float().cpu().numpy())
        _close(y, O.linear_f64(xs, Wr), Wr, xs, dtype)
    perm, rowinfo, layout = lin._mma_order()
    assert (layout is not None) == sortable and (lin.ids.data_ptr() != old_ptr) == sortable
    if sortable:
        assert layout.n_classes == len(set(widths)) and layout.first_pos[layout.n_classes] == 70
        assert bool((lin.nbits[perm.long()][1:] >= lin.nbits[perm.long()][:-1]).all())
    after = ext.decode_f32(lin.ids, lin.min_s, lin.nbits, lin.bit_off, 256, lin.tau_s, lin.esc_idx, lin.esc_vals)
    assert torch.equal(before, after)


def test_plane_tiles_change_no_result_and_survive_moves_subsets_and_fusion(monkeypatch):
    """The operator stores whole tiles in planes when it sorts the rows; results are those of rows kept back to back, bit
    for bit, at every M; a move of the module keeps the row layout; a row subset and a fusion of such modules still read
    the rows; QVB8_PLANES=0 switches the planes off."""
    from qvb8_amd.formats.qvb8.fuse import concat_linears
    enc = PK.encode_tensor(H.synth_weight(520, 1024, seed=11).to(DEV), 1e-3, restore="fp16",
                           force_escapes=[3, 1024 * 100 + 17, 1024 * 519 + 1000])
    flat, tiled = QVBandLinearV8.from_encoded(enc), QVBandLinearV8.from_encoded(enc)
    flat.plane_tiles = False
    xs = {M: torch.randn(M, 1024, generator=torch.Generator().manual_seed(M)).to(torch.bfloat16).to(DEV) for M in (1, 7, 40, 64, 200)}
    want = {M: flat(x) for M, x in xs.items()}
    for M, x in xs.items():
        assert torch.equal(want[M], tiled(x)), M
    assert tiled._planes and not flat._planes
    ref, Wr, x64 = _ref(enc, xs[7], saturate=True)
    _close(want[7], ref, Wr, x64, torch.bfloat16)
    tiled = tiled.to(torch.bfloat16)                          # any _apply drops the launch data; the sorted buffers stay
    assert tiled._mma_order()[2] is not None and tiled._planes
    for M, x in xs.items():
        assert torch.equal(want[M], tiled(x)), M
    rows = torch.arange(519, -1, -3, device=DEV)
    for M in (1, 40):
        assert torch.equal(flat.row_subset(rows)(xs[M]), tiled.row_subset(rows)(xs[M])), M
    enc2 = PK.encode_tensor(H.synth_weight(136, 1024, seed=12).to(DEV), 1e-3, restore="fp16")
    other = QVBandLinearV8.from_encoded(enc2).prepare()
    fused = concat_linears([tiled, other])[0]                 # members already stored in planes: sorted again as one weight
    assert fused._mma_order()[2] is not None and fused._planes
    for M in (1, 20):                                         # the tile kernel on both sides
        x = xs[200][:M].contiguous()
        assert torch.equal(fused(x), torch.cat([tiled(x), other(x)], dim=1)), M
    y = fused(xs[200][:100])
    for e, part in ((enc, y[:, :520]), (enc2, y[:, 520:])):
        ref, Wr, x64 = _ref(e, xs[200][:100], saturate=True)
        _close(part, ref, Wr, x64, torch.bfloat16)
    monkeypatch.setenv("QVB8_PLANES", "0")
    off = QVBandLinearV8.from_encoded(enc)
    assert torch.equal(want[40], off(xs[40])) and not off._planes


@pytest.mark.parametrize("seed", range(10))
def test_plane_tiles_seeded_shapes(seed):
    """Seeded random shapes and width mixes (rows that are no multiple of 16, runs shorter than a tile, widths the slicing
    cannot read, escapes): the operator with whole tiles in planes gives, bit for bit, what it gives with the rows back to
    back, and both agree with the oracle."""
    rng = np.random.default_rng(1000 + seed)
    Q = int(rng.integers(17, 400))
    P = int(rng.choice([128, 256, 384, 512, 1024]))
    pool = [list(range(4, 9)), [6, 7], [7], [5, 6, 7, 8], [4, 8], [6, 9, 7], [3, 6, 7]][int(rng.integers(0, 7))]
    n_kinds = int(rng.integers(1, len(pool) + 1))
    widths = [int(w) for w in rng.choice(pool, size=n_kinds, replace=False)]
    reps = [int(rng.integers(1, 40)) for _ in widths]
    pattern = [w for w, n in zip(widths, reps) for _ in range(n)]
    d = H.mixed_width_pack(Q, P, pattern, seed=seed)
    d["tau_s"] = d["tau_s"] * (1.0 / 64)
    n_esc = int(rng.integers(0, 6))
    if n_esc:
        d["esc_idx"] = np.sort(rng.choice(Q * P, n_esc, replace=False)).astype(np.int64)
        d["esc_vals"] = rng.normal(size=n_esc).astype(np.float32)
    a = H.to_device_args(d, DEV)

    def make(planes):
        m = QVBandLinearV8(min_s=a[1].clone(), nbits=a[2].clone(), bit_off=a[3].clone(), ids=a[0].clone(), Q=Q, P=P, tau_s=a[5].clone(),
                           esc_idx=a[6], esc_vals=a[7])
        m.plane_tiles = planes
        return m
    flat, tiled = make(False), make(True)
    Wr = O.reconstruct(d["min_s"], d["tau_s"], d["ids_dense"], d["esc_idx"], d["esc_vals"])
    for M in (1, 13, 40, 70):
        x = torch.randn(M, P, generator=torch.Generator().manual_seed(seed * 100 + M)).to(torch.bfloat16).to(DEV)
        y0, y1 = flat(x), tiled(x)
        assert torch.equal(y0, y1), (Q, P, pattern[:8], M)
        xs = O.sat_half(x.float().cpu().numpy())
        _close(y1, O.linear_f64(xs, Wr), Wr, xs, torch.bfloat16)
    assert not flat._planes
    from qvb8_amd import ext_qvb8 as ext
    dense = ext.decode_f32(tiled.ids, tiled.min_s, tiled.nbits, tiled.bit_off, P, tiled.tau_s, tiled.esc_idx, tiled.esc_vals)
    assert np.array_equal(dense.cpu().numpy().view(np.uint32), Wr.astype(np.float32).view(np.uint32))


@pytest.mark.parametrize("P,M", [(6144, 1), (6144, 8), (12288, 1), (12288, 3)])
def test_plane_tiles_long_rows_agree_with_the_oracle(P, M):
    """Rows beyond 4096 columns: with the rows in planes a workgroup may have twelve waves, so a row's partial sums are
    grouped differently than with the rows back to back and the two products may differ in the last bit -- each of them
    stays inside the oracle's bound, and the restored weight is the same bit for bit."""
    Q = 72
    d = H.mixed_width_pack(Q, P, [6] * 40 + [7] * 32, seed=P + M)
    d["tau_s"] = d["tau_s"] * (1.0 / 64)
    a = H.to_device_args(d, DEV)
    Wr = O.reconstruct(d["min_s"], d["tau_s"], d["ids_dense"], d["esc_idx"], d["esc_vals"])
    x = torch.randn(M, P, generator=torch.Generator().manual_seed(P + M)).to(torch.bfloat16).to(DEV)
    xs = O.sat_half(x.float().cpu().numpy())
    for planes in (False, True):
        m = QVBandLinearV8(min_s=a[1].clone(), nbits=a[2].clone(), bit_off=a[3].clone(), ids=a[0].clone(), Q=Q, P=P, tau_s=a[5].clone(),
                           esc_idx=a[6], esc_vals=a[7])
        m.plane_tiles = planes
        y = m(x)
        assert m._planes == planes
        _close(y, O.linear_f64(xs, Wr), Wr, xs, torch.bfloat16)
        from qvb8_amd import ext_qvb8 as ext
        dense = ext.decode_f32(m.ids, m.min_s, m.nbits, m.bit_off, P, m.tau_s, m.esc_idx, m.esc_vals)
        assert np.array_equal(dense.cpu().numpy().view(np.uint32), Wr.astype(np.float32).view(np.uint32))
