"""GPU parity of the QVB8R path (walk + dense restore, fused product, escape correction, module) against the oracle:
restored weights bit-exact with the QVB8 restore of the same ids, products within the GEMV tolerance."""
import numpy as np
import pytest
import torch

from oracle import qvb8_oracle as O
from oracle import qvb8r_oracle as R
from qvb8_amd import ext_qvb8 as ext8
from qvb8_amd import ext_qvb8r as ext
from qvb8_amd.formats.qvb8 import pack as PK
from qvb8_amd.formats.qvb8r import pack as RP
from qvb8_amd.formats.qvb8r.module import QVBandLinearV8R
from tests import helpers as H

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _make(Q, P, tau, seed, restore="fp16", force=None, **kw):
    W = H.synth_weight(Q, P, seed=seed).to(DEV)
    enc = PK.encode_tensor(W, tau, restore=restore, force_escapes=force, keep_ids=True)
    d = RP.transcode(enc, **kw)
    return W, enc, d


@pytest.mark.parametrize("Q,P,kw", [(64, 512, dict(rows_per_tile=3, n_classes=2)), (37, 128, dict(rows_per_tile=1)),
                                     (300, 1024, dict()), (20, 5120, dict(rows_per_tile=2)), (9, 8192, dict())])
def test_restore_bit_exact_and_ids(Q, P, kw):
    W, enc, d = _make(Q, P, 2e-3, seed=Q + P, force=[3, P * (Q - 1) + 77], **kw)
    lin = QVBandLinearV8R(d, device=DEV)
    want_ids = enc["ids_dense"].cpu().numpy().astype(np.int64)
    assert np.array_equal(R.ids(d), want_ids)                                  # the oracle's walk reads the stream back
    got_ids = ext.ids(P, *lin._core(), T=lin.T).cpu().numpy().astype(np.int64)
    assert np.array_equal(got_ids, want_ids)
    v8 = H.oracle_view(enc)
    for dt, narrow, tab in ((torch.float32, lambda a: a, False), (torch.float16, O.narrow_fp16, False), (torch.bfloat16, O.narrow_bf16, True)):
        ei, ev = (enc["esc_idx_bf16"], enc["esc_vals_bf16"]) if tab else (enc["esc_idx"], enc["esc_vals"])
        ref = narrow(O.reconstruct(v8["min_s"], v8["tau_s"], want_ids, ei.cpu().numpy(), ev.cpu().numpy()))
        got = lin.dense(dt).float().cpu().numpy()
        assert np.array_equal(got.view(np.uint32), ref.astype(np.float32).view(np.uint32)), dt
    # the certificate carries over: re-checked on the GPU against the original weights
    max_err, bad = ext8.certify(lin.dense(torch.float16), W, 2e-3)
    assert bad == 0 and max_err < 2e-3
    # compact chunk of a block range
    blocks = lin.blocks8.cpu().numpy()
    if len(blocks) > 1:
        b0, nb = 1, len(blocks) - 1
        t0 = int(blocks[b0, 1])
        base = int(lin.tiles[t0, 1])
        rows = Q - base
        Wc = ext.decode(*lin._core(), P, 2, b0, nb, base, rows, T=lin.T).cpu().numpy()
        full = lin.dense(torch.float32).cpu().numpy()
        band = O.reconstruct(v8["min_s"], v8["tau_s"], want_ids, np.zeros(0, np.int64), np.zeros(0, np.float32))
        assert np.array_equal(Wc.view(np.uint32), band[d["perm"][base:base + rows]].view(np.uint32))
        assert full.shape == (Q, P)


@pytest.mark.parametrize("M", [1, 2, 3, 4, 7, 8, 9, 16, 17, 31, 48])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
def test_product_small_m(M, dtype):
    Q, P = 150, 1024
    W, enc, d = _make(Q, P, 2e-3, seed=5, force=[10, P * 149 + 1023, P * 77 + 512], rows_per_tile=3)
    lin = QVBandLinearV8R(d, device=DEV)
    x = torch.randn(M, P, generator=torch.Generator().manual_seed(M)).to(dtype).to(DEV)
    x[0, 5] = 1.0e5 if dtype != torch.float16 else 6.0e4                     # no narrowing on this path: used as it is
    y = lin(x)
    assert y.dtype == dtype and y.shape == (M, Q)
    Wr = R.reconstruct(d, enc["esc_idx"].cpu().numpy(), enc["esc_vals"].cpu().numpy())
    xs = x.float().cpu().numpy()
    ref = O.linear_f64(xs, Wr)
    eps = {torch.float32: 0.0, torch.float16: 2.0 ** -11, torch.bfloat16: 2.0 ** -8}[dtype]
    tol = H.gemv_tolerance(ref, Wr, xs) + eps * np.abs(ref)
    diff = np.abs(y.float().cpu().numpy().astype(np.float64) - ref)
    assert np.all(diff <= tol), (float(diff.max()), float((diff / tol).max()))
    assert torch.equal(y, lin(x))                                             # reproducible


@pytest.mark.parametrize("Q,P", [(12, 28672), (40, 8192)])
def test_65b_row_lengths_against_the_oracle(Q, P):
    """Rows as long as the large-dense configuration's (hidden 8192, FFN 28672; one row per tile there): ids and restore
    bit for bit against the oracle's walk, the product of 1 and 16 rows against restore + float64 matmul."""
    W, enc, d = _make(Q, P, 2e-3, seed=Q + P, force=[5, P * (Q - 1) + P - 1])
    assert d["T"] == 1
    lin = QVBandLinearV8R(d, device=DEV)
    want_ids = R.ids(d)
    assert np.array_equal(want_ids, enc["ids_dense"].cpu().numpy().astype(np.int64))
    assert np.array_equal(ext.ids(P, *lin._core(), T=lin.T).cpu().numpy().astype(np.int64), want_ids)
    Wr = R.reconstruct(d, enc["esc_idx"].cpu().numpy(), enc["esc_vals"].cpu().numpy())
    assert np.array_equal(lin.dense(torch.float32).cpu().numpy().view(np.uint32), Wr.view(np.uint32))
    assert np.array_equal(lin.dense(torch.float16).cpu().numpy().view(np.uint16), O.narrow_fp16(Wr).astype(np.float16).view(np.uint16))
    for M in (1, 16):
        x = torch.randn(M, P, generator=torch.Generator().manual_seed(M)).to(torch.bfloat16).to(DEV)
        y = lin(x)
        xs = x.float().cpu().numpy()
        ref = O.linear_f64(xs, Wr)
        tol = H.gemv_tolerance(ref, Wr, xs) + 2.0 ** -8 * np.abs(ref)
        diff = np.abs(y.float().cpu().numpy().astype(np.float64) - ref)
        assert np.all(diff <= tol), (M, float((diff / tol).max()))


def test_walk_probe_walks_the_symbols_of_the_product_kernel():
    """The measurement aid that times the walk alone: it leaves, per row, tau_s times the sum over the 32 lanes of the
    exclusive-or of (symbol of the even step + symbol of the odd step) over the lane's step pairs -- the same symbols, in
    the same lanes, as the product kernel multiplies (symbol = id - the row's delta).  Nothing else is read: X is absent."""
    import ctypes
    from qvb8_amd import _lib
    Q, P = 90, 768
    W, enc, d = _make(Q, P, 2e-3, seed=21, rows_per_tile=4, n_classes=2)
    lin = QVBandLinearV8R(d, device=DEV)
    core = lin._core()
    c, _, _ = ext._core(*core, P)
    Y = torch.full((1, Q), float("nan"), dtype=torch.float32, device=DEV)
    lib = _lib.load()
    assert lib.qvb8r_walk_probe(ctypes.byref(c), lin.T, Y.data_ptr(), torch.cuda.current_stream().cuda_stream) == 0
    ids = ext.ids(P, *core, T=lin.T).cpu().numpy().astype(np.int64)
    drow = core[9].cpu().numpy().astype(np.int64)
    sym = (ids - drow[:, None]).reshape(Q, P // 64, 2, 32)
    assert sym.min() >= 0
    keep = np.bitwise_xor.reduce(sym[:, :, 0, :] + sym[:, :, 1, :], axis=1)          # [row, lane]
    want = (lin.tau_s.cpu().numpy().astype(np.float64) * keep.sum(1).astype(np.float64)).astype(np.float32)
    assert np.array_equal(Y.cpu().numpy()[0].view(np.uint32), want.view(np.uint32))
    assert lib.qvb8r_walk_probe(ctypes.byref(c), 0, Y.data_ptr(), None) != 0                    # bad rows-per-tile bound


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_matrix_core_rows_agree_with_single_row_walk(dtype):
    """Every row of a many-row call against the one-row kernel on the same row: the two differ only in the order of the
    fp32 additions (and, for fp32 X, in the 22-bit hi + lo split), far inside the product tolerance.  Row scales that
    differ by 2^40 between rows, a zero row and a ragged last batch (P = 640 is not a multiple of 256) are in."""
    Q, P, M = 100, 640, 21
    W, enc, d = _make(Q, P, 2e-3, seed=11, rows_per_tile=5, n_classes=2)
    lin = QVBandLinearV8R(d, device=DEV)
    x = torch.randn(M, P, generator=torch.Generator().manual_seed(3))
    x[3] *= 2.0 ** 20; x[4] *= 2.0 ** -20; x[5] = 0.0
    x = x.to(dtype).to(DEV)
    core = lin._core()
    many = ext.multi(x, *core, T=lin.T)
    for m in range(M):
        one = ext.gemv(x[m], *core, T=lin.T)
        scale = float(x[m].float().abs().max()) * float(P) * 2047.0 * float(lin.tau_s.abs().max())
        assert float((many[m] - one).abs().max()) <= 2.0 ** -18 * scale + 0.0, m
    assert float(many[5].abs().max()) == 0.0


def test_module_large_m_paths_and_packfile(tmp_path):
    Q, P = 96, 512
    W, enc, d = _make(Q, P, 2e-3, seed=8, force=[1, P * 50 + 3], rows_per_tile=4, n_classes=2)
    path = str(tmp_path / "t.qvb8r")
    RP.write_pack(path, d)
    bias = torch.linspace(-1, 1, Q)
    lin = QVBandLinearV8R.from_packfile(path, bias=bias, device=DEV)
    lin.CHUNK_BYTES = 2 * P * 40                                             # force several chunks
    lin.__init__(dict(RP.container.read(path)), bias=bias, device=DEV, path=path)
    assert len(lin.chunks) > 1
    Wr = R.reconstruct(d, enc["esc_idx"].cpu().numpy(), enc["esc_vals"].cpu().numpy())
    for M, dtype in ((30, torch.bfloat16), (70, torch.float16), (70, torch.float32)):
        x = torch.randn(M, P, generator=torch.Generator().manual_seed(M)).to(dtype).to(DEV)
        y = lin(x)
        xs = x.float().cpu().numpy()
        Wm = O.narrow_fp16(Wr) if M > 48 else Wr
        if M > 48:
            xs = O.sat_half(xs)
        ref = O.linear_f64(xs, Wm) + bias.double().numpy()
        eps = {torch.float32: 0.0, torch.float16: 2.0 ** -11, torch.bfloat16: 2.0 ** -8}[dtype]
        tol = H.gemv_tolerance(ref, Wm, xs) + eps * np.abs(ref)
        diff = np.abs(y.float().cpu().numpy().astype(np.float64) - ref)
        assert np.all(diff <= tol), (M, dtype, float((diff / tol).max()))
    before = lin.tau_s.clone()
    lin.to(torch.bfloat16)
    assert lin.tau_s.dtype == torch.float32 and torch.equal(lin.tau_s, before)


def test_argument_errors():
    W, enc, d = _make(16, 256, 2e-3, seed=2)
    lin = QVBandLinearV8R(d, device=DEV)
    with pytest.raises(RuntimeError):
        ext.multi(torch.zeros(49, 256, device=DEV), *lin._core(), T=lin.T)
    with pytest.raises(RuntimeError):
        ext.multi(torch.zeros(2, 256), *lin._core(), T=lin.T)               # host tensor
    with pytest.raises(RuntimeError):
        ext.decode(*lin._core(), 256, 2, 0, 99, -1, 0, T=lin.T)             # block range outside the schedule
    short = lin.words[:100].contiguous()
    with pytest.raises(RuntimeError):
        ext.gemv(torch.zeros(256, device=DEV), short, *lin._core()[1:], T=lin.T)   # stream without its pad


def test_same_input_fusion_against_the_oracle_and_the_members():
    """q/k/v-like siblings (different row counts, alphabets and tile heights, one with a bias, escapes in two) joined into
    one walk: every member's output equals its own launch bit for bit and the oracle's restore + float64 matmul within
    the product tolerance; the registry's finalize hook does the replacement on a model."""
    import torch.nn as nn
    from qvb8_amd.common import formats as F
    from qvb8_amd.common.fusion import FusedMember
    from qvb8_amd.formats.qvb8r.fuse import concat_linears
    P = 512
    lins, Wrs = [], []
    for i, (Q, kw, force) in enumerate(((96, dict(rows_per_tile=4, n_classes=2), [7, P * 90 + 500]), (40, dict(rows_per_tile=1), None),
                                        (33, dict(), [P * 32 + 1]))):
        W, enc, d = _make(Q, P, 2e-3, seed=70 + i, force=force, **kw)
        lins.append(QVBandLinearV8R(d, bias=torch.full((Q,), 0.25) if i == 1 else None, device=DEV))
        Wrs.append(R.reconstruct(d, enc["esc_idx"].cpu().numpy(), enc["esc_vals"].cpu().numpy()))
    fused, splits = concat_linears(lins)
    assert splits == [96, 136] and fused.out_features == 169
    for M, dtype in ((1, torch.bfloat16), (5, torch.float32), (20, torch.float16), (60, torch.bfloat16)):
        x = torch.randn(M, P, generator=torch.Generator().manual_seed(M)).to(dtype).to(DEV)
        parts = torch.tensor_split(fused(x), splits, -1)
        xs = x.float().cpu().numpy()
        for i, (part, lin, Wr) in enumerate(zip(parts, lins, Wrs)):
            if M <= 48:
                assert torch.equal(part, lin(x)), (M, dtype, i)
            Wm, xm = (O.narrow_fp16(Wr), O.sat_half(xs)) if M > 48 else (Wr, xs)
            ref = O.linear_f64(xm, Wm) + (lin.bias.double().cpu().numpy() if lin.bias is not None else 0.0)
            eps = {torch.float32: 0.0, torch.float16: 2.0 ** -11, torch.bfloat16: 2.0 ** -8}[dtype]
            tol = H.gemv_tolerance(ref, Wm, xm) + eps * np.abs(ref)
            diff = np.abs(part.float().cpu().numpy().astype(np.float64) - ref)
            assert np.all(diff <= tol), (M, dtype, i, float((diff / tol).max()))

    class Attn(nn.Module):
        def __init__(self):
            super().__init__()
            self.q_proj, self.k_proj, self.v_proj = lins
    class Block(nn.Module):
        def __init__(self):
            super().__init__()
            self.self_attn = Attn()
    blk = Block()
    x = torch.randn(2, P, generator=torch.Generator().manual_seed(9)).to(torch.bfloat16).to(DEV)
    want = [lin(x) for lin in lins]
    assert F.get_format("qvb8r").finalize(blk) == 1 and isinstance(blk.self_attn.k_proj, FusedMember)
    got = [blk.self_attn.q_proj(x), blk.self_attn.k_proj(x), blk.self_attn.v_proj(x)]
    for a, b in zip(got, want):
        assert torch.equal(a, b)
    assert not blk.self_attn._qvb8r_fused.holding()


@pytest.mark.parametrize("out_dtype", [torch.bfloat16, torch.float16, torch.float32])
def test_embedding_rows_walked_on_the_gpu(out_dtype, tmp_path):
    """QVBandEmbeddingV8R: looked-up rows (repeats, any order, 2-D index) equal the oracle's two-rounding lookup value over
    the oracle's walk of the same stream, escapes written over it, bit for bit; `weight` is every row; an index outside
    the table raises; the registry hands the class out for the format."""
    from qvb8_amd.common import formats as F
    from qvb8_amd.formats.qvb8r.module import QVBandEmbeddingV8R
    Q, P = 300, 640
    W, enc, d = _make(Q, P, 2e-3, seed=3, force=[5, P * 17 + 600, P * 299 + 1], rows_per_tile=3, n_classes=2)
    path = str(tmp_path / "emb.qvb8r")
    RP.write_pack(path, d)
    assert F.get_format("qvb8r").embedding is QVBandEmbeddingV8R
    emb = QVBandEmbeddingV8R.from_packfile(path, out_dtype=out_dtype, device=DEV)
    tok = torch.tensor([[17, 0, 299, 17], [5, 123, 298, 0]], device=DEV)
    got = emb(tok)
    assert got.dtype == out_dtype and got.shape == (2, 4, P)
    name = {torch.bfloat16: "bf16", torch.float16: "fp16", torch.float32: "fp32"}[out_dtype]
    ref = O.embedding_rows(tok.cpu().numpy().reshape(-1), d["min_s"], d["tau_s"], R.ids(d), P, d["esc_idx"], d["esc_val"], dtype=name)
    assert np.array_equal(got.float().cpu().numpy().reshape(-1, P).view(np.uint32), ref.astype(np.float32).view(np.uint32))
    full = emb.weight
    ref_all = O.embedding_rows(np.arange(Q), d["min_s"], d["tau_s"], R.ids(d), P, d["esc_idx"], d["esc_val"], dtype=name)
    assert np.array_equal(full.float().cpu().numpy().view(np.uint32), ref_all.astype(np.float32).view(np.uint32))
    with pytest.raises(IndexError):
        emb(torch.tensor([Q], device=DEV))
    before = emb.tau_s.clone()
    emb.to(torch.bfloat16)
    assert emb.tau_s.dtype == torch.float32 and torch.equal(emb.tau_s, before)
