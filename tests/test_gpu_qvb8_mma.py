"""GPU parity of the matrix-core path (qvb8_mma through ext.mma_tiles / ext.mma_multi) against the CPU oracle."""
import numpy as np
import pytest
import torch

from oracle import qvb8_oracle as O
from qvb8_amd import ext_qvb8 as ext
from qvb8_amd.formats.qvb8 import pack as PK
from tests import helpers as H

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _x(M, P, dtype, seed):
    g = torch.Generator().manual_seed(seed)
    return torch.randn(M, P, generator=g).to(dtype).to(DEV)


def _perm_by_width(nbits: torch.Tensor):
    return torch.argsort(nbits.to(torch.int16), stable=True).to(torch.int32)


def _check(d, args, x, y, saturate_ref):
    ids = H.oracle_ids(d) if "ids_dense" not in d else d["ids_dense"]
    Wr = O.reconstruct(d["min_s"], d["tau_s"], ids, d["esc_idx"], d["esc_vals"])
    xs = x.float().cpu().numpy()
    if saturate_ref:
        xs = O.sat_half(xs)
    ref = O.linear_f64(xs, Wr)
    tol = H.gemv_tolerance(ref, Wr, xs)
    diff = np.abs(y.cpu().numpy().astype(np.float64) - ref)
    assert y.dtype == torch.float32 and tuple(y.shape) == ref.shape
    assert np.all(diff <= tol), (float(diff.max()), float((diff / tol).max()), np.argwhere(diff > tol)[:5])
    return float((diff / tol).max())


@pytest.mark.parametrize("M", [1, 2, 5, 8, 15, 16, 17, 31, 32, 33, 48])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_mma_all_m(M, dtype):
    W = H.synth_weight(272, 4096, seed=M).to(DEV)          # 17 tiles: the last is ragged
    enc = PK.encode_tensor(W, 1e-3, restore="fp16+bf16")
    x = _x(M, 4096, dtype, M)
    perm = _perm_by_width(enc["nbits"])
    for p in (None, perm):
        y = ext.mma_tiles(x, *H.pack_args(enc), perm=p, saturate=False)
        _check(H.oracle_view(enc), None, x, y, saturate_ref=False)


@pytest.mark.parametrize("M,P", [(1, 4096), (3, 4096), (8, 4096), (1, 12288), (1, 17408), (2, 5120), (1, 28672),
                                 (9, 3072), (12, 2048), (16, 2048), (16, 1024), (13, 1280), (4, 12288), (5, 12288), (3, 17408)])
def test_activations_through_lds_change_no_bit(M, P, monkeypatch):
    """Small X is staged through LDS once (1, 4, 8 or 16 sixteen-byte pieces per thread; up to 8 rows whatever fits, more
    rows up to 64 KB); the same call with that path switched off fetches X per wave and panel in memory order and turns it
    into operand order through the wave's own piece of LDS -- the path every larger X takes (9..16 rows of 4096 columns,
    6.. rows of 12288).  Same arithmetic in the same order: identical bits."""
    W = H.synth_weight(80, P, seed=P + M).to(DEV)
    enc = PK.encode_tensor(W, 1e-3, restore="fp16", force_escapes=[9, P * 79 + P - 1])
    perm = _perm_by_width(enc["nbits"])
    for dtype, saturate in ((torch.bfloat16, True), (torch.float16, False), (torch.bfloat16, False)):
        x = _x(M, P, dtype, 7 * M)
        monkeypatch.setenv("QVB8_TILE_X_LDS", "1")
        y1 = ext.mma_tiles(x, *H.pack_args(enc), perm=perm, saturate=saturate)
        monkeypatch.setenv("QVB8_TILE_X_LDS", "0")
        y0 = ext.mma_tiles(x, *H.pack_args(enc), perm=perm, saturate=saturate)
        assert torch.equal(y1, y0), (dtype, saturate)
    _check(H.oracle_view(enc), None, x, y1, saturate_ref=False)


@pytest.mark.parametrize("M", [2, 5, 9, 12, 16])
def test_rows_in_planes_and_both_ways_of_fetching_x(M, monkeypatch):
    """The module's default storage (rows in planes, width order): X through LDS as a whole against X fetched per wave, bit
    for bit, and both against the oracle.  9 and more rows of 12288 columns exceed what LDS takes as a whole: that weight
    then takes the per-wave path either way and is checked against the oracle alone."""
    from qvb8_amd.formats.qvb8.module import QVBandLinearV8
    for Q, P in ((272, 2048), (96, 12288)):
        W = H.synth_weight(Q, P, seed=Q + M).to(DEV)
        enc = PK.encode_tensor(W, 1e-3, restore="fp16")
        lin = QVBandLinearV8.from_encoded(enc)
        x = _x(M, P, torch.bfloat16, 5 * M)
        monkeypatch.setenv("QVB8_TILE_X_LDS", "1")
        y1 = lin(x)
        monkeypatch.setenv("QVB8_TILE_X_LDS", "0")
        y0 = lin(x)
        assert torch.equal(y1, y0), (Q, P)
        d = H.oracle_view(enc)
        Wr = O.reconstruct(d["min_s"], d["tau_s"], d["ids_dense"] if "ids_dense" in d else H.oracle_ids(d), d["esc_idx"], d["esc_vals"])
        xs = O.sat_half(x.float().cpu().numpy())
        ref = O.linear_f64(xs, Wr)
        tol = H.gemv_tolerance(ref, Wr, xs) + 2.0 ** -8 * np.abs(ref)           # the module rounds to the caller's bf16
        diff = np.abs(y1.float().cpu().numpy().astype(np.float64) - ref)
        assert y1.dtype == torch.bfloat16 and np.all(diff <= tol), (Q, P, float((diff / tol).max()))


@pytest.mark.parametrize("Q,P,tau", [(1024, 4096, 1e-3), (200, 12288, 1e-3), (130, 768, 2e-3), (96, 2048, 2e-3),
                                     (64, 5120, 2e-3), (40, 17408, 2e-3), (24, 28672, 2e-3), (16, 128, 1e-3), (3, 256, 1e-3)])
def test_mma_shapes(Q, P, tau):
    W = H.synth_weight(Q, P, seed=P).to(DEV)
    enc = PK.encode_tensor(W, tau, restore="fp16+bf16")
    perm = _perm_by_width(enc["nbits"])
    for M, dtype in ((1, torch.bfloat16), (16, torch.float16), (24, torch.bfloat16)):
        x = _x(M, P, dtype, Q)
        y = ext.mma_tiles(x, *H.pack_args(enc), perm=perm, saturate=False)
        _check(H.oracle_view(enc), None, x, y, saturate_ref=False)


@pytest.mark.parametrize("Q,P,widths", [(40, 2176, [4, 5, 6, 7, 8]), (35, 128, list(range(1, 15))), (33, 4096, [7, 9, 6, 3]),
                                        (20, 6144, [7, 3, 12]), (64, 1024, [8]), (48, 1024, [4])])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_mma_mixed_widths_and_per_element_rows(Q, P, widths, dtype):
    d = H.mixed_width_pack(Q, P, widths, seed=11)
    args = H.to_device_args(d, DEV)
    for M in (1, 7, 20):
        x = _x(M, P, dtype, 3)
        for perm in (None, _perm_by_width(args[2])):
            y = ext.mma_tiles(x, *args, perm=perm, saturate=False)
            _check(d, None, x, y, saturate_ref=False)


def test_mma_escapes_and_determinism():
    W = H.synth_weight(128, 4096, seed=11).to(DEV)
    W[3, 17] = 1.5
    W[3, 4000] = -2.0
    W[90, 0] = 0.8
    enc = PK.encode_tensor(W, 1e-3, restore="fp16", max_nbits=7, force_escapes=[5 * 4096 + 9, 5 * 4096 + 10])
    assert enc["esc_idx"].numel() >= 5
    for M in (1, 12, 40):
        x = _x(M, 4096, torch.bfloat16, 5)
        y1 = ext.mma_tiles(x, *H.pack_args(enc), saturate=False)
        y2 = ext.mma_tiles(x, *H.pack_args(enc), saturate=False)
        assert torch.equal(y1, y2)
        _check(H.oracle_view(enc), None, x, y1, saturate_ref=False)


def test_mma_multi_reference_signature():
    W = H.synth_weight(256, 1024, seed=4).to(DEV)
    enc = PK.encode_tensor(W, 1e-3, restore="fp16+bf16")
    perm = _perm_by_width(enc["nbits"])
    tile_nb = torch.zeros((256 + 15) // 16, dtype=torch.int32, device=DEV)
    x32 = torch.randn(9, 1024, device=DEV) * 3
    x32[0, 0] = 1e6                                            # saturates in fp16 mode
    y = ext.mma_multi(x32, *H.pack_args(enc), perm, tile_nb)
    _check(H.oracle_view(enc), None, x32, y, saturate_ref=True)
    xb = x32.bfloat16()
    yb = ext.mma_multi(xb, *H.pack_args(enc, bf16_table=True), perm, tile_nb, True, None, 0)
    _check(H.oracle_view(enc, bf16_table=True), None, xb, yb, saturate_ref=False)
    with pytest.raises(RuntimeError, match="outside 1..48"):
        ext.mma_multi(torch.randn(49, 1024, device=DEV), *H.pack_args(enc), perm, tile_nb)
    Wodd = H.synth_weight(16, 192, seed=1).to(DEV)
    eo = PK.encode_tensor(Wodd, 1e-3)
    with pytest.raises(RuntimeError, match="P%128==0"):
        ext.mma_multi(torch.randn(2, 192, device=DEV), *H.pack_args(eo), None, None)


@pytest.mark.parametrize("M", [1, 7, 16, 20, 40])
def test_mma_bf16_activations_narrowed_on_load(M):
    """bf16 X with saturate=True: the kernel narrows X like saturating_half (clamp to +-65504, fp16, NaN kept) in
    registers; the oracle does the same narrowing on the CPU and multiplies the fp32 band value."""
    W = H.synth_weight(150, 2048, seed=40 + M).to(DEV)
    enc = PK.encode_tensor(W, 1e-3, restore="fp16", force_escapes=[5, 2048 * 3 + 17, 2048 * 149 + 2047])
    x = _x(M, 2048, torch.bfloat16, 90 + M)
    x[0, 3] = 3.0e5                                            # clamps to 65504
    x[M - 1, 100] = -1.0e30                                    # clamps to -65504
    x[0, 7] = 1.0e-6                                           # an fp16 subnormal after narrowing
    perm = _perm_by_width(enc["nbits"])
    y = ext.mma_tiles(x, *H.pack_args(enc), perm=perm, saturate=True)
    _check(H.oracle_view(enc), None, x, y, saturate_ref=True)
    # the unsaturated mode sees the huge activations as they are: the two modes must differ there
    y2 = ext.mma_tiles(x, *H.pack_args(enc), perm=perm, saturate=False)
    assert not torch.allclose(y[0], y2[0])
    xn = x.clone()
    xn[0, 11] = float("nan")
    yn = ext.mma_tiles(xn, *H.pack_args(enc), perm=perm, saturate=True)
    assert torch.isnan(yn[0]).all() and (M == 1 or not torch.isnan(yn[1:]).any())


# ---- 49..256 rows of X: the workgroup-tiled decode + GEMM kernel behind the same entry point ------------------------------

def _sorted_pack(d):
    """Device arguments of a hand-made pack with its rows copied into width order + row records + layout."""
    a = H.to_device_args(d, DEV)
    ids, min_s, nbits, bit_off, P, tau_s, ei, ev = a
    perm = _perm_by_width(nbits)
    srt = ext.sort_rows_by_width(ids, nbits, bit_off, P, perm)
    assert srt is not None
    ids, bit_off, layout = srt
    rowinfo = ext.mma_prepare(nbits, bit_off, tau_s, min_s, P, ids.numel(), perm)
    return (ids, min_s, nbits, bit_off, P, tau_s, ei, ev), perm, rowinfo, layout


@pytest.mark.parametrize("M", [33, 49, 64, 65, 100, 128, 129, 256])
@pytest.mark.parametrize("mode", ["fp16", "bf16_saturated", "bf16_operands"])
def test_gemm_many_rows(M, mode):
    """Three widths in one weight (each run of equal widths fills only part of its 256-row block), an odd number of
    256-column groups (uneven column ranges), token counts on both sides of the 64- and 128-row blocks."""
    Q, P = 300, 768
    widths = [7, 6, 5] if mode == "bf16_operands" else [8, 7, 4]
    d = H.mixed_width_pack(Q, P, widths, seed=M)
    d["tau_s"] = d["tau_s"] * (1.0 / 64)
    args, perm, rowinfo, layout = _sorted_pack(d)
    dtype = torch.float16 if mode == "fp16" else torch.bfloat16
    x = _x(M, P, dtype, M)
    if mode == "bf16_saturated":
        x[0, 3] = 1.0e5                                                      # narrowed to 65504 on the way into LDS
    y = ext.mma_tiles(x, *args, perm=perm, saturate=mode != "bf16_operands", rowinfo=rowinfo, layout=layout)
    _check(d, None, x, y, saturate_ref=mode == "bf16_saturated")
    # against the 16-row tile kernel on the same rows: only the order of the fp32 additions differs
    for m0 in (0, M - 7):
        small = ext.mma_tiles(x[m0:m0 + 7].contiguous(), *args, perm=perm, saturate=mode != "bf16_operands", rowinfo=rowinfo, layout=layout)
        ref = np.abs(small.cpu().numpy()).max() + 1e-30
        assert float((y[m0:m0 + 7] - small).abs().max()) <= 1e-4 * ref
    assert torch.equal(y, ext.mma_tiles(x, *args, perm=perm, saturate=mode != "bf16_operands", rowinfo=rowinfo, layout=layout))


@pytest.mark.parametrize("M", [1, 16, 40, 64, 100, 256])
@pytest.mark.parametrize("out_dtype", [torch.float16, torch.bfloat16])
def test_results_stored_as_16_bit_are_the_rounded_fp32_results(M, out_dtype):
    """QVB8_MMA_Y_F16 / _BF16 on every kernel behind qvb8_mma (tile kernel, both GEMM kernels, one and several column
    ranges): bit for bit what casting the fp32 result gives; refused for a weight with escapes."""
    for Q, P in ((300, 768), (136, 2048)):
        d = H.mixed_width_pack(Q, P, [7, 6, 5], seed=3 * M + Q)
        d["tau_s"] = d["tau_s"] * (1.0 / 64)
        args, perm, rowinfo, layout = _sorted_pack(d)
        x = _x(M, P, torch.bfloat16, M)
        kw = dict(perm=perm, saturate=True, rowinfo=rowinfo, layout=layout)
        y32 = ext.mma_tiles(x, *args, **kw)
        y16 = ext.mma_tiles(x, *args, out_dtype=out_dtype, **kw)
        assert y16.dtype == out_dtype and torch.equal(y16, y32.to(out_dtype))
    with_esc = list(args)
    with_esc[6] = torch.tensor([5], dtype=torch.int64, device=DEV)
    with_esc[7] = torch.tensor([0.25], dtype=torch.float32, device=DEV)
    with pytest.raises(RuntimeError):
        ext.mma_tiles(x, *with_esc, out_dtype=out_dtype, **kw)


def test_gemm_needs_layout_and_sliceable_widths():
    d = H.mixed_width_pack(64, 256, [9, 6], seed=1)
    args, perm, rowinfo, layout = _sorted_pack(d)
    x = _x(64, 256, torch.float16, 1)
    d2 = H.mixed_width_pack(64, 384, [6], seed=2)
    args2, perm2, rowinfo2, layout2 = _sorted_pack(d2)
    with pytest.raises(RuntimeError):
        ext.mma_tiles(_x(64, 384, torch.float16, 2), *args2, perm=perm2, rowinfo=rowinfo2, layout=layout2)   # P % 256 != 0
    with pytest.raises(RuntimeError):
        ext.mma_tiles(x, *args, perm=perm, rowinfo=rowinfo, layout=layout)   # width 9 is not sliced
    with pytest.raises(RuntimeError):
        ext.mma_tiles(x, *args, perm=perm, rowinfo=rowinfo, layout=None)     # M > 48 without a layout
    y = ext.mma_tiles(x[:48].contiguous(), *args, perm=perm, rowinfo=rowinfo, layout=layout)   # the tile kernel reads any width
    _check(d, None, x[:48], y, saturate_ref=False)


@pytest.mark.parametrize("Q,P,M", [(4096, 4096, 256), (1024, 12288, 64), (6144, 4096, 96)])
def test_gemm_real_shapes_with_escapes(Q, P, M):
    """Encoder-made packs at projection shapes (column ranges split over workgroups, two token blocks), escapes included,
    through the operator: bf16 in, bf16 out."""
    from qvb8_amd.formats.qvb8.module import QVBandLinearV8
    W = H.synth_weight(Q, P, seed=Q + M).to(DEV)
    enc = PK.encode_tensor(W, 1e-3, restore="fp16", force_escapes=[5, P * (Q // 2) + 77, P * (Q - 1) + P - 1])
    lin = QVBandLinearV8.from_encoded(enc)
    x = _x(M, P, torch.bfloat16, Q)
    y = lin(x)
    assert y.dtype == torch.bfloat16 and tuple(y.shape) == (M, Q)
    assert lin._gemm_ok(lin._mma_order()[2], False)
    v8 = H.oracle_view(enc)
    Wr = O.reconstruct(v8["min_s"], v8["tau_s"], H.oracle_ids(v8), v8["esc_idx"], v8["esc_vals"])
    xs = O.sat_half(x.float().cpu().numpy())
    ref = O.linear_f64(xs, Wr)
    tol = H.gemv_tolerance(ref, Wr, xs) + 2.0 ** -8 * np.abs(ref)
    diff = np.abs(y.float().cpu().numpy().astype(np.float64) - ref)
    assert np.all(diff <= tol), (float(diff.max()), float((diff / tol).max()))


def _sorted_planes(d):
    """As _sorted_pack, with every whole tile of one width stored in planes."""
    a = H.to_device_args(d, DEV)
    ids, min_s, nbits, bit_off, P, tau_s, ei, ev = a
    perm = _perm_by_width(nbits)
    srt = ext.sort_rows_by_width(ids, nbits, bit_off, P, perm, planes=True)
    assert srt is not None
    ids, bit_off, layout = srt
    assert ext.rows_in_planes(bit_off)
    rowinfo = ext.mma_prepare(nbits, bit_off, tau_s, min_s, P, ids.numel(), perm)
    return (ids, min_s, nbits, bit_off, P, tau_s, ei, ev), perm, rowinfo, layout


@pytest.mark.parametrize("Q,P,widths", [(300, 768, [7, 6, 5]), (136, 2048, [8, 4]), (64, 4096, [7]), (333, 256, [6, 9, 5])])
def test_rows_stored_in_planes_change_no_result(Q, P, widths):
    """The same pack with its rows back to back and with whole tiles stored in planes: the dense restore and the
    matrix-core products of every kernel behind qvb8_mma (with and without a row layout, with escapes) agree bit for bit; the GEMV kernel reads them too."""
    d = H.mixed_width_pack(Q, P, widths, seed=Q + P)
    d["tau_s"] = d["tau_s"] * (1.0 / 64)
    rng = np.random.default_rng(5)
    flat = np.sort(rng.choice(Q * P, 40, replace=False)).astype(np.int64)
    d["esc_idx"], d["esc_vals"] = flat, rng.normal(size=40).astype(np.float32)
    args_n, perm, rowinfo_n, layout_n = _sorted_pack(d)
    args_p, perm_p, rowinfo_p, layout_p = _sorted_planes(d)
    assert torch.equal(perm, perm_p)
    ids_n, min_s, nbits, off_n, _, tau_s, ei, ev = args_n
    ids_p, off_p = args_p[0], args_p[3]
    assert ids_n.numel() == ids_p.numel() and not torch.equal(ids_n, ids_p)
    back_ids, back_off = ext.rows_back_to_back(ids_p, nbits, off_p, P)           # the planes undone: the same bytes again
    assert torch.equal(back_ids, ids_n) and torch.equal(back_off, off_n)
    for fn in (ext.decode_f32, ext.decode, ext.decode_bf16):
        assert torch.equal(fn(ids_n, min_s, nbits, off_n, P, tau_s, ei, ev), fn(ids_p, min_s, nbits, off_p, P, tau_s, ei, ev))
    rows = torch.tensor([0, Q - 1, Q // 2, 17, 16, 0], device=DEV)               # the row lookup (embedding read) as well
    for dt in (torch.float32, torch.bfloat16):
        assert torch.equal(ext.lookup_rows(rows, ids_n, min_s, nbits, off_n, P, tau_s, ei, ev, dt),
                           ext.lookup_rows(rows, ids_p, min_s, nbits, off_p, P, tau_s, ei, ev, dt))
    x8 = _x(8, P, torch.float16, 1)
    _check(d, None, x8, ext.gemv_multi(x8, *args_p), saturate_ref=False)      # rows in planes are read element by element there
    sliceable = all(4 <= w <= 8 for w in widths) and P % 256 == 0
    for M in (1, 5, 16, 20, 40) + ((64, 100, 256) if sliceable else ()):
        x = _x(M, P, torch.bfloat16, M)
        want = ext.mma_tiles(x, *args_n, perm=perm, rowinfo=rowinfo_n, layout=layout_n)
        got = ext.mma_tiles(x, *args_p, perm=perm, rowinfo=rowinfo_p, layout=layout_p, planes=True)
        assert torch.equal(want, got), M
        if M <= 40:                                            # without the layout: the row records carry the planes
            assert torch.equal(ext.mma_tiles(x, *args_n, perm=perm, rowinfo=rowinfo_n),
                               ext.mma_tiles(x, *args_p, perm=perm, rowinfo=rowinfo_p, planes=True)), M
    _check(d, None, _x(3, P, torch.bfloat16, 3), ext.mma_tiles(_x(3, P, torch.bfloat16, 3), *args_p, perm=perm, rowinfo=rowinfo_p,
                                                              layout=layout_p, planes=True), saturate_ref=True)
    # a caller that leaves the statement out while the records mark rows as stored in planes: those rows come out as NaN
    # (their offset names a tile, not a row), every other row as usual -- never another row's values
    x = _x(2, P, torch.bfloat16, 9)
    left_out = ext.mma_tiles(x, *args_p, perm=perm, rowinfo=rowinfo_p)
    right = ext.mma_tiles(x, *args_p, perm=perm, rowinfo=rowinfo_p, planes=True)
    marked = ((off_p >> 62) & 1) == 1
    assert bool(marked.any()) and bool(torch.isnan(left_out[:, marked]).all())
    assert torch.equal(left_out[:, ~marked], right[:, ~marked])


@pytest.mark.parametrize("Q,P,widths", [(300, 768, [7, 6, 5]), (136, 256, [8, 4]), (333, 256, [6, 9, 5]), (40, 128, [5, 6, 7, 8]), (64, 128, [7])])
def test_rows_widened_to_whole_tiles_keep_every_value(Q, P, widths):
    """A few rows stored one width up so that every run of a width is a whole number of tiles: the dense restore is bit
    for bit what it was, no row got narrower, and every run below the last sliceable width is a multiple of 16 rows."""
    d = H.mixed_width_pack(Q, P, widths, seed=Q)
    ids, min_s, nbits, bit_off, _, tau_s, ei, ev = H.to_device_args(d, DEV)
    wide = ext.widen_rows_to_whole_tiles(ids, nbits, bit_off, P)
    counts = {w: widths_n for w, widths_n in zip(*[t.tolist() for t in torch.unique(nbits, return_counts=True)])}
    if all(n % 16 == 0 for w, n in sorted(counts.items())[:-1]):
        assert wide is None
        return
    ids2, nbits2, off2 = wide
    assert bool((nbits2 >= nbits).all()) and int((nbits2 != nbits).sum()) <= 15 * len(counts)
    assert torch.equal(ext.decode_f32(ids, min_s, nbits, bit_off, P, tau_s, ei, ev), ext.decode_f32(ids2, min_s, nbits2, off2, P, tau_s, ei, ev))
    runs = sorted(zip(*[t.tolist() for t in torch.unique(nbits2, return_counts=True)]))
    for (w, n), (w_next, _) in zip(runs[:-1], runs[1:]):
        assert n % 16 == 0 or w_next > 8, runs
