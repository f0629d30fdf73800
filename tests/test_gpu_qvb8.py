"""GPU parity: the HIP restore, certificate and GEMV against the CPU oracle.  All calls go through the C ABI
(qvb8_amd.ext_qvb8 -> ctypes -> libqvb8_amd.so)."""
import numpy as np
import pytest
import torch

from oracle import qvb8_oracle as O
from qvb8_amd import ext_qvb8 as ext
from qvb8_amd.formats.qvb8 import pack as PK
from tests import helpers as H

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _bits(t: torch.Tensor) -> np.ndarray:
    if t.dtype == torch.float32:
        return t.cpu().numpy().view(np.uint32)
    return t.cpu().view(torch.int16).numpy().view(np.uint16)


def _check_decode(d, args):
    ids = H.oracle_ids(d) if "ids_dense" not in d else d["ids_dense"]
    for fn, dt in ((ext.decode_f32, "fp32"), (ext.decode, "fp16"), (ext.decode_bf16, "bf16")):
        got = fn(*args)
        want = O.restore(d["min_s"], d["tau_s"], ids, d["esc_idx"], d["esc_vals"], dt)
        if dt == "fp32":
            assert np.array_equal(_bits(got), want.view(np.uint32)), dt
        elif dt == "fp16":
            assert np.array_equal(_bits(got), want.astype(np.float16).view(np.uint16)), dt
        else:
            assert np.array_equal(_bits(got), O.bf16_bits(want)), dt


@pytest.mark.parametrize("Q,P,widths", [
    (64, 4096, [7]), (48, 2048, [6]), (33, 768, [5, 6]), (40, 2080, [4, 5, 6, 7, 8]),      # dword-sliced path
    (29, 96, list(range(1, 15))), (17, 13, [3, 7, 11]), (9, 40, [2, 9, 14]), (5, 1, [14, 1]),  # per-element path
    (3, 6144, [7, 3, 12]),
])
def test_decode_bit_exact_hand_made_packs(Q, P, widths):
    d = H.mixed_width_pack(Q, P, widths, seed=Q * 131 + P)
    _check_decode(d, H.to_device_args(d, DEV))


def test_fp16_restore_rounds_the_fp32_value_not_the_exact_sum():
    """fp16 weights are fp16(fp32(fma(id, tau_s, min_s))): two roundings.  A pack big enough to hold values whose fp32
    rounding lands on an fp16 tie (where rounding the exact sum once gives the other neighbour) restores bit for bit;
    the results stored as fp16 by the matrix-core kernel follow the same rule."""
    Q, P = 256, 4096
    d = H.mixed_width_pack(Q, P, [8, 6], seed=77)
    d["tau_s"] = d["tau_s"] * (1.0 / 64)
    ids = d["ids_dense"]
    w32 = O.restore(d["min_s"], d["tau_s"], ids, d["esc_idx"], d["esc_vals"], "fp32")
    exact = d["min_s"].astype(np.float64)[:, None] + ids.astype(np.float64) * d["tau_s"].astype(np.float64)[:, None]
    want = w32.astype(np.float16).view(np.uint16)
    assert (want != exact.astype(np.float16).view(np.uint16)).sum() >= 8          # the case is in the pack
    args = H.to_device_args(d, DEV)
    assert np.array_equal(_bits(ext.decode(*args)), want)
    rows = torch.arange(Q, device=DEV)
    e0, v0 = torch.zeros(0, dtype=torch.int64, device=DEV), torch.zeros(0, device=DEV)
    got = ext.lookup_rows(rows, *args[:6], e0, v0, out_dtype=torch.float16)
    prod = (ids.astype(np.float32) * d["tau_s"][:, None]).astype(np.float32)
    assert np.array_equal(_bits(got), (d["min_s"][:, None] + prod).astype(np.float32).astype(np.float16).view(np.uint16))


def test_decode_golden_blob(golden):
    g = golden("ref_qvb8_blob.npz")
    d = O.parse_qvb8_blob(g["blob11"].tobytes())
    args = H.to_device_args(d, DEV)
    got = ext.decode_f32(*args)
    assert np.array_equal(_bits(got), g["dense"].view(np.uint32))
    g2 = golden("ref_qvbd_bf16.npz")
    d2 = O.parse_qvbd_blob(g2["blob"].tobytes())
    w16 = ext.decode(*H.to_device_args(d2, DEV))
    assert np.array_equal(_bits(w16), O.cpu_linear_weights(g2["blob"].tobytes()).astype(np.float16).view(np.uint16))


@pytest.mark.parametrize("restore", ["fp16", "fp16+bf16"])
def test_encoded_pack_restore_and_certificate(restore):
    W = H.synth_weight(192, 4096, seed=0).to(DEV)
    W[5, 100] = 0.9
    W[77, 4000] = -0.7
    enc = PK.encode_tensor(W, 1e-3, restore=restore, max_nbits=7, force_escapes=[12345, 99999])
    assert enc["esc_idx"].numel() >= 4
    d = H.oracle_view(enc)
    _check_decode(d, H.pack_args(enc))
    w16 = ext.decode(*H.pack_args(enc))
    err, bad = ext.certify(w16, W, 1e-3)
    assert bad == 0 and err < 1e-3
    assert err == pytest.approx(O.certificate_max_err(W.float().cpu().numpy(), w16.float().cpu().numpy()), abs=1e-12)
    if restore == "fp16+bf16":
        wb = ext.decode_bf16(*H.pack_args(enc, bf16_table=True))
        err, bad = ext.certify(wb, W, 1e-3)
        assert bad == 0 and err < 1e-3
    # without the escapes the certificate must fail: the check is not vacuous
    e0 = torch.zeros(0, dtype=torch.int64, device=DEV)
    v0 = torch.zeros(0, dtype=torch.float32, device=DEV)
    wbad = ext.decode(enc["ids"], enc["min_s"], enc["nbits"], enc["bit_off"], enc["P"], enc["tau_s"], e0, v0)
    err, bad = ext.certify(wbad, W, 1e-3)
    assert bad >= 2 and err > 0.1


def test_sat_half_matches_oracle():
    x = torch.tensor([1e9, -1e9, 65504.0, 65519.0, 65520.0, 3.14159, float("nan"), -0.0, 1e-7, 6e-5], device=DEV)
    for dt in (torch.float32, torch.bfloat16):
        xi = x.to(dt)
        got = ext.saturating_half(xi).float().cpu().numpy()
        want = O.sat_half(xi.float().cpu().numpy())
        assert np.array_equal(np.isnan(got), np.isnan(want))
        assert np.array_equal(got[~np.isnan(got)], want[~np.isnan(want)])


def _check_gemv(enc_or_d, args, M, x_dtype, seed=0, is_enc=True):
    d = H.oracle_view(enc_or_d) if is_enc else enc_or_d
    P, Q = d["P"], d["Q"]
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(M, P, generator=g).to(x_dtype).to(DEV)
    y = ext.gemv_multi(x, *args)
    assert y.dtype == torch.float32 and tuple(y.shape) == (M, Q)
    ids = H.oracle_ids(d) if "ids_dense" not in d else d["ids_dense"]
    Wr = O.reconstruct(d["min_s"], d["tau_s"], ids, d["esc_idx"], d["esc_vals"])
    xs = O.sat_half(x.float().cpu().numpy())
    ref = O.linear_f64(xs, Wr)
    tol = H.gemv_tolerance(ref, Wr, xs)
    diff = np.abs(y.cpu().numpy().astype(np.float64) - ref)
    assert np.all(diff <= tol), (float(diff.max()), float((diff / tol).max()))
    # bf16 outputs: within one bf16 step of the rounded reference
    yb = y.bfloat16().float().cpu().numpy()
    rb = O.narrow_bf16(ref.astype(np.float32))
    assert np.all(np.abs(yb - rb) <= 2.0 ** -7 * np.abs(rb) + tol)
    return y


@pytest.mark.parametrize("M", [1, 2, 3, 4, 5, 6, 7, 8])
def test_gemv_all_m_encoded_pack(M):
    W = H.synth_weight(320, 4096, seed=M).to(DEV)
    enc = PK.encode_tensor(W, 1e-3, restore="fp16")
    _check_gemv(enc, H.pack_args(enc), M, torch.bfloat16, seed=M)


@pytest.mark.parametrize("Q,P,tau", [(1024, 4096, 1e-3), (256, 12288, 1e-3), (130, 768, 2e-3), (96, 2048, 2e-3),
                                     (64, 5120, 2e-3), (40, 17408, 2e-3), (24, 28672, 2e-3)])
@pytest.mark.parametrize("x_dtype", [torch.bfloat16, torch.float16, torch.float32])
def test_gemv_shapes(Q, P, tau, x_dtype):
    W = H.synth_weight(Q, P, seed=P).to(DEV)
    enc = PK.encode_tensor(W, tau, restore="fp16")
    for M in (1, 3):
        _check_gemv(enc, H.pack_args(enc), M, x_dtype, seed=Q)


@pytest.mark.parametrize("Q,P,widths", [(40, 2080, [4, 5, 6, 7, 8]), (29, 96, list(range(1, 15))), (17, 13, [3, 7, 11]),
                                        (33, 4096, [7, 9, 6, 3]), (12, 6144, [7, 3, 12])])
def test_gemv_mixed_widths_and_per_element_rows(Q, P, widths):
    d = H.mixed_width_pack(Q, P, widths, seed=7)
    for M in (1, 4):
        _check_gemv(d, H.to_device_args(d, DEV), M, torch.float32, seed=3, is_enc=False)


def test_gemv_escapes_and_determinism():
    W = H.synth_weight(128, 4096, seed=11).to(DEV)
    W[3, 17] = 1.5
    W[3, 4000] = -2.0
    W[90, 0] = 0.8
    enc = PK.encode_tensor(W, 1e-3, restore="fp16", max_nbits=7, force_escapes=[5 * 4096 + 9, 5 * 4096 + 10])
    assert enc["esc_idx"].numel() >= 5
    y1 = _check_gemv(enc, H.pack_args(enc), 2, torch.bfloat16, seed=5)
    y2 = _check_gemv(enc, H.pack_args(enc), 2, torch.bfloat16, seed=5)
    assert torch.equal(y1, y2)
    # the correction is real: dropping the escapes moves row 3 by about x * 1.5
    e0 = torch.zeros(0, dtype=torch.int64, device=DEV)
    v0 = torch.zeros(0, dtype=torch.float32, device=DEV)
    g = torch.Generator().manual_seed(5)
    x = torch.randn(2, 4096, generator=g).to(torch.bfloat16).to(DEV)
    y0 = ext.gemv_multi(x, enc["ids"], enc["min_s"], enc["nbits"], enc["bit_off"], 4096, enc["tau_s"], e0, v0)
    assert (y0[:, 3] - y1[:, 3]).abs().max() > 0.1


def test_gemv_activation_saturation_and_nan():
    W = H.synth_weight(64, 2048, seed=2).to(DEV)
    enc = PK.encode_tensor(W, 1e-3)
    x = torch.zeros(1, 2048, device=DEV)
    x[0, 5] = 1e6
    x[0, 9] = -3e5
    _check_gemv_x(enc, x)
    x[0, 100] = float("nan")
    y = ext.gemv_multi(x, *H.pack_args(enc))
    assert torch.isnan(y).all()


def _check_gemv_x(enc, x):
    d = H.oracle_view(enc)
    y = ext.gemv_multi(x, *H.pack_args(enc))
    Wr = O.reconstruct(d["min_s"], d["tau_s"], H.oracle_ids(d))
    xs = O.sat_half(x.float().cpu().numpy())
    ref = O.linear_f64(xs, Wr)
    assert np.all(np.abs(y.cpu().numpy() - ref) <= 1e-3 * np.abs(ref) + 1e-3 * np.abs(xs).max() * 0.1)


def test_gemv_argument_errors():
    W = H.synth_weight(16, 256, seed=1).to(DEV)
    enc = PK.encode_tensor(W, 1e-3)
    x = torch.randn(9, 256, device=DEV)
    with pytest.raises(RuntimeError, match="outside the instantiated range"):
        ext.gemv_multi(x, *H.pack_args(enc))
    a = list(H.pack_args(enc))
    a[0] = torch.cat([torch.zeros(1, dtype=torch.uint8, device=DEV), enc["ids"]])[1:]
    with pytest.raises(RuntimeError, match="4-byte aligned"):
        ext.gemv_multi(x[:1], *a)
    with pytest.raises(RuntimeError, match="GPU tensors"):
        ext.gemv_multi(x[:1].cpu(), *H.pack_args(enc))


def test_forward_dispatch_small_and_large_m():
    W = H.synth_weight(256, 1024, seed=4).to(DEV)
    enc = PK.encode_tensor(W, 1e-3)
    d = H.oracle_view(enc)
    ids = H.oracle_ids(d)
    for M in (1, 8, 9, 40):
        x = torch.randn(M, 1024, device=DEV).to(torch.bfloat16)
        y = ext.forward(x, *H.pack_args(enc))
        assert y.dtype == torch.float32 and tuple(y.shape) == (M, 256)
        xs = O.sat_half(x.float().cpu().numpy())
        Wr = O.reconstruct(d["min_s"], d["tau_s"], ids)
        Wuse = Wr if M <= 8 else O.narrow_fp16(Wr)
        ref = O.linear_f64(xs, Wuse)
        assert np.all(np.abs(y.cpu().numpy() - ref) <= H.gemv_tolerance(ref, Wuse, xs))
