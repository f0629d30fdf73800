"""The QVB8 oracle against the reference's golden vectors, libm, and closed forms."""
import ctypes
import ctypes.util

import numpy as np
import pytest
import torch

from oracle import qvb8_oracle as O


def test_pack_known_answer_3bit():
    # eight 3-bit ids 1..7,0, LSB first: bits 001 010 011 100 101 110 111 000 from bit 0 upwards
    buf, off = O.pack_bits_rows(np.array([[1, 2, 3, 4, 5, 6, 7, 0]]), np.array([3]))
    assert buf[:3].tolist() == [0xD1, 0x58, 0x1F]
    assert buf[3:].tolist() == [0] * 8 and len(buf) == 3 + 8
    assert off.tolist() == [0]


def test_pack_known_answer_unaligned_rows():
    # row 0: three 3-bit ids (9 bits), row 1 starts at bit 9 with 5-bit ids
    ids = np.array([[5, 2, 7], [17, 1, 30]])
    buf, off = O.pack_bits_rows(ids, np.array([3, 5]))
    assert off.tolist() == [0, 9]
    stream = 0
    for k, (v, w, p) in enumerate([(5, 3, 0), (2, 3, 3), (7, 3, 6), (17, 5, 9), (1, 5, 14), (30, 5, 19)]):
        stream |= v << p
    want = [(stream >> (8 * i)) & 0xFF for i in range(3)]
    assert buf[:3].tolist() == want


def test_bits_against_reference_vectors(golden):
    g = golden("ref_bits.npz")
    for i in range(int(g["n_cases"])):
        ids, nb = g[f"c{i}_ids"], g[f"c{i}_nbits"]
        buf, off = O.pack_bits_rows(ids, nb)
        assert np.array_equal(buf, g[f"c{i}_buf"]), i
        assert np.array_equal(off.astype(np.int64), g[f"c{i}_off"])
        Q, P = ids.shape
        assert np.array_equal(O.unpack_bits_rows(g[f"c{i}_buf"], nb, g[f"c{i}_off"], Q, P), g[f"c{i}_back"])
        assert np.array_equal(g[f"c{i}_back"], ids)
        if Q > 1:
            assert np.array_equal(O.unpack_bits_rows(g[f"c{i}_buf"], nb[1:], g[f"c{i}_off"], Q, P, r0=1), g[f"c{i}_part"])


@pytest.mark.parametrize("P", [1, 7, 8, 13, 32, 96])
def test_bits_round_trip_all_widths(P):
    rng = np.random.default_rng(P)
    nb = np.arange(1, 15)
    ids = np.stack([rng.integers(0, 1 << int(w), P) for w in nb])
    buf, off = O.pack_bits_rows(ids, nb)
    assert len(buf) == (int(nb.sum()) * P + 7) // 8 + 8
    assert np.array_equal(O.unpack_bits_rows(buf, nb, off, len(nb), P), ids)
    # brute force, bit by bit
    bits = np.unpackbits(buf, bitorder="little")
    for r in (0, 6, 13):
        for c in (0, P - 1):
            p = int(off[r]) + c * int(nb[r])
            v = sum(int(bits[p + k]) << k for k in range(int(nb[r])))
            assert v == ids[r, c]


def _libm_fmaf():
    lib = ctypes.CDLL(ctypes.util.find_library("m"))
    lib.fmaf.restype = ctypes.c_float
    lib.fmaf.argtypes = [ctypes.c_float] * 3
    return lib.fmaf


def test_fma32_equals_libm_fmaf_exhaustive_ids():
    fmaf = _libm_fmaf()
    rng = np.random.default_rng(0)
    ids = np.arange(1 << 14, dtype=np.float32)
    for _ in range(6):
        ts = np.float32(abs(rng.normal(2e-3, 1e-3)) + 1e-6)
        m = np.float32(rng.normal(0, 0.1))
        got = O.fma32(ids, ts, np.full_like(ids, m))
        want = np.array([fmaf(float(i), float(ts), float(m)) for i in ids], np.float32)
        assert np.array_equal(got.view(np.uint32), want.view(np.uint32))
        f64 = (ids.astype(np.float64) * np.float64(ts) + np.float64(m)).astype(np.float32)
        assert np.array_equal(got.view(np.uint32), f64.view(np.uint32))


def test_fma32_and_reconstruct_against_reference_vectors(golden):
    g = golden("ref_restore.npz")
    out = O.fma32(g["fma_a"], g["fma_b"], g["fma_c"])
    assert np.array_equal(out.view(np.uint32), g["fma_out"].view(np.uint32))
    fmaf = _libm_fmaf()
    want = np.array([fmaf(float(a), float(b), float(c)) for a, b, c in zip(g["fma_a"], g["fma_b"], g["fma_c"])], np.float32)
    assert np.array_equal(out.view(np.uint32), want.view(np.uint32))
    rec = O.reconstruct(g["min_s"], g["tau_s"], g["ids"], g["esc_idx"], g["esc_vals"])
    assert np.array_equal(rec.view(np.uint32), g["rec"].view(np.uint32))
    assert np.array_equal(O.reconstruct(g["min_s"], g["tau_s"], g["ids"]).view(np.uint32), g["rec_plain"].view(np.uint32))
    # a dropped escape or a wrong row broadcast fails here
    assert not np.array_equal(g["rec"], g["rec_plain"])
    assert np.array_equal(np.nan_to_num(O.e4m3_lut(), nan=-1), np.nan_to_num(g["e4m3_lut"], nan=-1))


def test_e4m3_against_torch():
    codes = torch.arange(256, dtype=torch.uint8)
    t = codes.view(torch.float8_e4m3fn).float().numpy()
    lut = O.e4m3_lut()
    assert np.array_equal(np.isnan(t), np.isnan(lut))
    ok = ~np.isnan(t)
    assert np.array_equal(t[ok], lut[ok])


def test_narrowing_against_libraries():
    rng = np.random.default_rng(1)
    v = np.concatenate([rng.normal(0, 0.05, 20000), rng.normal(0, 1e-6, 2000), [0.0, -0.0, 65504.0, 65520.0, 1e-8, 70000.0],
                        rng.normal(0, 300, 2000)]).astype(np.float32)
    assert np.array_equal(O.narrow_bf16(v), torch.from_numpy(v).bfloat16().float().numpy())
    with np.errstate(over="ignore"):
        assert np.array_equal(O.narrow_fp16(v), torch.from_numpy(v).half().float().numpy())
    # ties to even on the bf16 grid: 1 + 2^-8 is halfway between 1 and 1 + 2^-7
    assert O.narrow_bf16(np.array([1 + 2.0 ** -8], np.float32))[0] == 1.0
    assert O.narrow_bf16(np.array([1 + 3 * 2.0 ** -8], np.float32))[0] == np.float32(1 + 2.0 ** -6)


def test_sat_half():
    x = np.array([1e9, -1e9, 65504.0, 65519.0, 3.14159, np.nan, -0.0], np.float32)
    y = O.sat_half(x)
    assert y[0] == 65504.0 and y[1] == -65504.0 and y[2] == 65504.0 and y[3] == 65504.0
    assert y[4] == np.float32(np.float16(3.14159)) and np.isnan(y[5])


def test_blob_readers_against_reference_vectors(golden):
    g = golden("ref_qvb8_blob.npz")
    d = O.parse_qvb8_blob(g["blob11"].tobytes())
    for k in ("min_s", "tau_s", "nbits", "bit_off", "buf", "esc_idx", "esc_vals"):
        assert np.array_equal(d[k], g[k]), k
    assert [d["Q"], d["P"], d["tau"]] == g["QPtau"].tolist()
    assert list(O.read_header(g["blob11"].tobytes())) == g["hdr"].tolist()
    dense = O.decode_tensor(g["blob11"].tobytes())
    assert np.array_equal(dense.view(np.uint32), g["dense"].view(np.uint32))
    for tag in ("v11s", "v10s"):
        dd = O.parse_qvb8_blob(g[f"blob{tag[1:3]}s"].tobytes())
        assert np.array_equal(dd["esc_idx"], g[f"{tag}_esc_idx"])
        assert np.array_equal(dd["esc_vals"].view(np.uint32), g[f"{tag}_esc_vals"].view(np.uint32))
        assert np.array_equal(O.decode_tensor(g[f"blob{tag[1:3]}s"].tobytes()).view(np.uint32), g[f"{tag}_dense"].view(np.uint32))
    assert np.array_equal(O.decode_tensor(g["blob9"].tobytes()).view(np.uint32), g["v9_dense"].view(np.uint32))
    # certificate of the golden tensor: fp16 restore within tau of the original
    W = g["W"]
    assert O.certificate_max_err(W, O.narrow_fp16(dense)) < 1e-3


@pytest.mark.parametrize("tag", ["bf16", "fp32"])
def test_qvbd_reader_against_reference_vectors(golden, tag):
    g = golden(f"ref_qvbd_{tag}.npz")
    d = O.parse_qvbd_blob(g["blob"].tobytes())
    for k in ("min_s", "tau_s", "nbits", "bit_off", "buf", "esc_idx", "esc_vals"):
        assert np.array_equal(d[k], g[k]), k
    assert d["source"] == bytes(g["source"]).decode() and d["restore"] == bytes(g["restore"]).decode()
    assert [d["Q"], d["P"]] == g["Qptau"][:2].tolist()
    assert np.float32(d["tau"]) == np.float32(g["Qptau"][2]) and np.float32(d["max_err"]) == np.float32(g["Qptau"][3])
    ids = O.unpack_bits_rows(d["buf"], d["nbits"], d["bit_off"], d["Q"], d["P"])
    assert np.array_equal(ids, g["codes"])
    W16 = O.cpu_linear_weights(g["blob"].tobytes())
    assert O.certificate_max_err(g["W"], W16) < 1e-3
    assert O.certificate_max_err(g["W"], W16) == pytest.approx(float(g["Qptau"][3]), abs=1e-9)


def test_reader_errors():
    with pytest.raises(O.OracleFormatError):
        O.parse_qvb8_blob(b"\0" * 80)
    with pytest.raises(O.OracleFormatError):
        O.parse_qvbd_blob(b"QVBX" + b"\0" * 60)


def test_router_topk_closed_form():
    logits = np.log(np.array([[0.1, 0.2, 0.3, 0.4]]))
    idx, w = O.router_topk(logits, 2)
    assert idx.tolist() == [[3, 2]]
    assert np.allclose(w, [[4 / 7, 3 / 7]])


def test_moe_reference_tiny_brute_force():
    rng = np.random.default_rng(3)
    E, H, I, T, k = 4, 8, 6, 3, 2
    Wgu = [rng.normal(0, 0.3, (2 * I, H)).astype(np.float32) for _ in range(E)]
    Wdn = [rng.normal(0, 0.3, (H, I)).astype(np.float32) for _ in range(E)]
    x = rng.normal(0, 1, (T, H)).astype(np.float16).astype(np.float32)
    idx, w = O.router_topk(rng.normal(0, 1, (T, E)), k)
    out = O.moe_reference(x, idx, w, Wgu, Wdn)
    t = 1
    want = np.zeros(H)
    for j in range(k):
        e = idx[t, j]
        y = Wgu[e].astype(np.float64) @ x[t]
        g, u = y[:I], y[I:]
        want += w[t, j] * (Wdn[e].astype(np.float64) @ (g / (1 + np.exp(-g)) * u))
    assert np.allclose(out[t], want, rtol=1e-12)


def test_moe_reference_relu2_by_hand():
    """The non-gated ReLU^2 branch on a case small enough to work out by hand: one token, one expert with weight 1/2
    and one with weight 1/4, integers throughout.  up(x) = (3, -2) -> relu^2 = (9, 0); down rows (1, 5) and (2, 7)."""
    x = np.array([[1.0, 2.0]], np.float32)
    W_up = [np.array([[1.0, 1.0], [0.0, -1.0]], np.float32), np.array([[-1.0, 0.0], [2.0, 1.0]], np.float32)]
    W_dn = [np.array([[1.0, 5.0], [2.0, 7.0]], np.float32), np.array([[3.0, 1.0], [0.0, -2.0]], np.float32)]
    idx = np.array([[0, 1]], np.int64)
    w = np.array([[0.5, 0.25]], np.float32)
    # expert 0: up = (3, -2), h = (9, 0), down = (9, 18); expert 1: up = (-1, 4), h = (0, 16), down = (16, -32)
    want = 0.5 * np.array([9.0, 18.0]) + 0.25 * np.array([16.0, -32.0])
    got = O.moe_reference(x, idx, w, W_up, W_dn, act="relu2")
    assert np.array_equal(got, want[None, :])
    # and it is not the gated form: the same call as gated SiLU needs an even number of up rows split in halves
    gated = O.moe_reference(x, idx, w, [np.vstack([u, u]) for u in W_up], W_dn)
    assert not np.allclose(gated, got)


def test_embedding_rows_two_roundings_closed_form():
    """The lookup value is fl(min + fl(id * tau)): checked against float64 arithmetic rounded explicitly at each step
    (id * tau is exact in float64: 14 + 24 bits; min + product of two floats is exact in float64 unless the exponents
    are more than 29 apart, which these magnitudes never are)."""
    rng = np.random.default_rng(5)
    Q, P = 40, 96
    nb = rng.integers(1, 15, Q)
    ids = np.stack([rng.integers(0, 1 << int(w), P) for w in nb])
    min_s = rng.normal(0, 0.1, Q).astype(np.float32)
    tau_s = (np.abs(rng.normal(2e-3, 1e-3, Q)) + 1e-6).astype(np.float32)
    rows = np.array([3, 3, 39, 0, 17, 3], np.int64)
    got = O.embedding_rows(rows, min_s, tau_s, ids, P)
    prod = (ids[rows].astype(np.float64) * tau_s[rows].astype(np.float64)[:, None]).astype(np.float32)
    want = (min_s[rows].astype(np.float64)[:, None] + prod.astype(np.float64)).astype(np.float32)
    assert got.dtype == np.float32 and got.shape == (6, P)
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))
    # from the fused value by at most the two rounding errors (half a unit of the product, half a unit of the sum,
    # plus the fused value's own half unit), and not always equal to it
    fused = O.band_values(min_s, tau_s, ids)[rows].astype(np.float64)
    bound = 0.5 * np.spacing(np.abs(prod)).astype(np.float64) + np.spacing(np.maximum(np.abs(got), np.abs(fused).astype(np.float32))).astype(np.float64)
    assert np.all(np.abs(got.astype(np.float64) - fused) <= bound)
    assert np.any(got.astype(np.float64) != fused)


def test_embedding_rows_known_answer_differs_from_fused():
    """id = 3, tau = 1 + 2^-23, min = -3: the product 3 + 3*2^-23 needs 26 bits and rounds to 3 + 2^-21 (tie to even),
    so the two-step value is 2^-21 while the fused one keeps the exact 3*2^-23."""
    tau = np.array([1.0 + 2.0 ** -23], np.float32)
    mn = np.array([-3.0], np.float32)
    ids = np.array([[3]])
    two = O.embedding_rows([0], mn, tau, ids, 1)
    one = O.band_values(mn, tau, ids)
    assert two[0, 0] == np.float32(2.0 ** -21)
    assert one[0, 0] == np.float32(3 * 2.0 ** -23)


def test_embedding_rows_escapes_and_narrowing():
    rng = np.random.default_rng(6)
    Q, P = 8, 32
    ids = rng.integers(0, 64, (Q, P))
    min_s = rng.normal(0, 0.1, Q).astype(np.float32)
    tau_s = np.full(Q, 2e-3, np.float32)
    esc_idx = np.array([2 * P + 5, 2 * P + 31, 7 * P + 0], np.int64)
    esc_vals = np.array([0.75, -1.5, 3.0e-5], np.float32)
    rows = np.array([7, 2, 2, 1], np.int64)
    out = O.embedding_rows(rows, min_s, tau_s, ids, P, esc_idx, esc_vals)
    assert out[0, 0] == esc_vals[2] and out[1, 5] == esc_vals[0] and out[2, 31] == esc_vals[1]
    plain = O.embedding_rows(rows, min_s, tau_s, ids, P)
    mask = np.ones_like(out, bool)
    mask[0, 0] = mask[1, 5] = mask[1, 31] = mask[2, 5] = mask[2, 31] = False
    assert np.array_equal(out[mask], plain[mask])
    h = O.embedding_rows(rows, min_s, tau_s, ids, P, esc_idx, esc_vals, dtype="fp16")
    assert np.array_equal(h, out.astype(np.float16).astype(np.float32))
    b = O.embedding_rows(rows, min_s, tau_s, ids, P, esc_idx, esc_vals, dtype="bf16")
    assert np.array_equal(b, torch.from_numpy(out).to(torch.bfloat16).float().numpy())


# ---- the dense MLP chain (gate / up -> SiLU * up -> down) -------------------------------------------------------------------

@pytest.mark.parametrize("dtype,tdt", [("bf16", "bfloat16"), ("fp16", "float16"), ("fp32", "float32")])
def test_swiglu_is_what_torch_computes_in_the_models_dtype(dtype, tdt):
    """`act_fn(gate) * up` on tensors of the model's dtype, by torch's CPU kernels (which compute silu in fp32 and round its
    result to the tensor's dtype, then round the product): an implementation that shares nothing with the oracle's.  A
    missing intermediate rounding, a sigmoid with the wrong sign or gate and up swapped all fail it.  fp32 results may
    differ in the last place (torch's expf against numpy's float64 exp); the narrow types must agree bit for bit except
    where a value lies within that last place of a rounding boundary -- counted, and bounded."""
    import torch
    import torch.nn.functional as F
    tdt = getattr(torch, tdt)
    g = torch.randn(1 << 16, generator=torch.Generator().manual_seed(3)) * 4.0
    u = torch.randn(1 << 16, generator=torch.Generator().manual_seed(4)) * 2.0
    g[:8] = torch.tensor([0.0, -0.0, 30.0, -30.0, 1e-6, -1e-6, 88.0, -88.0])
    g, u = g.to(tdt), u.to(tdt)
    want = (F.silu(g) * u).float().numpy()
    got = O.swiglu(g.float().numpy(), u.float().numpy(), dtype)
    assert got.dtype == np.float32
    if dtype == "fp32":
        assert np.all(np.abs(got - want) <= 2.0 ** -22 * np.abs(want) + 1e-37)
    else:
        differ = got.view(np.uint32) != want.view(np.uint32)
        assert differ.mean() < 2e-3, differ.mean()
        ulp = {"bf16": 2.0 ** -7, "fp16": 2.0 ** -10}[dtype]
        assert np.all(np.abs(got - want)[differ] <= ulp * np.abs(want)[differ] + 2.0 ** -24)
    swapped = O.swiglu(u.float().numpy(), g.float().numpy(), dtype)
    assert not np.array_equal(swapped.view(np.uint32), got.view(np.uint32))


def test_round_to_closed_forms():
    """One rounding to nearest even into each type: ties, the subnormal range of fp16, overflow to infinity."""
    v = np.array([1.0 + 2.0 ** -11, 1.0 + 3 * 2.0 ** -11, 2.0 ** -25, 3 * 2.0 ** -25, 65520.0, 65519.9], np.float64)
    assert np.array_equal(O.round_to(v, "fp16"), np.array([1.0, 1.0 + 2.0 ** -9, 0.0, 2.0 ** -23, np.inf, 65504.0], np.float32))
    v = np.array([1.0 + 2.0 ** -8, 1.0 + 3 * 2.0 ** -8, -1.0 - 2.0 ** -8], np.float64)
    assert np.array_equal(O.round_to(v, "bf16"), np.array([1.0, 1.0 + 2.0 ** -6, -1.0], np.float32))
    assert np.array_equal(O.round_to(np.array([1.0 + 2.0 ** -24, 1.0 + 3 * 2.0 ** -24]), "fp32"),
                          np.array([1.0, 1.0 + 2.0 ** -22], np.float32))


def test_mlp_reference_is_the_chain_of_its_parts():
    """With identity-like weights the chain reduces to the pointwise function: W_gate = W_up = I, W_down = I gives
    y = round(sat(swiglu(x, x))) for an x that fp16 holds exactly."""
    x = np.linspace(-4.0, 4.0, 64, dtype=np.float32).astype(np.float16).astype(np.float32)[None, :]
    I = np.eye(64, dtype=np.float32)
    y, h = O.mlp_reference(x, I, I, I, "bf16")
    assert np.array_equal(h, O.swiglu(O.round_to(x, "bf16"), O.round_to(x, "bf16"), "bf16"))
    assert np.array_equal(y, O.round_to(O.sat_half(h), "bf16"))
    y2, _ = O.mlp_reference(x, I, I, 2.0 * I, "bf16")
    assert np.array_equal(y2, O.round_to(2.0 * O.sat_half(h).astype(np.float64), "bf16"))
