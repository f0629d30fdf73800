"""Shared by the GPU parity tests: synthetic packs and oracle views of them."""
import numpy as np
import torch

from oracle import qvb8_oracle as O
from qvb8_amd.formats.qvb8 import pack as PK


def synth_weight(Q, P, seed=0, sigma=0.02, dtype=torch.bfloat16):
    g = torch.Generator().manual_seed(seed)
    return (sigma * torch.randn(Q, P, generator=g)).to(dtype)


def enc_to(enc: dict, device):
    return {k: (v.to(device) if torch.is_tensor(v) else v) for k, v in enc.items()}


def pack_args(enc: dict, bf16_table=False):
    """Positional pack operands in the extension's order after X."""
    ei = enc["esc_idx_bf16"] if bf16_table else enc["esc_idx"]
    ev = enc["esc_vals_bf16"] if bf16_table else enc["esc_vals"]
    return (enc["ids"], enc["min_s"], enc["nbits"], enc["bit_off"], enc["P"], enc["tau_s"], ei, ev)


def oracle_view(enc: dict, bf16_table=False) -> dict:
    """The encoded tensor as the oracle's dict (numpy, host)."""
    ei = enc["esc_idx_bf16"] if bf16_table else enc["esc_idx"]
    ev = enc["esc_vals_bf16"] if bf16_table else enc["esc_vals"]
    return dict(Q=enc["Q"], P=enc["P"], min_s=enc["min_s"].cpu().numpy(), tau_s=enc["tau_s"].cpu().numpy(),
                nbits=enc["nbits"].cpu().numpy().astype(np.int64), bit_off=enc["bit_off"].cpu().numpy(),
                buf=enc["ids"].cpu().numpy(), esc_idx=ei.cpu().numpy(), esc_vals=ev.cpu().numpy())


def oracle_ids(d: dict):
    return O.unpack_bits_rows(d["buf"], d["nbits"], d["bit_off"], d["Q"], d["P"])


def mixed_width_pack(Q, P, widths, seed=0):
    """A hand-made pack with the given row widths (cycled), random ids and metadata: exercises every
    width and unaligned rows without going through the encoder."""
    rng = np.random.default_rng(seed)
    nb = np.array([widths[i % len(widths)] for i in range(Q)], np.int64)
    ids = np.stack([rng.integers(0, 1 << int(w), P) for w in nb]).astype(np.int64)
    buf, off = O.pack_bits_rows(ids, nb)
    min_s = rng.normal(0, 0.08, Q).astype(np.float32)
    tau_s = (np.abs(rng.normal(2e-3, 5e-4, Q)) + 1e-5).astype(np.float32)
    return dict(Q=Q, P=P, min_s=min_s, tau_s=tau_s, nbits=nb, bit_off=off.astype(np.int64), buf=buf,
                esc_idx=np.zeros(0, np.int64), esc_vals=np.zeros(0, np.float32), ids_dense=ids)


def to_device_args(d: dict, device):
    t = lambda a, dt=None: torch.from_numpy(np.ascontiguousarray(a)).to(device if dt is None else device)
    return (t(d["buf"]), t(d["min_s"]), t(d["nbits"].astype(np.uint8)), t(d["bit_off"].astype(np.int64)), d["P"],
            t(d["tau_s"]), t(d["esc_idx"].astype(np.int64)), t(d["esc_vals"].astype(np.float32)))


def gemv_tolerance(y_ref: np.ndarray, W: np.ndarray, x: np.ndarray):
    """|y - y_ref| <= 1e-3*|y_ref| + atol, atol = 1e-3 * ||w_row|| * ||x|| / sqrt(P): the cancellation floor of a
    length-P dot product of these magnitudes."""
    P = W.shape[1]
    wn = np.linalg.norm(W.astype(np.float64), axis=1)
    xn = np.linalg.norm(x.astype(np.float64), axis=1)
    atol = 1e-3 * xn[:, None] * wn[None, :] / np.sqrt(P)
    return 1e-3 * np.abs(y_ref) + atol
