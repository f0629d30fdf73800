"""Writes the golden vectors under tests/golden/ by running the reference's own readers.

Run once, in the build container (the reference tree does not travel):
    python tests/golden/make_reference_vectors.py [/root/reference/src]

Inputs are produced by this repository's writers (or drawn at random with fixed
seeds); expected outputs are what the reference's Python functions return for them:
    qv_band.formats.qvb8.decode: pack_bits_rows, unpack_bits_rows, fma32, reconstruct,
        _e4m3_lut, _nbits_for, read_header, unpack_tensor, decode_tensor
    qv_band.formats.qvb8.pack_container: unpack_formula (fp16 restore)
    qv_band.formats.qvb8r.codec: slot_tables
    qv_band.formats.qvb8r.container: blocks_for, write/read, runtime_tables
Everything is stored as plain arrays in .npz files (no pickles).  The fixtures hold
data only: inputs and the outputs the reference gave.
"""
from __future__ import annotations

import os
import struct
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
sys.path.insert(0, ROOT)
REF_SRC = sys.argv[1] if len(sys.argv) > 1 else "/root/reference/src"
sys.path.insert(0, REF_SRC)

import qv_band.formats.qvb8.decode as RD            # noqa: E402
import qv_band.formats.qvb8.pack_container as RC    # noqa: E402
import qv_band.formats.qvb8r.codec as RK            # noqa: E402
import qv_band.formats.qvb8r.container as RF        # noqa: E402

import torch                                         # noqa: E402
from qvb8_amd.formats.qvb8 import decode as L       # noqa: E402
from qvb8_amd.formats.qvb8 import pack as PK        # noqa: E402
from qvb8_amd.formats.qvb8 import pack_container as C  # noqa: E402


def save(name, **arrs):
    np.savez_compressed(os.path.join(HERE, name), **arrs)
    print("wrote", name, {k: getattr(v, "shape", None) for k, v in arrs.items()})


def bits_vectors():
    rng = np.random.default_rng(1)
    out = {}
    cases = [(1, 8, [3]), (4, 16, [1, 14, 7, 6]), (5, 13, [5, 9, 2, 11, 7]), (3, 64, [7, 7, 6]),
             (6, 24, [8, 4, 12, 13, 3, 10]), (2, 1, [14, 1])]
    for i, (Q, P, nb) in enumerate(cases):
        nb = np.array(nb, np.int64)
        ids = np.stack([rng.integers(0, 1 << int(w), P) for w in nb]).astype(np.int64)
        buf, off = RD.pack_bits_rows(ids.astype(np.uint64), nb)
        back = RD.unpack_bits_rows(buf, nb, off.astype(np.int64), Q, P)
        # a partial read starting at row 1 with absolute offsets
        part = RD.unpack_bits_rows(buf, nb[1:], off.astype(np.int64), Q, P, r0=1) if Q > 1 else back[:0]
        out.update({f"c{i}_ids": ids, f"c{i}_nbits": nb, f"c{i}_buf": buf, f"c{i}_off": off.astype(np.int64),
                    f"c{i}_back": back, f"c{i}_part": part})
    out["n_cases"] = np.array(len(cases))
    out["nbits_for_in"] = np.array([0, 1, 2, 3, 4, 5, 8, 9, 64, 65, 128, 129, 16383, 16384, 16385], np.int64)
    out["nbits_for_out"] = RD._nbits_for(out["nbits_for_in"])
    save("ref_bits.npz", **out)


def restore_vectors():
    rng = np.random.default_rng(2)
    Q, P = 8, 96
    nb = rng.integers(1, 15, Q)
    ids = np.stack([rng.integers(0, 1 << int(w), P) for w in nb]).astype(np.int64)
    min_s = (rng.normal(0, 0.08, Q)).astype(np.float32)
    tau_s = (np.abs(rng.normal(2e-3, 5e-4, Q)) + 1e-5).astype(np.float32)
    esc_idx = np.sort(rng.choice(Q * P, 11, replace=False)).astype(np.int64)
    esc_vals = rng.normal(0, 1, 11).astype(np.float32)
    rec = RD.reconstruct(min_s, tau_s, ids, esc_idx, esc_vals)
    rec_plain = RD.reconstruct(min_s, tau_s, ids)
    # fma32 on near-cancelling operands: c close to -a*b
    a = rng.integers(0, 1 << 14, 4096).astype(np.float32)
    b = (np.abs(rng.normal(2e-3, 1e-3, 4096)) + 1e-6).astype(np.float32)
    c = (-(a.astype(np.float64) * b.astype(np.float64)) * (1 + rng.normal(0, 1e-6, 4096))).astype(np.float32)
    f = RD.fma32(a, b, c)
    save("ref_restore.npz", ids=ids, nbits=nb, min_s=min_s, tau_s=tau_s, esc_idx=esc_idx, esc_vals=esc_vals,
         rec=rec, rec_plain=rec_plain, fma_a=a, fma_b=b, fma_c=c, fma_out=f, e4m3_lut=RD._e4m3_lut())


def blob_vectors():
    torch.manual_seed(3)
    W = (0.02 * torch.randn(12, 64)).to(torch.bfloat16)
    W[3, 5] = 0.75
    W[7, 60] = -0.5
    enc = PK.encode_tensor(W, 1e-3, restore="fp16", max_nbits=7, force_escapes=[17, 200])
    blob11 = PK.to_qvb8_blob(enc)
    (min_s, tau_s, nbits, bit_off, buf, Q, P, tau, esc_idx, esc_vals) = RD.unpack_tensor(blob11)
    hdr = np.array(RD.read_header(blob11), np.float64)
    dense = RD.decode_tensor(blob11)
    out = dict(W=W.float().numpy(), blob11=np.frombuffer(blob11, np.uint8), min_s=min_s, tau_s=tau_s, nbits=nbits,
               bit_off=bit_off, buf=buf, QPtau=np.array([Q, P, tau], np.float64), esc_idx=esc_idx,
               esc_vals=esc_vals, hdr=hdr, dense=dense)
    # the same tensor with its escapes split into an fp32 pool and an FP8 pool (esc_mode 1), v11 and v10
    n = len(esc_idx)
    n8 = n // 2
    e8_idx, e32_idx = esc_idx[:n8], esc_idx[n8:]
    e32_vals = esc_vals[n8:]
    rng = np.random.default_rng(4)
    e8_codes = rng.integers(0, 127, n8).astype(np.uint8)
    e8_codes[0] |= 0x80
    s8 = (np.abs(rng.normal(0.01, 0.003, Q)) + 1e-4).astype(np.float32)
    body = (min_s.astype("<f4").tobytes() + tau_s.astype("<f4").tobytes() + nbits.astype(np.uint8).tobytes()
            + bit_off.astype("<u8").tobytes() + e32_idx.astype("<i8").tobytes() + e32_vals.astype("<f4").tobytes()
            + e8_idx.astype("<i8").tobytes() + e8_codes.tobytes() + s8.tobytes() + buf.tobytes())
    for ver, fmt in ((11, L._HEADER_FMT), (10, L._HEADER_FMT_V10)):
        blob = struct.pack(fmt, L.MAGIC, Q, P, ver, tau, n, 1, n8) + body
        r = RD.unpack_tensor(blob)
        out[f"blob{ver}s"] = np.frombuffer(blob, np.uint8)
        out[f"v{ver}s_esc_idx"] = r[8]
        out[f"v{ver}s_esc_vals"] = r[9]
        out[f"v{ver}s_dense"] = RD.decode_tensor(blob)
    blob9 = struct.pack(L._HEADER_FMT_V9, L.MAGIC, Q, P, 9, tau, n) + blob11[64:]
    out["blob9"] = np.frombuffer(blob9, np.uint8)
    out["v9_dense"] = RD.decode_tensor(blob9)
    save("ref_qvb8_blob.npz", **out)

    # QVBD container, fp16 restore, bf16 source (escapes as bf16 bits) and fp32 source
    for tag, Wt in (("bf16", W), ("fp32", W.float() * 1.0001)):
        e = PK.encode_tensor(Wt, 1e-3, restore="fp16", max_nbits=7, force_escapes=[17, 200])
        qb = PK.to_qvbd_blob(e)
        d = RC.unpack_formula(qb)
        d2 = RC.unpack_formula(qb, skip_bit_decode=True)
        assert d2["codes"] is None
        save(f"ref_qvbd_{tag}.npz", W=Wt.float().numpy(), blob=np.frombuffer(qb, np.uint8),
             Qptau=np.array([d["Q"], d["P"], d["tau"], d["max_err"]], np.float64),
             source=np.array(list(d["source"].encode()), np.uint8), restore=np.array(list(d["restore"].encode()), np.uint8),
             min_s=d["min_s"], tau_s=d["tau_s"], nbits=d["nbits"], bit_off=d["bit_off"], buf=d["buf"],
             codes=d["codes"], esc_idx=d["esc_idx"], esc_vals=d["esc_vals"],
             esc_idx_fp16=d["esc_idx_fp16"], esc_vals_fp16=d["esc_vals_fp16"],
             calc=np.array(RC.calc_method_of(qb)))


def qvb8r_vectors():
    rng = np.random.default_rng(5)
    K, N = 3, 40
    F = np.zeros((K, N), np.int64)
    for k in range(K):
        w = rng.random(N) ** 3 + 1e-3
        f = np.maximum(1, np.floor(w / w.sum() * 4096)).astype(np.int64)
        f = np.minimum(f, 1024)
        while f.sum() != 4096:
            i = int(rng.integers(0, N))
            if f.sum() < 4096 and f[i] < 1024:
                f[i] += 1
            elif f.sum() > 4096 and f[i] > 1:
                f[i] -= 1
        F[k] = f
    tab = RK.slot_tables(F.astype(np.uint16))
    tiles = np.array([[0, 0, 3], [0, 3, 3], [0, 6, 2], [1, 8, 4], [2, 12, 1], [2, 13, 4], [2, 17, 4], [2, 21, 4],
                      [2, 25, 4], [2, 29, 4], [2, 33, 4], [2, 37, 4], [2, 41, 4], [2, 45, 3]], np.int32)
    b8 = RF.blocks_for(tiles, 8)
    b16 = RF.blocks_for(tiles, 16)
    b2 = RF.blocks_for(tiles, 2)
    save("ref_qvb8r_tables.npz", F=F, tab=tab, tiles=tiles, blocks8=b8, blocks16=b16, blocks2=b2,
         consts=np.array([RK.PB, RK.MQ, RK.MAX_ID, RK.MAX_FREQ, RK.CENTRE, RK.ROWS_PER_TILE_DIV, RF.PAD_WORDS,
                          RF.VERSION], np.int64))


def qvb8r_file_vectors():
    """A .qvb8r file written by the REFERENCE's container.write from arrays this build's writer made, and what the
    reference's container.read / runtime_tables return for the file THIS build's container writes."""
    import tempfile
    from qvb8_amd.formats.qvb8r import codec as MK
    from qvb8_amd.formats.qvb8r import container as MC
    rng = np.random.default_rng(9)
    Q, P = 12, 256
    ids = np.clip(np.round(rng.normal(40, 8, (Q, P))), 0, 127).astype(np.int64)
    enc = MK.encode_ids(ids, n_classes=2, rows_per_tile=3)
    min_s = rng.normal(-0.08, 0.01, Q).astype(np.float32)
    tau_s = np.full(Q, 2e-3, np.float32)
    esc_idx = np.array([7, P * 5 + 9], np.int64)
    esc_val = np.array([0.5, -0.25], np.float32)
    esc_delta = np.array([0.41, -0.2], np.float32)
    cert = dict(tau=2e-3, restore="fp16")
    with tempfile.TemporaryDirectory() as td:
        ref_path = os.path.join(td, "ref.qvb8r")
        RF.write(ref_path, enc, Q, P, min_s, tau_s, esc_idx, esc_val, esc_delta, cert)
        ref_blob = open(ref_path, "rb").read()
        mine = MC.to_bytes(enc, Q, P, min_s, tau_s, esc_idx, esc_val, esc_delta, cert)
        d = RF.read(blob=mine)                                   # the reference's reader on this build's bytes
        tab, tiles, words, off = RF.runtime_tables(d)
    out = dict(ids=ids, min_s=min_s, tau_s=tau_s, esc_idx=esc_idx, esc_val=esc_val, esc_delta=esc_delta,
               ref_blob=np.frombuffer(ref_blob, np.uint8), my_blob=np.frombuffer(mine, np.uint8),
               rt_tab=tab, rt_tiles=tiles, rt_words=words, rt_off=off,
               hdr=np.array([d["Q"], d["P"], d["T"], d["K"], d["N"], d["PB"]], np.int64))
    for k in MC.ARRAYS:
        out["read_" + k] = np.asarray(d[k])
    save("ref_qvb8r_file.npz", **out)


if __name__ == "__main__":
    bits_vectors()
    restore_vectors()
    blob_vectors()
    qvb8r_vectors()
    qvb8r_file_vectors()
