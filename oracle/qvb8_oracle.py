"""CPU oracle for the QVB8 per-row virtual-band codec.  TEST INFRASTRUCTURE ONLY.

This file restates, in plain numpy, what the reference's readers and CPU restore
compute, so that the HIP kernels can be checked against it.  Nothing in the
shipped package may import it: only tests/, the smoke check and the CPU-baseline
leg of the benchmark do.

Every function names the reference source it follows (paths relative to the
reference tree, src/qv_band/...).

Pinning status (what fixes each function besides this file's own text):
  pack_bits_rows / unpack_bits_rows   hand-computed known answers, brute force over
                                      widths 1..14 and unaligned row starts, golden
                                      vectors produced by the reference's own
                                      pack_bits_rows / unpack_bits_rows
  fma32 / band_values / reconstruct   libm fmaf via ctypes (exhaustive over ids),
                                      float64 closed form, reference decode_tensor
                                      golden vectors
  embedding_rows                      float64 closed form rounded twice, a known answer
                                      on which the fused and the two-step value differ,
                                      agreement with reconstruct within one ulp
  narrow_fp16 / narrow_bf16           numpy.float16, torch.bfloat16
  e4m3_lut / e4m3_decode              torch.float8_e4m3fn
  parse_qvb8_blob / parse_qvbd_blob   golden vectors produced by the reference's
                                      unpack_tensor / unpack_formula
  sat_half                            closed form (clamp, then numpy.float16)
  gemv / mma / moe references         float64 matmul of the restored weights
  round_to                            closed forms (ties, fp16 subnormals, overflow)
  swiglu                              torch's CPU silu and multiply on bf16 / fp16 / fp32
                                      tensors (an independent implementation)
  mlp_reference                       identity weights reduce it to swiglu and sat_half
The synthetic ENCODER policy is not pinned by anything: the reference ships no
writer.  Any writer whose bytes the readers accept and whose restore meets the
certificate conforms.
"""
from __future__ import annotations

import struct

import numpy as np

# formats/qvb8/decode.py:53-55, 70-74, 86, 91
MAGIC = 0x38425651
VERSION = 11
HEADER_BYTES = 64
HDR_V11 = "<IIIIdQIQ20x"
HDR_V10 = "<IIIIdQIB27x"
HDR_V9 = "<IIIIdQ32x"
MAX_CERTIFIED_NBITS = 14
FP16_MANTISSA_BITS = 10

# formats/qvb8/pack_container.py:8-22
QVBD_MAGIC = b"QVBD"
QVBD_VERSION = 1
QVBD_HDR = "<4sBIIffBBB8x"
QVBD_HDR_BYTES = 32
SOURCE_CODES = {"bf16": 0, "fp8_block": 1, "q4_block": 2, "fp32": 3}
SOURCE_NAMES = {v: k for k, v in SOURCE_CODES.items()}
ESC32_WIDTH = {"bf16": 2, "fp8_block": 2, "q4_block": 2, "fp32": 4}
RESTORE_NAMES = {0: "fp16", 3: "fp16+bf16"}


class OracleFormatError(ValueError):
    """Stands in for the reference's Qvb8Error (common/errors.py:20-21)."""


# ---------------------------------------------------------------------------
# FP8 escape pool                                  formats/qvb8/decode.py:104-135
def e4m3_lut() -> np.ndarray:
    """All 256 E4M3FN bit patterns as float32 (decode.py:104-121)."""
    code = np.arange(256)
    sign = np.where(code & 0x80, -1.0, 1.0)
    expo = (code >> 3) & 0xF
    mant = code & 0x7
    sub = sign * mant * 2.0 ** -9
    nor = sign * (1.0 + mant / 8.0) * np.exp2(expo.astype(np.float64) - 7.0)
    val = np.where(expo == 0, sub, nor)
    val = np.where((expo == 15) & (mant == 7), np.nan, val)
    return val.astype(np.float32)


def e4m3_decode(codes: np.ndarray, s8_rows: np.ndarray) -> np.ndarray:
    """Stored value of an FP8 escape: fp32 product lut[code] * s8[row], narrowed to
    fp16, widened back (decode.py:127-135)."""
    with np.errstate(over="ignore", invalid="ignore"):
        prod = (e4m3_lut()[codes] * s8_rows.astype(np.float32)).astype(np.float32)
        return prod.astype(np.float16).astype(np.float32)


def combine_escapes(e32_idx, e32_vals, e8_idx, e8_codes, s8, P):
    """fp32 pool + FP8 pool -> one list ascending by flat index, stable
    (decode.py:144-161)."""
    if len(e8_idx) == 0:
        return np.asarray(e32_idx, np.int64), np.asarray(e32_vals, np.float32)
    e8_vals = e4m3_decode(np.asarray(e8_codes), np.asarray(s8)[np.asarray(e8_idx) // P])
    idx = np.concatenate([np.asarray(e32_idx, np.int64), np.asarray(e8_idx, np.int64)])
    val = np.concatenate([np.asarray(e32_vals, np.float32), e8_vals])
    order = np.argsort(idx, kind="stable")
    return idx[order], val[order]


# ---------------------------------------------------------------------------
# restore arithmetic                                formats/qvb8/decode.py:164-212
def fma32(a, b, c) -> np.ndarray:
    """a*b + c rounded once to fp32, by error-free transformations in fp32
    (decode.py:168-193: Dekker/Veltkamp TwoProduct, Knuth TwoSum)."""
    f = np.float32
    a = np.asarray(a, f)
    b = np.asarray(b, f)
    c = np.asarray(c, f)
    split = f(4097.0)                       # 2^12 + 1

    def halves(v):
        t = (split * v).astype(f)
        hi = (t - (t - v).astype(f)).astype(f)
        return hi, (v - hi).astype(f)

    p = (a * b).astype(f)
    ah, al = halves(a)
    bh, bl = halves(b)
    # exact error of the product: ((ah*bh - p) + ah*bl + al*bh) + al*bl
    e = (ah * bh).astype(f)
    e = (e - p).astype(f)
    e = (e + (ah * bl).astype(f)).astype(f)
    e = (e + (al * bh).astype(f)).astype(f)
    e = (e + (al * bl).astype(f)).astype(f)
    s = (c + p).astype(f)
    v = (s - c).astype(f)
    se = ((c - (s - v).astype(f)).astype(f) + (p - v).astype(f)).astype(f)
    return (s + (se + e).astype(f)).astype(f)


def band_values(min_s, tau_s, ids) -> np.ndarray:
    """fp32 band value of every element: fmaf(float(id), tau_s[row], min_s[row])
    (decode.py:196-209; kernels: qvb8_cuda.cu:551, 346-353)."""
    ids = np.asarray(ids)
    Q = ids.shape[0]
    ts = np.broadcast_to(np.asarray(tau_s, np.float32).reshape(-1, 1), ids.shape) \
        if np.ndim(tau_s) else np.float32(tau_s)
    m = np.broadcast_to(np.asarray(min_s, np.float32).reshape(Q, 1), ids.shape)
    return fma32(ids.astype(np.float32), ts, m)


def reconstruct(min_s, tau_s, ids, esc_idx=None, esc_vals=None) -> np.ndarray:
    """Band values with the escapes written over them (decode.py:196-212)."""
    out = np.array(band_values(min_s, tau_s, ids), np.float32, copy=True)
    if esc_idx is not None and len(esc_idx):
        out.reshape(-1)[np.asarray(esc_idx, np.int64)] = np.asarray(esc_vals, np.float32)
    return out


def narrow_fp16(v) -> np.ndarray:
    """fp32 -> fp16 (round to nearest even) -> fp32: the certified restore precision
    (backends_experts.py:67-72; qvb8_cuda.cu:686-688)."""
    with np.errstate(over="ignore"):
        return np.asarray(v, np.float32).astype(np.float16).astype(np.float32)


def narrow_bf16(v) -> np.ndarray:
    """fp32 -> bf16 (round to nearest even) -> fp32 (qvb8_cuda.cu:1699-1720).
    numpy has no bfloat16, so the rounding is done on the bit pattern."""
    u = np.ascontiguousarray(np.asarray(v, np.float32)).view(np.uint32).astype(np.uint64)
    nan = (u & 0x7FFFFFFF) > 0x7F800000
    r = (u + 0x7FFF + ((u >> 16) & 1)) & 0xFFFF0000
    r = np.where(nan, u | 0x00400000, r) & 0xFFFF0000
    return r.astype(np.uint32).view(np.float32).reshape(np.shape(v))


def bf16_bits(v) -> np.ndarray:
    """The 16-bit pattern of narrow_bf16(v)."""
    return (narrow_bf16(v).view(np.uint32) >> 16).astype(np.uint16)


def restore(min_s, tau_s, ids, esc_idx=None, esc_vals=None, dtype="fp32") -> np.ndarray:
    """Dense restore in one of the three precisions the kernels store.  Escapes are
    narrowed the same way (qvb8_cuda.cu:689-697, 1721-1725)."""
    w = reconstruct(min_s, tau_s, ids, esc_idx, esc_vals)
    if dtype == "fp16":
        return narrow_fp16(w)
    if dtype == "bf16":
        return narrow_bf16(w)
    if dtype == "fp32":
        return w
    raise ValueError(dtype)


def embedding_rows(rows, min_s, tau_s, ids, P: int, esc_idx=None, esc_vals=None, dtype="fp32") -> np.ndarray:
    """Rows `rows` of the table as the reference's embedding reads them (formats/qvb8/embedding.py:97-158): the band
    value is `min_s[r] + float(id) * tau_s[r]` as an fp32 multiply then an fp32 add (two roundings; the linear layers'
    restore fuses them), the escapes of the looked-up rows are written over it in fp32, and the result is narrowed once
    to the output dtype.  `ids` is the dense (Q, P) id matrix.  Returns fp32 holding the narrowed values."""
    rows = np.asarray(rows, np.int64).reshape(-1)
    idf = np.asarray(ids)[rows].astype(np.float32)
    ts = np.asarray(tau_s, np.float32)[rows].reshape(-1, 1)
    m = np.asarray(min_s, np.float32)[rows].reshape(-1, 1)
    prod = (idf * ts).astype(np.float32)
    out = (m + prod).astype(np.float32)
    if esc_idx is not None and len(esc_idx):
        ei = np.asarray(esc_idx, np.int64)
        er, ec = ei // P, ei - (ei // P) * P
        ev = np.asarray(esc_vals, np.float32)
        for i, r in enumerate(rows.tolist()):
            hit = er == r
            if hit.any():
                out[i, ec[hit]] = ev[hit]
    if dtype == "fp16":
        return narrow_fp16(out)
    if dtype == "bf16":
        return narrow_bf16(out)
    if dtype == "fp32":
        return out
    raise ValueError(dtype)


def certificate_max_err(w_orig, w_restored) -> float:
    """max |restored - original| over the tensor (README.md:26-27)."""
    a = np.asarray(w_orig, np.float64)
    b = np.asarray(w_restored, np.float64)
    return float(np.max(np.abs(a - b))) if a.size else 0.0


# ---------------------------------------------------------------------------
# bit packing                             formats/qvb8/decode.py:215-365, 30-43
def row_bit_offsets(nbits, P: int) -> np.ndarray:
    """Absolute bit of each row's first id; rows back to back (decode.py:215-221,
    pack_container.py:108-115)."""
    nb = np.asarray(nbits, np.int64)
    off = np.zeros(len(nb), np.int64)
    if len(nb) > 1:
        off[1:] = np.cumsum(nb[:-1] * P)
    return off


def payload_bytes(nbits, P: int) -> int:
    """Bytes of the id payload without the 8 pad bytes (pack_container.py:117-119)."""
    return (int(np.asarray(nbits, np.int64).sum()) * P + 7) // 8


def pack_bits_rows(ids, nbits):
    """(Q,P) ids -> (bytes uint8 incl. 8 zero pad bytes, bit_off uint64).  Element
    (r,c) occupies bits [bit_off[r]+c*nbits[r], +nbits[r]); stream bit k is bit k&7
    of byte k>>3; value LSB first (decode.py:286-314, 30-43)."""
    ids = np.asarray(ids, np.uint64)
    Q, P = ids.shape
    nb = np.asarray(nbits, np.int64)
    off = row_bit_offsets(nb, P)
    total = int((nb * P).sum())
    nbytes = (total + 7) // 8
    bits = np.zeros(nbytes * 8, np.uint8)
    for r in range(Q):
        w = int(nb[r])
        if w == 0 or P == 0:
            continue
        k = np.arange(w, dtype=np.uint64)
        rowbits = ((ids[r][:, None] >> k[None, :]) & np.uint64(1)).astype(np.uint8)
        bits[int(off[r]):int(off[r]) + w * P] = rowbits.reshape(-1)
    buf = np.zeros(nbytes + 8, np.uint8)
    if nbytes:
        buf[:nbytes] = np.packbits(bits, bitorder="little")
    return buf, off.astype(np.uint64)


def load_fields(buf, bit_pos, nb) -> np.ndarray:
    """Fields of width nb (array or scalar, <= 14... any <= 25) starting at absolute bit
    positions bit_pos: a 4-byte little-endian window at bit>>3, shifted by bit&7 and
    masked (qvb8_cuda.cu:42-55).  Needs 3 readable bytes past the last field's first
    byte, which the 8 pad bytes guarantee."""
    buf = np.asarray(buf, np.uint8)
    bit_pos = np.asarray(bit_pos, np.int64)
    by = bit_pos >> 3
    sh = (bit_pos & 7).astype(np.uint32)
    w = (buf[by].astype(np.uint32)
         | (buf[by + 1].astype(np.uint32) << np.uint32(8))
         | (buf[by + 2].astype(np.uint32) << np.uint32(16))
         | (buf[by + 3].astype(np.uint32) << np.uint32(24)))
    mask = (np.uint32(1) << np.asarray(nb, np.uint32)) - np.uint32(1)
    return ((w >> sh) & mask).astype(np.int64)


def unpack_bits_rows(buf, nbits, bit_off, Q: int, P: int, r0: int = 0) -> np.ndarray:
    """Inverse of pack_bits_rows: len(nbits) rows starting at absolute row r0, bit
    offsets absolute (decode.py:346-365)."""
    nb = np.asarray(nbits, np.int64)
    n = len(nb)
    out = np.zeros((n, P), np.int64)
    if n == 0 or P == 0:
        return out
    boff = np.asarray(bit_off).astype(np.int64)[r0:r0 + n]
    rows_per_block = max(1, (1 << 20) // max(1, P))
    cols = np.arange(P, dtype=np.int64)
    for i0 in range(0, n, rows_per_block):
        i1 = min(n, i0 + rows_per_block)
        pos = boff[i0:i1, None] + cols[None, :] * nb[i0:i1, None]
        out[i0:i1] = load_fields(buf, pos, np.broadcast_to(nb[i0:i1, None], pos.shape))
    return out


# ---------------------------------------------------------------------------
# blob readers
def read_header(blob: bytes):
    """(Q, P, tau, n_esc) from the first 64 bytes (decode.py:368-381)."""
    magic, Q, P, version, tau, n_esc = struct.unpack(HDR_V9, blob[:HEADER_BYTES])
    if magic != MAGIC:
        raise OracleFormatError(f"not a QVB8 blob (magic {magic:#x})")
    if version not in (9, VERSION):
        raise OracleFormatError(f"QVB8 version {version}")
    return Q, P, tau, n_esc


def parse_qvb8_blob(blob: bytes) -> dict:
    """Legacy standalone blob, versions 9/10/11 (decode.py:384-430)."""
    magic, _, _, version = struct.unpack_from("<IIII", blob, 0)
    if magic != MAGIC:
        raise OracleFormatError(f"not a QVB8 blob (magic {magic:#x})")
    if version not in (9, 10, VERSION):
        raise OracleFormatError(f"QVB8 version {version}")
    fmt = HDR_V10 if version == 10 else HDR_V11
    magic, Q, P, version, tau, n_esc, esc_mode, n_fp8 = struct.unpack(fmt, blob[:HEADER_BYTES])
    cur = HEADER_BYTES

    def take(dt, count):
        nonlocal cur
        a = np.frombuffer(blob, dt, count=count, offset=cur).copy()
        cur += a.nbytes
        return a

    min_s = take("<f4", Q)
    tau_s = take("<f4", Q)
    nbits = take(np.uint8, Q).astype(np.int64)
    bit_off = take("<u8", Q).astype(np.int64)
    if version == 9 or esc_mode == 0:
        esc_idx = take("<i8", n_esc)
        esc_vals = take("<f4", n_esc)
    else:
        if n_fp8 > n_esc:
            raise OracleFormatError(f"header says {n_fp8} FP8 escapes of {n_esc} total")
        n32 = n_esc - n_fp8
        e32_idx = take("<i8", n32)
        e32_vals = take("<f4", n32)
        e8_idx = take("<i8", n_fp8)
        e8_codes = take(np.uint8, n_fp8)
        s8 = take("<f4", Q)
        esc_idx, esc_vals = combine_escapes(e32_idx, e32_vals, e8_idx, e8_codes, s8, P)
    buf = np.frombuffer(blob, np.uint8, offset=cur).copy()
    return dict(Q=Q, P=P, tau=tau, version=version, min_s=min_s, tau_s=tau_s, nbits=nbits,
                bit_off=bit_off, buf=buf, esc_idx=esc_idx, esc_vals=esc_vals)


def parse_qvbd_blob(blob: bytes) -> dict:
    """QVBD container, formula packs (pack_container.py:33-41, 48-106).  The fp16
    escape table of an fp16+bf16 pack needs escape_tables.json and is not resolved
    here: esc_idx/esc_vals are the stored (full) list."""
    magic, ver, Q, P, tau, max_err, src, calc, rcode = struct.unpack(QVBD_HDR, blob[:QVBD_HDR_BYTES])
    if magic != QVBD_MAGIC:
        raise OracleFormatError(f"not a qvband blob (magic {magic!r})")
    if ver != QVBD_VERSION:
        raise OracleFormatError(f"qvband version {ver}")
    if rcode not in RESTORE_NAMES:
        raise OracleFormatError(f"restore code {rcode}")
    if calc != 0:
        raise OracleFormatError(f"calc_method {calc}")
    source = SOURCE_NAMES[src]
    cur = QVBD_HDR_BYTES

    def take(dt, count):
        nonlocal cur
        a = np.frombuffer(blob, dt, count=count, offset=cur).copy()
        cur += a.nbytes
        return a

    min_s = take("<f4", Q)
    tau_s = take("<f4", Q)
    nbits = take(np.uint8, Q)
    bit_off = row_bit_offsets(nbits, P)
    buf = take(np.uint8, payload_bytes(nbits, P) + 8)
    n_esc_total, n8 = struct.unpack_from("<QQ", blob, cur)
    cur += 16
    n32 = int(n_esc_total) - int(n8)
    e32_idx = take("<i8", n32)
    if ESC32_WIDTH[source] == 4:
        e32_vals = take("<u4", n32).view(np.float32)
    else:
        e32_vals = (take("<u2", n32).astype(np.uint32) << np.uint32(16)).view(np.float32)
    e8_idx = take("<i8", n8)
    e8_codes = take(np.uint8, n8)
    s8 = take("<f4", Q)
    esc_idx, esc_vals = combine_escapes(e32_idx, e32_vals, e8_idx, e8_codes, s8, P)
    return dict(Q=Q, P=P, tau=tau, max_err=max_err, source=source, restore=RESTORE_NAMES[rcode],
                min_s=min_s, tau_s=tau_s, nbits=nbits, bit_off=bit_off, buf=buf,
                esc_idx=esc_idx, esc_vals=esc_vals, s8=s8)


def parse_blob(blob: bytes) -> dict:
    """Either container, by magic (module.py:177-195)."""
    return parse_qvbd_blob(blob) if blob[:4] == QVBD_MAGIC else parse_qvb8_blob(blob)


def decode_tensor(blob: bytes) -> np.ndarray:
    """Dense fp32 reconstruction of a legacy blob (decode.py:433-438)."""
    d = parse_qvb8_blob(blob)
    ids = unpack_bits_rows(d["buf"], d["nbits"], d["bit_off"], d["Q"], d["P"])
    return reconstruct(d["min_s"], d["tau_s"], ids, d["esc_idx"], d["esc_vals"])


def cpu_linear_weights(blob: bytes) -> np.ndarray:
    """The dense weight the reference's CPU linear multiplies: QVBD packs are narrowed
    to fp16 (escapes included), legacy blobs stay fp32 (backends_experts.py:55-81)."""
    if blob[:4] == QVBD_MAGIC:
        d = parse_qvbd_blob(blob)
        ids = unpack_bits_rows(d["buf"], d["nbits"], d["bit_off"], d["Q"], d["P"])
        return narrow_fp16(reconstruct(d["min_s"], d["tau_s"], ids, d["esc_idx"], d["esc_vals"]))
    return decode_tensor(blob)


# ---------------------------------------------------------------------------
# operator references (what the kernels' outputs are compared with)
def sat_half(x) -> np.ndarray:
    """Activation narrowing: clamp to +-65504, round to fp16, NaN kept; returned
    widened to fp32 (qvb8_cuda.cu:761-764, 790-841)."""
    x = np.asarray(x, np.float32)
    c = np.where(x > 65504.0, np.float32(65504.0), np.where(x < -65504.0, np.float32(-65504.0), x))
    return c.astype(np.float16).astype(np.float32)


def linear_f64(x, W) -> np.ndarray:
    """x @ W^T in float64: the referee for every GEMV/GEMM output."""
    return np.asarray(x, np.float64) @ np.asarray(W, np.float64).T


def gemv_reference(x, d: dict, ids=None) -> np.ndarray:
    """M <= 8 GEMV semantics: fp32 band value (not narrowed), X saturated to fp16,
    escapes exact (qvb8_cuda.cu:375-453, 507-533, 1059-1166).  float64 accumulate."""
    if ids is None:
        ids = unpack_bits_rows(d["buf"], d["nbits"], d["bit_off"], d["Q"], d["P"])
    W = reconstruct(d["min_s"], d["tau_s"], ids, d.get("esc_idx"), d.get("esc_vals"))
    return linear_f64(sat_half(x), W)


def mma_reference(x, d: dict, bf16: bool, ids=None) -> np.ndarray:
    """Small-M tensor-core semantics: weight (and escape) rounded once to fp16, or to
    bf16 with bf16 activations; X saturated to fp16 in fp16 mode
    (qvb8_cuda.cu:1744-1751, 2443-2446, 2594)."""
    if ids is None:
        ids = unpack_bits_rows(d["buf"], d["nbits"], d["bit_off"], d["Q"], d["P"])
    W = reconstruct(d["min_s"], d["tau_s"], ids, d.get("esc_idx"), d.get("esc_vals"))
    if bf16:
        return linear_f64(narrow_bf16(x), narrow_bf16(W))
    return linear_f64(sat_half(x), narrow_fp16(W))


def silu(v):
    v = np.asarray(v, np.float64)
    return v / (1.0 + np.exp(-v))


def round_to(v, dtype: str) -> np.ndarray:
    """v (float64 or float32) rounded once, to nearest even, to "fp32" / "fp16" / "bf16", returned as float32."""
    v32 = np.asarray(v, np.float64).astype(np.float32)
    if dtype == "fp16":
        return narrow_fp16(v32)
    if dtype == "bf16":
        return narrow_bf16(v32)
    return v32


def swiglu(gate, up, dtype: str) -> np.ndarray:
    """silu(gate) * up as a model in `dtype` computes it: silu rounded to `dtype` before the multiply, the product rounded
    again (decode/fused_pointwise.py:60-67 `_swiglu_k`: "silu() returns the input dtype"; the eager code it replaces is
    `act_fn(gate_proj(x)) * up_proj(x)`, :143-148).  gate and up are taken as already holding values of `dtype`."""
    g = np.asarray(gate, np.float32).astype(np.float64)
    s = round_to(g / (1.0 + np.exp(-g)), dtype).astype(np.float64)
    return round_to(s * np.asarray(up, np.float32).astype(np.float64), dtype)


def mlp_reference(x, W_gate, W_up, W_down, dtype: str):
    """down_proj(act_fn(gate_proj(x)) * up_proj(x)) with packed linears, as the reference runs a dense MLP at decode
    (decode/fused_pointwise.py:194-204; each product = X saturated to fp16 times the fp32 band value, module.py:455-464,
    its result cast to the caller's `dtype`).  Products in float64.  Returns (y, h): y rounded to `dtype`, h = the
    intermediate in `dtype` (before the down product narrows it to saturated fp16)."""
    xs = sat_half(np.asarray(x, np.float32))
    g = round_to(linear_f64(xs, W_gate), dtype)
    u = round_to(linear_f64(xs, W_up), dtype)
    h = swiglu(g, u, dtype)
    y = linear_f64(sat_half(h), W_down)
    return round_to(y, dtype), h


def moe_reference(x, top_idx, top_w, W_gu: list, W_dn: list, act="silu") -> np.ndarray:
    """Per-token loop over the routed experts (backends_experts.py:228-272 semantics;
    fused kernel: qvb8_cuda.cu:937-992): h = act(gate)*up with gate = first half of the
    gate_up rows, out[t] = sum_j w[t,j] * down_e(h).  float64 throughout; x saturated
    to fp16 like every GEMV input."""
    xs = sat_half(x).astype(np.float64)
    T, k = top_idx.shape
    D = W_dn[0].shape[0]
    out = np.zeros((T, D))
    for t in range(T):
        for j in range(k):
            e = int(top_idx[t, j])
            y = W_gu[e].astype(np.float64) @ xs[t]
            if act == "silu":
                I = y.shape[0] // 2
                h = silu(y[:I]) * y[I:]
            else:                                   # relu^2, non-gated (qvb8_cuda.cu:995-1000)
                h = np.maximum(y, 0.0) ** 2
            out[t] += float(top_w[t, j]) * (W_dn[e].astype(np.float64) @ h)
    return out


def router_topk(logits, k: int):
    """softmax -> top-k -> renormalise (run/run_inference.py:92-100)."""
    z = np.asarray(logits, np.float64)
    z = z - z.max(-1, keepdims=True)
    p = np.exp(z)
    p /= p.sum(-1, keepdims=True)
    idx = np.argsort(-p, axis=-1, kind="stable")[:, :k]
    w = np.take_along_axis(p, idx, -1)
    w = w / w.sum(-1, keepdims=True)
    return idx.astype(np.int64), w.astype(np.float32)
