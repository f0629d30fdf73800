"""CPU tests of the host side: the package's own pack readers / writers against the reference's golden vectors, the
synthetic encoder's certificate, and the C-ABI library (loads, exports every symbol the header declares; no compute)."""
import ctypes
import json
import os
import re

import numpy as np
import pytest
import torch

from oracle import qvb8_oracle as O
from qvb8_amd.common.errors import EscapeTableError, Qvb8Error
from qvb8_amd.formats.qvb8 import decode as L
from qvb8_amd.formats.qvb8 import escape_split as ES
from qvb8_amd.formats.qvb8 import pack as PK
from qvb8_amd.formats.qvb8 import pack_container as C

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_legacy_reader_and_writer_against_reference_vectors(golden):
    g = golden("ref_qvb8_blob.npz")
    blob = g["blob11"].tobytes()
    min_s, tau_s, nb, off, buf, Q, P, tau, ei, ev = L.unpack_tensor(blob)
    for got, key in ((min_s, "min_s"), (tau_s, "tau_s"), (nb, "nbits"), (off, "bit_off"), (buf, "buf"), (ei, "esc_idx"), (ev, "esc_vals")):
        assert np.array_equal(np.asarray(got).astype(g[key].dtype), g[key]), key
    assert [Q, P, tau] == g["QPtau"].tolist()
    assert list(L.read_header(blob)) == g["hdr"].tolist()
    # the writer reproduces the reference's bytes
    again = L.pack_tensor(min_s, tau_s, nb, off, buf, Q, P, tau, ei, ev)
    assert again == blob
    # split-pool (FP8 E4M3) variants and version 9 read to the same escapes / dense values as the reference
    for tag, key in (("v11s", "blob11s"), ("v10s", "blob10s")):
        r = L.unpack_tensor(g[key].tobytes())
        assert np.array_equal(r[8], g[f"{tag}_esc_idx"])
        assert np.array_equal(np.asarray(r[9], np.float32).view(np.uint32), g[f"{tag}_esc_vals"].view(np.uint32))
    r9 = L.unpack_tensor(g["blob9"].tobytes())
    ids = O.unpack_bits_rows(r9[4], np.asarray(r9[2], np.int64), r9[3], r9[5], r9[6])
    dense = O.reconstruct(r9[0], r9[1], ids, r9[8], r9[9])
    assert np.array_equal(dense.view(np.uint32), g["v9_dense"].view(np.uint32))


@pytest.mark.parametrize("tag", ["bf16", "fp32"])
def test_container_reader_and_writer_against_reference_vectors(golden, tag):
    g = golden(f"ref_qvbd_{tag}.npz")
    blob = g["blob"].tobytes()
    assert C.calc_method_of(blob) == int(g["calc"]) == C.CALC_FORMULA
    d = C.unpack_formula(blob, skip_bit_decode=True)
    for k in ("min_s", "tau_s", "nbits", "bit_off", "buf", "esc_idx", "esc_vals", "esc_idx_fp16", "esc_vals_fp16"):
        assert np.array_equal(np.asarray(d[k]).astype(g[k].dtype), g[k]), k
    assert d["codes"] is None and d["source"] == bytes(g["source"]).decode() and d["restore"] == bytes(g["restore"]).decode()
    again = C.pack_formula(Q=d["Q"], P=d["P"], tau=d["tau"], max_err=d["max_err"], min_s=d["min_s"], tau_s=d["tau_s"],
                           nbits=d["nbits"], buf=d["buf"], esc_idx=d["esc_idx"], esc_vals=d["esc_vals"],
                           source=d["source"], restore=d["restore"])
    assert again == blob


def test_bit_packer_against_reference_vectors(golden):
    g = golden("ref_bits.npz")
    for c in range(int(g["n_cases"])):
        buf, off = L.pack_bits_rows(g[f"c{c}_ids"].astype(np.uint64), g[f"c{c}_nbits"])
        assert np.array_equal(buf, g[f"c{c}_buf"]) and np.array_equal(off, g[f"c{c}_off"]), c
    assert np.array_equal(L._nbits_for(g["nbits_for_in"]), g["nbits_for_out"])


@pytest.mark.parametrize("restore", ["fp16", "fp16+bf16"])
def test_encoder_certificate_and_round_trip(restore, tmp_path):
    g = torch.Generator().manual_seed(1)
    W = (0.02 * torch.randn(48, 256, generator=g)).to(torch.bfloat16)
    W[3, 5] = 0.9                                             # an outlier row: wider ids or escapes, still certified
    enc = PK.encode_tensor(W, 1e-3, restore=restore, force_escapes=[7, 256 * 47 + 255])
    d = dict(min_s=enc["min_s"].numpy(), tau_s=enc["tau_s"].numpy(), nbits=enc["nbits"].numpy().astype(np.int64),
             bit_off=enc["bit_off"].numpy(), buf=enc["ids"].numpy())
    assert np.array_equal(d["bit_off"], O.row_bit_offsets(d["nbits"], 256))
    ids = O.unpack_bits_rows(d["buf"], d["nbits"], d["bit_off"], 48, 256)
    Wf = W.float().numpy()
    r16 = O.restore(d["min_s"], d["tau_s"], ids, enc["esc_idx"].numpy(), enc["esc_vals"].numpy(), "fp16")
    assert O.certificate_max_err(Wf, r16) < 1e-3
    if restore == "fp16+bf16":
        rb = O.restore(d["min_s"], d["tau_s"], ids, enc["esc_idx_bf16"].numpy(), enc["esc_vals_bf16"].numpy(), "bf16")
        assert O.certificate_max_err(Wf, rb) < 1e-3
        assert max(O.certificate_max_err(Wf, r16), O.certificate_max_err(Wf, rb)) == pytest.approx(enc["max_err"], abs=1e-12)
    # file round trip through the container (+ escape_tables.json for the two-table pack)
    path = os.path.join(tmp_path, "w.qvband")
    PK.write_pack(path, enc)
    blob = open(path, "rb").read()
    back = C.unpack_formula(blob, fp16_list=ES.fp16_list_for(path), where=path)
    assert back["restore"] == restore and np.array_equal(back["buf"], d["buf"])
    assert np.array_equal(back["esc_idx_fp16"], enc["esc_idx"].numpy())
    assert np.array_equal(back["esc_idx"], enc["esc_idx_bf16"].numpy())
    # the oracle's independent reader agrees with the package's writer
    od = O.parse_qvbd_blob(blob)
    assert np.array_equal(od["buf"], d["buf"]) and np.array_equal(od["esc_idx"], enc["esc_idx_bf16"].numpy())


def test_escape_tables_missing_or_inconsistent(tmp_path):
    g = torch.Generator().manual_seed(2)
    W = (0.02 * torch.randn(8, 128, generator=g)).to(torch.bfloat16)
    enc = PK.encode_tensor(W, 1e-3, restore="fp16+bf16", force_escapes=[1, 130])
    path = os.path.join(tmp_path, "t.qvband")
    PK.write_pack(path, enc)
    tables = os.path.join(tmp_path, ES.TABLES_FILE)
    assert os.path.exists(tables) and "t.qvband" in json.load(open(tables))["tensors"]
    os.remove(tables)
    ES._CACHE.clear()
    assert ES.fp16_list_for(path) is None
    d = C.unpack_formula(open(path, "rb").read(), fp16_list=None)
    assert d["esc_idx_fp16"] is None                          # no fp16 table without the json: fp16 forwards must refuse
    assert isinstance(ES.fp16_missing_error("t.qvband"), EscapeTableError)
    with pytest.raises(EscapeTableError):
        ES.select_fp16(np.array([1, 130]), ("fp16", np.array([5]), 2, 1), "t.qvband")   # 5 is not an escape of the pack
    with pytest.raises(EscapeTableError):
        ES.select_fp16(np.array([1, 130]), ("fp16", np.array([1]), 3, 1), "t.qvband")   # written for another pack


def test_reader_and_encoder_errors():
    with pytest.raises(Qvb8Error):
        L.unpack_tensor(b"\0" * 80)
    with pytest.raises(Qvb8Error):
        C.unpack_formula(b"QVBX" + b"\0" * 60)
    with pytest.raises(Qvb8Error):
        PK.encode_tensor(torch.zeros(4), 1e-3)
    with pytest.raises(Qvb8Error):
        PK.encode_tensor(torch.full((2, 8), float("nan")), 1e-3)
    with pytest.raises(Qvb8Error):
        PK.encode_tensor(torch.zeros(2, 8), 1e-3, restore="bf16")
    e = PK.encode_tensor(torch.zeros(0, 8), 1e-3)
    assert e["Q"] == 0 and e["ids"].numel() == L.IDS_PAD_BYTES


def test_library_loads_and_exports_every_declared_symbol():
    from qvb8_amd import _lib
    header = open(os.path.join(ROOT, "include", "qvb8_amd.h")).read()
    body = re.sub(r"/\*.*?\*/", "", header, flags=re.S)
    declared = set(re.findall(r"\b(qvb8r?_[a-z0-9_]+)\s*\(", body))
    assert declared and declared == set(_lib.SYMBOLS)
    path = _lib.lib_path()
    if not os.path.exists(path):
        from qvb8_amd import build
        build.build(verbose=False)
    lib = ctypes.CDLL(path)
    for name in sorted(declared):
        assert hasattr(lib, name), name
    lib.qvb8_abi_version.restype = ctypes.c_int
    m = re.search(r"#define\s+QVB8_ABI_VERSION\s+(\d+)", header)
    assert m and lib.qvb8_abi_version() == int(m.group(1)) == _lib.EXPECTED_ABI
    lib.qvb8_last_error.restype = ctypes.c_char_p
    assert lib.qvb8_last_error() is not None
    # size queries are host-only arithmetic: callable without a GPU
    lib.qvb8_mma_rowinfo_bytes.restype = ctypes.c_int64
    lib.qvb8_mma_rowinfo_bytes.argtypes = [ctypes.c_int64]
    assert lib.qvb8_mma_rowinfo_bytes(4096) == 24 * 4096 and lib.qvb8_mma_rowinfo_bytes(0) == 0
    assert lib.qvb8_mma_rowinfo_bytes(5) == 8 * 6 + 16 * 5


def test_operators_fail_loudly_without_a_gpu():
    if torch.cuda.is_available():
        pytest.skip("needs a machine without a GPU")
    from qvb8_amd import ext_qvb8 as ext
    enc = PK.encode_tensor(torch.zeros(4, 128), 1e-3)
    with pytest.raises(RuntimeError):
        ext.decode(enc["ids"], enc["min_s"], enc["nbits"], enc["bit_off"], 128, enc["tau_s"], enc["esc_idx"], enc["esc_vals"])
    from qvb8_amd.formats.qvb8.module import QVBandLinearV8
    lin = QVBandLinearV8.from_encoded(enc)
    with pytest.raises(RuntimeError):
        lin(torch.zeros(1, 128))


def test_format_registry():
    from qvb8_amd.common import formats as F
    assert F.known_formats() == ("qvb8", "qvb8r", "qvband")
    spec = F.get_format("qvband")
    assert spec.linear.__name__ == "QVBandLinearV8" and spec.experts.__name__ == "QVBandExpertsV8"
    assert spec.filename("model.layers.0.mlp.up_proj.weight") == "model_layers_0_mlp_up_proj_weight.qvband"
    assert F.get_format("qvb8r").linear.__name__ == "QVBandLinearV8R" and F.get_format("qvb8r").experts is None
    with pytest.raises(NotImplementedError):
        F.require(F.get_format("qvb8r"), "experts")
    with pytest.raises(NotImplementedError):
        F.require(spec, "cpu_linear")
    with pytest.raises(ValueError):
        F.get_format("fp8n")


def test_plane_index_is_the_layout_the_header_describes():
    """ext_qvb8._plane_index against the layout written out with loops: step s of a tile = plane A (entry l = r + 16 (g % 4):
    dwords 0..3 of slice g of row r) then plane B (dwords 4..w-1), 256 w bytes per step."""
    import torch
    from qvb8_amd import ext_qvb8 as ext
    for P, w in ((128, 4), (256, 7), (384, 8), (128, 5)):
        to_planes, to_native = ext._plane_index(P, w, torch.device("cpu"))
        assert sorted(to_planes.tolist()) == sorted(to_native.tolist()) == list(range(16 * P // 32 * w))
        where = dict(zip(to_native.tolist(), to_planes.tolist()))
        for r in range(16):
            for g in range(P // 32):
                for d in range(w):
                    native = (r * (P // 32) + g) * w + d
                    step, entry = g // 4, r + 16 * (g % 4)
                    want = step * 64 * w + (entry * 4 + d if d < 4 else 256 + entry * (w - 4) + d - 4)
                    assert where[native] == want


def test_rows_widened_to_whole_tiles_on_the_host():
    """widen_rows_to_whole_tiles on CPU tensors: every id survives (read back field by field), no row gets narrower,
    every run of a width below the last is whole tiles."""
    import torch
    from qvb8_amd import ext_qvb8 as ext
    from tests import helpers as H
    for Q, P, widths in ((300, 128, [7, 6, 5]), (40, 128, [5, 6, 7, 8]), (31, 128, [6, 7]), (64, 128, [7]), (50, 128, [6, 9])):
        d = H.mixed_width_pack(Q, P, widths, seed=Q)
        ids, _, nbits, bit_off = H.to_device_args(d, "cpu")[:4]
        wide = ext.widen_rows_to_whole_tiles(ids, nbits, bit_off, P)
        if wide is None:
            counts = sorted(zip(*[t.tolist() for t in torch.unique(nbits, return_counts=True)]))
            assert all(n % 16 == 0 or nxt[0] > 8 for (_, n), nxt in zip(counts[:-1], counts[1:]))
            continue
        ids2, nb2, off2 = wide
        assert bool((nb2 >= nbits).all())
        buf = ids2.numpy()
        for q in range(Q):
            w = int(nb2[q])
            for c in (0, 1, 31, 32, P // 2, P - 1):
                pos = int(off2[q]) + c * w
                v = int.from_bytes(buf[pos >> 3:(pos >> 3) + 4].tobytes(), "little")
                assert (v >> (pos & 7)) & ((1 << w) - 1) == d["ids_dense"][q, c]
        runs = sorted(zip(*[t.tolist() for t in torch.unique(nb2, return_counts=True)]))
        for (w, n), (w_next, _) in zip(runs[:-1], runs[1:]):
            assert n % 16 == 0 or w_next > 8, runs


def test_tile_uniform_widths_and_repack_rows_on_the_host():
    """tile_uniform_widths gives every whole 16-row tile whose widths lie in 4..8 its largest width and leaves other rows
    alone; repack_rows stores the rows again in those widths, in row order from byte 0, every id unchanged (read back field
    by field); a regular stack is recognised, an irregular one is not."""
    import torch
    from qvb8_amd import ext_qvb8 as ext
    from tests import helpers as H
    for Q, P, widths in ((96, 128, [5, 6, 6, 6, 7]), (40, 64, [5, 6, 7, 8]), (64, 128, [7]), (50, 96, [6, 9, 3]), (37, 40, [4, 5])):
        d = H.mixed_width_pack(Q, P, widths, seed=Q)
        ids, _, nbits, bit_off = H.to_device_args(d, "cpu")[:4]
        target = ext.tile_uniform_widths(nbits)
        nb = nbits.to(torch.int64)
        whole = Q // 16 * 16
        tiles = nb[:whole].view(-1, 16)
        sliced = (tiles.amin(1) >= 4) & (tiles.amax(1) <= 8)
        want = torch.where(sliced[:, None], tiles.amax(1, keepdim=True).expand_as(tiles), tiles).reshape(-1)
        if target is None:
            assert torch.equal(want, nb[:whole])
            target = nbits
        else:
            assert torch.equal(target[:whole].to(torch.int64), want) and torch.equal(target[whole:], nbits[whole:])
        ids2, off2 = ext.repack_rows(ids, nbits, bit_off, P, target)
        row_bits = target.to(torch.int64) * P
        assert torch.equal(off2, torch.cumsum(row_bits, 0) - row_bits) and ids2.numel() == int(row_bits.sum()) // 8 + 8
        buf = ids2.numpy()
        for q in range(Q):
            w = int(target[q])
            for c in (0, 1, P // 2, P - 1):
                pos = int(off2[q]) + c * w
                v = int.from_bytes(buf[pos >> 3:(pos >> 3) + 4].tobytes(), "little")
                assert (v >> (pos & 7)) & ((1 << w) - 1) == d["ids_dense"][q, c]
    with pytest.raises(RuntimeError):
        ext.repack_rows(ids, nbits, bit_off, P, torch.full_like(nbits, 3))
    # two experts of 32 rows x 64 columns in 6 bits, back to back at a stride of 1600 bytes
    nb = torch.full((2, 32), 6, dtype=torch.uint8)
    off = (torch.arange(2).view(2, 1) * 1600 * 8 + torch.arange(32).view(1, 32) * 64 * 6).to(torch.int64)
    assert ext.stack_is_regular(nb, off, 64)
    off2 = off.clone(); off2[1, 5] += 8
    nb2 = nb.clone(); nb2[0, 3] = 5
    assert not ext.stack_is_regular(nb, off2, 64) and not ext.stack_is_regular(nb2, off, 64)


def test_unit_order_of_a_gate_up_pack():
    """Units of 16 outputs, gate rows then up rows, every row of a unit at the unit's widest width, widths ascending."""
    import torch
    from qvb8_amd.formats.qvb8.mlp import unit_order, UNIT
    inter = 96
    g = torch.Generator().manual_seed(5)
    nbits = torch.randint(3, 7, (2 * inter,), generator=g).to(torch.uint8)
    perm, new_nbits = unit_order(nbits, inter)
    perm = perm.to(torch.int64)
    assert sorted(perm.tolist()) == list(range(2 * inter))                     # a permutation of the rows
    blocks = perm.view(-1, 2, UNIT)
    assert torch.equal(blocks[:, 1], blocks[:, 0] + inter)                      # a unit's up rows follow its gate rows
    assert int(blocks[:, 0].max()) < inter
    stored = new_nbits.to(torch.int64)[perm].view(-1, 2 * UNIT)
    assert bool((stored == stored[:, :1]).all())                                 # one width per unit ...
    assert bool((stored[1:, 0] >= stored[:-1, 0]).all())                         # ... ascending over the units
    assert bool((new_nbits >= nbits.clamp(min=4)).all())                         # no row loses bits
    need = torch.maximum(nbits[:inter], nbits[inter:]).clamp(min=4).to(torch.int64)
    assert int(new_nbits.to(torch.int64).sum()) <= 2 * int(need.sum()) + 2 * UNIT * 3 * 4      # only the units at a width change are widened
    assert unit_order(nbits, inter - 1) is None and unit_order(nbits[:-1], inter) is None
    wide = nbits.clone(); wide[3] = 9
    assert unit_order(wide, inter) is None                                       # a row wider than 8 bits
