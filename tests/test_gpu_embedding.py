"""GPU parity: the row lookup (qvb8_lookup_rows through the C ABI) and QVBandEmbeddingV8 against the CPU oracle's
restatement of the reference's embedding read.  Bit-exact in every output dtype."""
import os

import numpy as np
import pytest
import torch

from oracle import qvb8_oracle as O
from qvb8_amd import ext_qvb8 as ext
from qvb8_amd.formats.qvb8 import pack as PK
from qvb8_amd.formats.qvb8.embedding import QVBandEmbeddingV8
from tests import helpers as H

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
DTYPES = ((torch.float32, "fp32"), (torch.float16, "fp16"), (torch.bfloat16, "bf16"))


def _same_bits(got: torch.Tensor, want_f32: np.ndarray, name: str) -> bool:
    if name == "fp32":
        return np.array_equal(got.cpu().numpy().view(np.uint32), want_f32.view(np.uint32))
    if name == "fp16":
        return np.array_equal(got.cpu().view(torch.int16).numpy().view(np.uint16), want_f32.astype(np.float16).view(np.uint16))
    return np.array_equal(got.cpu().view(torch.int16).numpy().view(np.uint16), O.bf16_bits(want_f32))


def _lookup(d, rows, dtype):
    ids, min_s, nbits, bit_off, P, tau_s, ei, ev = H.to_device_args(d, DEV)
    return ext.lookup_rows(torch.from_numpy(rows).to(DEV), ids, min_s, nbits, bit_off, P, tau_s, ei, ev, dtype)


@pytest.mark.parametrize("Q,P,widths", [
    (64, 4096, [7]), (48, 5120, [6, 7]), (40, 2080, [4, 5, 6, 7, 8]),                      # dword-sliced path
    (29, 96, list(range(1, 15))), (17, 13, [3, 7, 11]), (5, 1, [14, 1]), (6, 6144, [7, 3, 12]),   # per-element path
])
def test_lookup_rows_bit_exact_hand_made_packs(Q, P, widths):
    d = H.mixed_width_pack(Q, P, widths, seed=Q * 17 + P)
    rng = np.random.default_rng(Q + P)
    rows = np.concatenate([rng.integers(0, Q, 23), [0, Q - 1, Q - 1]]).astype(np.int64)      # repeats, both ends
    # escapes in some of the looked-up rows (first and last column included) and in rows nobody asks for
    esc = sorted({int(rows[0]) * P, int(rows[0]) * P + P - 1, (Q - 1) * P + P // 2, int(rows[5]) * P + P // 3})
    d["esc_idx"] = np.array(esc, np.int64)
    d["esc_vals"] = rng.normal(0, 0.5, len(esc)).astype(np.float32)
    for dtype, name in DTYPES:
        got = _lookup(d, rows, dtype)
        want = O.embedding_rows(rows, d["min_s"], d["tau_s"], d["ids_dense"], P, d["esc_idx"], d["esc_vals"], name)
        assert got.shape == (len(rows), P) and got.dtype == dtype
        assert _same_bits(got, want, name), name


def test_lookup_rows_is_the_two_step_value_not_the_fused_one():
    """On a pack where the two differ, the lookup follows the embedding's arithmetic and the dense restore the linear's."""
    d = H.mixed_width_pack(32, 4096, [7], seed=77)
    rows = np.arange(32, dtype=np.int64)
    got = _lookup(d, rows, torch.float32).cpu().numpy()
    two = O.embedding_rows(rows, d["min_s"], d["tau_s"], d["ids_dense"], 4096)
    one = O.band_values(d["min_s"], d["tau_s"], d["ids_dense"])
    assert np.any(two != one)
    assert np.array_equal(got.view(np.uint32), two.view(np.uint32))
    dense = ext.decode_f32(*H.to_device_args(d, DEV)).cpu().numpy()
    assert np.array_equal(dense.view(np.uint32), one.view(np.uint32))


def test_lookup_rows_edges():
    d = H.mixed_width_pack(12, 256, [6, 9], seed=3)
    # no rows: an empty result, no launch
    out = _lookup(d, np.zeros(0, np.int64), torch.bfloat16)
    assert out.shape == (0, 256)
    # a row number outside the table: that row is NaN, its neighbours are untouched
    rows = np.array([4, 12, -1, 11], np.int64)
    got = _lookup(d, rows, torch.float32).cpu().numpy()
    want = O.embedding_rows(np.array([4, 11]), d["min_s"], d["tau_s"], d["ids_dense"], 256)
    assert np.array_equal(got[[0, 3]].view(np.uint32), want.view(np.uint32))
    assert np.isnan(got[1]).all() and np.isnan(got[2]).all()
    ids, min_s, nbits, bit_off, P, tau_s, ei, ev = H.to_device_args(d, DEV)
    with pytest.raises(RuntimeError):
        ext.lookup_rows(torch.zeros(3, dtype=torch.int32, device=DEV), ids, min_s, nbits, bit_off, P, tau_s, ei, ev)
    with pytest.raises(RuntimeError):
        ext.lookup_rows(torch.zeros(3, dtype=torch.int64), ids, min_s, nbits, bit_off, P, tau_s, ei, ev)


def test_embedding_module_from_packfile(tmp_path):
    Q, P = 96, 512
    W = H.synth_weight(Q, P, seed=31).to(DEV)
    forced = [7 * P + 3, 7 * P + 511, 40 * P, 95 * P + 100]
    for restore, name in (("fp16", "emb.qvband"), ("fp16", "emb.qvb8")):
        enc = PK.encode_tensor(W, 1e-3, restore=restore, force_escapes=forced)
        path = os.path.join(tmp_path, name)
        PK.write_pack(path, enc)
        d = H.oracle_view(enc)
        ids_dense = H.oracle_ids(d)
        tokens = torch.tensor([[7, 0, 95], [40, 7, 3]], dtype=torch.int64)            # host ids: the result comes back to the host
        for dtype, dname in DTYPES:
            emb = QVBandEmbeddingV8.from_packfile(path, out_dtype=dtype, device=DEV)
            assert emb.num_embeddings == Q and emb.embedding_dim == P
            y = emb(tokens)
            assert y.shape == (2, 3, P) and y.dtype == dtype and y.device.type == "cpu"
            want = O.embedding_rows(tokens.reshape(-1).numpy(), d["min_s"], d["tau_s"], ids_dense, P, d["esc_idx"], d["esc_vals"], dname)
            assert _same_bits(y.reshape(-1, P), want, dname), (name, dname)
            y_dev = emb(tokens.to(DEV))
            assert y_dev.device.type == "cuda" and torch.equal(y_dev.cpu(), y)
        # within tau of the original weights (the lookup moves a value by an ulp at most, far inside the slack)
        emb = QVBandEmbeddingV8.from_packfile(path, out_dtype=torch.float32, device=DEV)
        all_rows = emb(torch.arange(Q, device=DEV))
        assert float((all_rows - W.float()).abs().max()) < 1e-3
        # the dense view leaves the escapes out, as the reference's does; casting the module keeps the fp32 metadata
        w = emb.weight.cpu().numpy()
        assert np.array_equal(w.view(np.uint32), O.embedding_rows(np.arange(Q), d["min_s"], d["tau_s"], ids_dense, P).view(np.uint32))
        rows = emb._decode_rows(torch.tensor([40, 7], device=DEV)).cpu().numpy()
        assert np.array_equal(rows.view(np.uint32), w[[40, 7]].view(np.uint32))
        before = emb.tau_s.clone()
        emb.to(torch.bfloat16)
        assert emb.tau_s.dtype == torch.float32 and torch.equal(emb.tau_s, before) and emb.esc_vals.dtype == torch.float32


def test_embedding_index_outside_the_table():
    """Where the reference's gathers fail on an index outside the table, this operator writes a row of NaN (no host read,
    the other rows right); with check_indices it raises IndexError before any launch."""
    Q, P = 40, 256
    enc = PK.encode_tensor(H.synth_weight(Q, P, seed=5).to(DEV), 1e-3, restore="fp16")
    a = H.pack_args(enc)
    emb = QVBandEmbeddingV8(min_s=a[1], nbits=a[2], bit_off=a[3], ids=a[0], Q=Q, P=P, tau_s=a[5], esc_idx=a[6], esc_vals=a[7],
                            out_dtype=torch.float32)
    tokens = torch.tensor([3, Q, 39, -2], device=DEV)
    y = emb(tokens)
    assert bool(y[1].isnan().all()) and bool(y[3].isnan().all())
    assert torch.equal(y[[0, 2]], emb(torch.tensor([3, 39], device=DEV))) and not bool(y[[0, 2]].isnan().any())
    emb.check_indices = True
    with pytest.raises(IndexError):
        emb(tokens)
    assert torch.equal(emb(torch.tensor([3, 39], device=DEV)), y[[0, 2]])


def test_embedding_fp16_output_of_a_two_table_pack_needs_its_fp16_list(tmp_path):
    from qvb8_amd.common.errors import EscapeTableError
    W = H.synth_weight(32, 256, seed=2).to(DEV)
    enc = PK.encode_tensor(W, 1e-3, restore="fp16+bf16", force_escapes=[5, 300])
    path = os.path.join(tmp_path, "two.qvband")
    with open(path, "wb") as fh:                      # the pack alone, without escape_tables.json beside it
        fh.write(PK.to_qvbd_blob(enc))
    QVBandEmbeddingV8.from_packfile(path, out_dtype=torch.bfloat16, device=DEV)        # the full list: fine
    with pytest.raises(EscapeTableError):
        QVBandEmbeddingV8.from_packfile(path, out_dtype=torch.float16, device=DEV)


def test_registry_names_the_embedding():
    from qvb8_amd.common.formats import get_format
    assert get_format("qvb8").embedding is QVBandEmbeddingV8 and get_format("qvband").embedding is QVBandEmbeddingV8


def test_lookup_rows_refusals_through_the_c_abi():
    """Argument errors come back as a status and a message, nothing is launched."""
    from qvb8_amd import _lib
    lib = _lib.load()
    d = H.mixed_width_pack(8, 256, [6], seed=1)
    ids, min_s, nbits, bit_off, P, tau_s, _, _ = H.to_device_args(d, DEV)
    rows = torch.zeros(4, dtype=torch.int64, device=DEV)
    out = torch.empty(4 * P + 8, dtype=torch.float32, device=DEV)
    st = torch.cuda.current_stream().cuda_stream

    def call(rows_ptr=rows.data_ptr(), n=4, Q=8, out_dtype=_lib.F32, out_ptr=out.data_ptr(), esc=(None, None, 0), ids_ptr=ids.data_ptr()):
        return lib.qvb8_lookup_rows(rows_ptr, n, ids_ptr, ids.numel(), min_s.data_ptr(), tau_s.data_ptr(), nbits.data_ptr(),
                                    bit_off.data_ptr(), Q, P, esc[0], esc[1], esc[2], out_dtype, out_ptr, st)
    assert call() == 0
    assert call(n=0, rows_ptr=None) == 0                          # nothing to look up
    for bad in (dict(out_dtype=7), dict(rows_ptr=None), dict(out_ptr=out.data_ptr() + 4), dict(out_ptr=None), dict(n=-1),
                dict(esc=(None, None, 3)), dict(Q=0), dict(ids_ptr=ids.data_ptr() + 1)):
        assert call(**bad) != 0, bad
        assert lib.qvb8_last_error().decode().startswith("qvb8_lookup_rows"), bad
