"""Host logic of the banded KV cache on the CPU: the codec (bit packing, widths, certificate, truncation) and the id layout
with its tile table, against the oracle's restatement.  No kernel is called."""
import numpy as np
import pytest
import torch

from oracle import kv_attn_oracle as A
from qvb8_amd.kv import codec as C
from qvb8_amd.kv import fused_attn as FA


@pytest.mark.parametrize("bits,n", [(1, 9), (4, 64), (6, 1000), (7, 77), (8, 5), (11, 333), (16, 40)])
def test_pack_ids_is_lsb_first_and_round_trips(bits, n):
    g = torch.Generator().manual_seed(bits * 100 + n)
    ids = torch.randint(0, 1 << bits, (n,), generator=g)
    packed = C.pack_ids(ids, bits)
    assert packed.dtype == torch.uint8 and packed.numel() == (n * bits + 7) // 8
    assert torch.equal(C.unpack_ids(packed, bits, n), ids)
    # the same bytes as the weight format's bit packing of one row (LSB first, fields back to back)
    from oracle import qvb8_oracle as O
    want = O.pack_bits_rows(ids.numpy()[None, :], np.array([bits]))
    buf = want[0] if isinstance(want, tuple) else want
    assert np.array_equal(packed.numpy(), np.asarray(buf)[:packed.numel()])


def test_known_bytes_of_three_bit_ids():
    ids = torch.tensor([1, 2, 3, 4, 5, 6, 7, 0])
    assert C.pack_ids(ids, 3).tolist() == [0xD1, 0x58, 0x1F]


def test_band_kv_heads_matches_the_oracle_codec_on_the_cpu():
    torch.manual_seed(4)
    x = (torch.randn(3, 50, 32) * torch.rand(3, 1, 32) * 4).to(torch.bfloat16)
    x[1, :, 5] = 0.75                                                # a constant channel
    for bits, tau in ((6, 0.0), (4, 0.05), (6, 0.003)):
        got = C.band_kv_heads(x, torch.bfloat16, bits, tau=tau)
        want = A.band_kv(x.float().numpy(), bits, tau, "bf16")
        for h, (bk, (ids, mn, step, b)) in enumerate(zip(got, want)):
            assert bk.bits == b and bk.orig_shape == (50, 32) and bk.orig_dtype == torch.bfloat16
            assert np.array_equal(bk.min_s.numpy(), mn) and np.array_equal(bk.tau_s.numpy(), step)
            assert np.array_equal(bk.ids().numpy(), ids)
            assert bk.nbytes() == (50 * 32 * b + 7) // 8 + 8 * 32
            if tau > 0:
                assert float((bk.decode_all_torch(dtype=torch.bfloat16).float() - x[h].float()).abs().max()) <= tau
            assert np.array_equal(bk.decode_all_torch().numpy(), A.decode_kv(ids, mn, step))
            cut = bk.truncate(7)
            assert cut.orig_shape == (7, 32) and torch.equal(cut.ids(), bk.ids()[:7]) and bk.truncate(50) is bk
            with pytest.raises(ValueError):
                bk.truncate(0)
    assert got[1].ids()[:, 5].abs().max() == 0
    with pytest.raises(C.KVCertificateError):
        C.band_kv_heads(torch.tensor([[[0.0], [1.1], [3e4]]]), torch.float32, 6, tau=1e-9)       # 16 bits: steps of 0.46


def test_layout_and_tile_table_from_segments():
    torch.manual_seed(6)
    seg_len = [40, 9, 64]
    segs_k = [C.band_kv_heads(torch.randn(2, sl, 128).to(torch.bfloat16), torch.bfloat16, 6, tau=0.1) for sl in seg_len]
    segs_v = [C.band_kv_heads(torch.randn(2, sl, 128).to(torch.bfloat16), torch.bfloat16, 5) for sl in seg_len]
    lay = FA.layout_from_segments(segs_k, segs_v, seg_len, "cpu")
    assert lay.ki.shape == (113, 2, 128) and lay.ki.dtype == torch.uint8 and lay.n == 113
    ts, tl, tseg = A.tile_table(seg_len)
    assert np.array_equal(lay.t_start.numpy(), ts) and np.array_equal(lay.t_len.numpy(), tl) and np.array_equal(lay.t_seg.numpy(), tseg)
    assert lay.n_tiles == 2 + 1 + 2 and int(lay.t_len.max()) <= FA.BLOCK_N
    pos = 0
    for si, sl in enumerate(seg_len):
        for h in range(2):
            bk = segs_k[si][h]
            mid, step, c = A.centre_form(bk.min_s.numpy(), bk.tau_s.numpy(), bk.bits)
            assert np.array_equal(lay.kmin[si, h].numpy(), mid) and np.array_equal(lay.kstep[si, h].numpy(), step) and float(lay.kc[si, h]) == c
            assert torch.equal(lay.ki[pos:pos + sl, h].to(torch.int64), bk.ids())
            assert float(lay.vc[si, h]) == (2 ** segs_v[si][h].bits - 1) / 2
        pos += sl
    with pytest.raises(ValueError):
        FA.QVLayout(lay.ki, lay.vi, lay.kmin, lay.kstep, lay.vmin, lay.vstep, seg_len, "cpu", block_n=64)
    # more than 8 bits: no byte layout; on request 16-bit patterns in int16
    tight = C.band_kv_heads((torch.randn(1, 16, 128) * 4).to(torch.bfloat16), torch.bfloat16, 6, tau=0.004)
    assert tight[0].bits > 8 and FA.layout_from_segments([tight], [tight], [16], "cpu") is None
    wide = FA.layout_from_segments([tight], [tight], [16], "cpu", allow_wide=True)
    assert wide.ki.dtype == torch.int16
    assert torch.equal(wide.ki[:, 0].to(torch.int64) & 0xFFFF, tight[0].ids())


def test_split_planner_rules():
    assert FA.rows_per_workgroup(6, 256) == 16 and FA.rows_per_workgroup(24, 256) == 32 and FA.rows_per_workgroup(96, 256) == 32
    assert FA.rows_per_workgroup(96, 128) == 64 and FA.rows_per_workgroup(17, 128) == 32


def test_take_rows_and_unband_keep_every_value():
    torch.manual_seed(8)
    x = torch.randn(2, 30, 16).to(torch.bfloat16)
    heads = C.band_kv_heads(x, torch.bfloat16, 6, tau=0.1)
    full = C.unband_kv_4d(heads, 1, 2)
    assert full.shape == (1, 2, 30, 16) and full.dtype == torch.bfloat16
    assert float((full[0].float() - x.float()).abs().max()) <= 0.1
    rows = torch.tensor([0, 3, 4, 29])
    sub = heads[0].take_rows(rows)
    assert sub.orig_shape == (4, 16) and sub.bits == heads[0].bits and sub.min_s is heads[0].min_s
    assert torch.equal(sub.decode_all(), heads[0].decode_all()[rows])          # the same values, bit for bit
    assert torch.equal(heads[0].decode_row(3), heads[0].decode_all()[3])
    assert heads[0].take_rows(torch.arange(30)) is heads[0] and heads[0].outlier_count == 0
    with pytest.raises(ValueError):
        heads[0].take_rows(torch.tensor([30]))
    assert C.unband_kv_4d([], 1, 2).shape == (1, 2, 0, 0)
