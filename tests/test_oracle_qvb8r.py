"""CPU tests of the QVB8R side: the oracle's walk pinned by closed forms, round trips and (where it was built) the
reference's own compiled CPU codec; the product's writer and container against the oracle and the reference vectors."""
import numpy as np
import pytest

from oracle import qvb8_oracle as O
from oracle import qvb8r_oracle as R
from qvb8_amd.common.errors import QVB8RFormatError
from qvb8_amd.formats.qvb8r import codec as K
from qvb8_amd.formats.qvb8r import container as C


def _ids(Q, P, seed, sigma=9.0, centre=40.0):
    rng = np.random.default_rng(seed)
    shift = rng.integers(-6, 7, Q)[:, None]
    return np.clip(np.round(rng.normal(centre, sigma, (Q, P))) + shift, 0, 127).astype(np.int64)


def test_tables_and_blocks_against_reference_vectors(golden):
    g = golden("ref_qvb8r_tables.npz")
    assert np.array_equal(R.slot_tables(g["F"]), g["tab"]) and np.array_equal(K.slot_tables(g["F"]), g["tab"])
    for n in (2, 8, 16):
        assert np.array_equal(R.blocks_for(g["tiles"], n), g[f"blocks{n}"])
        assert np.array_equal(C.blocks_for(g["tiles"], n), g[f"blocks{n}"])
    assert g["consts"].tolist() == [K.PB, K.MQ, K.MAX_ID, K.MAX_FREQ, K.CENTRE, K.ROWS_PER_TILE_DIV, C.PAD_WORDS, C.VERSION]


def test_single_lane_rans_closed_form():
    """Textbook rANS on one lane, done with Python integers: the walk's arithmetic (x' = f * (x >> 12) + slot - cum) must
    invert the textbook encoder step x' = ((x // f) << 12) + x % f + cum, and a state below 2^32 takes one 32-bit word."""
    F = np.array([[1024, 1024, 1024, 512, 512]], np.int64)          # a frequency is at most 1024 (10 bits hold f - 1)
    cum = [0, 1024, 2048, 3072, 3584]
    tab = R.slot_tables(F)[0]
    rng = np.random.default_rng(1)
    syms = rng.integers(0, 5, 64).tolist()
    x, words = 1 << 32, []
    for i in range(len(syms) - 2, -1, -2):                       # pairs, backwards
        s1, s2 = syms[i], syms[i + 1]
        f1, f2 = int(F[0, s1]), int(F[0, s2])
        if x >= (f1 * f2) << 40:
            words.append(x & 0xFFFFFFFF)
            x >>= 32
        x = ((x // f2) << 12) + x % f2 + cum[s2]
        x = ((x // f1) << 12) + x % f1 + cum[s1]
    words.reverse()
    got, ptr = [], 0
    for _ in range(len(syms) // 2):
        for _h in range(2):
            E = int(tab[x & 4095])
            got.append(E & 2047)
            x = ((E >> 22) + 1) * (x >> 12) + ((E >> 11) & 2047)
        if x < 1 << 32:
            x = (x << 32) | words[ptr]
            ptr += 1
    assert got == syms and ptr == len(words) and x == 1 << 32


@pytest.mark.parametrize("Q,P,classes,rows_per_tile", [(8, 128, 1, 3), (96, 256, 3, None), (40, 4096, 2, 2), (5, 512, 1, 1)])
def test_writer_round_trip_through_the_oracle_walk(Q, P, classes, rows_per_tile):
    ids = _ids(Q, P, seed=Q + P)
    enc = K.encode_ids(ids, n_classes=classes, rows_per_tile=rows_per_tile)
    d = dict(enc, P=P, Q=Q)
    assert np.array_equal(R.ids(d), ids)
    assert sorted(enc["perm"].tolist()) == list(range(Q)) and enc["freq"].astype(np.int64).sum(1).tolist() == [4096] * enc["K"]
    assert int(enc["tiles"][:, 2].sum()) == Q and enc["T"] == int(enc["tiles"][:, 2].max())
    assert enc["states"].min() >= 1 << 32                      # decoder invariant at the start of every tile
    # the oracle's own C encoder (a restatement of the reference's) produces the same words and states tile by tile
    F = enc["freq"].astype(np.int64)
    Cm = np.concatenate([np.zeros((F.shape[0], 1), np.int64), np.cumsum(F, 1)[:, :-1]], 1)
    sym_sorted = (ids - enc["drow"].astype(np.int64)[:, None])[enc["perm"]].astype(np.int16)
    off = enc["tile_off"].astype(np.int64)
    for t, (k, r0, nr) in enumerate(enc["tiles"].tolist()):
        w, st = R.encode_tile(sym_sorted[r0:r0 + nr], F[k], Cm[k])
        assert np.array_equal(w, enc["words"][off[t]:off[t + 1]]) and np.array_equal(st, enc["states"][t]), t


def test_against_the_reference_compiled_codec():
    ref = R.reference_module()
    if ref is None:
        pytest.skip("oracle/_ref was not built here (needs the reference tree): the walk stays pinned by the round trip")
    import torch
    Q, P = 24, 512
    ids = _ids(Q, P, seed=11)
    enc = K.encode_ids(ids, n_classes=2, rows_per_tile=3)
    F = enc["freq"].astype(np.int64)
    Cm = np.concatenate([np.zeros((F.shape[0], 1), np.int64), np.cumsum(F, 1)[:, :-1]], 1)
    sym_sorted = (ids - enc["drow"].astype(np.int64)[:, None])[enc["perm"]].astype(np.int16)
    # (1) the reference's encoder, given the same symbols / tiles / tables, emits the same stream
    words, off, states = ref.encode(torch.from_numpy(np.ascontiguousarray(sym_sorted)), torch.from_numpy(enc["tiles"].astype(np.int64)),
                                    torch.from_numpy(F), torch.from_numpy(Cm))
    assert np.array_equal(words.numpy().view(np.uint32), enc["words"])
    assert np.array_equal(off.numpy(), enc["tile_off"].astype(np.int64))
    assert np.array_equal(states.numpy().view(np.uint64), enc["states"])
    # (2) the reference's row decoder reads this build's stream back: value = m + fl(id * t) in its embedding flavour
    tab = K.slot_tables(enc["freq"])
    inv = np.empty(Q, np.int32); inv[enc["perm"]] = np.arange(Q, dtype=np.int32)
    row_tile = np.repeat(np.arange(len(enc["tiles"]), dtype=np.int32), enc["tiles"][:, 2])
    mn = np.zeros(Q, np.float32); ts = np.ones(Q, np.float32)
    wpad = np.concatenate([enc["words"], np.zeros(C.PAD_WORDS, np.uint32)])
    t = lambda a: torch.from_numpy(np.ascontiguousarray(a))
    out = ref.embed_rows(t(np.arange(Q, dtype=np.int64)), t(wpad.view(np.int32)), t(enc["tile_off"].astype(np.int64)),
                         t(enc["states"].view(np.int64)), t(enc["tiles"].astype(np.int64)), t(tab.view(np.int32)), t(inv), t(row_tile),
                         t(mn), t(ts), t(enc["drow"].astype(np.int32)), t(np.zeros(Q + 1, np.int64)), t(np.zeros(0, np.int32)),
                         t(np.zeros(0, np.float32)), P)
    assert np.array_equal(out.numpy().astype(np.int64), ids)       # min 0, step 1: the value IS the id
    assert np.array_equal(ref.row_hist(t(sym_sorted), int(enc["N"])).numpy().sum(0), np.bincount(sym_sorted.reshape(-1), minlength=int(enc["N"])))


def test_container_round_trip_and_restore_invariant(tmp_path):
    """QVB8R restore == QVB8 restore of the same ids (the format's defining invariant), through the file."""
    Q, P = 32, 256
    rng = np.random.default_rng(3)
    ids = _ids(Q, P, seed=3)
    min_s = rng.normal(-0.08, 0.01, Q).astype(np.float32)
    tau_s = np.full(Q, 2e-3, np.float32)
    esc_idx = np.array([5, P * 7 + 100, P * 31 + 255], np.int64)
    esc_val = np.array([0.5, -0.25, 0.125], np.float32)
    band = O.reconstruct(min_s, tau_s, ids, np.zeros(0, np.int64), np.zeros(0, np.float32))
    esc_delta = esc_val - band.reshape(-1)[esc_idx]
    enc = K.encode_ids(ids)
    path = str(tmp_path / "w.qvb8r")
    n = C.write(path, enc, Q, P, min_s, tau_s, esc_idx, esc_val, esc_delta, cert=dict(tau=2e-3, restore="fp16"))
    blob = open(path, "rb").read()
    assert n == len(blob) and len(blob) % 4 == 0
    d = C.read(path)
    od = R.read_container(blob)                                  # the oracle's independent reader
    for k in C.ARRAYS:
        assert np.array_equal(d[k], od[k]), k
    assert (d["Q"], d["P"], d["T"], d["K"], d["N"], d["PB"]) == (Q, P, enc["T"], enc["K"], enc["N"], 12) and d["cert"]["restore"] == "fp16"
    assert all(off % 64 == 0 for off, _, _ in d["arrays"].values())
    want = O.reconstruct(min_s, tau_s, ids, esc_idx, esc_val)
    assert np.array_equal(R.reconstruct(od).view(np.uint32), want.view(np.uint32))
    tab, tiles, words, off = C.runtime_tables(d)
    otab, otiles, owords, ooff = R.runtime_tables(od)
    assert np.array_equal(tab, otab) and np.array_equal(words, owords) and len(words) == len(d["words"]) + 2048
    assert tiles.dtype == np.int64 and off.dtype == np.int64 and np.array_equal(off, ooff)
    # damaged files are refused
    bad = bytearray(blob); bad[200] ^= 1
    with pytest.raises(QVB8RFormatError):
        C.read(blob=bytes(bad))
    with pytest.raises(QVB8RFormatError):
        C.read(blob=b"QVBX" + blob[4:])
    v1 = bytearray(blob); v1[4:8] = np.uint32(1).tobytes()
    with pytest.raises(QVB8RFormatError):
        C.read(blob=bytes(v1))


def test_writer_limits():
    with pytest.raises(QVB8RFormatError):
        K.encode_ids(np.zeros((4, 100), np.int64))               # P % 128
    wide = np.zeros((2, 128), np.int64); wide[0, 0] = 5000
    with pytest.raises(QVB8RFormatError):
        K.encode_ids(wide)                                       # a row spanning more than 2048 symbols
    const = np.full((3, 128), 17, np.int64)                      # a constant tensor still codes (1 symbol <= 1024 / 4096)
    e = K.encode_ids(const)
    assert np.array_equal(R.ids(dict(e, P=128, Q=3)), const)
    f = K.quantise_frequencies(np.array([10**6, 1, 0, 3]))
    assert f.sum() == 4096 and f.max() <= 1024 and f[1] >= 1 and f[3] >= 1


def test_container_against_the_reference_reader_and_writer(golden):
    """The reference's container.write output for this build's arrays is reproduced byte for byte, and what the
    reference's container.read / runtime_tables returned for this build's file equals what the readers here return."""
    g = golden("ref_qvb8r_file.npz")
    ids, Q, P = g["ids"], int(g["hdr"][0]), int(g["hdr"][1])
    enc = K.encode_ids(ids, n_classes=2, rows_per_tile=3)
    mine = C.to_bytes(enc, Q, P, g["min_s"], g["tau_s"], g["esc_idx"], g["esc_val"], g["esc_delta"], dict(tau=2e-3, restore="fp16"))
    assert mine == g["my_blob"].tobytes() == g["ref_blob"].tobytes()
    for reader in (lambda b: C.read(blob=b), R.read_container):
        d = reader(g["ref_blob"].tobytes())
        for k in C.ARRAYS:
            assert np.array_equal(np.asarray(d[k]), g["read_" + k]) and np.asarray(d[k]).dtype == g["read_" + k].dtype, k
        assert [d["Q"], d["P"], d["T"], d["K"], d["N"], d["PB"]] == g["hdr"].tolist()
    d = C.read(blob=mine)
    for got, want in zip(C.runtime_tables(d), (g["rt_tab"], g["rt_tiles"], g["rt_words"], g["rt_off"])):
        assert np.array_equal(got, want) and got.dtype == want.dtype
    for got, want in zip(R.runtime_tables(R.read_container(mine)), (g["rt_tab"], g["rt_tiles"], g["rt_words"], g["rt_off"])):
        assert np.array_equal(got, want)
    assert np.array_equal(R.ids(R.read_container(mine)), ids)


def test_concat_is_the_members_stacked():
    """Joining tensors (same row length, different alphabets, classes and rows per tile) gives a tensor whose walk yields
    the members' ids stacked in order, whose restore is the members' restores stacked, and whose escapes follow their
    rows; the split points are the members' row counts.  The joined tensor also survives the file round trip."""
    from qvb8_amd.formats.qvb8r import codec, container, fuse
    rng = np.random.default_rng(11)
    P, members = 256, []
    for Q, spread, kw in ((40, 9, dict(rows_per_tile=3, n_classes=2)), (7, 30, dict(rows_per_tile=1)), (65, 4, dict(n_classes=3))):
        ids = np.clip(np.rint(rng.normal(60, spread, (Q, P))), 0, 2000).astype(np.int64)
        enc = codec.encode_ids(ids, **kw)
        ei = np.sort(rng.choice(Q * P, 5, replace=False)).astype(np.int64)
        d = dict(enc, Q=Q, P=P, PB=codec.PB, min_s=rng.normal(0, 0.1, Q).astype(np.float32),
                 tau_s=(np.abs(rng.normal(2e-3, 1e-4, Q)) + 1e-5).astype(np.float32), esc_idx=ei,
                 esc_val=rng.normal(0, 1, 5).astype(np.float32), esc_delta=rng.normal(0, 1e-3, 5).astype(np.float32), cert={})
        members.append((ids, d))
    joined, splits = fuse.concat([d for _, d in members])
    assert splits == [40, 47] and joined["Q"] == 112 and joined["K"] == 6 and joined["T"] == 16
    assert joined["N"] == max(d["N"] for _, d in members)
    assert np.array_equal(R.ids(joined), np.vstack([ids for ids, _ in members]))
    assert np.array_equal(R.reconstruct(joined).view(np.uint32), np.vstack([R.reconstruct(d) for _, d in members]).view(np.uint32))
    assert np.array_equal(joined["esc_delta"], np.concatenate([d["esc_delta"] for _, d in members]))
    blob = container.to_bytes(joined, joined["Q"], P, joined["min_s"], joined["tau_s"], joined["esc_idx"], joined["esc_val"],
                              joined["esc_delta"], {})
    back = container.read(blob=blob)
    assert np.array_equal(R.ids(back), R.ids(joined))
    with pytest.raises(ValueError):
        fuse.concat([members[0][1], dict(members[1][1], P=128)])
