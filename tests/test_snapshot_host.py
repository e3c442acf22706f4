"""Snapshot images composed by the library's host code against the reference's goldens:
the `file` FNV-1a-64 column of turbovec/tests/encode_fingerprint.rs:83-92 (8 cells,
calibrated slot-addressed indexes, TV7 images) and the seven sha256 digests of
benchmarks/hillclimb/data/parity_base_{x86,arm}.json (id-map and slot-addressed images at
every mutation stage, generator benchmarks/hillclimb/parity_mutate.py:31-84; those
digests were taken when to_bytes() still emitted the flat version-6 container).  No GPU:
codes and scales come from the oracle's encode, the image from tv_host_snapshot_*."""
import hashlib
import json
import os

import numpy as np
import pytest

from golden_data import FINGERPRINT, fingerprint_seed, parity_fixture_inputs

HERE = os.path.dirname(os.path.abspath(__file__))


@pytest.fixture(scope="module")
def T():
    from turbovec_amd import _lib
    _lib.lib()
    return _lib


def sha(b):
    return hashlib.sha256(b).hexdigest()


@pytest.mark.parametrize("row", FINGERPRINT, ids=[f"{r[0]}x{r[1]}" for r in FINGERPRINT])
def test_fingerprint_file_column(T, oracle, row):
    O = oracle
    dim, bits, _wb, _wc, _wcal, _wcodes, _wscales, wfile = row
    v = O.lcg_vectors(2000, dim, fingerprint_seed(dim, bits))
    rot = O.Rotation(dim)
    b, c = T.host_codebook(bits, dim)
    sh, sc = O.fit_calibration(rot, v, c)
    packed, scales = O.encode(rot, v, bits, (sh, sc))
    seq = O.repack_seq(packed, 2000, bits, dim)
    img = T.snapshot_compose(dim, bits, b, c, seq, 2000, scales, calibration=(sh, sc))
    assert O.fnv1a(np.frombuffer(img, np.uint8)) == wfile
    # and back
    assert T.snapshot_info(img) == (7, 0, dim, bits, dim, 2000)
    back = T.snapshot_extract(img)
    assert np.array_equal(back["seq"], seq) and np.array_equal(back["scales"].view(np.uint32), scales.view(np.uint32))
    assert np.array_equal(back["shift"], sh) and np.array_equal(back["scale"], sc)
    assert np.array_equal(back["centroids"], c) and np.array_equal(back["boundaries"], b)
    assert back["ids"] is None


@pytest.fixture(scope="module")
def parity_state(oracle):
    O = oracle
    base, warm, singles, _q = parity_fixture_inputs()
    rot = O.Rotation(768)
    packed, scales = O.encode(rot, np.concatenate([base, warm, singles]), 4)
    gold = json.load(open(os.path.join(HERE, "golden", "parity_base.json")))
    return packed, scales, gold


def test_parity_fixture_images(T, oracle, parity_state):
    O = oracle
    packed, scales, gold = parity_state
    b, c = T.host_codebook(4, 768)

    def image(n, seq=None, sc=None, ids=None):
        seq = O.repack_seq(packed[:n], n, 4, 768) if seq is None else seq
        sc = scales[:n] if sc is None else sc
        return T.snapshot_compose(768, 4, b, c, seq, n, sc, ids=ids, format=6)   # the digests hash the flat container

    assert sha(image(20000, ids=np.arange(20000, dtype=np.uint64))) == gold["sha256_after_bulk"]
    assert sha(image(21000, ids=np.arange(21000, dtype=np.uint64))) == gold["sha256_after_append"]
    assert sha(image(21050, ids=np.arange(21050, dtype=np.uint64))) == gold["sha256_after_singles"]
    assert sha(image(20000)) == gold["sha256_tq_after_bulk"]

    # 500 removes by id (id_map.rs:520-567): swap-and-pop of codes, scales and the id table
    n = 21050
    seq = O.repack_seq(packed, n, 4, 768)
    sc = scales.copy()
    ids = list(range(n))
    slot_of = {x: x for x in ids}
    for rid in range(500):
        slot = slot_of.pop(rid)
        last = n - 1
        O.swap_remove_seq(seq, sc, n, 4, 768, slot)
        if slot != last:
            ids[slot] = ids[last]
            slot_of[ids[slot]] = slot
        ids.pop()
        n -= 1
    img = image(n, seq=seq, sc=sc[:n], ids=np.array(ids, np.uint64))
    assert sha(img) == gold["sha256_after_idremove"]
    # from_bytes(to_bytes()) round trip keeps the bytes
    back = T.snapshot_extract(img)
    assert back["format"] == 6 and back["kind"] == 1
    again = T.snapshot_compose(768, 4, back["boundaries"], back["centroids"], back["seq"], back["n"], back["scales"],
                               ids=back["ids"], format=6)
    assert sha(again) == gold["sha256_roundtrip"]
    # the same state re-contained as a TV7 image and back loses nothing
    v7 = T.snapshot_compose(768, 4, b, c, seq, n, sc[:n], ids=np.array(ids, np.uint64))
    b7 = T.snapshot_extract(v7)
    assert np.array_equal(b7["seq"], back["seq"]) and np.array_equal(b7["ids"], back["ids"])
    assert np.array_equal(b7["scales"].view(np.uint32), back["scales"].view(np.uint32))

    n = 20000
    seq = O.repack_seq(packed[:n], n, 4, 768)
    sc = scales[:n].copy()
    for _ in range(500):
        n = O.swap_remove_seq(seq, sc, n, 4, 768, 0)
    assert sha(image(n, seq=seq, sc=sc[:n])) == gold["sha256_tq_after_swap"]


def test_image_validation(T, oracle):
    O = oracle
    dim, bits, n = 64, 4, 70                      # 2 units + 6 tail rows
    rng = np.random.default_rng(0)
    v = rng.standard_normal((n, dim)).astype(np.float32)
    packed, scales = O.encode(O.Rotation(dim), v, bits)
    seq = O.repack_seq(packed, n, bits, dim)
    b, c = T.host_codebook(bits, dim)
    ids = rng.permutation(1 << 40)[:n].astype(np.uint64) if False else (np.arange(n, dtype=np.uint64) * np.uint64(7919) + np.uint64(3))
    img = T.snapshot_compose(dim, bits, b, c, seq, n, scales, ids=ids)
    assert len(img) == len(T.snapshot_compose(dim, bits, b, c, seq, 64, scales[:64], ids=ids[:64]))  # tail rides in the header
    back = T.snapshot_extract(img)
    assert back["kind"] == 1 and np.array_equal(back["ids"], ids) and np.array_equal(back["seq"], seq)
    empty = T.snapshot_compose(dim, bits, b, c, np.zeros(0, np.uint8), 0, np.zeros(0, np.float32))
    assert T.snapshot_info(empty) == (7, 0, dim, bits, 0, 0)
    raw = bytearray(img)
    for pos, why in ((0, "not a TV7"), (4, "revision"), (30, "superblock checksum"), (len(raw) // 3, None)):
        bad = bytearray(raw)
        bad[pos] ^= 0x5A
        if why is None:
            # unit bytes carry no checksum of their own (io_v7.rs "What is checksummed"): still loads
            T.snapshot_info(bytes(bad))
            continue
        with pytest.raises(T.TurbovecHipError, match=why) as e:
            T.snapshot_info(bytes(bad))
        assert e.value.status == 10
    sb_len = 23 + 15 * 4 + 16 * 4 + 4 + 4
    bad = bytearray(raw)
    bad[sb_len + 20] ^= 1                          # inside the header's tail rows
    with pytest.raises(T.TurbovecHipError, match="header checksum"):
        T.snapshot_info(bytes(bad))
    with pytest.raises(T.TurbovecHipError, match="length"):
        T.snapshot_info(bytes(raw[:-1]))
    with pytest.raises(T.TurbovecHipError):
        T.snapshot_info(bytes(raw[:10]))
