"""Device-side ingest (tv_index_add) against the reference's encode goldens and the oracle.

The eight (dim, bits) cells of turbovec/tests/encode_fingerprint.rs:83-92 pin
codes and scales produced on the GPU by their FNV-1a-64 hashes; seeded Gaussian
rows are compared with the oracle byte for byte, including chunked adds
(encode is batch-independent, lib.rs:738-746) and degenerate rows.
"""
import numpy as np
import pytest

from golden_data import FINGERPRINT, fingerprint_seed
from helpers import OracleIndex, bits_equal, unit_gaussian

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def T():
    from turbovec_amd import _lib
    _lib.lib()
    return _lib


@pytest.mark.parametrize("row", FINGERPRINT, ids=[f"{r[0]}x{r[1]}" for r in FINGERPRINT])
def test_fingerprint_cells_encoded_on_device(T, oracle, row):
    O = oracle
    dim, bits, _wb, _wc, _wcal, wcodes, wscales, _wfile = row
    v = O.lcg_vectors(2000, dim, fingerprint_seed(dim, bits))
    rot = O.Rotation(dim)
    _b, c = O.codebook(bits, dim)
    ix = T.NativeIndex(dim, bits)
    ix.calibrate(v)                                # the fixture calibrates before it adds
    sh, sc = ix.calibration()
    assert O.fnv1a(np.concatenate([sh, sc])) == _wcal          # the fit itself: rotated on the device, ranked on the host
    osh, osc = O.fit_calibration(rot, v, c)
    assert bits_equal(sh, osh) and bits_equal(sc, osc)
    ix.add(v)
    assert len(ix) == 2000
    seq, scales = ix.download_seq()
    packed = O.seq_to_packed(seq, 2000, bits, dim)
    assert O.fnv1a(packed) == wcodes
    assert O.fnv1a(scales) == wscales
    ix.close()


@pytest.mark.parametrize("dim,bits", [(128, 4), (1536, 4), (1536, 2), (3072, 4), (64, 3), (8, 2)])
def test_add_matches_oracle_and_is_batch_independent(T, oracle, dim, bits):
    O = oracle
    n = 1000
    v = unit_gaussian(n, dim, seed=dim + bits) * np.float32(3.7)      # not unit length: the norm matters
    v[5] = 0.0                                                        # zero row -> scale 0
    v[6] = v[7]                                                       # duplicate rows -> identical codes
    v[8] *= np.float32(1e-12)                                         # below MIN_INPUT_NORM
    oidx = OracleIndex(O, dim, bits, v)
    one = T.NativeIndex(dim, bits)
    one.add(v)
    seq, scales = one.download_seq()
    assert np.array_equal(seq, oidx.seq)
    assert bits_equal(scales, oidx.scales)
    chunked = T.NativeIndex(dim, bits)
    for a, b in ((0, 1), (1, 33), (33, 64), (64, 700), (700, n)):
        chunked.add(v[a:b])
    seq2, scales2 = chunked.download_seq()
    assert np.array_equal(seq2, seq) and bits_equal(scales2, scales)
    # a search over the device-encoded index equals the oracle's over its own encode
    q = unit_gaussian(7, dim, seed=99)
    s, i = one.search(q, 10)
    os_, oi = oidx.search(q, 10)
    assert np.array_equal(i, oi) and bits_equal(s, os_)
    one.close()
    chunked.close()


def test_add_after_mutations_and_validation(T, oracle):
    O = oracle
    dim, bits = 256, 4
    v = unit_gaussian(300, dim, seed=1)
    ix = T.NativeIndex(dim, bits)
    ix.add(v[:200])
    ix.swap_remove(3)
    ix.add(v[200:])
    order = list(range(200))
    order[3] = 199
    order = order[:199] + list(range(200, 300))
    oidx = OracleIndex(O, dim, bits, v[order])
    seq, scales = ix.download_seq()
    assert np.array_equal(seq, oidx.seq) and bits_equal(scales, oidx.scales)
    bad = v[:4].copy()
    bad[2, 17] = np.nan
    with pytest.raises(T.TurbovecHipError) as e:
        ix.add(bad)
    assert e.value.status == 2 and len(ix) == 299      # nothing was added
    bad[2, 17] = 2e16
    with pytest.raises(T.TurbovecHipError):
        ix.add(bad)
    ix.add(np.zeros((0, dim), np.float32))
    assert len(ix) == 299
    ix.close()


# ---- the whole device pipeline against the reference's byte-level goldens ----
def test_fingerprint_file_bytes_from_the_device(T, oracle):
    """add on the device -> tv_index_to_bytes == the `file` column (encode_fingerprint.rs:83-92)."""
    O = oracle
    for row in FINGERPRINT:
        dim, bits, _wb, _wc, _wcal, _wcodes, _wscales, wfile = row
        v = O.lcg_vectors(2000, dim, fingerprint_seed(dim, bits))
        _b, c = O.codebook(bits, dim)
        sh, sc = O.fit_calibration(O.Rotation(dim), v, c)
        ix = T.NativeIndex(dim, bits)
        ix.set_calibration(sh, sc)
        ix.add(v)
        img = ix.to_bytes()
        assert O.fnv1a(np.frombuffer(img, np.uint8)) == wfile
        back, ids = T.NativeIndex.from_bytes(img)
        assert ids is None and len(back) == 2000 and back.to_bytes() == img
        q = v[:5]
        s0, i0 = ix.search(q, 10)
        s1, i1 = back.search(q, 10)
        assert np.array_equal(i0, i1) and bits_equal(s0, s1)
        ix.close()
        back.close()


def test_parity_fixture_digests_from_the_device(T):
    """benchmarks/hillclimb/parity_mutate.py:31-84 replayed on the host mirror: every to_bytes()
    digest of the run (flat version-6 container, which is what the digests were taken over)."""
    import hashlib
    import json
    import os
    from golden_data import parity_fixture_inputs
    from turbovec_amd.index import IdMapIndex, TurboQuantIndex
    gold = json.load(open(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "parity_base.json")))
    base, warm, singles, queries = parity_fixture_inputs()
    N, BATCH = len(base), len(warm)

    def sha6(idx, ids=None):
        return hashlib.sha256(idx._ix.to_bytes(ids=ids, format=6)).hexdigest()

    def ids_of(m):
        return np.asarray(m._slot_to_id, np.uint64)

    ix = IdMapIndex(dim=768, bit_width=4)
    ix.add_with_ids(base, np.arange(N, dtype=np.uint64))
    assert sha6(ix._inner, ids_of(ix)) == gold["sha256_after_bulk"] and len(ix) == gold["len_after_bulk"]
    ix.add_with_ids(warm, np.arange(N, N + BATCH, dtype=np.uint64))
    assert sha6(ix._inner, ids_of(ix)) == gold["sha256_after_append"]
    for i in range(len(singles)):
        ix.add_with_ids(singles[i:i + 1], np.array([N + BATCH + i], dtype=np.uint64))
    assert sha6(ix._inner, ids_of(ix)) == gold["sha256_after_singles"] and len(ix) == gold["len_after_singles"]
    ix._inner._ix.set_score_mode(T.SCORE_L_CLASSIC)          # the fixture's floats come from the LUT kernel
    s, g = ix.search(queries, 10)
    assert np.array_equal(g, np.array(gold["search_ids"], np.uint64)) and bits_equal(s, np.array(gold["search_scores"], np.float32))
    for i in range(500):
        assert ix.remove(i)
    assert sha6(ix._inner, ids_of(ix)) == gold["sha256_after_idremove"] and len(ix) == gold["len_after_idremove"]
    s, g = ix.search(queries, 10)
    assert np.array_equal(g, np.array(gold["post_remove_ids"], np.uint64)) and bits_equal(s, np.array(gold["post_remove_scores"], np.float32))
    again = IdMapIndex.from_bytes(ix.to_bytes())
    assert sha6(again._inner, ids_of(again)) == gold["sha256_roundtrip"]
    assert again.to_bytes() == ix.to_bytes()

    tq = TurboQuantIndex(dim=768, bit_width=4)
    tq.add(base)
    assert sha6(tq) == gold["sha256_tq_after_bulk"]
    for _ in range(500):
        tq.swap_remove(0)
    assert sha6(tq) == gold["sha256_tq_after_swap"] and len(tq) == gold["tq_len"]
    tq._ix.set_score_mode(T.SCORE_L_CLASSIC)
    s, i = tq.search(queries, 10)
    assert np.array_equal(i, np.array(gold["tq_ids"])) and bits_equal(s, np.array(gold["tq_scores"], np.float32))


def test_write_and_load(T, tmp_path):
    from turbovec_amd.index import IdMapIndex, TurboQuantIndex
    v = unit_gaussian(100, 128, seed=3)
    a = TurboQuantIndex(128, 4)
    a.add(v)
    p = tmp_path / "a.tv"
    a.write(p)
    b = TurboQuantIndex.load(p)
    assert len(b) == 100 and b.to_bytes() == a.to_bytes() and open(p, "rb").read() == a.to_bytes()
    s0, i0 = a.search(v[:3], 5)
    s1, i1 = b.search(v[:3], 5)
    assert np.array_equal(i0, i1) and bits_equal(s0, s1)
    m = IdMapIndex(128, 2)
    m.add_with_ids(v, np.arange(100, dtype=np.uint64) + np.uint64(1 << 50))
    m.remove((1 << 50) + 7)
    pm = tmp_path / "m.tvim"
    m.write(pm)
    m2 = IdMapIndex.load(pm)
    assert len(m2) == 99 and not m2.contains((1 << 50) + 7) and m2.to_bytes() == m.to_bytes()
    _s, g = m2.search(v[20:21], 1)
    assert g[0, 0] == (1 << 50) + 20
    with pytest.raises(FileNotFoundError):
        a.write(tmp_path / "missing" / "a.tv")
    with pytest.raises(FileNotFoundError):
        TurboQuantIndex.load(tmp_path / "nope.tv")
    bad = tmp_path / "bad.tv"
    bad.write_bytes(b"TV7\0garbage")
    with pytest.raises(OSError):
        TurboQuantIndex.load(bad)
    with pytest.raises(OSError):
        TurboQuantIndex.load(pm)                     # an id-map image is not a slot-addressed index
