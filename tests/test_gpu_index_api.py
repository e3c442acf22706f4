"""The host-side index objects, exercised the way the reference's own Python tests
exercise theirs (turbovec-python/tests/test_index.py, test_filtering.py,
test_id_map.py, test_argument_errors.py): shapes, clamping, filters, errors."""
import numpy as np
import pytest

from helpers import OracleIndex, bits_equal

pytestmark = pytest.mark.gpu

DIM = 128


def unit_vectors(n, dim=DIM, seed=0):
    rng = np.random.default_rng(seed)
    v = rng.standard_normal((n, dim)).astype(np.float32)
    v /= np.linalg.norm(v, axis=1, keepdims=True) + 1e-9
    return v


@pytest.fixture(scope="module")
def api():
    from turbovec_amd import index
    return index


# ---- TurboQuantIndex: construction, add, search shape -------------------
def test_new_reports_dim_and_bit_width(api):
    idx = api.TurboQuantIndex(dim=DIM, bit_width=3)
    assert (idx.dim, idx.bit_width, len(idx)) == (DIM, 3, 0)


@pytest.mark.parametrize("bad", [0, 1, 5, 8])
def test_constructor_rejects_bad_bit_width(api, bad):
    with pytest.raises(ValueError):
        api.TurboQuantIndex(dim=DIM, bit_width=bad)
    with pytest.raises(ValueError):
        api.IdMapIndex(dim=DIM, bit_width=bad)


@pytest.mark.parametrize("bad", [0, 7, 12, 16392])
def test_constructor_rejects_bad_dim(api, bad):
    with pytest.raises(ValueError):
        api.TurboQuantIndex(dim=bad, bit_width=4)


def test_add_is_incremental_and_search_shape(api):
    idx = api.TurboQuantIndex(DIM, 4)
    idx.add(unit_vectors(60, seed=1))
    idx.add(unit_vectors(40, seed=2))
    assert len(idx) == 100
    s, i = idx.search(unit_vectors(5, seed=3), 10)
    assert s.shape == (5, 10) and i.shape == (5, 10)
    assert s.dtype == np.float32 and i.dtype == np.int64
    assert np.all(np.diff(s, axis=1) <= 0)


def test_self_query_recall_at_1(api):
    v = unit_vectors(200, dim=512, seed=4)
    idx = api.TurboQuantIndex(512, 4)
    idx.add(v)
    _, i = idx.search(v, 1)
    assert (i[:, 0] == np.arange(200)).mean() >= 0.99      # turbovec/src/kernel_tests.rs:439-459


def test_batch_query_matches_individual(api):
    idx = api.TurboQuantIndex(DIM, 4)
    idx.add(unit_vectors(300, seed=5))
    q = unit_vectors(9, seed=6)
    s, i = idx.search(q, 7)
    for r in range(len(q)):
        s1, i1 = idx.search(q[r:r + 1], 7)
        assert bits_equal(s1[0], s[r]) and np.array_equal(i1[0], i[r])


def test_search_on_empty_index_and_k_clamp(api):
    idx = api.TurboQuantIndex(DIM, 4)
    s, i = idx.search(unit_vectors(2), 5)
    assert s.shape == (2, 0) and i.shape == (2, 0)
    idx.add(unit_vectors(7, seed=7))
    s, i = idx.search(unit_vectors(2), 50)
    assert s.shape == (2, 7)
    s, i = idx.search(unit_vectors(2), 1 << 40)
    assert s.shape == (2, 7)
    s, i = idx.search(np.zeros((0, DIM), np.float32), 3)
    assert s.shape == (0, 3)
    s, i = idx.search(unit_vectors(2), 0)
    assert s.shape == (2, 0)


def test_swap_remove(api, oracle):
    v = unit_vectors(50, seed=8)
    idx = api.TurboQuantIndex(DIM, 4)
    idx.add(v)
    assert idx.swap_remove(10) == 49 and len(idx) == 49
    assert idx.swap_remove(48) == 48 and len(idx) == 48       # removing the last: no swap
    order = list(range(50))
    order[10] = 49
    order = order[:48]
    ref = OracleIndex(oracle, DIM, 4, v[order])
    q = unit_vectors(4, seed=9)
    s, i = idx.search(q, 48)
    os_, oi = ref.search(q, 48)
    assert np.array_equal(i, oi) and bits_equal(s, os_)
    for bad in (-1, 48, 1 << 70):
        with pytest.raises(IndexError):
            idx.swap_remove(bad)


def test_argument_errors(api):
    idx = api.TurboQuantIndex(DIM, 4)
    idx.add(unit_vectors(20))
    with pytest.raises(TypeError, match="vectors must be a 2-D float32 array, got 2-D float64"):
        idx.add(unit_vectors(3).astype(np.float64))
    with pytest.raises(TypeError, match="got list"):
        idx.add([[0.0] * DIM])
    with pytest.raises(TypeError, match="queries must be a 2-D float32 array, got 1-D float32"):
        idx.search(unit_vectors(1)[0], 3)
    with pytest.raises(ValueError, match="C-contiguous"):
        idx.search(unit_vectors(4, dim=2 * DIM)[:, ::2], 3)
    with pytest.raises(ValueError, match="C-contiguous"):
        idx.add(unit_vectors(4, dim=2 * DIM)[:, ::2])
    with pytest.raises(ValueError, match="query dim 64 does not match index dim 128"):
        idx.search(unit_vectors(2, dim=64), 3)
    with pytest.raises(ValueError, match="does not match index dim"):
        idx.add(unit_vectors(2, dim=64))
    with pytest.raises(ValueError, match="non-negative"):
        idx.search(unit_vectors(1), -1)
    with pytest.raises(TypeError):
        idx.search(unit_vectors(1), 2.5)
    q = unit_vectors(2)
    q[1, 3] = np.nan
    with pytest.raises(ValueError):
        idx.search(q, 3)
    q[1, 3] = np.inf
    with pytest.raises(ValueError):
        idx.search(q, 3)
    bad = unit_vectors(2)
    bad[0, 0] = 1e17
    with pytest.raises(ValueError):
        idx.add(bad)
    assert len(idx) == 20
    with pytest.raises(TypeError):
        idx.search(unit_vectors(1), 3, np.ones(20, bool))        # mask is keyword-only


# ---- mask= ---------------------------------------------------------------
def test_mask_semantics(api):
    n = 200
    idx = api.TurboQuantIndex(DIM, 4)
    idx.add(unit_vectors(n, seed=10))
    q = unit_vectors(4, seed=11)
    s0, i0 = idx.search(q, 10)
    s1, i1 = idx.search(q, 10, mask=None)
    s2, i2 = idx.search(q, 10, mask=np.ones(n, bool))
    assert bits_equal(s0, s1) and bits_equal(s0, s2) and np.array_equal(i0, i1) and np.array_equal(i0, i2)
    allowed = [3, 7, 19, 42, 88, 121, 150, 175, 198]
    m = np.zeros(n, bool)
    m[allowed] = True
    s, i = idx.search(q, 5, mask=m)
    assert s.shape == (4, 5) and set(i.ravel()) <= set(allowed)
    s, i = idx.search(q, 20, mask=m)
    assert s.shape == (4, 9)                                   # effective k = popcount(mask)
    s, i = idx.search(q, 10, mask=np.zeros(n, bool))
    assert s.shape == (4, 0)
    # masked top-k == full ranking filtered afterwards, bitwise (turbovec/tests/filtering.rs:63-114)
    sf, if_ = idx.search(q, n)
    rng = np.random.default_rng(12)
    m = rng.random(n) < 0.3
    s, i = idx.search(q, 10, mask=m)
    for r in range(4):
        keep = m[if_[r]]
        assert np.array_equal(i[r], if_[r][keep][:10]) and bits_equal(s[r], sf[r][keep][:10])
    with pytest.raises(ValueError, match="mask length 199 does not match index size 200"):
        idx.search(q, 5, mask=np.ones(n - 1, bool))
    with pytest.raises(TypeError, match="mask must be a 1-D bool array"):
        idx.search(q, 5, mask=np.ones(n, np.int64))
    with pytest.raises(ValueError, match="C-contiguous"):
        idx.search(q, 5, mask=np.ones(2 * n, bool)[::2])
    # any non-zero byte is true
    raw = np.zeros(n, np.uint8)
    raw[allowed] = [2, 255, 1, 128, 3, 7, 64, 200, 9]
    s, i = idx.search(q, 20, mask=raw.view(bool))
    assert s.shape == (4, 9) and set(i.ravel()) == set(allowed)


# ---- IdMapIndex ------------------------------------------------------------
def test_id_map_add_search_remove(api):
    idx = api.IdMapIndex(DIM, 4)
    v = unit_vectors(100, seed=13)
    ids = (np.arange(100, dtype=np.uint64) * 1000 + 17)
    idx.add_with_ids(v, ids)
    assert len(idx) == 100 and idx.contains(17) and 99017 in idx and not idx.contains(5)
    assert not idx.contains(-3) and not idx.contains(1 << 70)
    s, got = idx.search(v[:10], 1)
    assert got.dtype == np.uint64 and (got[:, 0] == ids[:10]).mean() >= 0.9
    assert idx.remove(17) is True and idx.remove(17) is False and idx.remove(1 << 80) is False
    assert len(idx) == 99 and not idx.contains(17)
    idx.add_with_ids(v[:1], np.array([17], np.uint64))           # re-add the same id
    assert idx.contains(17) and len(idx) == 100
    # every remaining id still finds itself after a run of removes
    for x in ids[10:40]:
        assert idx.remove(int(x))
    alive = np.array([x for x in ids if idx.contains(int(x))], np.uint64)
    rows = np.array([np.where(ids == x)[0][0] for x in alive])
    _, got = idx.search(v[rows], 1)
    assert (got[:, 0] == alive).mean() >= 0.9
    with pytest.raises(ValueError, match="already present"):
        idx.add_with_ids(v[:1], np.array([alive[0]], np.uint64))
    with pytest.raises(ValueError, match="more than once"):
        idx.add_with_ids(v[:2], np.array([5, 5], np.uint64))
    with pytest.raises(TypeError, match="ids must be a 1-D uint64 array"):
        idx.add_with_ids(v[:2], np.array([5, 6], np.int64))
    with pytest.raises(ValueError, match="ids count mismatch"):
        idx.add_with_ids(v[:2], np.array([5], np.uint64))


def test_allowlist_semantics(api):
    n = 400
    idx = api.IdMapIndex(DIM, 4)
    v = unit_vectors(n, seed=14)
    rng = np.random.default_rng(15)
    ids = rng.permutation(1 << 20)[:n].astype(np.uint64) + np.uint64(1 << 40)
    idx.add_with_ids(v, ids)
    q = unit_vectors(5, seed=16)
    s0, g0 = idx.search(q, 10)
    s1, g1 = idx.search(q, 10, allowlist=None)
    assert bits_equal(s0, s1) and np.array_equal(g0, g1)
    allow = ids[[1, 5, 9, 100, 399, 7, 8, 250]]
    s, g = idx.search(q, 5, allowlist=allow)
    assert s.shape == (5, 5) and set(g.ravel()) <= set(allow.tolist())
    # allowlist smaller than k: rows of exactly n_allowed, no padding; duplicates collapse
    small = ids[:16]
    s, g = idx.search(q, 100, allowlist=np.concatenate([small, small[:4]]))
    assert s.shape == (5, 16) and g.shape == (5, 16)
    for r in range(5):
        assert set(g[r].tolist()) == set(small.tolist())
    s, g = idx.search(q, 10, allowlist=small)
    assert s.shape == (5, 10)
    s, g = idx.search(np.zeros((0, DIM), np.float32), 100, allowlist=np.array([ids[0]] * 3, np.uint64))
    assert s.shape == (0, 1)
    # allowlisted top-k == the full ranking restricted to the allowlist
    sf, gf = idx.search(q, n)
    aset = set(allow.tolist())
    s, g = idx.search(q, 8, allowlist=allow)
    for r in range(5):
        keep = np.array([x in aset for x in gf[r].tolist()])
        assert np.array_equal(g[r], gf[r][keep][:8]) and bits_equal(s[r], sf[r][keep][:8])
    with pytest.raises(ValueError, match="allowlist is empty"):
        idx.search(q, 5, allowlist=np.zeros(0, np.uint64))
    with pytest.raises(KeyError, match="not present in index"):
        idx.search(q, 5, allowlist=np.array([ids[0], 12345], np.uint64))
    with pytest.raises(TypeError, match="allowlist must be a 1-D uint64 array"):
        idx.search(q, 5, allowlist=np.array([1, 2], np.int64))
    with pytest.raises(TypeError):
        idx.search(q, 5, allow)                                   # keyword-only
    # a mutation moves slots: the allowlist follows ids, not slots
    assert idx.remove(int(ids[1]))
    s, g = idx.search(q, 100, allowlist=ids[[5, 9, 399]])
    assert s.shape == (5, 3) and set(g[0].tolist()) == set(ids[[5, 9, 399]].tolist())


def test_calibrate_before_add(api):
    v = unit_vectors(600, dim=256, seed=21) * np.linspace(0.2, 3.0, 256, dtype=np.float32)   # anisotropic
    v /= np.linalg.norm(v, axis=1, keepdims=True)
    idx = api.TurboQuantIndex(256, 4)
    assert idx.calibration_state == "uncalibrated"
    idx.calibrate(v)
    assert idx.calibration_state == "calibrated"
    idx.add(v)
    _, i = idx.search(v[:100], 1)
    assert (i[:, 0] == np.arange(100)).mean() >= 0.99
    again = api.TurboQuantIndex.from_bytes(idx.to_bytes())
    assert again.calibration_state == "calibrated" and again.to_bytes() == idx.to_bytes()
    with pytest.raises(NotImplementedError):
        idx.calibrate(v)
    with pytest.raises(ValueError):
        api.TurboQuantIndex(256, 4).calibrate(v[:1])
    with pytest.raises(TypeError):
        api.TurboQuantIndex(256, 4).calibrate(v.astype(np.float64))


# test_pickle_copy.py in the reference's Python suite: pickle / copy / deepcopy go through
# from_bytes(to_bytes()) and yield an independent index with the same answers
def test_pickle_and_copy_round_trip(api):
    import copy
    import pickle
    TurboQuantIndex, IdMapIndex = api.TurboQuantIndex, api.IdMapIndex
    rng = np.random.default_rng(21)
    v = rng.standard_normal((300, 64)).astype(np.float32)
    q = rng.standard_normal((3, 64)).astype(np.float32)
    idx = TurboQuantIndex(dim=64, bit_width=4)
    idx.add(v)
    want = idx.search(q, 5)
    for clone in (pickle.loads(pickle.dumps(idx)), copy.copy(idx), copy.deepcopy(idx)):
        assert len(clone) == 300 and clone.to_bytes() == idx.to_bytes()
        got = clone.search(q, 5)
        assert np.array_equal(got[1], want[1]) and np.array_equal(got[0], want[0])
    clone = copy.deepcopy(idx)
    clone.swap_remove(0)
    assert len(idx) == 300 and len(clone) == 299          # independent of the original
    im = IdMapIndex(dim=64, bit_width=2)
    ids = np.arange(1000, 1300, dtype=np.uint64)
    im.add_with_ids(v, ids)
    want = im.search(q, 5)
    clone = pickle.loads(pickle.dumps(im))
    got = clone.search(q, 5)
    assert np.array_equal(got[1], want[1]) and np.array_equal(got[0], want[0])
    assert clone.contains(1005) and not clone.contains(5)
