"""Parity of the HIP search path (through the C ABI) against the CPU oracle and
the reference's golden fixture.  Bar: integer accumulators, returned slots and
float scores all bit-exact (the float arithmetic is reproduced operation by
operation, so the 1e-5 relative tolerance the task allows is not needed)."""
import json
import os
import threading

import numpy as np
import pytest

from golden_data import parity_fixture_inputs
from helpers import OracleIndex, bits_equal, to_native, unit_gaussian

pytestmark = pytest.mark.gpu
HERE = os.path.dirname(os.path.abspath(__file__))


@pytest.fixture(scope="module")
def T():
    from turbovec_amd import _lib
    _lib.lib()
    return _lib


def omode(O, name):
    return getattr(O, "MODE_" + name)


def tmode(T, name):
    return getattr(T, "SCORE_" + name)


CASES = [
    # dim, bits, n, nq, k, mode
    (128, 4, 1000, 5, 10, "P"),
    (128, 4, 10007, 40, 10, "P"),          # ragged tail block, two query tiles
    (1536, 4, 5000, 33, 10, "P"),
    (3072, 4, 2100, 9, 10, "P"),
    (768, 4, 4099, 3, 1, "P"),
    (200, 4, 3000, 4, 7, "P"),             # byte groups not a multiple of 32 (padded chunk)
    (128, 4, 3000, 7, 10, "L_CLASSIC"),
    (1536, 4, 3000, 5, 10, "L_CLASSIC"),   # three 256-group flush batches
    (128, 4, 3000, 7, 10, "L_U32"),
    (128, 2, 3000, 7, 10, "L_U32"),
    (1536, 2, 3000, 9, 10, "L_U32"),
    (1536, 2, 3000, 2, 10, "L_CLASSIC"),
    (64, 3, 1500, 3, 10, "L_U32"),
    (1000, 2, 2000, 3, 5, "L_U32"),        # B = 8 rotation blocks
    (128, 4, 3000, 7, 10, "L_SCALAR"),     # the definition: every LUT term added in f32, one by one
    (1536, 2, 3000, 3, 10, "L_SCALAR"),
    (200, 4, 3000, 4, 7, "L_SCALAR"),      # padded last chunk: the chain stops at the last real group
    (64, 3, 1500, 3, 100, "L_SCALAR"),     # k beyond the per-lane lists
    (128, 4, 3000, 3, 100, "P"),           # k beyond the per-lane lists: radix select
    (64, 3, 500, 3, 500, "L_U32"),         # k = n: full ranking
    (128, 2, 5000, 2, 1000, "L_U32"),
]


@pytest.mark.parametrize("dim,bits,n,nq,k,mode", CASES, ids=lambda v: str(v))
def test_search_bit_exact(T, oracle, dim, bits, n, nq, k, mode):
    O = oracle
    oidx = OracleIndex(O, dim, bits, unit_gaussian(n, dim, seed=dim + bits + n))
    q = unit_gaussian(nq, dim, seed=1)
    ix = to_native(T, oidx, tmode(T, mode))
    # query preparation: rotated rows, and per-query scale / bias of the active tables
    qrot, qs, qb = ix.debug_prepare(q)
    want_rot = np.stack([oidx.rot.apply(x) for x in q])
    assert bits_equal(qrot, want_rot)
    _, cen = O.codebook(bits, dim)
    for qi in range(nq):
        if mode == "P":
            _, _, _, sc = O.build_permute_dot(want_rot[qi], cen, dim)
            assert qs[qi] == sc and qb[qi] == 0
        else:
            _, sc, bi = O.build_lut(want_rot[qi], cen, bits, dim)
            assert qs[qi] == sc and qb[qi] == bi
    # integer accumulators and float scores of every (query, slot)
    os_, oi, oacc, oraw = oidx.search(q, k, mode=omode(O, mode), dump=True)
    acc, raw = ix.debug_scan(q)
    assert np.array_equal(acc, oacc)
    assert bits_equal(raw, oraw)
    # the search proper
    s, i = ix.search(q, k)
    assert np.array_equal(i, oi)
    assert bits_equal(s, os_)
    ix.close()


def test_auto_mode_is_what_a_vnni_host_runs(T, oracle):
    O = oracle
    for bits, want in ((4, "P"), (2, "L_U32"), (3, "L_U32")):
        oidx = OracleIndex(O, 128, bits, unit_gaussian(700, 128, seed=bits))
        q = unit_gaussian(3, 128, seed=2)
        ix = to_native(T, oidx)
        s, i = ix.search(q, 10)
        os_, oi = oidx.search(q, 10, mode=omode(O, want))
        assert np.array_equal(i, oi) and bits_equal(s, os_)
        ix.close()


# ---- the reference's own end-to-end fixture ----
@pytest.fixture(scope="module")
def fixture_state(oracle):
    base, warm, singles, queries = parity_fixture_inputs()
    gold = json.load(open(os.path.join(HERE, "golden", "parity_base.json")))
    return base, warm, singles, queries, gold


def test_reference_fixture_ids_and_scores(T, oracle, fixture_state):
    """benchmarks/hillclimb/data/parity_base_x86.json: IdMapIndex 21 050 x 768
    4-bit, 20 queries, k=10, built by bulk add + batch append + 50 single
    appends; the classic u8-LUT path reproduces all 200 floats bit for bit."""
    O = oracle
    base, warm, singles, queries, gold = fixture_state
    o_base = OracleIndex(O, 768, 4, base)
    ix = to_native(T, o_base, T.SCORE_L_CLASSIC)
    o_warm = OracleIndex(O, 768, 4, warm)
    ix.append_rows(o_warm.rows(), o_warm.scales)             # add(batch)
    o_single = OracleIndex(O, 768, 4, singles)
    rows = o_single.rows()
    for r in range(len(singles)):                            # add(one row) x 50
        ix.append_rows(rows[r:r + 1], o_single.scales[r:r + 1])
    assert len(ix) == gold["len_after_singles"]
    s, i = ix.search(queries, 10)
    assert np.array_equal(i, np.array(gold["search_ids"]))
    assert bits_equal(s, np.array(gold["search_scores"], np.float32))
    # appended index == one-shot upload of the same rows (encode is batch independent)
    o_all = OracleIndex(O, 768, 4, np.concatenate([base, warm, singles]))
    seq, sc = ix.download_seq()
    assert np.array_equal(seq, o_all.seq) and np.array_equal(sc, o_all.scales)

    # 500 removes by id, mirrored as swap-and-pop (id_map.rs:520-567)
    n = len(ix)
    ids = list(range(n))
    slot_of = {x: x for x in ids}
    for rid in range(500):
        slot = slot_of.pop(rid)
        last = n - 1
        ix.swap_remove(slot)
        if slot != last:
            ids[slot] = ids[last]
            slot_of[ids[slot]] = slot
        ids.pop()
        n -= 1
    assert len(ix) == gold["len_after_idremove"]
    s, i = ix.search(queries, 10)
    assert np.array_equal(np.array(ids)[i], np.array(gold["post_remove_ids"]))
    assert bits_equal(s, np.array(gold["post_remove_scores"], np.float32))
    ix.close()


def test_reference_fixture_swap_remove_zero(T, oracle, fixture_state):
    O = oracle
    base, _, _, queries, gold = fixture_state
    oidx = OracleIndex(O, 768, 4, base)
    ix = to_native(T, oidx, T.SCORE_L_CLASSIC)
    for _ in range(500):
        ix.swap_remove(0)
    assert len(ix) == gold["tq_len"]
    s, i = ix.search(queries, 10)
    assert np.array_equal(i, np.array(gold["tq_ids"]))
    assert bits_equal(s, np.array(gold["tq_scores"], np.float32))
    # vacated lanes are zero: the device copy equals the oracle's after the same removals
    seq, sc = ix.download_seq()
    oseq, osc, n = oidx.seq.copy(), oidx.scales.copy(), oidx.n
    for _ in range(500):
        n = O.swap_remove_seq(oseq, osc, n, 4, 768, 0)
    assert np.array_equal(seq, oseq[: len(seq)]) and np.array_equal(sc, osc[:n])
    ix.close()


# ---- benchmark config 1: 100k x 128 4-bit, 1000 queries, k=10, full check ----
def test_config1_full(T, oracle):
    O = oracle
    oidx = OracleIndex(O, 128, 4, unit_gaussian(100_000, 128, seed=0))
    q = unit_gaussian(1000, 128, seed=1)
    ix = to_native(T, oidx)
    s, i = ix.search(q, 10)
    os_, oi = oidx.search(q, 10)
    assert np.array_equal(i, oi)
    assert bits_equal(s, os_)
    ix.close()


# ---- filtering: turbovec/tests/filtering.rs ----
@pytest.mark.parametrize("bits,mode", [(4, "P"), (2, "L_U32"), (4, "L_CLASSIC"), (2, "L_SCALAR")])
def test_mask_semantics(T, oracle, bits, mode):
    O = oracle
    dim, n, nq = 128, 4000, 6
    oidx = OracleIndex(O, dim, bits, unit_gaussian(n, dim, seed=7))
    q = unit_gaussian(nq, dim, seed=8)
    ix = to_native(T, oidx, tmode(T, mode))
    full_s, full_i = ix.search(q, n)                          # k = n ranking
    ofs, ofi = oidx.search(q, n, mode=omode(O, mode))
    assert np.array_equal(full_i, ofi) and bits_equal(full_s, ofs)
    rng = np.random.default_rng(3)
    masks = {
        "random 10%": rng.random(n) < 0.1,
        "1% (most blocks skipped)": rng.random(n) < 0.01,
        "contiguous 5%": np.arange(n) // 200 == 7,
        "all true": np.ones(n, bool),
        "three slots": np.isin(np.arange(n), [3, 777, 3999]),
        "last slot only": np.arange(n) == n - 1,
    }
    for name, m in masks.items():
        words, allowed = T.pack_mask(m)
        for k in (1, 10, 50):
            s, i = ix.search(q, k, mask_words=words)
            k_eff = min(k, allowed)
            assert s.shape == (nq, k_eff), name
            for qi in range(nq):                              # == unmasked ranking filtered post hoc
                keep = [j for j in range(n) if m[full_i[qi, j]]][:k_eff]
                assert i[qi].tolist() == full_i[qi, keep].tolist(), (name, k)
                assert bits_equal(s[qi], full_s[qi, keep]), (name, k)
            os_, oi = oidx.search(q, k, mask_words=words, mode=omode(O, mode))
            assert np.array_equal(i, oi) and bits_equal(s, os_)
    words, allowed = T.pack_mask(np.zeros(n, bool))           # all-false -> empty, filtering.rs:154
    s, i = ix.search(q, 10, mask_words=words)
    assert s.shape == (nq, 0) and i.shape == (nq, 0)
    with pytest.raises(T.TurbovecHipError) as e:              # lib.rs:1427-1434
        ix.search(q, 10, mask_words=np.zeros(3, np.uint64))
    assert e.value.status == T.ERR_MASK_LENGTH_MISMATCH
    # bits at or past n are ignored (search.rs:2996-2998)
    words, _ = T.pack_mask(masks["three slots"])
    words = words.copy()
    words[-1] |= np.uint64(1) << np.uint64(63)
    s, i = ix.search(q, 10, mask_words=words)
    assert s.shape == (nq, 3)
    ix.close()


# ---- shapes at the edges (lib.rs:1355-1402, search.rs:3226-3229, kernel_correctness.rs:184-240) ----
def test_degenerate_shapes(T, oracle):
    O = oracle
    dim = 64
    ix = T.NativeIndex(dim, 4)
    q = unit_gaussian(3, dim, seed=1)
    s, i = ix.search(q, 5)                                    # empty index -> k_eff 0
    assert s.shape == (3, 0)
    oidx = OracleIndex(O, dim, 4, unit_gaussian(45, dim, seed=2))
    ix.upload_seq(oidx.seq, oidx.n, oidx.scales)
    s, i = ix.search(np.zeros((0, dim), np.float32), 5)       # nq = 0
    assert s.shape == (0, 5)
    s, i = ix.search(q, 0)                                    # k = 0
    assert s.shape == (3, 0)
    s, i = ix.search(q, 1000)                                 # k > n clamps to n
    os_, oi = oidx.search(q, 1000)
    assert s.shape == (3, 45) and np.array_equal(i, oi) and bits_equal(s, os_)
    for n in (1, 31, 32, 33, 64, 65):                         # tail sizes around the block width
        o2 = OracleIndex(O, dim, 4, unit_gaussian(n, dim, seed=n))
        ix.upload_seq(o2.seq, o2.n, o2.scales)
        s, i = ix.search(q, 10)
        os_, oi = o2.search(q, 10)
        assert np.array_equal(i, oi) and bits_equal(s, os_), n
    ix.close()
    with pytest.raises(T.TurbovecHipError):
        T.NativeIndex(12, 4)                                  # dim not a multiple of 8
    with pytest.raises(T.TurbovecHipError):
        T.NativeIndex(64, 5)


def test_ties_and_zero_scale_rows(T, oracle):
    """Duplicate rows tie bitwise and must come back lowest slot first; zero
    rows get scale 0 (encode.rs:446) and score +-0.0, which tie with each other."""
    O = oracle
    dim = 128
    uniq = unit_gaussian(60, dim, seed=5)
    v = np.concatenate([uniq, np.zeros((7, dim), np.float32), uniq, uniq[:11], np.zeros((3, dim), np.float32)])
    for bits, mode in ((4, "P"), (4, "L_CLASSIC"), (2, "L_U32")):
        oidx = OracleIndex(O, dim, bits, v)
        assert (oidx.scales == 0).sum() == 10
        ix = to_native(T, oidx, tmode(T, mode))
        q = unit_gaussian(5, dim, seed=6)
        for k in (5, 20, 64, len(v)):
            s, i = ix.search(q, k)
            os_, oi = oidx.search(q, k, mode=omode(O, mode))
            assert np.array_equal(i, oi), (bits, mode, k)
            assert bits_equal(s, os_), (bits, mode, k)
        ix.close()


def test_tqplus_calibration(T, oracle):
    O = oracle
    dim, bits = 256, 4
    v = O.lcg_vectors(2500, dim, 0xBADC0DE)
    rot = O.Rotation(dim)
    _, cen = O.codebook(bits, dim)
    cal = O.fit_calibration(rot, v, cen)
    oidx = OracleIndex(O, dim, bits, v, calibration=cal)
    q = O.lcg_vectors(6, dim, 77)
    for mode in ("P", "L_CLASSIC", "L_SCALAR"):
        ix = to_native(T, oidx, tmode(T, mode))
        s, i = ix.search(q, 10)
        os_, oi = oidx.search(q, 10, mode=omode(O, mode))
        assert np.array_equal(i, oi) and bits_equal(s, os_)
        _, qs, qb = ix.debug_prepare(q)
        assert np.all(qb != 0)                                # the f64 bias correction landed
        ix.close()


# ---- batch_matches_single.rs:57-84, kernel_correctness.rs:243-347 ----
def test_batch_equals_single_and_is_deterministic(T, oracle):
    O = oracle
    dim = 128
    oidx = OracleIndex(O, dim, 4, unit_gaussian(6000, dim, seed=9))
    ix = to_native(T, oidx)
    for nq in (1, 7, 8, 9, 23, 50, 70):
        q = unit_gaussian(nq, dim, seed=100 + nq)
        s, i = ix.search(q, 10)
        for qi in range(nq):
            s1, i1 = ix.search(q[qi:qi + 1], 10)
            assert np.array_equal(i1[0], i[qi]) and bits_equal(s1[0], s[qi])
        s2, i2 = ix.search(q, 10)
        assert np.array_equal(i2, i) and bits_equal(s2, s)
    ix.close()


# query_scale_invariance.rs: ids invariant under power-of-two query scaling
def test_query_scale_invariance(T, oracle):
    dim = 128
    oidx = OracleIndex(oracle, dim, 4, unit_gaussian(3000, dim, seed=12))
    q = unit_gaussian(4, dim, seed=13)
    for mode in ("P", "L_U32"):
        ix = to_native(T, oidx, tmode(T, mode))
        _, base = ix.search(q, 10)
        for e in (-60, -20, 10, 40):
            _, i = ix.search(q * np.float32(2.0 ** e), 10)
            assert np.array_equal(i, base)
        ix.close()


# concurrent_search.rs / kernel_correctness.rs:315-347: 8 threads x 16 searches identical
def test_concurrent_searches(T, oracle):
    dim = 128
    oidx = OracleIndex(oracle, dim, 4, unit_gaussian(5000, dim, seed=14))
    ix = to_native(T, oidx)
    q = unit_gaussian(9, dim, seed=15)
    want_s, want_i = ix.search(q, 10)
    bad = []

    def worker():
        for _ in range(16):
            s, i = ix.search(q, 10)
            if not (np.array_equal(i, want_i) and bits_equal(s, want_s)):
                bad.append(1)

    threads = [threading.Thread(target=worker) for _ in range(8)]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    assert not bad
    ix.close()


def test_layout_round_trip_and_mutations(T, oracle):
    O = oracle
    for dim, bits in ((200, 2), (64, 3), (1536, 4)):
        n = 333
        oidx = OracleIndex(O, dim, bits, unit_gaussian(n, dim, seed=dim))
        ix = to_native(T, oidx)
        seq, sc = ix.download_seq()
        assert np.array_equal(seq, oidx.seq) and np.array_equal(sc, oidx.scales)
        # append in ragged pieces == one-shot
        ix2 = T.NativeIndex(dim, bits)
        rows = oidx.rows()
        for a, b in ((0, 1), (1, 40), (40, 41), (41, 300), (300, 333)):
            ix2.append_rows(rows[a:b], oidx.scales[a:b])
        seq2, sc2 = ix2.download_seq()
        assert np.array_equal(seq2, oidx.seq) and np.array_equal(sc2, oidx.scales)
        # removals in the middle, at the end, down to empty tail blocks
        oseq, osc, on = oidx.seq.copy(), oidx.scales.copy(), n
        rng = np.random.default_rng(1)
        for _ in range(120):
            idx = int(rng.integers(0, on))
            ix2.swap_remove(idx)
            on = O.swap_remove_seq(oseq, osc, on, bits, dim, idx)
        seq3, sc3 = ix2.download_seq()
        assert np.array_equal(seq3, oseq[: len(seq3)]) and np.array_equal(sc3, osc[:on])
        q = unit_gaussian(3, dim, seed=3)
        s, i = ix2.search(q, 10)
        os_, oi = O.search(oidx.rot, oseq[: len(seq3)], osc[:on], q, 10, bits, dim, on)
        assert np.array_equal(i, oi) and bits_equal(s, os_)
        with pytest.raises(T.TurbovecHipError) as e:
            ix2.swap_remove(on)
        assert e.value.status == T.ERR_INDEX_OUT_OF_RANGE
        ix.close()
        ix2.close()


def test_handed_over_tables_are_used(T, oracle):
    """tv_index_set_tables: the caller's own rotation and centroids replace the
    derived ones."""
    O = oracle
    dim = 64
    oidx = OracleIndex(O, dim, 4, unit_gaussian(500, dim, seed=1))
    ix = to_native(T, oidx)
    q = unit_gaussian(2, dim, seed=2)
    rot0, _, _ = ix.debug_prepare(q)
    signs, perms, cen, _ = ix.tables()
    flipped = signs.copy()
    flipped[0] = -flipped[0]                                  # negating round 0 negates the output
    ix.set_tables(signs=flipped)
    rot1, _, _ = ix.debug_prepare(q)
    assert bits_equal(rot1, -rot0)
    ix.set_tables(signs=signs, perms=perms, centroids=cen)
    rot2, _, _ = ix.debug_prepare(q)
    assert bits_equal(rot0, rot2)
    ix.close()


# ---- benchmark-sized inputs: size-independent properties ----
def test_random_codes_scale_properties(T):
    """1M x 1536 4-bit of uniform random code bytes and scales (configuration 2 itself, on encoded
    Gaussian rows, is in test_gpu_configs.py): the top-k the
    search returns equals an independent ranking of the dumped per-slot scores;
    batches of 1, 64 and 1024 agree row by row; top-10 is a prefix of top-32."""
    dim, bits, n = 1536, 4, 1_000_000
    G = dim // 2
    rng = np.random.default_rng(0)
    seq = rng.integers(0, 256, size=((n + 31) // 32) * G * 32, dtype=np.uint8)
    scales = (rng.random(n, dtype=np.float32) * np.float32(0.2) + np.float32(0.9))
    ix = T.NativeIndex(dim, bits)
    ix.upload_seq(seq, n, scales)
    q = unit_gaussian(1024, dim, seed=1)
    s, i = ix.search(q, 10)
    acc, raw = ix.debug_scan(q[:4])
    for qi in range(4):
        order = np.lexsort((np.arange(n), -raw[qi].astype(np.float64)))[:10]
        assert i[qi].tolist() == order.tolist()
        assert bits_equal(s[qi], raw[qi][order])
    s64, i64 = ix.search(q[:64], 10)
    assert np.array_equal(i64, i[:64]) and bits_equal(s64, s[:64])
    s1, i1 = ix.search(q[5:6], 10)
    assert np.array_equal(i1[0], i[5]) and bits_equal(s1[0], s[5])
    s32, i32 = ix.search(q[:40], 32)
    assert np.array_equal(i32[:, :10], i[:40]) and bits_equal(s32[:, :10], s[:40])
    assert np.all(np.diff(s32.astype(np.float64), axis=1) <= 0)   # sorted descending
    # 50% random slot mask (config 5's filter): every returned slot allowed, equals filtered ranking
    m = rng.random(n) < 0.5
    words, allowed = T.pack_mask(m)
    sm, im = ix.search(q[:4], 10, mask_words=words)
    assert m[im].all()
    for qi in range(4):
        order = np.lexsort((np.arange(n), -raw[qi].astype(np.float64)))
        order = order[m[order]][:10]
        assert im[qi].tolist() == order.tolist()
    ix.close()


# ---- sample-then-filter path (n above the candidate capacity) ----
@pytest.mark.parametrize("bits,mode", [(4, "P"), (2, "L_U32"), (4, "L_CLASSIC"), (4, "L_SCALAR")])
def test_sampled_path_matches_oracle_and_full_path(T, oracle, bits, mode):
    O = oracle
    dim, n, nq = 128, 40_003, 37
    oidx = OracleIndex(O, dim, bits, unit_gaussian(n, dim, seed=31))
    q = unit_gaussian(nq, dim, seed=32)
    ix = to_native(T, oidx, tmode(T, mode))
    rng = np.random.default_rng(5)
    masks = [None, rng.random(n) < 0.5, rng.random(n) < 0.01, (np.arange(n) > 30_000) & (np.arange(n) < 32_000)]
    for m in masks:
        words = None if m is None else T.pack_mask(m)[0]
        for k in (1, 10, 32, 33, 100, 128, 200, 256, 257, 1000, 1500):   # (64, 128, 256 leading keys kept by the selection's merge tree; full sort beyond)
            s, i = ix.search(q, k, mask_words=words)
            os_, oi = oidx.search(q, k, mask_words=words, mode=omode(O, mode))
            assert np.array_equal(i, oi), (mode, k)
            assert bits_equal(s, os_), (mode, k)
            for path in (1, 2):                   # full-range lists; one tile per launch
                ix.set_path(path)
                s2, i2 = ix.search(q, k, mask_words=words)
                ix.set_path(0)
                assert np.array_equal(i2, i) and bits_equal(s2, s)
    assert ix.overflow_redos() == 0
    ix.close()


def test_candidate_overflow_is_redone_exactly(T, oracle):
    """An index ordered against the sampler: every block the sampling pass reads
    holds poor matches and all the others hold near-duplicates of the query, so
    the floor is low, the candidate buffer overflows, and the query is scanned
    once more from a raised floor, with the same exact answer."""
    O = oracle
    dim, bits, n = 64, 4, 64 * 32 * 24
    rng = np.random.default_rng(8)
    q = unit_gaussian(3, dim, seed=9)
    v = -np.tile(q[0], (n, 1)) + 0.3 * rng.standard_normal((n, dim)).astype(np.float32)   # poor matches
    block = np.arange(n) // 32
    good = block % 4 != 0                           # k=10 -> the sampler reads every 64th block (a multiple of 4)
    v[good] = np.tile(q[0], (int(good.sum()), 1)) + 0.3 * rng.standard_normal((int(good.sum()), dim)).astype(np.float32)
    oidx = OracleIndex(O, dim, bits, v.astype(np.float32))
    ix = to_native(T, oidx)
    s, i = ix.search(q, 10)
    os_, oi = oidx.search(q, 10)
    assert np.array_equal(i, oi) and bits_equal(s, os_)
    assert ix.overflow_redos() >= 1
    # the repeated pass samples other blocks (half a stride in) and starts from the raised floor:
    # it settles the query without the exact path
    assert ix.exact_redos() == 0
    ix.close()


def test_all_equal_scores(T, oracle):
    """Every row identical: all scores tie bitwise, far more ties than the
    candidate buffer holds; the lowest slots must come back."""
    O = oracle
    dim, bits, n = 64, 4, 50_000
    row = unit_gaussian(1, dim, seed=3)
    oidx = OracleIndex(O, dim, bits, np.tile(row, (n, 1)))
    ix = to_native(T, oidx)
    q = unit_gaussian(2, dim, seed=4)
    for k in (10, 100):
        s, i = ix.search(q, k)
        assert np.array_equal(i, np.tile(np.arange(k), (2, 1)))
        os_, oi = oidx.search(q, k)
        assert np.array_equal(i, oi) and bits_equal(s, os_)
    ix.close()


# ---- u8-LUT batches, u32 epilogue: sixteen queries per pass, tables streamed through LDS ----
# 1536 x 2-bit: 12 chunks (configuration 3's row); 200 x 2-bit: 2 chunks, the second mostly padding;
# 1000 x 2-bit: 8 chunks, rotation blocks of 8; 64 x 3-bit: one chunk (its pair is half padding);
# 1536 x 4-bit: 24 chunks.  Query counts leave last tiles of 16, 9 (the sixteen-query scan), 8 and 1
# (the whole-table scans).
@pytest.mark.parametrize("dim,bits,n,nq,mode", [
    (1536, 2, 20_011, 40, "L_U32"), (1536, 2, 9_001, 25, "L_U32"), (200, 2, 30_000, 33, "L_U32"),
    (1000, 2, 12_000, 16, "L_U32"), (64, 3, 40_003, 48, "L_U32"), (1536, 4, 9_001, 17, "L_U32"),
    (1120, 2, 17_000, 9, "L_U32"),            # 9 chunks: the last pair is half padding
    (1536, 4, 9_001, 17, "L_CLASSIC"),        # the classic epilogue: three flush batches of 256 groups
    (1536, 2, 20_011, 40, "L_CLASSIC"),       # 12 chunks: a flush after 8 and one at the end
    (1120, 2, 17_000, 9, "L_CLASSIC"), (200, 2, 30_000, 33, "L_CLASSIC")])
def test_lut_sixteen_query_scan_matches_oracle(T, oracle, dim, bits, n, nq, mode):
    O = oracle
    oidx = OracleIndex(O, dim, bits, unit_gaussian(n, dim, seed=51))
    q = unit_gaussian(nq, dim, seed=52)
    ix = to_native(T, oidx, tmode(T, mode))
    rng = np.random.default_rng(7)
    for m in (None, rng.random(n) < 0.5, rng.random(n) < 0.003, (np.arange(n) >= 5_000) & (np.arange(n) < 7_000)):
        words = None if m is None else T.pack_mask(m)[0]
        for k in (1, 10, 100):
            s, i = ix.search(q, k, mask_words=words)
            os_, oi = oidx.search(q, k, mask_words=words, mode=omode(O, mode))
            assert np.array_equal(i, oi), k
            assert bits_equal(s, os_), k
            assert ix.queries_per_launch() == min(nq, 16)
            ix.set_path(8)                        # at most 8 queries per pass, whole tables in LDS
            s2, i2 = ix.search(q, k, mask_words=words)
            ix.set_path(0)
            assert np.array_equal(i2, i) and bits_equal(s2, s)
            assert ix.queries_per_launch() <= 8
    assert ix.overflow_redos() == 0
    ix.close()


# ---- one u8-LUT query: byte-table scan, first sampling level without floors (best row per block) ----
@pytest.mark.parametrize("dim,bits,n,mode", [(1536, 2, 20_011, "L_U32"), (128, 2, 60_003, "L_U32"), (64, 3, 40_003, "L_U32"),
                                             (256, 4, 30_000, "L_CLASSIC"), (1536, 4, 9_001, "L_U32")])
def test_lut_single_query_matches_oracle(T, oracle, dim, bits, n, mode):
    O = oracle
    oidx = OracleIndex(O, dim, bits, unit_gaussian(n, dim, seed=61))
    ix = to_native(T, oidx, tmode(T, mode))
    rng = np.random.default_rng(9)
    for qi, m in enumerate((None, rng.random(n) < 0.5, rng.random(n) < 0.003, (np.arange(n) >= 5_000) & (np.arange(n) < 7_000))):
        q = unit_gaussian(1, dim, seed=70 + qi)
        words = None if m is None else T.pack_mask(m)[0]
        for k in (1, 10, 100, 128, 129):
            s, i = ix.search(q, k, mask_words=words)
            os_, oi = oidx.search(q, k, mask_words=words, mode=omode(O, mode))
            assert np.array_equal(i, oi), k
            assert bits_equal(s, os_), k
    strides, _ = ix.sampling_plan(1, 10)
    assert len(strides) == 2                      # one level without floors, then the full scan
    strides, _ = ix.sampling_plan(1, 129)         # beyond the floorless level's k: the row-level ladder
    assert len(strides) >= 2
    assert ix.overflow_redos() == 0
    ix.close()


# ---- batched permute-dot scan (more than 32 queries per launch) ----
# dims 256/512/1536: weights of several tiles resident in LDS (1536 with 97 queries: the wide
# kernel, one pass for all); 3072 and 2560: streamed in slices, by the instance for two, three
# or four tiles of queries (45, 70, 131 queries);
# 2624 (41 chunks, odd): no batched kernel applies, the single-tile scan serves the batch.
@pytest.mark.parametrize("dim,n,nq", [(256, 40_003, 200), (1536, 20_011, 97), (1536, 9_001, 70), (512, 70_000, 129),
                                      (3072, 12_345, 131), (2560, 9_001, 70), (3072, 7_001, 45), (2624, 5_003, 40)])
def test_batched_scan_matches_oracle(T, oracle, dim, n, nq):
    O = oracle
    oidx = OracleIndex(O, dim, 4, unit_gaussian(n, dim, seed=41))
    q = unit_gaussian(nq, dim, seed=42)
    ix = to_native(T, oidx)
    rng = np.random.default_rng(6)
    for m in (None, rng.random(n) < 0.5, rng.random(n) < 0.003, (np.arange(n) >= 9_000) & (np.arange(n) < 11_000)):
        words = None if m is None else T.pack_mask(m)[0]
        for k in (1, 10, 100):
            s, i = ix.search(q, k, mask_words=words)
            os_, oi = oidx.search(q, k, mask_words=words)
            assert np.array_equal(i, oi), k
            assert bits_equal(s, os_), k
            ix.set_path(2)
            s2, i2 = ix.search(q, k, mask_words=words)
            ix.set_path(0)
            assert np.array_equal(i2, i) and bits_equal(s2, s)
    ix.close()
