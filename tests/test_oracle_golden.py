"""Pins the CPU oracle against every known answer the reference holds for the search path."""
import json
import os

import numpy as np
import pytest

from golden_data import (CODEBOOK, FINGERPRINT, ROT_DIM8, ROT_DIM24, ROT_DIM64, ROT_DIM128,
                         fingerprint_seed, parity_fixture_inputs)

HERE = os.path.dirname(os.path.abspath(__file__))


def bits_of(a):
    return [int(x) for x in np.asarray(a, np.float32).view(np.uint32)]


# ---- rotation: turbovec/tests/rotation_determinism.rs:36-96 ----
def test_rotation_golden_bits(oracle):
    O = oracle
    assert bits_of(O.Rotation(8).apply(np.arange(8, dtype=np.float32) - 3.5)) == ROT_DIM8
    in24 = np.array([(i * 7 % 11) - 5.0 for i in range(24)], np.float32)
    assert bits_of(O.Rotation(24).apply(in24)) == ROT_DIM24
    in64 = np.array([(i * 13 % 29) - 14.0 for i in range(64)], np.float32)
    assert bits_of(O.Rotation(64).apply(in64)) == ROT_DIM64


# turbovec/src/rotation.rs:1198-1213
def test_rotation_golden_dim128(oracle):
    e0 = np.zeros(128, np.float32)
    e0[0] = 1.0
    out = bits_of(oracle.Rotation(128).apply(e0))
    fold = 0
    for b in out:
        fold = (((fold << 1) | (fold >> 31)) & 0xFFFFFFFF) ^ b
    assert (fold, out[0], out[1], out[2], out[3]) == ROT_DIM128


# turbovec/src/rotation.rs:1231 -- apply_scaled_into == apply of the pre-scaled row, bitwise
@pytest.mark.parametrize("dim", [8, 24, 64, 128, 200, 768, 1000, 1024, 1536, 3072])
def test_apply_scaled_equals_apply_of_scaled(oracle, dim):
    rng = np.random.default_rng(dim)
    v = rng.standard_normal(dim).astype(np.float32)
    inv = np.float32(0.37)
    a = oracle.Rotation(dim).apply(v * inv)
    b = oracle.Rotation(dim).apply_scaled(v, inv)
    assert bits_of(a) == bits_of(b)


# rotation.rs:1294: norm preserved to 1e-4; orthogonality: rotating e_i gives unit columns
@pytest.mark.parametrize("dim", [128, 1536, 3072])
def test_rotation_is_orthogonal(oracle, dim):
    rot = oracle.Rotation(dim)
    rng = np.random.default_rng(1)
    x = rng.standard_normal(dim).astype(np.float32)
    y = rng.standard_normal(dim).astype(np.float32)
    rx, ry = rot.apply(x), rot.apply(y)
    assert abs(np.linalg.norm(rx) - np.linalg.norm(x)) / np.linalg.norm(x) < 1e-4
    assert abs(float(rx @ ry) - float(x @ y)) < 1e-3 * np.linalg.norm(x) * np.linalg.norm(y)
    assert rot.block == (dim & -dim)
    for r in range(2):
        assert sorted(rot.perm(r).tolist()) == list(range(dim))
        assert set(np.abs(rot.signs(r)).tolist()) == {1.0}


# ---- codebook: turbovec/tests/codebook_determinism.rs:91-98 ----
@pytest.mark.parametrize("dim,bits,wb,wc", CODEBOOK)
def test_codebook_fnv(oracle, dim, bits, wb, wc):
    b, c = oracle.codebook(bits, dim)
    assert oracle.fnv1a(c) == wc
    assert oracle.fnv1a(b) == wb


# codebook.rs:184-210 invariants, incl. the (128,4) cell that has no hash golden
@pytest.mark.parametrize("dim,bits", [(128, 4), (128, 2), (1536, 4), (3072, 4), (1536, 2)])
def test_codebook_invariants(oracle, dim, bits):
    b, c = oracle.codebook(bits, dim)
    assert len(c) == 1 << bits and len(b) == (1 << bits) - 1
    assert np.all(np.diff(c) > 0) and np.all(np.diff(b) > 0)
    for i in range(len(b)):
        assert b[i] == np.float32((c[i] + c[i + 1]) * np.float32(0.5))
    # symmetric Beta => antisymmetric codebook up to solver noise
    assert np.allclose(c, -c[::-1], atol=1e-6)


# kernel_tests.rs:316-337: codebook MSE*dim at dim 1536 within 5% of 0.1175 / 0.009497 (2/4-bit)
@pytest.mark.parametrize("bits,want", [(2, 0.1175), (4, 0.009497)])
def test_codebook_mse_matches_paper(oracle, bits, want):
    dim = 1536
    b, c = oracle.codebook(bits, dim)
    # coordinate of a uniform unit vector ~ N(0, 1/dim) at this dim
    rng = np.random.default_rng(0)
    x = rng.standard_normal(400000) / np.sqrt(dim)
    codes = np.searchsorted(b.astype(np.float64), x, side="left")
    mse = np.mean((x - c[codes]) ** 2) * dim
    assert abs(mse - want) / want < 0.05


# ---- encode: turbovec/tests/encode_fingerprint.rs:83-92 (calibration, codes, scales) ----
@pytest.mark.parametrize("row", FINGERPRINT, ids=lambda r: f"{r[0]}x{r[1]}")
def test_encode_fingerprint(oracle, row):
    O = oracle
    dim, bits, wb, wc, wcal, wcodes, wscales, _wfile = row
    v = O.lcg_vectors(2000, dim, fingerprint_seed(dim, bits))
    rot = O.Rotation(dim)
    b, c = O.codebook(bits, dim)
    assert O.fnv1a(b) == wb and O.fnv1a(c) == wc
    sh, sc = O.fit_calibration(rot, v, c)
    assert O.fnv1a(np.concatenate([sh, sc])) == wcal
    packed, scales = O.encode(rot, v, bits, (sh, sc))
    assert O.fnv1a(packed) == wcodes
    assert O.fnv1a(scales) == wscales


# ---- layouts: turbovec/src/pack.rs:964-1008 byte placement, round trip ----
@pytest.mark.parametrize("bits", [2, 3, 4])
def test_seq_layout_byte_map(oracle, bits):
    O = oracle
    dim, n = 64, 70
    rng = np.random.default_rng(bits)
    codes = rng.integers(0, 1 << bits, size=(n, dim), dtype=np.uint8)
    # bit-plane pack by hand: plane p byte c bit (7-k) = bit p of code at dim 8c+k
    packed = np.zeros((n, bits * dim // 8), np.uint8)
    for p in range(bits):
        for cc in range(dim // 8):
            byte = np.zeros(n, np.uint8)
            for k in range(8):
                byte |= (((codes[:, 8 * cc + k] >> p) & 1) << (7 - k)).astype(np.uint8)
            packed[:, p * (dim // 8) + cc] = byte
    seq = O.repack_seq(packed, n, bits, dim)
    cpb = 8 // bits
    field = 4 if bits == 3 else bits
    G = dim // cpb
    assert G == O.n_byte_groups(bits, dim)
    assert len(seq) == ((n + 31) // 32) * G * 32
    want = np.zeros_like(seq)
    for v in range(n):
        for g in range(G):
            byte = 0
            for cidx in range(cpb):
                byte |= int(codes[v, g * cpb + cidx]) << ((cpb - 1 - cidx) * field)
            want[((v // 32) * G + g) * 32 + v % 32] = byte
    assert np.array_equal(seq, want)            # padding lanes stay zero
    assert np.array_equal(O.seq_to_packed(seq, n, bits, dim), packed)


# ---- Mode P builder: turbovec/src/search.rs:4596-4616 (slot placement, zero = -128*sum w) ----
def test_permute_dot_slot_map_and_zero(oracle):
    O = oracle
    dim = 64
    _, cen = O.codebook(4, dim)
    q = np.zeros(dim, np.float32)
    q[2 * 5] = 1.0      # even dim of group 5 -> high nibble weight of group 5
    q[2 * 6 + 1] = -0.5  # odd dim of group 6 -> low nibble weight
    levels, w, zero, scale = O.build_permute_dot(q, cen, dim)
    assert w[(5 // 4) * 8 + 4 + 5 % 4] == 127
    assert w[(6 // 4) * 8 + 6 % 4] == -64 or w[(6 // 4) * 8 + 6 % 4] == -63
    assert zero == -128 * int(w.astype(np.int32).sum())
    cs = np.float32(np.abs(cen).max()) / np.float32(127.0)
    want_levels = np.clip(np.sign(cen / cs) * np.floor(np.abs(cen / cs) + np.float32(0.5)), -127, 127)
    assert np.array_equal(levels, want_levels.astype(np.int8))
    assert levels[15] == 127 and levels[0] == -127
    assert scale == np.float32(cs * (np.float32(1.0) / np.float32(127.0)))


# ---- Mode L builder invariants: turbovec/src/kernel_tests.rs:823-883 ----
@pytest.mark.parametrize("bits,dim", [(4, 128), (2, 128), (3, 64), (4, 1536), (2, 1536)])
def test_lut_invariants(oracle, bits, dim):
    O = oracle
    _, cen = O.codebook(bits, dim)
    rng = np.random.default_rng(5)
    q = rng.standard_normal(dim).astype(np.float32)
    lut, scale, bias = O.build_lut(q, cen, bits, dim)
    assert lut.max() <= 127
    pair = lut.reshape(-1, 2, 16).astype(np.int32)
    assert (pair[:, 0].max(axis=1) + pair[:, 1].max(axis=1)).max() <= 255
    assert pair.min(axis=2).max() == 0          # every sub-table has its min subtracted
    assert lut.max() == 127                     # the widest sub-table spans the full range
    for e in (-20, 7, 30):                      # bytes invariant to power-of-two query scaling
        lut2, scale2, bias2 = O.build_lut(q * np.float32(2.0 ** e), cen, bits, dim)
        assert np.array_equal(lut, lut2)
        assert scale2 == np.float32(scale * np.float32(2.0 ** e))
    lut0, scale0, bias0 = O.build_lut(np.zeros(dim, np.float32), cen, bits, dim)
    assert not lut0.any() and np.isfinite(scale0) and bias0 == 0


# LUT values against an independent numpy evaluation (float64 check of the rounding target)
def test_lut_matches_numpy_model(oracle):
    O = oracle
    bits, dim = 2, 64
    _, cen = O.codebook(bits, dim)
    rng = np.random.default_rng(9)
    q = rng.standard_normal(dim).astype(np.float32)
    lut, scale, bias = O.build_lut(q, cen, bits, dim)
    G = dim // 4
    vals = np.zeros((G, 2, 16), np.float32)
    for g in range(G):
        for sub in range(2):
            for nv in range(16):
                d0 = 4 * g + 2 * sub
                vals[g, sub, nv] = np.float32(np.float32(0) + q[d0] * cen[nv >> 2]) + q[d0 + 1] * cen[nv & 3]
    mins = vals.min(axis=2)
    span = (vals.max(axis=2) - mins).max()
    assert scale == np.float32(span / np.float32(127))
    want = np.floor((vals - mins[:, :, None]) * (np.float32(1) / scale) + np.float32(0.5))
    assert np.array_equal(lut.reshape(G, 2, 16), np.clip(want, 0, 127).astype(np.uint8))
    b = np.float32(0)
    for g in range(G):
        b = np.float32(b + np.float32(mins[g, 0] + mins[g, 1]))
    assert bias == b


# ---- scan integers by brute force on tiny inputs (decode codes, sum tables) ----
@pytest.mark.parametrize("bits,mode_name", [(4, "P"), (4, "L_CLASSIC"), (2, "L_U32"), (3, "L_U32"), (4, "L_SCALAR")])
def test_scan_integers_brute_force(oracle, bits, mode_name):
    O = oracle
    mode = getattr(O, "MODE_" + mode_name)
    dim, n, nq = 64, 75, 3
    rng = np.random.default_rng(11)
    v = rng.standard_normal((n, dim)).astype(np.float32)
    q = rng.standard_normal((nq, dim)).astype(np.float32)
    rot = O.Rotation(dim)
    packed, scales = O.encode(rot, v, bits)
    seq = O.repack_seq(packed, n, bits, dim)
    _, cen = O.codebook(bits, dim)
    s, idx, acc, raw = O.search(rot, seq, scales, q, n, bits, dim, n, mode=mode, dump=True)
    cpb = 8 // bits
    G = dim // cpb
    bytes_ = np.zeros((n, G), np.int64)
    for vi in range(n):
        for g in range(G):
            bytes_[vi, g] = seq[((vi // 32) * G + g) * 32 + vi % 32]
    for qi in range(nq):
        qr = rot.apply(q[qi])
        if mode == O.MODE_P:
            levels, w, zero, scale = O.build_permute_dot(qr, cen, dim)
            # decode every dimension's code, dot with the per-dimension weight
            codes = np.zeros((n, dim), np.int64)
            codes[:, 0::2] = bytes_ >> 4
            codes[:, 1::2] = bytes_ & 15
            wd = np.zeros(dim, np.int64)
            for g in range(G):
                wd[2 * g + 1] = w[(g // 4) * 8 + g % 4]
                wd[2 * g] = w[(g // 4) * 8 + 4 + g % 4]
            want = (levels.astype(np.int64)[codes] * wd[None, :]).sum(axis=1)
            assert np.array_equal(acc[qi], want)
            # the biased-u8 formulation the x86 kernel uses nets out to the same integer
            want_biased = ((levels.astype(np.int64)[codes] + 128) * wd[None, :]).sum(axis=1) + zero
            assert np.array_equal(want, want_biased)
            sc = (np.float32(1) * acc[qi].astype(np.float32) * scale) * scales
        else:
            lut, scale, bias = O.build_lut(qr, cen, bits, dim)
            lut = lut.reshape(G, 32).astype(np.int64)
            want = np.zeros(n, np.int64)
            for g in range(G):
                want += lut[g, bytes_[:, g] >> 4] + lut[g, 16 + (bytes_[:, g] & 15)]
            assert np.array_equal(acc[qi], want)
            sc = (acc[qi].astype(np.float32) * scale + bias) * scales
        assert np.allclose(raw[qi], sc, rtol=2e-5, atol=2e-4)  # cancellation of acc*scale against bias
        # ranking = total order (score desc, slot asc) over the raw scores
        order = sorted(range(n), key=lambda j: (-float(raw[qi, j]), j))
        assert idx[qi].tolist() == order
        assert np.array_equal(s[qi], raw[qi][order])


# ---- end to end: benchmarks/hillclimb/data/parity_base_{x86,arm}.json ----
@pytest.fixture(scope="module")
def parity_state(oracle):
    O = oracle
    base, warm, singles, queries = parity_fixture_inputs()
    rot = O.Rotation(768)
    allv = np.concatenate([base, warm, singles])
    packed, scales = O.encode(rot, allv, 4)
    gold = json.load(open(os.path.join(HERE, "golden", "parity_base.json")))
    return rot, packed, scales, queries, gold


def _eq_bits(a, b):
    return np.array_equal(np.asarray(a, np.float32).view(np.uint32), np.asarray(b, np.float32).view(np.uint32))


def test_parity_fixture_search(oracle, parity_state):
    """The fixture's 200 scores are reproduced bit-for-bit by the classic u8-LUT
    path (search.rs:516-582), which therefore pins the LUT builder, the integer
    scan, the flush epilogue and the top-k order.  The int8 permute-dot path
    gives different floats (it post-dates the fixture)."""
    O = oracle
    rot, packed, scales, queries, gold = parity_state
    n = len(scales)
    assert n == gold["len_after_singles"]
    seq = O.repack_seq(packed, n, 4, 768)
    s, i = O.search(rot, seq, scales, queries, 10, 4, 768, n, mode=O.MODE_L_CLASSIC)
    assert np.array_equal(i, np.array(gold["search_ids"]))
    assert _eq_bits(s, gold["search_scores"])
    # the other epilogues of the same integer sums agree to float rounding and keep the ids
    for mode in (O.MODE_L_SCALAR, O.MODE_L_U32):
        s2, i2 = O.search(rot, seq, scales, queries, 10, 4, 768, n, mode=mode)
        assert np.array_equal(i2, i)
        assert np.allclose(s2, s, rtol=2e-5)
    sp, ip = O.search(rot, seq, scales, queries, 10, 4, 768, n, mode=O.MODE_P)
    assert not _eq_bits(sp, gold["search_scores"])
    # lib.rs:3395-3428 demands >= 75 % top-k overlap between the two 4-bit modes
    overlap = np.mean([len(set(a) & set(b)) / 10 for a, b in zip(ip.tolist(), i.tolist())])
    assert overlap >= 0.75


def test_parity_fixture_after_removes(oracle, parity_state):
    O = oracle
    rot, packed, scales, queries, gold = parity_state
    n = len(scales)
    seq = O.repack_seq(packed, n, 4, 768)
    sc = scales.copy()
    ids = list(range(n))
    slot_of = {x: x for x in ids}
    for rid in range(500):                       # id_map.rs:520-567 swap-and-pop mirror
        slot = slot_of.pop(rid)
        last = n - 1
        O.swap_remove_seq(seq, sc, n, 4, 768, slot)
        if slot != last:
            ids[slot] = ids[last]
            slot_of[ids[slot]] = slot
        ids.pop()
        n -= 1
    assert n == gold["len_after_idremove"]
    s, i = O.search(rot, seq, sc, queries, 10, 4, 768, n, mode=O.MODE_L_CLASSIC)
    assert np.array_equal(np.array(ids)[i], np.array(gold["post_remove_ids"]))
    assert _eq_bits(s, gold["post_remove_scores"])
    # vacated lanes are zero, i.e. the buffer equals a from-scratch repack (lib.rs:2978-3003)
    repacked = O.repack_seq(O.seq_to_packed(seq, n, 4, 768), n, 4, 768)
    assert np.array_equal(seq[: len(repacked)], repacked)
    assert not seq[len(repacked):].any()


def test_parity_fixture_tq_swap_remove(oracle, parity_state):
    O = oracle
    rot, packed, scales, queries, gold = parity_state
    n = 20000
    seq = O.repack_seq(packed[:n], n, 4, 768)
    sc = scales[:n].copy()
    for _ in range(500):
        n = O.swap_remove_seq(seq, sc, n, 4, 768, 0)
    assert n == gold["tq_len"]
    s, i = O.search(rot, seq, sc, queries, 10, 4, 768, n, mode=O.MODE_L_CLASSIC)
    assert np.array_equal(i, np.array(gold["tq_ids"]))
    assert _eq_bits(s, gold["tq_scores"])


# ---- top-k / mask semantics: turbovec/tests/filtering.rs ----
def test_topk_heap_equals_total_order_with_ties(oracle):
    """Duplicate rows give bitwise-tied scores; the k<=1024 heap path
    (search.rs:244-252) and the sort path must both return the lowest slots."""
    O = oracle
    dim, bits = 64, 4
    rng = np.random.default_rng(3)
    uniq = rng.standard_normal((40, dim)).astype(np.float32)
    v = np.concatenate([uniq, uniq, uniq[:13]])   # many exact duplicates
    n = len(v)
    rot = O.Rotation(dim)
    packed, scales = O.encode(rot, v, bits)
    seq = O.repack_seq(packed, n, bits, dim)
    q = rng.standard_normal((4, dim)).astype(np.float32)
    full_s, full_i, acc, raw = O.search(rot, seq, scales, q, n, bits, dim, n, dump=True)
    for qi in range(4):
        order = sorted(range(n), key=lambda j: (-float(raw[qi, j]), j))
        assert full_i[qi].tolist() == order
    for k in (1, 5, 17, 64):                     # prefix property, filtering.rs:684-706
        s, i = O.search(rot, seq, scales, q, k, bits, dim, n)
        assert np.array_equal(i, full_i[:, :k]) and _eq_bits(s, full_s[:, :k])


def test_mask_semantics(oracle):
    O = oracle
    dim, bits, n = 64, 2, 300
    rng = np.random.default_rng(4)
    v = rng.standard_normal((n, dim)).astype(np.float32)
    q = rng.standard_normal((5, dim)).astype(np.float32)
    rot = O.Rotation(dim)
    packed, scales = O.encode(rot, v, bits)
    seq = O.repack_seq(packed, n, bits, dim)
    full_s, full_i = O.search(rot, seq, scales, q, n, bits, dim, n)
    mask = rng.random(n) < 0.1
    mask[64:160] = False                          # whole blocks without an allowed slot
    words, allowed = O.pack_mask(mask)
    assert allowed == int(mask.sum())
    s, i = O.search(rot, seq, scales, q, 20, bits, dim, n, mask_words=words)
    k_eff = min(20, allowed)
    assert s.shape == (5, k_eff)
    for qi in range(5):                           # masked == unmasked ranking filtered post hoc
        keep = [j for j in range(n) if mask[full_i[qi, j]]][:k_eff]
        assert i[qi].tolist() == full_i[qi, keep].tolist()
        assert _eq_bits(s[qi], full_s[qi, keep])
    all_true, _ = O.pack_mask(np.ones(n, bool))   # all-true mask == no mask, filtering.rs:117
    s2, i2 = O.search(rot, seq, scales, q, 10, bits, dim, n, mask_words=all_true)
    assert np.array_equal(i2, full_i[:, :10])
    none, _ = O.pack_mask(np.zeros(n, bool))      # all-false mask -> empty, filtering.rs:154
    s3, i3 = O.search(rot, seq, scales, q, 10, bits, dim, n, mask_words=none)
    assert s3.shape == (5, 0)
    few = np.zeros(n, bool)
    few[[3, 77, 200]] = True                      # n_allowed < k clamps, filtering.rs:133
    w3, _ = O.pack_mask(few)
    s4, i4 = O.search(rot, seq, scales, q, 10, bits, dim, n, mask_words=w3)
    assert s4.shape == (5, 3) and set(i4[0].tolist()) == {3, 77, 200}


def test_query_validation(oracle):
    O = oracle
    q = np.ones(16, np.float32)
    assert O.validate_queries(q, 8) == (O.OK, 0)
    assert O.validate_queries(q[:15], 8)[0] == O.ERR_QUERY_BUFFER_NOT_MULTIPLE_OF_DIM
    for bad in (np.nan, np.inf, -np.inf, 1e16, -2e16):
        q2 = q.copy()
        q2[11] = bad
        assert O.validate_queries(q2, 8) == (O.ERR_INVALID_QUERY_VALUE, 11)
    q2 = q.copy()
    q2[3] = np.float32(9.99e15)
    assert O.validate_queries(q2, 8)[0] == O.OK


# The throughput-oriented twin the CPU baseline times must give the same answer.
@pytest.mark.parametrize("dim,bits,n", [(1536, 4, 3000), (1536, 2, 3000), (128, 4, 5003), (64, 3, 700)])
def test_search_fast_equals_search(oracle, dim, bits, n):
    O = oracle
    rng = np.random.default_rng(21)
    v = rng.standard_normal((n, dim)).astype(np.float32)
    q = rng.standard_normal((37, dim)).astype(np.float32)
    rot = O.Rotation(dim)
    packed, scales = O.encode(rot, v, bits)
    seq = O.repack_seq(packed, n, bits, dim)
    s, i = O.search(rot, seq, scales, q, 10, bits, dim, n)
    s2, i2 = O.search_fast(rot, seq, scales, q, 10, bits, dim, n, n_threads=4)
    assert np.array_equal(i, i2) and _eq_bits(s, s2)
    words, _ = O.pack_mask(rng.random(n) < 0.03)
    s, i = O.search(rot, seq, scales, q, 10, bits, dim, n, mask_words=words)
    s2, i2 = O.search_fast(rot, seq, scales, q, 10, bits, dim, n, mask_words=words, n_threads=3)
    assert np.array_equal(i, i2) and _eq_bits(s, s2)


# The reference's AVX-512 VNNI production kernel, restated (search.rs:1392-1567 over the vector-major
# layout, pack.rs:1269-1271): same slots and score bits as the scalar statement of mode P, ragged last
# block, masks, fewer than eight queries in the last group, ties.  Skipped on a host without VNNI.
@pytest.mark.parametrize("dim,n,nq", [(1536, 3003, 37), (128, 5003, 9), (768, 70, 3), (64, 32, 8)])
def test_search_vnni_equals_search(oracle, dim, n, nq):
    O = oracle
    if not O.have_vnni():
        pytest.skip("host has no AVX-512 VNNI")
    rng = np.random.default_rng(23)
    v = rng.standard_normal((n, dim)).astype(np.float32)
    v[n // 2] = v[n // 3]                                   # a duplicate row: equal scores, lower slot first
    q = rng.standard_normal((nq, dim)).astype(np.float32)
    rot = O.Rotation(dim)
    packed, scales = O.encode(rot, v, 4)
    seq = O.repack_seq(packed, n, 4, dim)
    vm = O.seq_to_vector_major(seq, n, 4, dim)
    # layout: byte of (block b, group g, lane l) sits at b*G*32 + (g/4)*128 + (l/16)*64 + (l%16)*4 + g%4
    G = dim // 2
    for (b, g, l) in [(0, 0, 0), (0, 5, 17), ((n - 1) // 32, G - 1, (n - 1) % 32), (1 % ((n + 31) // 32), 6, 31)]:
        assert vm[b * G * 32 + (g // 4) * 128 + (l // 16) * 64 + (l % 16) * 4 + g % 4] == seq[(b * G + g) * 32 + l]
    for k in (1, 10, 64):
        s, i = O.search(rot, seq, scales, q, k, 4, dim, n, mode=O.MODE_P)
        for threads in (1, 5):
            s2, i2 = O.search_vnni(rot, vm, scales, q, k, dim, n, n_threads=threads)
            assert np.array_equal(i, i2) and _eq_bits(s, s2)
    for frac in (0.5, 0.03):
        words, _ = O.pack_mask(rng.random(n) < frac)
        s, i = O.search(rot, seq, scales, q, 10, 4, dim, n, mask_words=words, mode=O.MODE_P)
        s2, i2 = O.search_vnni(rot, vm, scales, q, 10, dim, n, mask_words=words, n_threads=3)
        assert np.array_equal(i, i2) and _eq_bits(s, s2)
