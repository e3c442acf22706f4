"""Edges of what the C ABI accepts: the longest row (16384 dimensions, lib.rs:101), re-uploads
over a larger index, row scales far outside the encoder's range."""
import numpy as np
import pytest

from helpers import OracleIndex, bits_equal, to_native, unit_gaussian

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def T():
    from turbovec_amd import _lib
    _lib.lib()
    return _lib


@pytest.mark.parametrize("dim,bits", [(16384, 4), (16384, 2), (10248, 4), (8, 4), (16, 2)])
def test_add_and_search_at_the_dimension_limits(T, oracle, dim, bits):
    """Encode on the device and search at the largest dimension tv_index_create accepts (and just
    past the row length at which the ingest kernel's scratch used to outgrow a workgroup's LDS,
    and at the shortest rows): codes, scales and results equal the oracle's."""
    n, nq = 150, 5
    v = unit_gaussian(n, dim, seed=dim + bits)
    v *= np.linspace(0.5, 2.0, n, dtype=np.float32)[:, None]
    oidx = OracleIndex(oracle, dim, bits, v)
    ix = T.NativeIndex(dim, bits)
    ix.add(v)
    seq, scales = ix.download_seq()
    assert np.array_equal(seq, oidx.seq)
    assert bits_equal(scales, oidx.scales)
    q = unit_gaussian(nq, dim, seed=3)
    for k in (1, 10):
        s, i = ix.search(q, k)
        os_, oi = oidx.search(q, k)
        assert np.array_equal(i, oi) and bits_equal(s, os_)
    ix.close()


def test_calibrate_at_the_dimension_limit(T, oracle):
    dim, bits, n = 16384, 4, 64
    v = unit_gaussian(n, dim, seed=11)
    rot = oracle.Rotation(dim)
    _, cen = oracle.codebook(bits, dim)
    cal = oracle.fit_calibration(rot, v, cen)
    ix = T.NativeIndex(dim, bits)
    ix.calibrate(v)
    sh, sc = ix.calibration()
    assert bits_equal(sh, cal[0]) and bits_equal(sc, cal[1])
    ix.add(v)
    oidx = OracleIndex(oracle, dim, bits, v, calibration=cal)
    seq, scales = ix.download_seq()
    assert np.array_equal(seq, oidx.seq) and bits_equal(scales, oidx.scales)
    ix.close()


@pytest.mark.parametrize("bits", [2, 4])
def test_upload_over_a_larger_index_leaves_no_stale_lanes(T, oracle, bits):
    """upload_seq replaces the contents: rows appended afterwards must land in zeroed blocks, so
    the bytes read back (whole padded blocks) equal a from-scratch index of the same rows."""
    dim = 128
    big = OracleIndex(oracle, dim, bits, unit_gaussian(1000, dim, seed=1))
    small_rows = unit_gaussian(75, dim, seed=2)
    small = OracleIndex(oracle, dim, bits, small_rows[:40])
    whole = OracleIndex(oracle, dim, bits, small_rows)
    ix = to_native(T, big)
    ix.upload_seq(small.seq, small.n, small.scales)
    ix.append_rows(whole.rows()[40:], whole.scales[40:])
    seq, scales = ix.download_seq()
    assert np.array_equal(seq, whole.seq)
    assert bits_equal(scales, whole.scales)
    data = ix.to_bytes(format=6)
    fresh = to_native(T, whole)
    assert data == fresh.to_bytes(format=6)
    q = unit_gaussian(4, dim, seed=3)
    s, i = ix.search(q, 10)
    os_, oi = whole.search(q, 10)
    assert np.array_equal(i, oi) and bits_equal(s, os_)
    ix.close(); fresh.close()


def test_wide_scan_with_subnormal_and_huge_row_scales(T, oracle):
    """Row scales a foreign snapshot could hold: subnormal (their reciprocal overflows), close to
    the largest float, and blocks of all-zero scales.  The wide kernel's accumulator bound must
    not lose a candidate: results equal the oracle's bit for bit."""
    dim, n, nq = 1536, 4_003, 200
    oidx = OracleIndex(oracle, dim, 4, unit_gaussian(n, dim, seed=61))
    rng = np.random.default_rng(62)
    block = np.arange(n) // 32
    kind = rng.integers(0, 5, size=block.max() + 1)[block]
    factors = np.ones(n, np.float32)
    factors[kind == 0] = np.float32(1e-42)          # every row of the block subnormal
    factors[kind == 1] = rng.choice(np.array([1e-44, 1e-40, 1e-35, 1.0], np.float32), size=int((kind == 1).sum()))
    factors[kind == 2] = np.float32(1e37)
    factors[kind == 3] = np.float32(0.0)
    oidx.scales = (oidx.scales * factors).astype(np.float32)
    q = unit_gaussian(nq, dim, seed=63)
    ix = to_native(T, oidx)
    for m in (None, kind != 2, kind == 0, (kind == 0) | (kind == 3)):       # with the huge blocks allowed, and not
        words = None if m is None else T.pack_mask(m)[0]
        for k in (1, 10, 100):
            s, i = ix.search(q, k, mask_words=words)
            assert ix.queries_per_launch() == nq
            os_, oi = oidx.search(q, k, mask_words=words)
            assert np.array_equal(i, oi) and bits_equal(s, os_), k
    ix.close()
