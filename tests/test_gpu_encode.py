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
    sh, sc = O.fit_calibration(rot, v, c)          # the fixture calibrates before it adds
    ix = T.NativeIndex(dim, bits)
    ix.set_calibration(sh, sc)
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
