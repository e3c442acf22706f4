"""Seeded sweep over shapes the fixed cases do not pin down: dims whose byte-group count is
not a multiple of the 32-group chunk, odd chunk counts, ragged last blocks, every bit
width and score mode, masks of every density, k from 1 to past the list and sampled-path
limits, batches around the tile sizes.  Each case is compared with the oracle bit for bit
(ids, float scores, and the integer sums of the first queries)."""
import numpy as np
import pytest

from helpers import OracleIndex, bits_equal, to_native, unit_gaussian

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def T():
    from turbovec_amd import _lib
    _lib.lib()
    return _lib


def cases():
    rng = np.random.default_rng(2024)
    out = []
    dims = [8, 16, 24, 40, 72, 104, 136, 200, 264, 328, 520, 776, 1000, 1032, 1544, 2056]
    for i in range(36):
        bits = int(rng.choice([2, 3, 4]))
        dim = int(rng.choice(dims))
        n = int(rng.choice([1, 5, 31, 32, 33, 64, 100, 257, 1000, 4097, 9000, 20_011, 40_000]))
        nq = int(rng.choice([1, 2, 3, 5, 8, 9, 31, 33, 65, 97, 130]))
        k = int(rng.choice([1, 2, 10, 16, 17, 32, 33, 100, 513, 600]))
        if bits == 4:
            mode = str(rng.choice(["AUTO", "P", "L_CLASSIC", "L_U32"]))
        else:
            mode = str(rng.choice(["AUTO", "L_CLASSIC", "L_U32"]))
        mask = str(rng.choice(["none", "half", "sparse", "run", "one", "allbutone"]))
        out.append((i, dim, bits, n, nq, k, mode, mask))
    return out


@pytest.mark.parametrize("case", cases(), ids=lambda c: "c%02d-d%d-b%d-n%d-q%d-k%d-%s-%s" % c)
def test_random_shape(T, oracle, case):
    O = oracle
    i, dim, bits, n, nq, k, mode, mask = case
    rng = np.random.default_rng(1000 + i)
    v = unit_gaussian(n, dim, seed=2000 + i)
    if n > 40:
        v[7] = v[3]                                   # exact ties
        v[11] *= 0.0                                  # zero row
    oidx = OracleIndex(O, dim, bits, v)
    omode = {"AUTO": 0, "P": O.MODE_P, "L_CLASSIC": O.MODE_L_CLASSIC, "L_U32": O.MODE_L_U32}[mode]
    tmode = {"AUTO": None, "P": T.SCORE_P, "L_CLASSIC": T.SCORE_L_CLASSIC, "L_U32": T.SCORE_L_U32}[mode]
    ix = to_native(T, oidx, mode=tmode)
    q = unit_gaussian(nq, dim, seed=3000 + i) * np.float32(rng.uniform(0.1, 30.0))
    m = None
    if mask == "half":
        m = rng.random(n) < 0.5
    elif mask == "sparse":
        m = rng.random(n) < 0.02
    elif mask == "run":
        m = np.zeros(n, bool); a = n // 3; m[a:a + max(1, n // 10)] = True
    elif mask == "one":
        m = np.zeros(n, bool); m[n // 2] = True
    elif mask == "allbutone":
        m = np.ones(n, bool); m[0] = False
    words = None if m is None else T.pack_mask(m)[0]
    s, idx = ix.search(q, k, mask_words=words)
    os_, oi = oidx.search(q, k, mask_words=words, mode=omode)
    assert s.shape == os_.shape
    assert np.array_equal(idx, oi)
    assert bits_equal(s, os_)
    if m is not None and idx.size:
        assert m[idx].all()
    acc, raw = ix.debug_scan(q[:2])
    _s, _i, oacc, oraw = oidx.search(q[:2], k, mode=omode, dump=True)
    assert np.array_equal(acc, oacc) and bits_equal(raw, oraw)
    ix.set_path(1)                                    # exact list / select path
    s2, i2 = ix.search(q, k, mask_words=words)
    ix.set_path(0)
    assert np.array_equal(i2, idx) and bits_equal(s2, s)
    ix.close()
