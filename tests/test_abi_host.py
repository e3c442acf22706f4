"""CPU-side checks of the product library: it loads, exports every symbol the
header declares, and its host-only derivations match the reference's goldens.
No kernel is launched here."""
import ctypes
import os
import re

import numpy as np
import pytest

from golden_data import CODEBOOK, ROT_DIM8, ROT_DIM24, ROT_DIM64

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.fixture(scope="module")
def T():
    from turbovec_amd import _lib
    _lib.lib()
    return _lib


def test_library_exports_every_declared_symbol(T):
    header = open(os.path.join(ROOT, "include", "turbovec_hip.h")).read()
    declared = set(re.findall(r"\b(tv_[a-z0-9_]+)\s*\(", header))
    declared -= {"tv_index"}
    assert declared == set(T.EXPORTS), declared ^ set(T.EXPORTS)
    handle = ctypes.CDLL(T.LIB_PATH)
    for name in sorted(declared):
        assert hasattr(handle, name), name


def test_status_strings(T):
    L = T.lib()
    assert L.tv_status_string(0) == b"ok"
    assert b"allowlist is empty" in L.tv_status_string(T.ERR_ALLOWLIST_EMPTY)
    assert b"mask length" in L.tv_status_string(T.ERR_MASK_LENGTH_MISMATCH)


def _apply(signs, perms, block, inv, x):
    """Scalar rotation (rotation.rs:265-320) driven by the library's tables."""
    x = np.asarray(x, np.float32)
    for r in range(2):
        y = (x[perms[r]] * signs[r]).astype(np.float32)
        for off in range(0, len(y), block):
            blk = y[off:off + block]
            ln = 1
            while ln < block:
                for i in range(0, block, 2 * ln):
                    a = blk[i:i + ln].copy()
                    b = blk[i + ln:i + 2 * ln].copy()
                    blk[i:i + ln] = a + b
                    blk[i + ln:i + 2 * ln] = a - b
                ln *= 2
            y[off:off + block] = blk * inv
        x = y
    return x


def test_host_rotation_tables_match_reference_goldens(T):
    cases = [(8, np.arange(8, dtype=np.float32) - 3.5, ROT_DIM8),
             (24, np.array([(i * 7 % 11) - 5.0 for i in range(24)], np.float32), ROT_DIM24),
             (64, np.array([(i * 13 % 29) - 14.0 for i in range(64)], np.float32), ROT_DIM64)]
    for dim, x, gold in cases:
        signs, perms, block, inv = T.host_rotation_tables(dim)
        assert block == (dim & -dim)
        out = _apply(signs, perms, block, inv, x)
        assert [int(v) for v in out.view(np.uint32)] == gold


@pytest.mark.parametrize("dim", [128, 1536, 3072])
def test_host_rotation_tables_match_oracle(T, oracle, dim):
    signs, perms, block, inv = T.host_rotation_tables(dim)
    rot = oracle.Rotation(dim)
    for r in range(2):
        assert np.array_equal(signs[r], rot.signs(r))
        assert np.array_equal(perms[r], rot.perm(r))
    assert block == rot.block


@pytest.mark.parametrize("dim,bits,wb,wc", CODEBOOK)
def test_host_codebook_matches_reference_fnv(T, oracle, dim, bits, wb, wc):
    b, c = T.host_codebook(bits, dim)
    assert oracle.fnv1a(c) == wc
    assert oracle.fnv1a(b) == wb


def test_host_codebook_dim128_matches_oracle(T, oracle):
    b, c = T.host_codebook(4, 128)
    ob, oc = oracle.codebook(4, 128)
    assert np.array_equal(b, ob) and np.array_equal(c, oc)


def test_validate_queries_and_pack_mask(T, oracle):
    q = np.ones(24, np.float32)
    assert T.validate_queries(q, 8) == (T.OK, 0)
    assert T.validate_queries(q[:23], 8)[0] == T.ERR_QUERY_BUFFER_NOT_MULTIPLE_OF_DIM
    for bad in (np.nan, np.inf, -np.inf, 1e16):
        q2 = q.copy()
        q2[17] = bad
        assert T.validate_queries(q2, 8) == (T.ERR_INVALID_QUERY_VALUE, 17)
        assert oracle.validate_queries(q2, 8) == (T.ERR_INVALID_QUERY_VALUE, 17)
    rng = np.random.default_rng(0)
    for n in (0, 1, 63, 64, 65, 1000):
        m = rng.random(n) < 0.3
        words, allowed = T.pack_mask(m)
        owords, oallowed = oracle.pack_mask(m)
        assert np.array_equal(words, owords) and allowed == oallowed == int(m.sum())
    # any non-zero byte counts as true (turbovec-python/src/lib.rs:87-130)
    words, allowed = T.pack_mask(np.array([0, 2, 255, 0, 1], np.uint8))
    assert words[0] == 0b10110 and allowed == 3


def test_missing_library_fails_loudly(T, monkeypatch, tmp_path):
    import turbovec_amd._lib as L
    monkeypatch.setattr(L, "_lib", None)
    monkeypatch.setattr(L, "LIB_PATH", str(tmp_path / "nope.so"))
    with pytest.raises(ImportError):
        L.lib()
