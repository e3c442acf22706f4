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


_C_TO_RUST = {
    "int": "c_int", "size_t": "usize", "float": "c_float", "double": "c_double", "void": "c_void",
    "uint8_t": "u8", "uint32_t": "u32", "uint64_t": "u64", "int32_t": "i32", "int64_t": "i64",
    "tv_index": "tv_index", "char": "c_char",
}


def _rust_type(c_decl):
    """'const float *queries' -> ('queries', '*const c_float'); 'tv_index **out' -> ('out', '*mut *mut tv_index')."""
    c_decl = c_decl.strip()
    m = re.match(r"^(const\s+)?(\w+)\s*(\*{0,2})\s*(\w+)$", c_decl)
    assert m, c_decl
    const, base, stars, name = m.groups()
    t = _C_TO_RUST[base]
    for depth in range(len(stars)):
        innermost = depth == 0
        t = ("*const " if (const and innermost) else "*mut ") + t
    return name, t


def test_rust_bindings_match_the_header():
    """rust/turbovec-hip-sys/src/lib.rs cannot be compiled here (no Rust toolchain): keep it equal to
    the C header mechanically -- every entry point, argument names, order and types, return types,
    and the status / score-mode constants."""
    header = open(os.path.join(ROOT, "include", "turbovec_hip.h")).read()
    rust = open(os.path.join(ROOT, "rust", "turbovec-hip-sys", "src", "lib.rs")).read()
    c_protos = re.findall(r"^(int|size_t|const char \*)\s*(tv_\w+)\s*\(([^;]*?)\)\s*;", header, flags=re.M | re.S)
    r_protos = {name: (args, ret) for name, args, ret in
                re.findall(r"pub fn (tv_\w+)\(([^)]*)\)\s*(?:->\s*([^;]+))?;", rust)}
    assert {p[1] for p in c_protos} == set(r_protos), {p[1] for p in c_protos} ^ set(r_protos)
    for ret, name, args in c_protos:
        want_ret = {"int": "c_int", "size_t": "usize", "const char *": "*const c_char"}[ret]
        assert r_protos[name][1].strip() == want_ret, name
        c_args = [a for a in (x.strip() for x in " ".join(args.split()).split(",")) if a and a != "void"]
        r_args = [a.strip() for a in r_protos[name][0].split(",") if a.strip()]
        assert len(c_args) == len(r_args), name
        for ca, ra in zip(c_args, r_args):
            rname, rtype = (x.strip() for x in ra.split(":"))
            assert (rname, rtype) == _rust_type(ca), (name, ca, ra)
    for cname, value in re.findall(r"^\s*(TV_[A-Z0-9_]+)\s*=\s*(\d+)", header, flags=re.M):
        assert re.search(rf"pub const {cname}: c_int = {value};", rust), cname


def test_integration_doc_lists_every_binding_entry_point():
    """The integration guide at the repository root names every non-diagnostic entry point of the header."""
    header = open(os.path.join(ROOT, "include", "turbovec_hip.h")).read()
    doc = open(os.path.join(ROOT, "INTEGRATION.md")).read()
    declared = set(re.findall(r"\b(tv_[a-z0-9_]+)\s*\(", header)) - {"tv_index"}
    missing = {n for n in declared if not n.startswith("tv_debug_") and n not in doc}
    assert not missing, missing


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
