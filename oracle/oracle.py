"""ctypes binding of the CPU oracle (oracle/libtv_oracle.so).

TEST INFRASTRUCTURE: the checker for the HIP search path.  Imported only by
tests, the smoke check and the CPU-baseline leg of the benchmark; the product
package never imports it.
"""
import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libtv_oracle.so")

MODE_AUTO, MODE_L_SCALAR, MODE_L_CLASSIC, MODE_L_U32, MODE_P = 0, 1, 2, 3, 4

OK = 0
ERR_QUERY_BUFFER_NOT_MULTIPLE_OF_DIM = 1
ERR_INVALID_QUERY_VALUE = 2
ERR_MASK_LENGTH_MISMATCH = 3
ERR_ALLOWLIST_EMPTY = 4
ERR_UNKNOWN_ID = 5
ERR_BAD_ARGUMENT = 6


def build():
    """Compile the oracle with gcc (always recompiles)."""
    subprocess.check_call(["make", "-B", "-C", _HERE, "libtv_oracle.so"], stdout=subprocess.DEVNULL)


def _load():
    if not os.path.exists(_LIB_PATH):
        build()
    lib = C.CDLL(_LIB_PATH)
    vp, sz, i32, f32p = C.c_void_p, C.c_size_t, C.c_int, C.c_void_p
    lib.tvo_rotation_new.restype = vp
    lib.tvo_rotation_new.argtypes = [i32]
    lib.tvo_rotation_free.argtypes = [vp]
    lib.tvo_rotation_block.argtypes = [vp]
    lib.tvo_rotation_signs.restype = C.POINTER(C.c_float)
    lib.tvo_rotation_signs.argtypes = [vp, i32]
    lib.tvo_rotation_perm.restype = C.POINTER(C.c_uint32)
    lib.tvo_rotation_perm.argtypes = [vp, i32]
    lib.tvo_rotation_apply.argtypes = [vp, f32p]
    lib.tvo_rotation_apply_scaled.argtypes = [vp, f32p, C.c_float, f32p]
    lib.tvo_beta_cdf.restype = C.c_double
    lib.tvo_beta_cdf.argtypes = [C.c_double, C.c_double]
    lib.tvo_beta_pdf.restype = C.c_double
    lib.tvo_beta_pdf.argtypes = [C.c_double, C.c_double]
    lib.tvo_codebook.argtypes = [i32, i32, f32p, f32p]
    lib.tvo_norm.restype = C.c_float
    lib.tvo_norm.argtypes = [f32p, i32]
    lib.tvo_fit_calibration.argtypes = [vp, f32p, sz, i32, f32p, i32, f32p, f32p]
    lib.tvo_encode.argtypes = [vp, f32p, sz, i32, i32, f32p, f32p, f32p, f32p, vp, f32p]
    lib.tvo_n_byte_groups.restype = sz
    lib.tvo_n_byte_groups.argtypes = [i32, i32]
    lib.tvo_seq_len.restype = sz
    lib.tvo_seq_len.argtypes = [sz, i32, i32]
    lib.tvo_repack_seq.argtypes = [vp, sz, i32, i32, vp]
    lib.tvo_seq_to_packed.argtypes = [vp, sz, i32, i32, vp]
    lib.tvo_swap_remove_seq.restype = sz
    lib.tvo_swap_remove_seq.argtypes = [vp, f32p, sz, i32, i32, sz]
    lib.tvo_build_lut.argtypes = [f32p, f32p, i32, i32, vp, f32p, f32p]
    lib.tvo_build_permute_dot.argtypes = [f32p, f32p, i32, vp, vp, vp, f32p]
    lib.tvo_calibrate_query.argtypes = [f32p, f32p, f32p, i32, f32p, f32p]
    lib.tvo_search.argtypes = [i32, f32p, sz, vp, vp, f32p, f32p, f32p, f32p, i32, i32, sz, sz, vp,
                               f32p, vp, vp, vp, f32p, i32]
    lib.tvo_search_fast.argtypes = [f32p, sz, vp, vp, f32p, f32p, i32, i32, sz, sz, vp, f32p, vp, vp, i32]
    lib.tvo_have_vnni.restype = i32
    lib.tvo_seq_to_vector_major.argtypes = [vp, sz, i32, i32, vp]
    lib.tvo_search_vnni.argtypes = [f32p, sz, vp, vp, f32p, f32p, i32, sz, sz, vp, f32p, vp, vp, i32]
    lib.tvo_validate_queries.argtypes = [f32p, sz, i32, vp]
    lib.tvo_pack_mask.restype = sz
    lib.tvo_pack_mask.argtypes = [vp, sz, vp]
    lib.tvo_lcg_vectors.argtypes = [sz, C.c_uint64, f32p]
    lib.tvo_fnv1a.restype = C.c_uint64
    lib.tvo_fnv1a.argtypes = [vp, sz]
    return lib


_lib = None


def lib():
    global _lib
    if _lib is None:
        _lib = _load()
    return _lib


def _p(a):
    return None if a is None else a.ctypes.data


def _f32(a):
    return np.ascontiguousarray(a, dtype=np.float32)


class Rotation:
    """turbovec/src/rotation.rs Rotation."""

    def __init__(self, dim):
        self.dim = dim
        self.h = lib().tvo_rotation_new(dim)
        if not self.h:
            raise ValueError("rotation dim must be a positive multiple of 8 and <= 16384")

    def __del__(self):
        if getattr(self, "h", None):
            lib().tvo_rotation_free(self.h)
            self.h = None

    @property
    def block(self):
        return lib().tvo_rotation_block(self.h)

    def signs(self, rnd):
        return np.ctypeslib.as_array(lib().tvo_rotation_signs(self.h, rnd), (self.dim,)).copy()

    def perm(self, rnd):
        return np.ctypeslib.as_array(lib().tvo_rotation_perm(self.h, rnd), (self.dim,)).copy()

    def apply(self, row):
        v = _f32(row).copy()
        lib().tvo_rotation_apply(self.h, _p(v))
        return v

    def apply_scaled(self, row, inv):
        src = _f32(row)
        dst = np.empty_like(src)
        lib().tvo_rotation_apply_scaled(self.h, _p(src), C.c_float(inv), _p(dst))
        return dst


_codebook_memo = {}


def codebook(bits, dim):
    """(boundaries, centroids) -- turbovec/src/codebook.rs:50."""
    key = (bits, dim)
    if key not in _codebook_memo:
        b = np.zeros((1 << bits) - 1, np.float32)
        c = np.zeros(1 << bits, np.float32)
        rc = lib().tvo_codebook(bits, dim, _p(b), _p(c))
        if rc != 0:
            raise ValueError("bad codebook shape")
        _codebook_memo[key] = (b, c)
    b, c = _codebook_memo[key]
    return b.copy(), c.copy()


def fit_calibration(rot, vectors, centroids):
    v = _f32(vectors)
    n, dim = v.shape
    sh = np.zeros(dim, np.float32)
    sc = np.ones(dim, np.float32)
    cen = _f32(centroids)
    lib().tvo_fit_calibration(rot.h, _p(v), n, dim, _p(cen), len(cen), _p(sh), _p(sc))
    return sh, sc


def encode(rot, vectors, bits, calibration=None):
    """Returns (packed bit-plane rows (n, bits*dim/8) u8, scales (n,) f32)."""
    v = _f32(vectors)
    n, dim = v.shape
    b, c = codebook(bits, dim)
    packed = np.zeros((n, bits * dim // 8), np.uint8)
    scales = np.zeros(n, np.float32)
    sh = sc = None
    if calibration is not None:
        sh, sc = _f32(calibration[0]), _f32(calibration[1])
    lib().tvo_encode(rot.h, _p(v), n, dim, bits, _p(b), _p(c), _p(sh), _p(sc), _p(packed), _p(scales))
    return packed, scales


def n_byte_groups(bits, dim):
    return lib().tvo_n_byte_groups(bits, dim)


def repack_seq(packed, n, bits, dim):
    packed = np.ascontiguousarray(packed, np.uint8)
    out = np.zeros(lib().tvo_seq_len(n, bits, dim), np.uint8)
    lib().tvo_repack_seq(_p(packed), n, bits, dim, _p(out))
    return out


def seq_to_packed(seq, n, bits, dim):
    seq = np.ascontiguousarray(seq, np.uint8)
    out = np.zeros((n, bits * dim // 8), np.uint8)
    lib().tvo_seq_to_packed(_p(seq), n, bits, dim, _p(out))
    return out


def swap_remove_seq(seq, scales, n, bits, dim, idx):
    """In place on seq/scales (numpy arrays); returns new n."""
    return lib().tvo_swap_remove_seq(_p(seq), _p(scales), n, bits, dim, idx)


def build_lut(q_rot, centroids, bits, dim):
    q = _f32(q_rot)
    cen = _f32(centroids)
    lut = np.zeros(n_byte_groups(bits, dim) * 32, np.uint8)
    s = C.c_float()
    b = C.c_float()
    lib().tvo_build_lut(_p(q), _p(cen), bits, dim, _p(lut), C.addressof(s), C.addressof(b))
    return lut, np.float32(s.value), np.float32(b.value)


def build_permute_dot(q_rot, centroids, dim):
    q = _f32(q_rot)
    cen = _f32(centroids)
    levels = np.zeros(16, np.int8)
    w = np.zeros(dim, np.int8)
    zero = C.c_int32()
    s = C.c_float()
    lib().tvo_build_permute_dot(_p(q), _p(cen), dim, _p(levels), _p(w), C.addressof(zero), C.addressof(s))
    return levels, w, zero.value, np.float32(s.value)


def pack_mask(mask_bools):
    m = np.ascontiguousarray(mask_bools).view(np.uint8)
    words = np.zeros((len(m) + 63) // 64, np.uint64)
    allowed = lib().tvo_pack_mask(_p(m), len(m), _p(words))
    return words, allowed


def validate_queries(queries_flat, dim):
    q = _f32(queries_flat).ravel()
    bad = C.c_size_t(0)
    rc = lib().tvo_validate_queries(_p(q), q.size, dim, C.addressof(bad))
    return rc, bad.value


def search(rot, seq, scales, queries, k, bits, dim, n, mask_words=None, mode=MODE_AUTO,
           calibration=None, dump=False, n_threads=8):
    """turbovec/src/search.rs:3206 over the sequential-blocked layout.

    Returns (scores (nq,k_eff) f32, indices (nq,k_eff) i64[, acc (nq,n) i32, raw scores (nq,n)]).
    """
    q = _f32(queries).reshape(-1, dim)
    nq = q.shape[0]
    _, cen = codebook(bits, dim)
    seq = np.ascontiguousarray(seq, np.uint8)
    scales = _f32(scales)
    n_allowed = n
    if mask_words is not None:
        mask_words = np.ascontiguousarray(mask_words, np.uint64)
        n_allowed = int(sum(bin(int(w)).count("1") for w in mask_words)) if len(mask_words) < 4096 else \
            int(np.unpackbits(mask_words.view(np.uint8)).sum())
    kk = min(k, n, n_allowed)
    out_s = np.zeros((nq, kk), np.float32)
    out_i = np.zeros((nq, kk), np.int64)
    k_eff = C.c_size_t(0)
    acc = sc = None
    if dump:
        acc = np.zeros((nq, n), np.int32)
        sc = np.zeros((nq, n), np.float32)
    sh = ts = None
    if calibration is not None:
        sh, ts = _f32(calibration[0]), _f32(calibration[1])
    rc = lib().tvo_search(mode, _p(q), nq, rot.h, _p(seq), _p(cen), _p(scales), _p(sh), _p(ts),
                          bits, dim, n, k, _p(mask_words), _p(out_s), _p(out_i), C.addressof(k_eff),
                          _p(acc), _p(sc), n_threads)
    if rc != 0:
        raise RuntimeError(f"tvo_search failed rc={rc}")
    assert k_eff.value == kk, (k_eff.value, kk)
    if dump:
        return out_s, out_i, acc, sc
    return out_s, out_i


def search_fast(rot, seq, scales, queries, k, bits, dim, n, mask_words=None, n_threads=8):
    """Throughput-oriented twin of search() (modes P / L_U32, uncalibrated, k <= 1024)."""
    q = _f32(queries).reshape(-1, dim)
    nq = q.shape[0]
    _, cen = codebook(bits, dim)
    seq = np.ascontiguousarray(seq, np.uint8)
    scales = _f32(scales)
    n_allowed = n
    if mask_words is not None:
        mask_words = np.ascontiguousarray(mask_words, np.uint64)
        n_allowed = int(np.unpackbits(mask_words.view(np.uint8)).sum())
    kk = min(k, n, n_allowed)
    assert kk <= 1024
    out_s = np.zeros((nq, kk), np.float32)
    out_i = np.zeros((nq, kk), np.int64)
    k_eff = C.c_size_t(0)
    rc = lib().tvo_search_fast(_p(q), nq, rot.h, _p(seq), _p(cen), _p(scales), bits, dim, n, k,
                               _p(mask_words), _p(out_s), _p(out_i), C.addressof(k_eff), n_threads)
    if rc != 0:
        raise RuntimeError(f"tvo_search_fast failed rc={rc}")
    return out_s, out_i


def have_vnni():
    return bool(lib().tvo_have_vnni())


def seq_to_vector_major(seq, n, bits, dim):
    """The layout the reference keeps at rest on VNNI hosts (pack.rs:1269-1271, :1347-1358)."""
    seq = np.ascontiguousarray(seq, np.uint8)
    out = np.zeros_like(seq)
    if lib().tvo_seq_to_vector_major(_p(seq), n, bits, dim, _p(out)) != 0:
        raise ValueError("vector-major needs a multiple of 4 byte-groups")
    return out


def search_vnni(rot, vm, scales, queries, k, dim, n, mask_words=None, n_threads=8):
    """The reference's AVX-512 VNNI permute-dot kernel (4-bit) over vector-major codes."""
    q = _f32(queries).reshape(-1, dim)
    nq = q.shape[0]
    _, cen = codebook(4, dim)
    vm = np.ascontiguousarray(vm, np.uint8)
    scales = _f32(scales)
    n_allowed = n
    if mask_words is not None:
        mask_words = np.ascontiguousarray(mask_words, np.uint64)
        n_allowed = int(np.unpackbits(mask_words.view(np.uint8)).sum())
    kk = min(k, n, n_allowed)
    assert kk <= 1024
    out_s = np.zeros((nq, kk), np.float32)
    out_i = np.zeros((nq, kk), np.int64)
    k_eff = C.c_size_t(0)
    rc = lib().tvo_search_vnni(_p(q), nq, rot.h, _p(vm), _p(cen), _p(scales), dim, n, k,
                               _p(mask_words), _p(out_s), _p(out_i), C.addressof(k_eff), n_threads)
    if rc != 0:
        raise RuntimeError(f"tvo_search_vnni failed rc={rc}")
    return out_s, out_i


def lcg_vectors(n, dim, seed):
    out = np.zeros(n * dim, np.float32)
    lib().tvo_lcg_vectors(n * dim, C.c_uint64(seed), _p(out))
    return out.reshape(n, dim)


def fnv1a(arr):
    a = np.ascontiguousarray(arr)
    b = a.view(np.uint8).ravel()
    return lib().tvo_fnv1a(_p(b), b.size)
