"""ctypes binding of libturbovec_hip.so (the C ABI declared in include/turbovec_hip.h).

There is no CPU fallback: if the library is missing or a call fails, this raises.
"""
import ctypes as C
import os

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libturbovec_hip.so")

OK = 0
ERR_QUERY_BUFFER_NOT_MULTIPLE_OF_DIM = 1
ERR_INVALID_QUERY_VALUE = 2
ERR_MASK_LENGTH_MISMATCH = 3
ERR_ALLOWLIST_EMPTY = 4
ERR_UNKNOWN_ID = 5
ERR_BAD_ARGUMENT = 6
ERR_HIP = 7
ERR_NO_DEVICE = 8
ERR_INDEX_OUT_OF_RANGE = 9

SCORE_AUTO, SCORE_L_SCALAR, SCORE_L_CLASSIC, SCORE_L_U32, SCORE_P = 0, 1, 2, 3, 4

# every symbol include/turbovec_hip.h declares
EXPORTS = [
    "tv_status_string", "tv_last_error", "tv_index_create", "tv_index_destroy", "tv_index_set_tables",
    "tv_index_set_calibration", "tv_index_set_score_mode", "tv_index_get_tables", "tv_index_upload_seq",
    "tv_index_upload_seq_dev", "tv_index_append_rows", "tv_index_add", "tv_index_add_dev", "tv_index_calibrate", "tv_index_get_calibration", "tv_index_swap_remove", "tv_index_download_seq", "tv_index_len", "tv_index_dim",
    "tv_index_bits", "tv_validate_queries", "tv_pack_mask", "tv_search", "tv_search_dev", "tv_debug_scan",
    "tv_debug_prepare", "tv_last_scan_ms", "tv_debug_queries_per_launch", "tv_index_device_ptrs", "tv_host_rotation_tables", "tv_host_codebook",
    "tv_debug_stream_probe", "tv_debug_mfma_probe", "tv_debug_set_path", "tv_debug_overflow_redos",
    "tv_host_snapshot_len", "tv_host_snapshot_compose", "tv_host_snapshot_info", "tv_host_snapshot_extract",
    "tv_index_to_bytes", "tv_index_from_bytes", "tv_search_dev_noalloc", "tv_noalloc_scratch_bytes",
    "tv_debug_exact_redos", "tv_debug_sampling_plan", "tv_debug_merged_calls", "tv_debug_level_repeats", "tv_debug_workspace_bytes",
]

_lib = None


class TurbovecHipError(RuntimeError):
    def __init__(self, status, detail=""):
        self.status = status
        super().__init__(f"turbovec_hip status {status}: {detail}")


def lib():
    """Load the built library; raises if it has not been built."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise ImportError(
            f"{LIB_PATH} is missing: build it with `python -m turbovec_amd.build` (hipcc, gfx950). "
            "The search path has no CPU fallback.")
    L = C.CDLL(LIB_PATH)
    vp, sz, i32 = C.c_void_p, C.c_size_t, C.c_int
    L.tv_status_string.restype = C.c_char_p
    L.tv_status_string.argtypes = [i32]
    L.tv_last_error.restype = C.c_char_p
    L.tv_index_create.argtypes = [i32, i32, i32, C.POINTER(vp)]
    L.tv_index_destroy.argtypes = [vp]
    L.tv_index_set_tables.argtypes = [vp, vp, vp, vp]
    L.tv_index_set_calibration.argtypes = [vp, vp, vp]
    L.tv_index_set_score_mode.argtypes = [vp, i32]
    L.tv_index_get_tables.argtypes = [vp, vp, vp, vp, vp]
    L.tv_index_upload_seq.argtypes = [vp, vp, sz, vp]
    L.tv_index_upload_seq_dev.argtypes = [vp, vp, sz, vp]
    L.tv_index_append_rows.argtypes = [vp, vp, vp, sz]
    L.tv_index_add.argtypes = [vp, vp, sz]
    L.tv_index_calibrate.argtypes = [vp, vp, sz]
    L.tv_index_get_calibration.argtypes = [vp, vp, vp, C.POINTER(sz)]
    L.tv_host_snapshot_len.restype = sz
    L.tv_host_snapshot_len.argtypes = [i32, i32, i32, i32, sz, sz]
    L.tv_host_snapshot_compose.argtypes = [i32, i32, i32, i32, vp, vp, sz, vp, vp, vp, sz, vp, vp, vp]
    L.tv_host_snapshot_info.argtypes = [vp, sz, C.POINTER(i32), C.POINTER(i32), C.POINTER(i32), C.POINTER(i32), C.POINTER(sz), C.POINTER(sz)]
    L.tv_host_snapshot_extract.argtypes = [vp, sz, vp, vp, vp, vp, vp, vp, vp]
    L.tv_index_to_bytes.argtypes = [vp, vp, i32, vp, sz, C.POINTER(sz)]
    L.tv_index_from_bytes.argtypes = [vp, sz, i32, C.POINTER(vp), vp]
    L.tv_index_add_dev.argtypes = [vp, vp, sz]
    L.tv_index_swap_remove.argtypes = [vp, sz]
    L.tv_index_download_seq.argtypes = [vp, vp, vp]
    L.tv_index_len.restype = sz
    L.tv_index_len.argtypes = [vp]
    L.tv_index_dim.argtypes = [vp]
    L.tv_index_bits.argtypes = [vp]
    L.tv_validate_queries.argtypes = [vp, sz, i32, C.POINTER(sz)]
    L.tv_pack_mask.argtypes = [vp, sz, vp, C.POINTER(sz)]
    L.tv_search.argtypes = [vp, vp, sz, sz, vp, sz, vp, vp, C.POINTER(sz)]
    L.tv_search_dev.argtypes = [vp, vp, sz, sz, vp, sz, vp, vp, C.POINTER(sz)]
    L.tv_search_dev_noalloc.argtypes = [vp, vp, sz, sz, vp, sz, vp, vp, C.POINTER(sz)]
    L.tv_noalloc_scratch_bytes.restype = sz
    L.tv_noalloc_scratch_bytes.argtypes = []
    L.tv_debug_scan.argtypes = [vp, vp, sz, vp, vp]
    L.tv_debug_prepare.argtypes = [vp, vp, sz, vp, vp, vp]
    L.tv_last_scan_ms.argtypes = [vp, C.POINTER(C.c_float), C.POINTER(i32)]
    L.tv_debug_queries_per_launch.argtypes = [vp, C.POINTER(i32)]
    L.tv_index_device_ptrs.argtypes = [vp, C.POINTER(vp), C.POINTER(vp), C.POINTER(sz)]
    L.tv_debug_set_path.argtypes = [vp, i32]
    L.tv_debug_overflow_redos.argtypes = [vp, C.POINTER(sz)]
    L.tv_debug_exact_redos.argtypes = [vp, C.POINTER(sz)]
    L.tv_debug_workspace_bytes.argtypes = [vp, C.POINTER(sz), C.POINTER(sz)]
    L.tv_debug_level_repeats.argtypes = [vp, i32, C.POINTER(sz)]
    L.tv_debug_merged_calls.argtypes = [vp, C.POINTER(sz)]
    L.tv_debug_sampling_plan.argtypes = [vp, sz, sz, vp, vp, sz, C.POINTER(sz)]
    L.tv_debug_stream_probe.argtypes = [vp, vp, vp, sz, i32, C.POINTER(C.c_float)]
    L.tv_debug_mfma_probe.argtypes = [vp, i32, i32, C.POINTER(C.c_float), C.POINTER(C.c_double)]
    L.tv_host_rotation_tables.argtypes = [i32, vp, vp, C.POINTER(i32), C.POINTER(C.c_float)]
    L.tv_host_codebook.argtypes = [i32, i32, vp, vp]
    _lib = L
    return L


def check(status):
    if status != OK:
        L = lib()
        detail = L.tv_status_string(status).decode()
        extra = L.tv_last_error().decode()
        raise TurbovecHipError(status, detail + (": " + extra if extra else ""))


def ptr(a):
    return None if a is None else a.ctypes.data


class NativeIndex:
    """Thin owner of a tv_index handle (device-resident codes, scales and tables)."""

    def __init__(self, dim, bits, device=0):
        h = C.c_void_p()
        check(lib().tv_index_create(dim, bits, device, C.byref(h)))
        self.h = h
        self.dim, self.bits = dim, bits
        self.n_byte_groups = dim // (8 // bits)

    def close(self):
        h, self.h = getattr(self, "h", None), None
        if h and _lib is not None:
            _lib.tv_index_destroy(h)

    __del__ = close

    def __len__(self):
        return lib().tv_index_len(self.h)

    def set_score_mode(self, mode):
        check(lib().tv_index_set_score_mode(self.h, mode))

    def set_calibration(self, shift, scale):
        if shift is None:
            check(lib().tv_index_set_calibration(self.h, None, None))
            return
        sh = np.ascontiguousarray(shift, np.float32)
        sc = np.ascontiguousarray(scale, np.float32)
        assert sh.shape == (self.dim,) and sc.shape == (self.dim,)
        check(lib().tv_index_set_calibration(self.h, ptr(sh), ptr(sc)))

    def set_tables(self, signs=None, perms=None, centroids=None):
        s = None if signs is None else np.ascontiguousarray(signs, np.float32)
        p = None if perms is None else np.ascontiguousarray(perms, np.uint32)
        c = None if centroids is None else np.ascontiguousarray(centroids, np.float32)
        check(lib().tv_index_set_tables(self.h, ptr(s), ptr(p), ptr(c)))

    def tables(self):
        signs = np.zeros((2, self.dim), np.float32)
        perms = np.zeros((2, self.dim), np.uint32)
        cen = np.zeros(1 << self.bits, np.float32)
        bnd = np.zeros((1 << self.bits) - 1, np.float32)
        check(lib().tv_index_get_tables(self.h, ptr(signs), ptr(perms), ptr(cen), ptr(bnd)))
        return signs, perms, cen, bnd

    def upload_seq(self, seq_codes, n, scales):
        seq = np.ascontiguousarray(seq_codes, np.uint8)
        sc = np.ascontiguousarray(scales, np.float32)
        assert seq.size == ((n + 31) // 32) * self.n_byte_groups * 32, "sequential-blocked size mismatch"
        assert sc.size == n
        check(lib().tv_index_upload_seq(self.h, ptr(seq), n, ptr(sc)))

    def upload_seq_dev(self, d_seq_ptr, n, d_scales_ptr):
        check(lib().tv_index_upload_seq_dev(self.h, d_seq_ptr, n, d_scales_ptr))

    def append_rows(self, rows, scales):
        r = np.ascontiguousarray(rows, np.uint8).reshape(-1, self.n_byte_groups)
        sc = np.ascontiguousarray(scales, np.float32)
        assert len(sc) == len(r)
        check(lib().tv_index_append_rows(self.h, ptr(r), ptr(sc), len(r)))

    def add(self, vectors):
        """Encode raw float32 rows on the device and append them (tv_index_add)."""
        v = np.ascontiguousarray(vectors, np.float32).reshape(-1, self.dim)
        check(lib().tv_index_add(self.h, ptr(v), len(v)))

    def calibrate(self, sample):
        """Fit and commit the TQ+ pair from sample rows (tv_index_calibrate); empty index only."""
        v = np.ascontiguousarray(sample, np.float32).reshape(-1, self.dim)
        check(lib().tv_index_calibrate(self.h, ptr(v), len(v)))

    def calibration(self):
        n = C.c_size_t(0)
        check(lib().tv_index_get_calibration(self.h, None, None, C.byref(n)))
        if n.value == 0:
            return None
        sh, sc = np.zeros(n.value, np.float32), np.zeros(n.value, np.float32)
        check(lib().tv_index_get_calibration(self.h, ptr(sh), ptr(sc), C.byref(n)))
        return sh, sc

    def add_dev(self, d_vectors_ptr, n):
        check(lib().tv_index_add_dev(self.h, d_vectors_ptr, n))

    def swap_remove(self, idx):
        check(lib().tv_index_swap_remove(self.h, idx))

    def to_bytes(self, ids=None, format=7):
        """Snapshot image (tv_index_to_bytes); ids (uint64, one per slot) makes it an id-map image."""
        idp = None
        if ids is not None:
            ids = np.ascontiguousarray(ids, np.uint64)
            assert len(ids) == len(self)
            idp = ptr(ids)
        n = C.c_size_t(0)
        check(lib().tv_index_to_bytes(self.h, idp, format, None, 0, C.byref(n)))
        out = np.zeros(n.value, np.uint8)
        check(lib().tv_index_to_bytes(self.h, idp, format, ptr(out), n.value, C.byref(n)))
        return out.tobytes()

    @classmethod
    def from_bytes(cls, data, device=0):
        """(index, ids or None) from a snapshot image (tv_index_from_bytes)."""
        _fmt, kind, dim, bits, n_calib, n = snapshot_info(data)
        buf = np.frombuffer(data, np.uint8)
        ids = np.zeros(n, np.uint64) if kind == 1 else None
        h = C.c_void_p()
        check(lib().tv_index_from_bytes(ptr(buf), len(buf), device, C.byref(h), ptr(ids) if ids is not None else None))
        self = cls.__new__(cls)
        self.h = h
        self.dim, self.bits = dim, bits
        self.n_byte_groups = dim // (4 if bits == 2 else 2)
        return self, ids

    def download_seq(self):
        n = len(self)
        seq = np.zeros(((n + 31) // 32) * self.n_byte_groups * 32, np.uint8)
        sc = np.zeros(n, np.float32)
        check(lib().tv_index_download_seq(self.h, ptr(seq), ptr(sc)))
        return seq, sc

    def search(self, queries, k, mask_words=None):
        q = np.ascontiguousarray(queries, np.float32).reshape(-1, self.dim)
        nq = q.shape[0]
        n = len(self)
        cap = min(k, n)
        out_s = np.zeros((nq, cap), np.float32)
        out_i = np.zeros((nq, cap), np.int64)
        k_eff = C.c_size_t(0)
        mw = None if mask_words is None else np.ascontiguousarray(mask_words, np.uint64)
        check(lib().tv_search(self.h, ptr(q), nq, k, ptr(mw), 0 if mw is None else mw.size, ptr(out_s), ptr(out_i),
                              C.byref(k_eff)))
        ke = k_eff.value
        if ke == cap:
            return out_s, out_i
        return (np.ascontiguousarray(out_s.ravel()[: nq * ke].reshape(nq, ke)),
                np.ascontiguousarray(out_i.ravel()[: nq * ke].reshape(nq, ke)))

    def search_dev(self, d_queries_ptr, nq, k, d_out_scores_ptr, d_out_idx_ptr, d_mask_ptr=None, n_allowed=0):
        k_eff = C.c_size_t(0)
        check(lib().tv_search_dev(self.h, d_queries_ptr, nq, k, d_mask_ptr, n_allowed, d_out_scores_ptr,
                                  d_out_idx_ptr, C.byref(k_eff)))
        return k_eff.value

    def search_dev_noalloc(self, d_queries_ptr, nq, k, d_out_scores_ptr, d_out_idx_ptr, d_mask_ptr=None, n_allowed=0):
        """tv_search_dev on the library's fixed scratch array: no device allocation inside the call."""
        k_eff = C.c_size_t(0)
        check(lib().tv_search_dev_noalloc(self.h, d_queries_ptr, nq, k, d_mask_ptr, n_allowed, d_out_scores_ptr,
                                          d_out_idx_ptr, C.byref(k_eff)))
        return k_eff.value

    def debug_scan(self, queries):
        q = np.ascontiguousarray(queries, np.float32).reshape(-1, self.dim)
        n = len(self)
        acc = np.zeros((q.shape[0], n), np.int32)
        sc = np.zeros((q.shape[0], n), np.float32)
        check(lib().tv_debug_scan(self.h, ptr(q), q.shape[0], ptr(acc), ptr(sc)))
        return acc, sc

    def debug_prepare(self, queries):
        q = np.ascontiguousarray(queries, np.float32).reshape(-1, self.dim)
        rot = np.zeros_like(q)
        scale = np.zeros(q.shape[0], np.float32)
        bias = np.zeros(q.shape[0], np.float32)
        check(lib().tv_debug_prepare(self.h, ptr(q), q.shape[0], ptr(rot), ptr(scale), ptr(bias)))
        return rot, scale, bias

    def last_scan_ms(self):
        ms = C.c_float(0)
        n = C.c_int(0)
        check(lib().tv_last_scan_ms(self.h, C.byref(ms), C.byref(n)))
        return ms.value, n.value

    def queries_per_launch(self):
        n = C.c_int(0)
        check(lib().tv_debug_queries_per_launch(self.h, C.byref(n)))
        return n.value

    def set_path(self, force_full_lists):
        check(lib().tv_debug_set_path(self.h, int(force_full_lists)))

    def overflow_redos(self):
        c = C.c_size_t(0)
        check(lib().tv_debug_overflow_redos(self.h, C.byref(c)))
        return c.value

    def exact_redos(self):
        c = C.c_size_t(0)
        check(lib().tv_debug_exact_redos(self.h, C.byref(c)))
        return c.value

    def workspace_bytes(self):
        """(search workspace, host-call staging) bytes the index holds on the device."""
        a, b = C.c_size_t(0), C.c_size_t(0)
        check(lib().tv_debug_workspace_bytes(self.h, C.byref(a), C.byref(b)))
        return a.value, b.value

    def level_repeats(self, track=-1):
        """Sampling levels that ran twice so far (counted while tracking is on; track=1/0 switches it)."""
        c = C.c_size_t(0)
        check(lib().tv_debug_level_repeats(self.h, track, C.byref(c)))
        return c.value

    def merged_calls(self):
        """Search calls so far that were served by another caller's launch."""
        c = C.c_size_t(0)
        check(lib().tv_debug_merged_calls(self.h, C.byref(c)))
        return c.value

    def sampling_plan(self, nq, k):
        """(strides, repeat_offsets) of the sampling ladder a search of nq queries for the k best runs on the
        index as it stands; the last stride is 1 (the full scan).  Empty when the search does not sample."""
        strides, offs = np.zeros(32, np.uint32), np.zeros(32, np.uint32)
        c = C.c_size_t(0)
        check(lib().tv_debug_sampling_plan(self.h, nq, k, ptr(strides), ptr(offs), 32, C.byref(c)))
        return strides[:c.value].copy(), offs[:c.value].copy()

    def mfma_probe(self, iters=2000, reps=3):
        """int8 operations per second of the batched scan's MFMA loop alone (registers x LDS, no HBM)."""
        ms, ops = C.c_float(0), C.c_double(0)
        check(lib().tv_debug_mfma_probe(self.h, iters, reps, C.byref(ms), C.byref(ops)))
        return ops.value / (ms.value * 1e-3)

    def stream_probe(self, d_src_ptr, d_dst_ptr, nbytes, reps=5):
        """Mean ms per launch of a read-sum (d_dst_ptr None) or copy kernel over nbytes."""
        ms = C.c_float(0)
        check(lib().tv_debug_stream_probe(self.h, d_src_ptr, d_dst_ptr, nbytes, reps, C.byref(ms)))
        return ms.value

    def device_ptrs(self):
        a, b, s = C.c_void_p(), C.c_void_p(), C.c_size_t()
        check(lib().tv_index_device_ptrs(self.h, C.byref(a), C.byref(b), C.byref(s)))
        return a.value, b.value, s.value


def validate_queries(queries_flat, dim):
    q = np.ascontiguousarray(queries_flat, np.float32).ravel()
    bad = C.c_size_t(0)
    rc = lib().tv_validate_queries(ptr(q), q.size, dim, C.byref(bad))
    return rc, bad.value


def pack_mask(mask_bytes):
    m = np.ascontiguousarray(mask_bytes).view(np.uint8).ravel()
    words = np.zeros((m.size + 63) // 64, np.uint64)
    allowed = C.c_size_t(0)
    check(lib().tv_pack_mask(ptr(m), m.size, ptr(words), C.byref(allowed)))
    return words, allowed.value


def snapshot_info(data):
    buf = np.frombuffer(data, np.uint8)
    fmt, kind, dim, bits = C.c_int(0), C.c_int(0), C.c_int(0), C.c_int(0)
    n_calib, n = C.c_size_t(0), C.c_size_t(0)
    check(lib().tv_host_snapshot_info(ptr(buf), len(buf), C.byref(fmt), C.byref(kind), C.byref(dim), C.byref(bits),
                                      C.byref(n_calib), C.byref(n)))
    return fmt.value, kind.value, dim.value, bits.value, n_calib.value, n.value


def snapshot_compose(dim, bits, boundaries, centroids, seq, n, scales, calibration=None, ids=None, format=7):
    """Host-only: the snapshot image of an index given in the persisted layout."""
    kind = 0 if ids is None else 1
    b = np.ascontiguousarray(boundaries, np.float32)
    c = np.ascontiguousarray(centroids, np.float32)
    sh = sc = None
    n_calib = 0
    if calibration is not None:
        sh = np.ascontiguousarray(calibration[0], np.float32)
        sc = np.ascontiguousarray(calibration[1], np.float32)
        n_calib = len(sh)
    seq = np.ascontiguousarray(seq, np.uint8)
    scales = np.ascontiguousarray(scales, np.float32)
    if ids is not None:
        ids = np.ascontiguousarray(ids, np.uint64)
    out = np.zeros(lib().tv_host_snapshot_len(format, dim, bits, kind, n_calib, n), np.uint8)
    check(lib().tv_host_snapshot_compose(format, dim, bits, kind, ptr(b), ptr(c), n_calib,
                                         ptr(sh) if sh is not None else None, ptr(sc) if sc is not None else None,
                                         ptr(seq) if n else None, n, ptr(scales) if n else None,
                                         ptr(ids) if ids is not None and n else None, ptr(out)))
    return out.tobytes()


def snapshot_extract(data):
    """Host-only: (dict of arrays) unpacked from a snapshot image."""
    fmt, kind, dim, bits, n_calib, n = snapshot_info(data)
    buf = np.frombuffer(data, np.uint8)
    G = dim // (4 if bits == 2 else 2)
    nl = 1 << bits
    out = dict(format=fmt, kind=kind, dim=dim, bits=bits, n=n,
               boundaries=np.zeros(nl - 1, np.float32), centroids=np.zeros(nl, np.float32),
               shift=np.zeros(n_calib, np.float32), scale=np.zeros(n_calib, np.float32),
               seq=np.zeros(((n + 31) // 32) * G * 32, np.uint8), scales=np.zeros(((n + 31) // 32) * 32, np.float32),
               ids=np.zeros(((n + 31) // 32) * 32, np.uint64))
    check(lib().tv_host_snapshot_extract(ptr(buf), len(buf), ptr(out["boundaries"]), ptr(out["centroids"]),
                                         ptr(out["shift"]), ptr(out["scale"]), ptr(out["seq"]), ptr(out["scales"]),
                                         ptr(out["ids"])))
    out["scales"] = out["scales"][:n]
    out["ids"] = out["ids"][:n] if kind == 1 else None
    return out


def host_rotation_tables(dim):
    """The rotation tables the library derives for `dim` (no GPU needed)."""
    signs = np.zeros((2, dim), np.float32)
    perms = np.zeros((2, dim), np.uint32)
    block = C.c_int(0)
    inv = C.c_float(0)
    check(lib().tv_host_rotation_tables(dim, ptr(signs), ptr(perms), C.byref(block), C.byref(inv)))
    return signs, perms, block.value, np.float32(inv.value)


def host_codebook(bits, dim):
    """(boundaries, centroids) the library derives (no GPU needed)."""
    b = np.zeros((1 << bits) - 1, np.float32)
    c = np.zeros(1 << bits, np.float32)
    check(lib().tv_host_codebook(bits, dim, ptr(b), ptr(c)))
    return b, c
