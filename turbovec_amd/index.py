"""Host-side mirror of the reference's index objects for the search path.

`TurboQuantIndex` and `IdMapIndex` keep the names, argument meaning, result
shapes and exception types of the reference's Python surface
(turbovec-python/src/lib.rs:601-690 search, :1129-1250 id-map search, :1000-1063
add_with_ids, :1063-1100 remove; turbovec/src/lib.rs:1345-1485
try_search_with_mask; turbovec/src/id_map.rs:664-712 try_search_with_allowlist,
:520-567 remove) and hand every piece of arithmetic to the HIP library through
its C ABI: encode on add, lane moves on swap_remove, and the whole search.  The
id <-> slot tables stay on the host, as in the reference.  There is no CPU
search here: without the built library every method raises ImportError.

Snapshots: `to_bytes` / `from_bytes` / `write` / `load` produce and read the
reference's image bytes (turbovec/src/io_v7.rs; lib.rs:2167 to_bytes, id_map.rs:971)
through tv_index_to_bytes / tv_index_from_bytes.

Pickling, `copy` and `deepcopy` go through `from_bytes(to_bytes())`, as the
reference's bindings reduce them (turbovec-python/src/lib.rs `__reduce__`).

Not mirrored (outside the search path): sync (the incremental container),
calibrate on a populated index (re-encoding stored rows).
"""
import os
import threading

import numpy as np

from . import _lib as T

_MAX_DIM = 16384            # turbovec/src/lib.rs:101
_MAX_INPUT_MAGNITUDE = 1e16  # turbovec/src/lib.rs:109


def _desc(obj):
    if isinstance(obj, np.ndarray):
        return f"{obj.ndim}-D {obj.dtype}"
    return type(obj).__name__


def _f32_2d(name, obj):
    """turbovec-python/src/lib.rs:56-62: no silent casts, the error names the argument."""
    if not isinstance(obj, np.ndarray) or obj.dtype != np.float32 or obj.ndim != 2 or not obj.dtype.isnative:
        raise TypeError(f"{name} must be a 2-D float32 array, got {_desc(obj)}")
    if not obj.flags.c_contiguous:
        raise ValueError(f"{name} must be C-contiguous; call np.ascontiguousarray(...) first")
    return obj


def _size(name, obj):
    """turbovec-python/src/lib.rs:153-175 extract_size."""
    if isinstance(obj, (bool, int, np.integer)) or hasattr(obj, "__index__"):
        v = int(obj)
        if v < 0:
            raise ValueError(f"{name} must be a non-negative integer, got {v}")
        if v >= 1 << 64:
            raise ValueError(f"{name} must fit in an unsigned 64-bit integer, got {v}")
        return v
    raise TypeError(f"{name} must be an integer, got {type(obj).__name__}")


def _check_values(name, arr, what):
    """turbovec/src/lib.rs:1363-1380, encode.rs:76-83: every value finite and |x| < 1e16."""
    ok = np.abs(arr) < _MAX_INPUT_MAGNITUDE          # NaN compares false
    if not ok.all():
        r, c = np.argwhere(~ok)[0]
        raise ValueError(f"{what} {r} has a non-finite or out-of-range value at coordinate {c} "
                         f"(must be finite with magnitude < 1e16)")


class TurboQuantIndex:
    """Slot-addressed index; `search` returns (scores float32, slots int64), shape (nq, k_eff)."""

    def __init__(self, dim, bit_width=4, device=0):
        dim = _size("dim", dim)
        bit_width = _size("bit_width", bit_width)
        if bit_width not in (2, 3, 4):
            raise ValueError(f"bit_width must be 2, 3, or 4, got {bit_width}")
        if dim == 0 or dim % 8 != 0:
            raise ValueError(f"dim must be a positive multiple of 8, got {dim}")
        if dim > _MAX_DIM:
            raise ValueError(f"dim {dim} exceeds maximum {_MAX_DIM}")
        self._ix = T.NativeIndex(dim, bit_width, device)
        self._lock = threading.RLock()       # mutators exclude each other and searches (the reference's RwLock)

    # -- shape -----------------------------------------------------------
    @property
    def dim(self):
        return self._ix.dim

    @property
    def bit_width(self):
        return self._ix.bits

    def __len__(self):
        return len(self._ix)

    def prepare(self):
        """Idempotent; the device copy of the index is always search-ready."""
        return None

    def calibrate(self, sample):
        """Fit the TQ+ pair from `sample` and commit it (lib.rs:2599); before the first add only."""
        v = _f32_2d("sample", sample)
        if v.shape[1] != self.dim:
            raise ValueError(f"sample dim {v.shape[1]} does not match index dim {self.dim}")
        if len(v) < 2:
            raise ValueError("calibration needs at least 2 rows")
        _check_values("sample", v, "sample row")
        with self._lock:
            if len(self._ix):
                raise NotImplementedError("calibrate on a populated index (re-encoding stored rows) is not built")
            self._ix.calibrate(v)

    @property
    def calibration_state(self):
        return "uncalibrated" if self._ix.calibration() is None else "calibrated"

    def set_calibration(self, shift, scale):
        """Hand over a fitted TQ+ pair (turbovec/src/lib.rs:2599); affects later adds and searches."""
        with self._lock:
            self._ix.set_calibration(shift, scale)

    # -- snapshots ---------------------------------------------------------
    def to_bytes(self):
        with self._lock:
            return self._ix.to_bytes()

    @classmethod
    def from_bytes(cls, data, device=0):
        return cls._adopt(*_load_image(data, device, want_kind=0))

    def __reduce__(self):
        """pickle, copy.copy and copy.deepcopy rebuild through from_bytes(to_bytes()), as the
        reference's bindings do (turbovec-python/src/lib.rs:268-287, 828-833): the copy is a
        separate index with its own device memory."""
        return (type(self).from_bytes, (self.to_bytes(),))

    @classmethod
    def _adopt(cls, native, _ids):
        self = cls.__new__(cls)
        self._ix = native
        self._lock = threading.RLock()
        return self

    def write(self, path):
        _write_atomically(path, self.to_bytes())

    @classmethod
    def load(cls, path, device=0):
        with open(path, "rb") as f:
            return cls.from_bytes(f.read(), device)

    # -- mutation ----------------------------------------------------------
    def add(self, vectors):
        v = _f32_2d("vectors", vectors)
        if v.shape[1] != self.dim:
            raise ValueError(f"vector dim {v.shape[1]} does not match index dim {self.dim}")
        if len(v) == 0:
            return
        _check_values("vectors", v, "vector")
        with self._lock:
            self._ix.add(v)

    def swap_remove(self, idx):
        """Move the last vector into slot idx; returns the slot it came from (lib.rs:2864-3028)."""
        try:
            i = int(idx)
        except (TypeError, ValueError):
            raise TypeError(f"idx must be an integer, got {type(idx).__name__}")
        with self._lock:
            n = len(self._ix)
            if i < 0 or i >= n:
                raise IndexError(f"swap_remove index {i} out of range for index of size {n}")
            self._ix.swap_remove(i)
            return n - 1

    # -- search ------------------------------------------------------------
    def search(self, queries, k, *, mask=None):
        q = _f32_2d("queries", queries)
        k = _size("k", k)
        m = None
        if mask is not None:
            if not isinstance(mask, np.ndarray) or mask.dtype != np.bool_ or mask.ndim != 1:
                raise TypeError(f"mask must be a 1-D bool array, got {_desc(mask)}")
            if not mask.flags.c_contiguous:
                raise ValueError("mask must be C-contiguous; call np.ascontiguousarray(...) first")
            # read as raw bytes: every non-zero byte is true (turbovec-python/src/lib.rs:87-130)
            m = np.frombuffer(np.ndarray.tobytes(mask), np.uint8)
        if q.shape[1] != self.dim:
            raise ValueError(f"query dim {q.shape[1]} does not match index dim {self.dim}")
        q = q.copy()                                    # snapshot, as the binding does (:617-629)
        _check_values("queries", q, "query")
        with self._lock:
            n = len(self._ix)
            if m is not None and len(m) != n:
                raise ValueError(f"mask length {len(m)} does not match index size {n}")
            return self._search_locked(q, k, m)

    def _search_locked(self, q, k, mask_bytes):
        n = len(self._ix)
        words, n_allowed = (None, n)
        if mask_bytes is not None:
            words, n_allowed = T.pack_mask(mask_bytes)
        k_eff = min(k, n, n_allowed)
        if len(q) == 0 or k_eff == 0:
            return np.zeros((len(q), k_eff), np.float32), np.zeros((len(q), k_eff), np.int64)
        k_lib = min(k, n)                               # the library clamps again; keep the argument small
        return self._ix.search(q, k_lib, mask_words=words)


def _load_image(data, device, want_kind):
    """Corrupt or foreign bytes surface as a plain OSError, as the reference's loaders do."""
    try:
        info = T.snapshot_info(data)
        if info[1] != want_kind:
            raise OSError("image holds %s index" % ("an id-map" if info[1] == 1 else "a slot-addressed"))
        return T.NativeIndex.from_bytes(data, device)
    except T.TurbovecHipError as e:
        raise OSError(str(e)) from None


def _write_atomically(path, data):
    """Temp sibling + rename: the destination never holds a torn image."""
    path = os.fspath(path)
    d = os.path.dirname(path) or "."
    if not os.path.isdir(d):
        raise FileNotFoundError(f"cannot write {path!r}: directory {d!r} does not exist")
    tmp = f"{path}.tmp.{os.getpid()}"
    with open(tmp, "wb") as f:
        f.write(data)
        f.flush()
        os.fsync(f.fileno())
    os.replace(tmp, path)


class IdMapIndex:
    """Index addressed by external uint64 ids; `search` returns (scores, ids uint64)."""

    def __init__(self, dim, bit_width=4, device=0):
        self._inner = TurboQuantIndex(dim, bit_width, device)
        self._slot_to_id = []            # id_map.rs:181: slot -> external id
        self._id_to_slot = {}

    @property
    def dim(self):
        return self._inner.dim

    @property
    def bit_width(self):
        return self._inner.bit_width

    def __len__(self):
        return len(self._slot_to_id)

    def prepare(self):
        return None

    def to_bytes(self):
        with self._inner._lock:
            return self._inner._ix.to_bytes(ids=np.asarray(self._slot_to_id, np.uint64))

    @classmethod
    def from_bytes(cls, data, device=0):
        native, ids = _load_image(data, device, want_kind=1)
        self = cls.__new__(cls)
        self._inner = TurboQuantIndex._adopt(native, None)
        self._slot_to_id = ids.tolist()
        self._id_to_slot = {x: i for i, x in enumerate(self._slot_to_id)}
        if len(self._id_to_slot) != len(self._slot_to_id):
            raise OSError("image holds duplicate ids")
        return self

    def __reduce__(self):
        """See TurboQuantIndex.__reduce__ (turbovec-python/src/lib.rs:1462-1468)."""
        return (type(self).from_bytes, (self.to_bytes(),))

    def write(self, path):
        _write_atomically(path, self.to_bytes())

    @classmethod
    def load(cls, path, device=0):
        with open(path, "rb") as f:
            return cls.from_bytes(f.read(), device)

    def contains(self, id):
        try:
            v = int(id)
        except (TypeError, ValueError):
            raise TypeError(f"id must be an integer, got {type(id).__name__}")
        return 0 <= v < (1 << 64) and v in self._id_to_slot

    __contains__ = contains

    def add_with_ids(self, vectors, ids):
        v = _f32_2d("vectors", vectors)
        if not isinstance(ids, np.ndarray) or ids.dtype != np.uint64 or ids.ndim != 1:
            raise TypeError(f"ids must be a 1-D uint64 array, got {_desc(ids)}")
        if v.shape[1] != self.dim:
            raise ValueError(f"vector dim {v.shape[1]} does not match index dim {self.dim}")
        if len(ids) != len(v):
            raise ValueError(f"ids count mismatch: expected {len(v)}, got {len(ids)}")
        # validate every id before anything is added (id_map.rs:396-460)
        seen = set()
        for x in ids.tolist():
            if x in self._id_to_slot:
                raise ValueError(f"id {x} is already present in the index")
            if x in seen:
                raise ValueError(f"id {x} appears more than once in this batch")
            seen.add(x)
        if len(v) == 0:
            return
        with self._inner._lock:
            self._inner.add(v)
            base = len(self._slot_to_id)
            for off, x in enumerate(ids.tolist()):
                self._id_to_slot[x] = base + off
                self._slot_to_id.append(x)

    def remove(self, id):
        """id_map.rs:520-567: inner swap_remove first, then the tables."""
        try:
            v = int(id)
        except (TypeError, ValueError):
            raise TypeError(f"id must be an integer, got {type(id).__name__}")
        with self._inner._lock:
            slot = self._id_to_slot.get(v) if 0 <= v < (1 << 64) else None
            if slot is None:
                return False
            last = len(self._slot_to_id) - 1
            self._inner.swap_remove(slot)
            del self._id_to_slot[v]
            if slot != last:
                moved = self._slot_to_id[last]
                self._slot_to_id[slot] = moved
                self._id_to_slot[moved] = slot
            self._slot_to_id.pop()
            return True

    def search(self, queries, k, *, allowlist=None):
        q = _f32_2d("queries", queries)
        k = _size("k", k)
        allow = None
        if allowlist is not None:
            if not isinstance(allowlist, np.ndarray) or allowlist.dtype != np.uint64 or allowlist.ndim != 1:
                raise TypeError(f"allowlist must be a 1-D uint64 array, got {_desc(allowlist)}")
            allow = allowlist.tolist()
            if len(allow) == 0:
                raise ValueError("allowlist is empty")          # SearchError::AllowlistEmpty
        if q.shape[1] != self.dim:
            raise ValueError(f"query dim {q.shape[1]} does not match index dim {self.dim}")
        q = q.copy()
        _check_values("queries", q, "query")
        with self._inner._lock:
            mask_bytes = None
            if allow is not None:
                unknown = []
                for x in allow:
                    if x not in self._id_to_slot:
                        unknown.append(x)
                        if len(unknown) > 5:
                            break
                if unknown:
                    raise KeyError(f"allowlist contains id(s) not present in index: {unknown[:5]}"
                                   f"{', ...' if len(unknown) > 5 else ''}")
                mask_bytes = np.zeros(len(self._slot_to_id), np.uint8)      # duplicates collapse here
                mask_bytes[[self._id_to_slot[x] for x in allow]] = 1
            scores, slots = self._inner._search_locked(q, k, mask_bytes)
            table = np.asarray(self._slot_to_id, np.uint64)
            ids = table[slots] if slots.size else np.zeros(slots.shape, np.uint64)
            return scores, ids
