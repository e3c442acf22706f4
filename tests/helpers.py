"""Shared builders for the parity tests: the oracle plays the part of the
reference crate (it encodes the seeded vectors and answers the search), the
HIP library answers the same search through its C ABI."""
import numpy as np


def unit_gaussian(n, dim, seed):
    """i.i.d. N(0,1) rows, L2-normalised in float32 (the benchmark configs' generator)."""
    rng = np.random.default_rng(seed)
    v = rng.standard_normal((n, dim), dtype=np.float32)
    v /= np.linalg.norm(v, axis=1, keepdims=True).astype(np.float32)
    return v


class OracleIndex:
    """Encoded index held on the host in the reference's persisted layout."""

    def __init__(self, O, dim, bits, vectors, calibration=None):
        self.O, self.dim, self.bits = O, dim, bits
        self.rot = O.Rotation(dim)
        self.calibration = calibration
        self.n = len(vectors)
        self.packed, self.scales = O.encode(self.rot, vectors, bits, calibration)
        self.seq = O.repack_seq(self.packed, self.n, bits, dim)

    def search(self, q, k, mask_words=None, mode=0, dump=False):
        return self.O.search(self.rot, self.seq, self.scales, q, k, self.bits, self.dim, self.n,
                             mask_words=mask_words, mode=mode, calibration=self.calibration, dump=dump)

    def rows(self):
        """Per-vector code bytes (n, G): what extract_codes_flat yields (pack.rs:306)."""
        G = self.O.n_byte_groups(self.bits, self.dim)
        nb = (self.n + 31) // 32
        return np.ascontiguousarray(
            self.seq.reshape(nb, G, 32).transpose(0, 2, 1).reshape(nb * 32, G)[: self.n])


def to_native(T, oidx, mode=None):
    ix = T.NativeIndex(oidx.dim, oidx.bits)
    if mode is not None:
        ix.set_score_mode(mode)
    if oidx.calibration is not None:
        ix.set_calibration(*oidx.calibration)
    ix.upload_seq(oidx.seq, oidx.n, oidx.scales)
    return ix


def bits_equal(a, b):
    a = np.ascontiguousarray(a, np.float32)
    b = np.ascontiguousarray(b, np.float32)
    return a.shape == b.shape and np.array_equal(a.view(np.uint32), b.view(np.uint32))


def ladder_for(T, dim, bits, n, nq, k):
    """(strides, repeat_offsets) of the sampling ladder the library runs for nq queries, k best, on an index of
    n rows of this shape (the ladder depends on nothing else): asked of a throw-away index of zero rows."""
    probe = T.NativeIndex(dim, bits)
    probe.append_rows(np.zeros((n, probe.n_byte_groups), np.uint8), np.zeros(n, np.float32))
    plan = probe.sampling_plan(nq, k)
    probe.close()
    return plan
