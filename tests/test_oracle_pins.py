"""Pins the oracle functions for which the reference holds no golden vector.

The reference has no known answer written by its int8 permute-dot kernel, by the
u32 / scalar LUT epilogues, by `calibrate_queries`, or for the (128, 4) codebook
cell.  What those functions must return is nevertheless fixed by mathematics:
each test below evaluates an independent model -- exact rational arithmetic
rounded once per IEEE operation, a closed-form conditional mean instead of a
quadrature, numpy float32 element operations -- and demands bit equality with
the oracle.  Every test also shows that its inputs separate the intended
definition from the plausible wrong ones (round-half-even for half-away, the
two nibble weights swapped, multiply-then-add for a fused multiply-add, a float32
or exactly summed bias correction, the opposite sign): the model evaluated the
wrong way must disagree with the oracle on the same inputs.
"""
import math
from fractions import Fraction

import numpy as np
import pytest

from golden_data import CODEBOOK, FINGERPRINT


# --------------------------------------------------------------------------
# IEEE-754 rounding of an exact rational, written out (round to nearest, ties
# to even; gradual underflow), so that no float arithmetic of the platform is
# trusted by the models below.
# --------------------------------------------------------------------------
def _round_ieee(x, precision, emin):
    if x == 0:
        return Fraction(0)
    sign = -1 if x < 0 else 1
    ax = abs(x)
    e = ax.numerator.bit_length() - ax.denominator.bit_length()
    if Fraction(2) ** e > ax:
        e -= 1
    elif Fraction(2) ** (e + 1) <= ax:
        e += 1
    assert Fraction(2) ** e <= ax < Fraction(2) ** (e + 1)
    e = max(e, emin)
    ulp = Fraction(2) ** (e - precision + 1)
    qn = ax / ulp
    n = qn.numerator // qn.denominator
    r = qn - n
    if r > Fraction(1, 2) or (r == Fraction(1, 2) and (n & 1)):
        n += 1
    return sign * n * ulp


def r32(x):
    return _round_ieee(Fraction(x), 24, -126)


def r64(x):
    return _round_ieee(Fraction(x), 53, -1022)


def F(x):
    """Exact value of a float32 / float64 / int."""
    return Fraction(int(x)) if isinstance(x, (int, np.integer)) else Fraction(float(x))


def test_rounding_helper_against_known_cases():
    # ties to even at the 24-bit boundary, subnormals, and agreement with numpy's casts
    assert r32(Fraction(2 ** 24 + 1)) == 2 ** 24
    assert r32(Fraction(2 ** 24 + 3)) == 2 ** 24 + 4
    assert r32(Fraction(1, 2 ** 150)) == 0
    assert r32(Fraction(3, 2 ** 150)) == Fraction(2, 2 ** 149)
    rng = np.random.default_rng(0)
    for v in rng.standard_normal(200) * 10.0 ** rng.integers(-30, 30, 200):
        assert float(r32(F(v))) == float(np.float32(v))
    for a, b in rng.standard_normal((200, 2)):
        assert float(r64(F(a) + F(b))) == float(np.float64(a) + np.float64(b))
        assert float(r64(F(a) * F(b))) == float(np.float64(a) * np.float64(b))


def round_half_away(t):
    """f32::round of float32 values, exactly (the float64 sum |t| + 0.5 is exact)."""
    t64 = np.asarray(t, np.float32).astype(np.float64)
    return np.copysign(np.floor(np.abs(t64) + 0.5), t64)


# --------------------------------------------------------------------------
# (a) build_permute_dot -- turbovec/src/search.rs:2806-2846
# --------------------------------------------------------------------------
def model_permute_dot(q, cen, rounding="away", swap=False):
    q = np.asarray(q, np.float32)
    cen = np.asarray(cen, np.float32)
    one, c127 = np.float32(1.0), np.float32(127.0)
    rnd = round_half_away if rounding == "away" else (lambda t: np.rint(np.asarray(t, np.float32).astype(np.float64)))
    cmax = np.float32(np.abs(cen).max())
    cs = np.float32(cmax / c127) if cmax > 0 else one
    levels = np.clip(rnd(cen / cs), -127, 127).astype(np.int8)
    qmax = np.float32(np.abs(q).max())
    qs = np.float32(qmax / c127)
    if qs >= np.finfo(np.float32).tiny:
        inv = np.float32(one / qs)
    else:
        qs, inv = one, one
    w = np.clip(rnd(q * inv), -127, 127).astype(np.int8)
    hi, lo = w[0::2], w[1::2]            # even dimension -> high nibble, odd -> low
    if swap:
        hi, lo = lo, hi
    weights = np.concatenate([lo.reshape(-1, 4), hi.reshape(-1, 4)], axis=1).ravel()
    zero = -128 * int(w.astype(np.int64).sum())
    return levels, weights, zero, np.float32(cs * qs)


def _same_tables(a, b):
    return (np.array_equal(a[0], b[0]) and np.array_equal(a[1], b[1]) and a[2] == b[2]
            and np.float32(a[3]).view(np.uint32) == np.float32(b[3]).view(np.uint32))


@pytest.mark.parametrize("dim", [128, 1536, 3072])
def test_permute_dot_matches_independent_model(oracle, dim):
    O = oracle
    _, cen = O.codebook(4, dim)
    rng = np.random.default_rng(dim)
    rot = O.Rotation(dim)
    for i in range(120):
        q = rng.standard_normal(dim).astype(np.float32)
        if i % 3 == 0:
            q = rot.apply(q / np.linalg.norm(q))            # what the search feeds the builder
        elif i % 3 == 1:
            q *= np.float32(2.0 ** int(rng.integers(-60, 40)))
        got = O.build_permute_dot(q, cen, dim)
        assert _same_tables(got, model_permute_dot(q, cen)), i
    # a query too small for 1/qs: unit scales, all-zero weights (search.rs:2826-2827)
    tiny = np.full(dim, 1e-38, np.float32)
    got = O.build_permute_dot(tiny, cen, dim)
    assert _same_tables(got, model_permute_dot(tiny, cen))
    assert not got[1].any() and got[3] == model_permute_dot(tiny, cen)[3]
    zero_q = np.zeros(dim, np.float32)
    assert _same_tables(O.build_permute_dot(zero_q, cen, dim), model_permute_dot(zero_q, cen))


def test_permute_dot_half_way_cases_round_away_and_clamp(oracle):
    O = oracle
    dim = 64
    _, cen = O.codebook(4, dim)
    # |q|max = 127 makes qs = inv_qs = 1 exactly, so q itself is what gets rounded
    q = np.zeros(dim, np.float32)
    q[0] = 127.0
    q[1] = -127.0
    halves = [0.5, -0.5, 1.5, -1.5, 2.5, -2.5, 63.5, -64.5, 126.5, -126.5, 0.49999997, -0.49999997]
    q[2:2 + len(halves)] = halves
    levels, w, zero, scale = O.build_permute_dot(q, cen, dim)
    by_dim = np.zeros(dim, np.int64)
    for g in range(dim // 2):
        by_dim[2 * g + 1] = w[(g // 4) * 8 + g % 4]
        by_dim[2 * g] = w[(g // 4) * 8 + 4 + g % 4]
    assert by_dim[:2].tolist() == [127, -127]
    assert by_dim[2:2 + len(halves)].tolist() == [1, -1, 2, -2, 3, -3, 64, -65, 127, -127, 0, 0]
    assert _same_tables((levels, w, zero, scale), model_permute_dot(q, cen))
    # the same inputs tell the wrong definitions apart
    assert not _same_tables((levels, w, zero, scale), model_permute_dot(q, cen, rounding="even"))
    assert not _same_tables((levels, w, zero, scale), model_permute_dot(q, cen, swap=True))


# --------------------------------------------------------------------------
# (c) calibrate_queries -- turbovec/src/search.rs:3154-3186
# --------------------------------------------------------------------------
def model_bias_corr(q_rot, shift, how="f64_sequential", sign=-1):
    if how == "f64_sequential":         # bc -= f64(q) * f64(shift): the product is exact in f64
        bc = Fraction(0)
        for a, b in zip(q_rot, shift):
            bc = r64(bc + sign * r64(F(a) * F(b)))
        return r32(bc)
    if how == "f32_sequential":
        bc = Fraction(0)
        for a, b in zip(q_rot, shift):
            bc = r32(bc + sign * r32(F(a) * F(b)))
        return bc
    if how == "exact":
        return r32(sum((sign * F(a) * F(b) for a, b in zip(q_rot, shift)), Fraction(0)))
    if how == "reversed":
        bc = Fraction(0)
        for a, b in zip(q_rot[::-1], shift[::-1]):
            bc = r64(bc + sign * r64(F(a) * F(b)))
        return r32(bc)
    raise ValueError(how)


def _calibrate(O, q_rot, shift, scale):
    import ctypes as C
    q_rot, shift, scale = (np.ascontiguousarray(a, np.float32) for a in (q_rot, shift, scale))
    out = np.zeros_like(q_rot)
    bc = C.c_float()
    O.lib().tvo_calibrate_query(q_rot.ctypes.data, shift.ctypes.data, scale.ctypes.data, len(q_rot),
                                out.ctypes.data, C.addressof(bc))
    return out, np.float32(bc.value)


def test_calibrate_query_matches_exact_model(oracle):
    O = oracle
    rng = np.random.default_rng(21)
    for dim in (8, 64, 1536):
        for _ in range(6):
            q = rng.standard_normal(dim).astype(np.float32)
            shift = (rng.standard_normal(dim) * 0.05).astype(np.float32)
            scale = rng.uniform(0.7, 1.4, dim).astype(np.float32)
            q_cal, bc = _calibrate(O, q, shift, scale)
            assert np.array_equal(q_cal.view(np.uint32), (q / scale).view(np.uint32))
            assert F(bc) == model_bias_corr(q, shift)
    # no pair: copy and +0.0 (search.rs:3161-3164)
    import ctypes as C
    q = rng.standard_normal(16).astype(np.float32)
    out = np.zeros_like(q)
    bc = C.c_float(7.0)
    O.lib().tvo_calibrate_query(q.ctypes.data, None, None, 16, out.ctypes.data, C.addressof(bc))
    assert np.array_equal(out, q) and bc.value == 0.0


def test_calibrate_query_inputs_separate_the_wrong_sums(oracle):
    O = oracle
    # products 2^60, 1, -2^60, 1, 2^-30, -1, 3 * 2^-30: the sequential f64 sum loses the first 1
    # next to 2^60 and keeps 2^-30 next to the second, ending at -2^-28; a float32 accumulator
    # loses the 2^-30 as well, the exact sum keeps everything and rounds to -1, the reversed
    # order ends at 0
    q = np.array([2.0 ** 30, 1.0, -(2.0 ** 30), 1.0, 1.0, -1.0, 3.0, 0.0], np.float32)
    shift = np.array([2.0 ** 30, 1.0, 2.0 ** 30, 1.0, 2.0 ** -30, 1.0, 2.0 ** -30, 5.0], np.float32)
    scale = np.ones(8, np.float32)
    _, bc = _calibrate(O, q, shift, scale)
    want = model_bias_corr(q, shift)
    assert F(bc) == want == -Fraction(1, 2 ** 28)
    for how in ("f32_sequential", "exact", "reversed"):
        assert model_bias_corr(q, shift, how) != want, how
    assert model_bias_corr(q, shift, sign=+1) != want


# --------------------------------------------------------------------------
# (b) float epilogues of the scan -- search.rs:1519-1524 (P: fused), :1174-1177
#     (L-u32: multiply, add), :3113-3128 (L-scalar), :516-582 (L-classic)
# --------------------------------------------------------------------------
def _seq_bytes(seq, n, G):
    nb = (n + 31) // 32
    return seq.reshape(nb, G, 32).transpose(0, 2, 1).reshape(nb * 32, G)[:n].astype(np.int64)


def epilogue_p(acc, scale, bias, vs, fused=True):
    a = r32(F(acc))                                   # cvtepi32_ps rounds to nearest even
    t = r32(a * F(scale) + F(bias)) if fused else r32(r32(a * F(scale)) + F(bias))
    return r32(t * F(vs))


def epilogue_u32(acc, scale, bias, vs, fused=False):
    a = r32(F(acc))
    t = r32(a * F(scale) + F(bias)) if fused else r32(r32(a * F(scale)) + F(bias))
    return r32(t * F(vs))


def _calibrated_case(O, dim, bits, n, seed):
    rng = np.random.default_rng(seed)
    v = rng.standard_normal((n, dim)).astype(np.float32)
    v /= np.linalg.norm(v, axis=1, keepdims=True)
    rot = O.Rotation(dim)
    _, cen = O.codebook(bits, dim)
    cal = O.fit_calibration(rot, v, cen)
    packed, scales = O.encode(rot, v, bits, cal)
    seq = O.repack_seq(packed, n, bits, dim)
    return rng, v, rot, cen, cal, seq, scales


def test_mode_p_scores_match_exact_model_on_calibrated_index(oracle):
    O = oracle
    dim, bits, n = 1536, 4, 64
    rng, v, rot, cen, cal, seq, scales = _calibrated_case(O, dim, bits, n, 31)
    seq = seq.copy()
    G = dim // 2
    q = rng.standard_normal((4, dim)).astype(np.float32)
    q /= np.linalg.norm(q, axis=1, keepdims=True)
    # rows 0 and 1 are crafted against query 0: every nibble takes the outermost level on the
    # side of its weight's sign (row 0) or against it (row 1), the largest sums this query has
    qr0 = rot.apply(q[0])
    qc0 = qr0 / cal[1]
    _, w0, _, _ = model_permute_dot(qc0, cen)
    sgn = np.zeros(dim, np.int64)
    for g in range(G):
        sgn[2 * g + 1] = w0[(g // 4) * 8 + g % 4]
        sgn[2 * g] = w0[(g // 4) * 8 + 4 + g % 4]
    hi_nib = np.where(sgn[0::2] >= 0, 15, 0)
    lo_nib = np.where(sgn[1::2] >= 0, 15, 0)
    row = (hi_nib << 4 | lo_nib).astype(np.uint8)
    for g in range(G):
        seq[g * 32 + 0] = row[g]
        seq[g * 32 + 1] = row[g] ^ 0xFF
    s, idx, acc, raw = O.search(rot, seq, scales, q, n, bits, dim, n, mode=O.MODE_P, calibration=cal, dump=True)
    by = _seq_bytes(seq, n, G)
    codes = np.zeros((n, dim), np.int64)
    codes[:, 0::2] = by >> 4
    codes[:, 1::2] = by & 15
    differs_unfused = 0
    for qi in range(len(q)):
        qr = rot.apply(q[qi])
        q_cal = (qr / cal[1]).astype(np.float32)
        bias = model_bias_corr(qr, cal[0])               # 0.0 + bias_corr
        levels, w, zero, scale = model_permute_dot(q_cal, cen)
        wd = np.zeros(dim, np.int64)
        for g in range(G):
            wd[2 * g + 1] = w[(g // 4) * 8 + g % 4]
            wd[2 * g] = w[(g // 4) * 8 + 4 + g % 4]
        want_acc = (levels.astype(np.int64)[codes] * wd[None, :]).sum(axis=1)
        assert np.array_equal(acc[qi], want_acc)
        assert bias != 0
        for j in range(n):
            want = epilogue_p(int(want_acc[j]), scale, bias, scales[j])
            assert F(raw[qi, j]) == want, (qi, j)
            differs_unfused += epilogue_p(int(want_acc[j]), scale, bias, scales[j], fused=False) != want
        order = sorted(range(n), key=lambda j: (-float(raw[qi, j]), j))
        assert idx[qi].tolist() == order
    assert differs_unfused > 0          # these inputs tell fma from multiply-then-add


def test_mode_p_accumulators_beyond_2_pow_24_round_to_even(oracle):
    O = oracle
    dim, bits, n = 1536, 4, 32
    rot = O.Rotation(dim)
    _, cen = O.codebook(bits, dim)
    G = dim // 2
    # every weight must be +-127 for the sums to pass 2^24: the calibration pair shapes what the
    # builder sees -- q_cal = q_rot / scale_tq with scale_tq = |q_rot| is +-1 exactly
    rng = np.random.default_rng(5)
    q = rng.standard_normal((1, dim)).astype(np.float32)
    qr = rot.apply(q[0])
    assert np.all(qr != 0)
    tq_scale = np.abs(qr).astype(np.float32)
    tq_shift = (rng.standard_normal(dim) * 0.01).astype(np.float32)
    q_cal = (qr / tq_scale).astype(np.float32)
    assert set(np.abs(q_cal).tolist()) == {1.0}
    levels, w, zero, scale = model_permute_dot(q_cal, cen)
    assert set(np.abs(w).tolist()) == {127}
    sgn = np.zeros(dim, np.int64)
    for g in range(G):
        sgn[2 * g + 1] = w[(g // 4) * 8 + g % 4]
        sgn[2 * g] = w[(g // 4) * 8 + 4 + g % 4]
    seq = np.zeros(G * 32, np.uint8)
    codes = np.zeros((n, dim), np.int64)
    for lane in range(n):
        # lane 0: all outermost levels with the weights; later lanes flip a growing share of
        # dimensions to inner levels so the sums sweep a range of odd and even values > 2^24
        c = np.where(sgn >= 0, 15, 0)
        flip = rng.random(dim) < lane * 0.004
        c = np.where(flip, np.where(sgn >= 0, 15 - rng.integers(1, 3, dim), rng.integers(1, 3, dim)), c)
        if lane % 2:
            c = 15 - c                                   # and the negative side
        codes[lane] = c
        seq[np.arange(G) * 32 + lane] = (c[0::2] << 4 | c[1::2]).astype(np.uint8)
    scales = rng.uniform(0.5, 1.5, n).astype(np.float32)
    s, idx, acc, raw = O.search(rot, seq, scales, q, n, bits, dim, n, mode=O.MODE_P,
                                calibration=(tq_shift, tq_scale), dump=True)
    want_acc = (levels.astype(np.int64)[codes] * sgn[None, :]).sum(axis=1)
    assert np.array_equal(acc[0], want_acc)
    assert (np.abs(want_acc) > 2 ** 24).sum() >= 16 and (want_acc % 2 != 0).any()
    bias = model_bias_corr(qr, tq_shift)
    inexact = 0
    for j in range(n):
        assert F(raw[0, j]) == epilogue_p(int(want_acc[j]), scale, bias, scales[j]), j
        inexact += r32(F(int(want_acc[j]))) != int(want_acc[j])
    assert inexact > 0                  # some of the integers really are rounded by the conversion


@pytest.mark.parametrize("bits", [2, 3, 4])
def test_l_u32_scores_match_exact_model_on_calibrated_index(oracle, bits):
    O = oracle
    dim, n = 256, 96
    rng, v, rot, cen, cal, seq, scales = _calibrated_case(O, dim, bits, n, 40 + bits)
    G = O.n_byte_groups(bits, dim)
    q = rng.standard_normal((3, dim)).astype(np.float32)
    s, idx, acc, raw = O.search(rot, seq, scales, q, n, bits, dim, n, mode=O.MODE_L_U32, calibration=cal, dump=True)
    by = _seq_bytes(seq, n, G)
    differs_fused = 0
    for qi in range(len(q)):
        qr = rot.apply(q[qi])
        q_cal = (qr / cal[1]).astype(np.float32)
        lut, scale, lbias = model_lut(q_cal, cen, bits)
        bias = r32(F(lbias) + model_bias_corr(qr, cal[0]))       # lut.bias += bias_corr (search.rs:3261)
        want_acc = np.zeros(n, np.int64)
        for g in range(G):
            want_acc += lut[g, 0, by[:, g] >> 4] + lut[g, 1, by[:, g] & 15]
        assert np.array_equal(acc[qi], want_acc)
        for j in range(n):
            want = epilogue_u32(int(want_acc[j]), scale, bias, scales[j])
            assert F(raw[qi, j]) == want, (qi, j)
            differs_fused += epilogue_u32(int(want_acc[j]), scale, bias, scales[j], fused=True) != want
    assert differs_fused > 0            # these inputs tell multiply-then-add from fma


def test_l_scalar_and_l_classic_scores_match_exact_model(oracle):
    O = oracle
    dim, bits, n = 1024, 4, 40      # 512 byte-groups: two flush periods of the classic epilogue
    rng, v, rot, cen, cal, seq, scales = _calibrated_case(O, dim, bits, n, 50)
    G = dim // 2
    q = rng.standard_normal((2, dim)).astype(np.float32)
    by = _seq_bytes(seq, n, G)
    out = {m: O.search(rot, seq, scales, q, n, bits, dim, n, mode=m, calibration=cal, dump=True)
           for m in (O.MODE_L_SCALAR, O.MODE_L_CLASSIC)}
    for qi in range(len(q)):
        qr = rot.apply(q[qi])
        q_cal = (qr / cal[1]).astype(np.float32)
        lut, scale, lbias = model_lut(q_cal, cen, bits)
        bias = r32(F(lbias) + model_bias_corr(qr, cal[0]))
        fs = F(scale)
        for j in range(n):
            hi = lut[np.arange(G), 0, by[j] >> 4]
            lo = lut[np.arange(G), 1, by[j] & 15]
            # scalar (search.rs:3113-3128): two separate multiply-adds per group, in group order
            sc = bias
            for g in range(G):
                sc = r32(sc + r32(fs * int(hi[g])))
                sc = r32(sc + r32(fs * int(lo[g])))
            assert F(out[O.MODE_L_SCALAR][3][qi, j]) == r32(sc * F(scales[j])), (qi, j)
            # classic (search.rs:516-582): fa = fma(scale, f32(sum of 256 groups), fa)
            fa = bias
            for g0 in range(0, G, 256):
                part = int(hi[g0:g0 + 256].sum() + lo[g0:g0 + 256].sum())
                fa = r32(fs * part + fa)
            assert F(out[O.MODE_L_CLASSIC][3][qi, j]) == r32(fa * F(scales[j])), (qi, j)


# --------------------------------------------------------------------------
# Mode-L table build for every bit width -- search.rs:2856-2994
# --------------------------------------------------------------------------
def model_lut(q, cen, bits):
    """(lut[G][2][16] int64, scale f32, bias f32) from numpy float32 element operations."""
    q = np.asarray(q, np.float32)
    cen = np.asarray(cen, np.float32)
    cpb = 8 // bits
    cpn = cpb // 2
    G = len(q) // cpb
    vals = np.zeros((G, 2, 16), np.float32)
    for sub in range(2):
        for nv in range(16):
            s = np.zeros(G, np.float32)
            for c in range(cpn):
                code = (nv >> ((cpn - 1 - c) * bits)) & ((1 << bits) - 1)
                s = (s + q[sub * cpn + c::cpb][:G] * cen[code]).astype(np.float32)
            vals[:, sub, nv] = s
    mins = vals.min(axis=2)
    span = np.float32((vals.max(axis=2) - mins).max())
    scale = np.float32(span / np.float32(127)) if span > 0 else np.float32(1)
    if scale >= np.finfo(np.float32).tiny:
        inv = np.float32(np.float32(1) / scale)
    else:
        scale = inv = np.float32(1)
    lut = np.clip(round_half_away((vals - mins[:, :, None]) * inv), 0, 127).astype(np.int64)
    bias = np.float32(0)
    for g in range(G):
        bias = np.float32(bias + np.float32(mins[g, 0] + mins[g, 1]))
    return lut, scale, bias


@pytest.mark.parametrize("bits,dim", [(2, 128), (3, 128), (4, 128), (2, 1536), (3, 1024), (4, 3072)])
def test_lut_matches_independent_model_every_bit_width(oracle, bits, dim):
    O = oracle
    _, cen = O.codebook(bits, dim)
    rng = np.random.default_rng(100 * bits + dim)
    G = O.n_byte_groups(bits, dim)
    for i in range(8):
        q = rng.standard_normal(dim).astype(np.float32)
        if i % 2:
            q = O.Rotation(dim).apply(q / np.linalg.norm(q))
        lut, scale, bias = O.build_lut(q, cen, bits, dim)
        mlut, mscale, mbias = model_lut(q, cen, bits)
        assert np.array_equal(lut.reshape(G, 2, 16), mlut)
        assert scale.view(np.uint32) == mscale.view(np.uint32) and bias.view(np.uint32) == mbias.view(np.uint32)


# --------------------------------------------------------------------------
# Scores approximate the true inner product (kernel_tests.rs:401-419 asks the mean
# self-score to sit within 0.005 of 1): a dropped or mis-signed bias correction, a
# wrong scale or transposed weights fail this without any reference-held vector.
# --------------------------------------------------------------------------
@pytest.mark.parametrize("bits,mode_name,tol", [(4, "P", 0.005), (4, "L_U32", 0.005), (2, "L_U32", 0.005),
                                                (4, "L_CLASSIC", 0.005), (3, "L_U32", 0.005)])
def test_scores_estimate_inner_products(oracle, bits, mode_name, tol):
    O = oracle
    dim, n = 1536, 500
    mode = getattr(O, "MODE_" + mode_name)
    for calibrated in (False, True):
        rng = np.random.default_rng(7)
        v = rng.standard_normal((n, dim)).astype(np.float32)
        v /= np.linalg.norm(v, axis=1, keepdims=True)
        rot = O.Rotation(dim)
        _, cen = O.codebook(bits, dim)
        cal = O.fit_calibration(rot, v, cen) if calibrated else None
        packed, scales = O.encode(rot, v, bits, cal)
        seq = O.repack_seq(packed, n, bits, dim)
        q = v[:40]
        s, idx, acc, raw = O.search(rot, seq, scales, q, 1, bits, dim, n, mode=mode, calibration=cal, dump=True)
        self_scores = raw[np.arange(40), np.arange(40)]
        assert abs(float(self_scores.mean()) - 1.0) < tol
        true = (q.astype(np.float64) @ v.astype(np.float64).T)
        err = raw.astype(np.float64) - true
        # cross scores: unbiased, error of the size of the quantisation noise
        assert abs(err.mean()) < 2e-3
        assert np.sqrt((err ** 2).mean()) < {2: 0.012, 3: 0.006, 4: 0.004}[bits]
        if calibrated:
            # flipping the sign of the bias correction moves every score by 2 * sum(q_rot * shift)
            qr = np.stack([rot.apply(x) for x in q])
            bc = -(qr.astype(np.float64) @ cal[0].astype(np.float64))
            if np.abs(bc).mean() > 1e-3:
                assert np.abs(err).mean() < np.abs(err - 2 * (bc[:, None] * scales[None, :])).mean()


# --------------------------------------------------------------------------
# (d) the codebook, every cell including (128, 4): an independent Lloyd-Max whose
#     cell probabilities come from scipy's regularised incomplete beta function and
#     whose conditional means are closed-form (no quadrature, no continued fraction
#     of ours): for the density f(x) = (1 - x^2)^(a-1) / (2^(2a-1) B(a, a)) on [-1, 1],
#     the integral of x f(x) over [lo, hi] is ((1-lo^2)^a - (1-hi^2)^a) / (2a 2^(2a-1) B(a,a)).
# --------------------------------------------------------------------------
def independent_codebook(bits, dim, iters=200, tol=1e-12):
    sp = pytest.importorskip("scipy.special")
    a = (dim - 1.0) / 2.0
    n_levels = 1 << bits
    std = math.sqrt(2.0 * a / ((2.0 * a + 1.0) * 4.0 * a))
    spread = 3.0 * std
    c = np.array([-spread + 2.0 * spread * i / (n_levels - 1.0) for i in range(n_levels)], np.float64)
    log_norm = (2.0 * a - 1.0) * math.log(2.0) + sp.betaln(a, a)

    def first_moment(lo, hi):
        def part(x):
            return 0.0 if abs(x) >= 1.0 else math.exp(a * math.log1p(-x * x) - log_norm)
        return (part(lo) - part(hi)) / (2.0 * a)

    for _ in range(iters):
        edges = np.concatenate([[-1.0], (c[:-1] + c[1:]) / 2.0, [1.0]])
        new = c.copy()
        for i in range(n_levels):
            lo, hi = edges[i], edges[i + 1]
            prob = sp.betainc(a, a, (hi + 1.0) / 2.0) - sp.betainc(a, a, (lo + 1.0) / 2.0)
            if prob >= 1e-15:
                new[i] = first_moment(lo, hi) / prob
        change = np.abs(new - c).max()
        c = new
        if change < tol:
            break
    c32 = c.astype(np.float32)
    b32 = ((c32[:-1] + c32[1:]) * np.float32(0.5)).astype(np.float32)
    return b32, c32


_PINNED_CELLS = sorted({(d, b) for d, b, _, _ in CODEBOOK} | {(r[0], r[1]) for r in FINGERPRINT})


@pytest.mark.parametrize("dim,bits", _PINNED_CELLS + [(128, 4), (128, 2), (128, 3)])
def test_codebook_matches_independent_lloyd_max(oracle, dim, bits):
    b, c = oracle.codebook(bits, dim)
    mb, mc = independent_codebook(bits, dim)
    assert np.array_equal(c.view(np.uint32), mc.view(np.uint32))
    assert np.array_equal(b.view(np.uint32), mb.view(np.uint32))


def test_independent_lloyd_max_reproduces_the_reference_hashes(oracle):
    # the model itself is anchored on the reference's goldens (codebook_determinism.rs:91-98),
    # so its answer for the cell without a golden carries their weight
    for dim, bits, wb, wc in CODEBOOK:
        mb, mc = independent_codebook(bits, dim)
        assert oracle.fnv1a(mc) == wc and oracle.fnv1a(mb) == wb
