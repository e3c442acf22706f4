"""The wide scan skips the float epilogue of a tile when no accumulator of a lane reaches an
integer bound derived from the query's floor.  The bound must be conservative: whenever the
exact float score of an accumulator reaches the floor, the accumulator reaches the bound.
This restates the bound's arithmetic (tv_kernels3.hip: WideQuery, k_scan_p4_wide) in float32
numpy and tries to break it with accumulators placed right at the decision point."""
import numpy as np

F = np.float32


def fma32(a, b, c):
    # a * b is exact in float64 for float32 inputs; the sum rounds once to float64, then to float32
    return F(np.float64(a) * np.float64(b) + np.float64(c))


def exact_pass(acc, qs, qb, vs, tau):
    s = F(fma32(F(acc), qs, qb) * vs)
    return s >= tau


ALWAYS = -2**31


def bound_of(qs, qb, tau, vmax):
    with np.errstate(over="ignore", divide="ignore", invalid="ignore", under="ignore"):
        bounded = (F(1e-30) <= tau <= F(1e30) and F(1e-30) <= qs <= F(1e30) and abs(qb) <= F(1e30)
                   and np.isfinite(F(tau / qs)))
        if not bounded:
            return ALWAYS                  # ta = -inf in the kernel: every tile is scored
        if vmax > F(1e30) or 0 < vmax < F(1e-30):
            return ALWAYS                  # the block is flagged: always scored
        inv = F(F(1.0) / vmax)
        ta = F(F(tau / qs) * F(1.0 - 1e-5))
        rb = F(qb / qs)
        tb = F(F(rb + F(F(1e-5) * abs(rb))) + F(2.0))
        bf = F(fma32(ta, inv, -tb) - F(1.0))
    if np.isnan(bf):
        return 0
    return int(np.clip(np.trunc(np.float64(bf)), -2**31, 2**31 - 1))


def test_bound_never_rejects_a_passing_accumulator():
    rng = np.random.default_rng(7)
    checked = 0
    for _ in range(4000):
        qs = F(10.0 ** rng.uniform(-9, -1))
        qb = F(rng.choice([0.0, 1.0, -1.0]) * 10.0 ** rng.uniform(-6, 1))
        vmax = F(10.0 ** rng.uniform(-3, 3))
        vs = F(vmax * F(rng.uniform(0.0, 1.0)))            # any allowed row scale in [0, vmax]
        if rng.random() < 0.3:
            vs = vmax
        # a floor that an accumulator of realistic size (|acc| < 2^25) can sit on
        acc0 = int(rng.integers(-2**24, 2**25))
        tau = F(fma32(F(acc0), qs, qb) * vs)
        if not (tau > 0 and np.isfinite(tau)):
            continue
        bound = bound_of(qs, qb, tau, vmax)
        for d in range(-6, 7):
            acc = acc0 + d
            if exact_pass(acc, qs, qb, vs, tau):
                checked += 1
                assert acc >= bound, (qs, qb, vmax, vs, tau, acc, bound)
    assert checked > 10000


def test_bound_is_not_vacuous():
    """At the block's largest row scale the bound sits within a small margin of the decision point."""
    rng = np.random.default_rng(8)
    gaps = []
    for _ in range(500):
        qs = F(10.0 ** rng.uniform(-7, -3))
        qb = F(rng.uniform(-0.5, 0.5))
        vmax = F(rng.uniform(0.5, 2.0))
        acc0 = int(rng.integers(2**18, 2**23))
        tau = F(fma32(F(acc0), qs, qb) * vmax)
        if not tau > 0:
            continue
        gaps.append((acc0 - bound_of(qs, qb, tau, vmax)) / acc0)
    gaps = np.array(gaps)
    assert (gaps >= 0).all()
    assert np.median(gaps) < 1e-3   # the margin is a small fraction of the accumulator


def test_bound_survives_extreme_row_scales():
    """Row scales from the smallest subnormal to the largest float (an uploaded snapshot may hold
    anything), query scales down to where tau / qs overflows: a passing accumulator is never
    rejected."""
    rng = np.random.default_rng(9)
    checked = extreme = 0
    with np.errstate(over="ignore", under="ignore", invalid="ignore"):
        for _ in range(6000):
            qs = F(10.0 ** rng.uniform(-38, 2))
            qb = F(rng.choice([0.0, 1.0, -1.0]) * 10.0 ** rng.uniform(-30, 10))
            vmax = F(10.0 ** rng.uniform(-45, 38.5))
            if vmax == 0:
                continue
            vs = vmax if rng.random() < 0.5 else F(vmax * F(rng.uniform(0.0, 1.0)))
            acc0 = int(rng.integers(-2**24, 2**25))
            tau = F(fma32(F(acc0), qs, qb) * vs)
            if not (tau > 0 and np.isfinite(tau)):
                continue
            bound = bound_of(qs, qb, tau, vmax)
            extreme += vmax < 1e-38 or vmax > 1e30 or not np.isfinite(F(tau / qs))
            for d in range(-3, 4):
                acc = acc0 + d
                if exact_pass(acc, qs, qb, vs, tau):
                    checked += 1
                    assert acc >= bound, (qs, qb, vmax, vs, tau, acc, bound)
    assert checked > 5000 and extreme > 500
