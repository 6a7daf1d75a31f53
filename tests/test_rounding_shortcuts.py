"""CPU checks of the arithmetic shortcuts the HIP quantizers take on the way to bit-exact output.

The kernels replace `clamp(nearest_int(v))` by an add-and-truncate, and the IEEE division in front of it by a
multiplication with a reciprocal wherever the product stays clear of every rounding boundary; a lane that comes closer
takes the division.  These tests restate both in numpy float32 (IEEE, like the device arithmetic) and drive them with
inputs placed on and around the boundaries, where a wrong margin or constant would show."""
import numpy as np

C = np.float32(0.49999997)  # the largest float below 0.5
assert C == np.nextafter(np.float32(0.5), np.float32(0))


def round_half_away(v):
    v = np.asarray(v, dtype=np.float32)
    with np.errstate(invalid="ignore"):
        t = np.trunc(v)
        r = np.where(np.abs(v - t) >= np.float32(0.5), t + np.copysign(np.float32(1), v), t)
    return r.astype(np.float32)


def nearest_int_clamped(v, lo, hi):
    """`(v.round() as i32).clamp(lo, hi)`: NaN -> 0, saturating."""
    r = round_half_away(v)
    r = np.where(np.isnan(r), np.float32(0), r)
    return np.clip(r, lo, hi).astype(np.int32)


def shortcut_signed(v, lo, hi):
    """|v| + C, sign put back, truncated with saturation and NaN -> 0, clamped."""
    v = np.asarray(v, dtype=np.float32)
    with np.errstate(invalid="ignore"):
        a = (np.abs(v) + C).astype(np.float32)
        t = np.trunc(np.copysign(a, v))
    t = np.where(np.isnan(t), np.float32(0), t)
    return np.clip(t, lo, hi).astype(np.int32)


def shortcut_0_15(v):
    v = np.asarray(v, dtype=np.float32)
    w = np.where(np.isnan(v), np.float32(0), np.clip(v, np.float32(0), np.float32(15))).astype(np.float32)
    return np.trunc((w + C).astype(np.float32)).astype(np.int32)


def boundary_cloud(lo, hi, spread=6):
    """every n + 0.5 in [lo, hi] with its neighbours up to `spread` ulps away, plus the integers' neighbours"""
    out = []
    for n in np.arange(lo - 2, hi + 2):
        for c in (np.float32(n), np.float32(n + 0.5)):
            up = down = c
            out.append(c)
            for _ in range(spread):
                up = np.nextafter(up, np.float32(np.inf))
                down = np.nextafter(down, np.float32(-np.inf))
                out += [up, down]
    return np.array(out, dtype=np.float32)


def test_add_and_truncate_equals_round_half_away():
    rng = np.random.default_rng(1)
    v = np.concatenate([
        boundary_cloud(-40, 40),
        rng.uniform(-40, 40, 2_000_000).astype(np.float32),
        (rng.standard_normal(200_000) * 1e-3).astype(np.float32),
        rng.integers(0, 2**32, 2_000_000, dtype=np.uint64).astype(np.uint32).view(np.float32),  # any bit pattern
        np.array([0.0, -0.0, np.inf, -np.inf, np.nan, 3e38, -3e38, 2**31, -2**31, 2**23 + 1, 8388607.5, 4194304.5],
                 dtype=np.float32),
    ])
    assert np.array_equal(shortcut_signed(v, -32, 31), nearest_int_clamped(v, -32, 31))
    assert np.array_equal(shortcut_signed(v, -127, 127), nearest_int_clamped(v, -127, 127))
    assert np.array_equal(shortcut_0_15(v), nearest_int_clamped(v, 0, 15))
    # the one float where adding 0.5 itself would fail
    assert shortcut_0_15(C) == 0 and np.trunc(C + np.float32(0.5)) == 1


def _quotients_near_boundaries(rng, n, lo, hi):
    """(numerator, denominator) pairs whose quotient lies within about 1e-4 of some k + 0.5, k in [lo, hi)"""
    den = np.exp(rng.uniform(np.log(1e-6), np.log(10.0), n)).astype(np.float32)
    den *= rng.choice(np.array([-1, 1], dtype=np.float32), n)
    k = rng.integers(lo, hi, n).astype(np.float64) + 0.5
    delta = rng.choice(np.array([0, 1e-7, 3e-7, 1e-6, 2e-6, 4e-6, 8e-6, 1.5e-5, 3e-5, 1e-4]), n) * rng.choice([-1, 1], n)
    num = ((k + delta) * den.astype(np.float64)).astype(np.float32)
    return num, den


def test_multiplying_by_the_reciprocal_rounds_like_the_division_outside_the_margin():
    """Requantization: the reciprocal is itself a correctly rounded division; margin 8e-6 for |quotient| < 33."""
    rng = np.random.default_rng(2)
    for lo, hi in ((0, 15), (-32, 31)):
        num, den = _quotients_near_boundaries(rng, 3_000_000, lo - 1, hi + 1)
        exact = nearest_int_clamped((num / den).astype(np.float32), lo, hi)
        q = (num * (np.float32(1) / den).astype(np.float32)).astype(np.float32)
        fast = shortcut_signed(q, lo, hi)
        sure = np.abs(np.abs(q - fast.astype(np.float32)) - np.float32(0.5)) >= np.float32(8e-6)
        assert sure.mean() > 0.2 and (~sure).mean() > 0.2  # both sides are exercised
        assert np.array_equal(fast[sure], exact[sure])
        assert (fast != exact).any()  # and the margin is needed: inside it the two do differ


def test_a_reciprocal_one_ulp_off_rounds_like_the_division_outside_the_wider_margin():
    """Coordinate descent of the Q6_K search: hardware reciprocal (one ulp), margin 2e-5."""
    rng = np.random.default_rng(3)
    num, den = _quotients_near_boundaries(rng, 3_000_000, -33, 32)
    den = np.abs(den)  # the kernel only divides by positive sums
    exact = nearest_int_clamped((num / den).astype(np.float32), -32, 31)
    r = (np.float32(1) / den).astype(np.float32)
    for rcp in (r, np.nextafter(r, np.float32(np.inf)), np.nextafter(r, np.float32(0))):
        q = (num * rcp).astype(np.float32)
        fast = shortcut_signed(q, -32, 31)
        sure = np.abs(np.abs(q - fast.astype(np.float32)) - np.float32(0.5)) >= np.float32(2e-5)
        assert sure.mean() > 0.1
        assert np.array_equal(fast[sure], exact[sure])
