"""The identity behind the costs-only relaxation: for binary64 round-to-nearest,

    min_i fl(fl(f_i + t_i) + c)  ==  fl(min_i fl(f_i + t_i) + c)

because x -> fl(x + c) is monotone (x <= y implies fl(x + c) <= fl(y + c)).  The reference evaluates
the left side (csrc/dp_core.cpp:68,70); the kernel evaluates the right side and adds c once per cell.
Checked here on the CPU with numpy (IEEE binary64, same rounding as the device's v_add_f64) over
operands chosen to provoke rounding: magnitudes spread over the whole exponent range, values one ulp
apart, subnormals, negatives, exact cancellations and +inf.  The ARGMIN of the two sides does differ
(asserted too), which is why the kernel never takes it from the right-hand side."""
import numpy as np


def _both_sides(pre, c):
    left = np.min(pre + c[:, None], axis=1)
    right = np.min(pre, axis=1) + c
    return left, right


def _same_bits(a, b):
    return np.array_equal(a.view(np.int64), b.view(np.int64))


def test_random_operands_over_the_exponent_range():
    rng = np.random.Generator(np.random.PCG64(2024))
    n, k = 200_000, 16
    for scale_f, scale_c in ((0, 0), (0, 40), (40, 0), (-300, -300), (300, 300), (0, -40), (-1000, -1000)):
        f = rng.standard_normal((n, k)) * 2.0 ** (scale_f + rng.integers(-8, 9, size=(n, k)))
        t = rng.standard_normal((n, k)) * 2.0 ** (scale_f + rng.integers(-8, 9, size=(n, k)))
        c = rng.standard_normal(n) * 2.0 ** (scale_c + rng.integers(-8, 9, size=n))
        with np.errstate(over="ignore", invalid="raise"):
            pre = f + t
            left, right = _both_sides(pre, c)
        assert _same_bits(left, right), (scale_f, scale_c)


def test_neighbouring_values_cancellation_subnormals_and_inf():
    rng = np.random.Generator(np.random.PCG64(7))
    n, k = 100_000, 12
    base = rng.uniform(1.0, 2.0, size=(n, 1))
    steps = rng.integers(0, 6, size=(n, k)).astype(np.float64)
    pre = base + steps * 2.0 ** -52                      # candidates a few ulps apart
    for c in (2.0 ** 20 * rng.integers(1, 5, size=n).astype(np.float64),      # swallows the differences
              -base[:, 0],                                                    # exact cancellation with one of them
              -(base[:, 0] + 2.0 ** -52),
              np.full(n, 5e-324), np.full(n, -5e-324), np.zeros(n), np.full(n, np.inf)):
        left, right = _both_sides(pre, c)
        assert _same_bits(left, right)
    pre_inf = pre.copy()
    pre_inf[rng.uniform(size=pre.shape) < 0.3] = np.inf  # infeasible sources
    pre_inf[:100] = np.inf                               # ... all of them
    left, right = _both_sides(pre_inf, rng.uniform(0.5, 30.0, size=n))
    assert _same_bits(left, right)
    tiny = rng.integers(-4, 5, size=(n, k)).astype(np.float64) * 5e-324       # subnormal sums
    left, right = _both_sides(tiny, rng.integers(-4, 5, size=n).astype(np.float64) * 5e-324 + 0.0)
    assert np.array_equal(left, right)                   # equal as numbers (a zero may differ in sign)


def test_the_argmin_is_not_preserved():
    """Two candidates that differ before + c and collide after it: the reference's lowest-index rule
    then picks another source than the argmin of the pre-sums -- the reason the backtrack recomputes
    the full candidates."""
    pre = np.array([[1.0 + 2.0 ** -50, 1.0]])
    c = np.array([2.0 ** 20])
    cand = pre + c[:, None]
    assert cand[0, 0] == cand[0, 1]
    assert int(np.argmin(cand[0])) == 0 and int(np.argmin(pre[0])) == 1
    left, right = _both_sides(pre, c)
    assert _same_bits(left, right)
