"""Comparison helpers shared by the tests."""
import numpy as np

from oracle.numpy_oracle import (  # noqa: F401  (re-exported for the tests)
    _square_sum64, check_sum_forward, forward_sum_bound, sum_tolerances)


def ulp_distance(a, b):
    """Largest distance, in units in the last place, between two float arrays
    of the same dtype (NaNs must coincide; +0 and -0 are 1 apart... treated as
    equal here because both are the same real number)."""
    a = np.asarray(a)
    b = np.asarray(b)
    assert a.dtype == b.dtype and a.shape == b.shape, (a.dtype, b.dtype, a.shape, b.shape)
    nan_a, nan_b = np.isnan(a), np.isnan(b)
    assert np.array_equal(nan_a, nan_b), 'NaN positions differ'
    it = {2: np.int16, 4: np.int32, 8: np.int64}[a.dtype.itemsize]
    ia = a.view(it).astype(np.int64)
    ib = b.view(it).astype(np.int64)
    sign = np.int64(1) << (8 * a.dtype.itemsize - 1)
    ia = np.where(ia < 0, -(ia + sign), ia)
    ib = np.where(ib < 0, -(ib + sign), ib)
    d = np.abs(ia - ib)
    d[nan_a] = 0
    return int(d.max()) if d.size else 0


def assert_ulp(got, expect, max_ulp=1):
    got = np.asarray(got)
    expect = np.asarray(expect)
    assert got.dtype == expect.dtype, (got.dtype, expect.dtype)
    assert got.shape == expect.shape, (got.shape, expect.shape)
    if got.dtype.kind == 'f':
        d = ulp_distance(got, expect)
        assert d <= max_ulp, 'max ulp distance %d > %d' % (d, max_ulp)
    else:
        assert np.array_equal(got, expect)


def assert_exact(got, expect):
    got = np.asarray(got)
    expect = np.asarray(expect)
    assert got.dtype == expect.dtype, (got.dtype, expect.dtype)
    assert got.shape == expect.shape, (got.shape, expect.shape)
    assert np.array_equal(got, expect, equal_nan=got.dtype.kind in 'fc')


def assert_sum_close(got, expect, addends_abs_sum, dtype, data=None, axis=None):
    """Two bounds on a floating-point sum whose order differs from NumPy's.

    Backward: ``|got - expect| <= rtol * sum(|addends|)``, which any summation
    order of the same addends meets.  On data that cancels this is very wide
    (the sum of |a| dwarfs the result), so when the addends themselves are
    given (``data``, ``axis``) the forward bound of ``forward_sum_bound`` must
    hold as well: that one a missing partial result does break."""
    got = np.asarray(got)
    expect = np.asarray(expect)
    assert got.dtype == expect.dtype, (got.dtype, expect.dtype)
    assert got.shape == expect.shape, (got.shape, expect.shape)
    rtol = sum_tolerances(dtype)
    err = np.abs(got.astype(np.float64) - expect.astype(np.float64))
    bound = rtol * np.asarray(addends_abs_sum, dtype=np.float64) + 1e-300
    assert np.all(err <= bound), 'max err/bound = %g' % float(np.max(err / bound))
    if data is not None:
        ratio = check_sum_forward(got, data, axis, dtype)
        assert ratio <= 1.0, 'forward bound: max err/bound = %g' % ratio
        return ratio
    return None


def shaped_random(shape, dtype, seed=0, scale=10):
    """Seeded test data: uniform in [0, scale) for numbers, random bits for bool."""
    rng = np.random.default_rng(seed)
    dt = np.dtype(dtype)
    if dt.kind == 'b':
        return rng.integers(0, 2, shape).astype(dt)
    if dt.kind == 'u':
        return rng.integers(0, scale, shape).astype(dt)
    if dt.kind == 'i':
        return rng.integers(-scale, scale, shape).astype(dt)
    return (rng.random(shape) * 2 * scale - scale).astype(dt)
