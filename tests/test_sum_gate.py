"""The floating-point sum gate must be able to fail.

``helpers.assert_sum_close`` holds a sum to two bounds.  The backward bound
(rtol * sum|a|) alone is blind on data that cancels: for N(0,1) addends sum|a|
is ~0.8 N while the result is only ~sqrt(N): at 2**28 addends rtol * sum|a| is
about 2100 where a missing partial result of 2**17 addends changes the sum by
about 360.  These tests pin that the forward bound
(rtol * max(|ref64|, sigma * sqrt(N))) accepts every honest summation order and
rejects a dropped or doubled block of addends.  CPU only."""
import numpy as np
import pytest

from helpers import assert_sum_close, check_sum_forward, forward_sum_bound


def _orders(a):
    """The same addends summed in orders a GPU reduction may use."""
    flat = a.reshape(-1)
    yield np.sum(flat)                                         # NumPy pairwise
    yield np.add.reduce(flat.reshape(-1, 256), axis=0).sum()   # strided lanes, then a tree
    yield np.add.reduce(flat.reshape(256, -1), axis=1).sum()   # contiguous runs, then a tree
    acc = np.zeros(1024, a.dtype)
    for part in flat.reshape(-1, 1024):                        # plain running sums per lane
        acc += part
    yield acc.sum()


@pytest.mark.parametrize('dtype', ['float32', 'float64'])
def test_every_summation_order_passes(dtype):
    rng = np.random.default_rng(3)
    a = rng.standard_normal((2048, 2048)).astype(dtype)
    for got in _orders(a):
        assert check_sum_forward(np.asarray(got, dtype=dtype), a, None, dtype) <= 1.0


@pytest.mark.parametrize('dtype', ['float32', 'float64'])
def test_missing_or_doubled_partial_is_rejected(dtype):
    rng = np.random.default_rng(3)
    n = 2048
    a = rng.standard_normal((n, n)).astype(dtype)
    splits = 2048                       # a full reduction cut into this many partials
    chunk = a.size // splits
    honest = np.sum(a)
    mag = np.abs(a).sum(dtype=np.float64)
    for k in (0, 7, splits - 1):
        dropped = np.asarray(
            float(honest) - a.reshape(-1)[k * chunk:(k + 1) * chunk].sum(dtype=np.float64),
            dtype=dtype)
        doubled = np.asarray(2 * float(honest) - float(dropped), dtype=dtype)
        assert check_sum_forward(dropped, a, None, dtype) > 1.0
        assert check_sum_forward(doubled, a, None, dtype) > 1.0
        with pytest.raises(AssertionError):
            assert_sum_close(dropped, np.asarray(honest), mag, dtype, data=a, axis=None)
    assert_sum_close(np.asarray(honest), np.asarray(honest), mag, dtype, data=a, axis=None)


def test_axis_sums_missing_rows_are_rejected():
    rng = np.random.default_rng(4)
    a = rng.standard_normal((512, 4096), dtype=np.float32)
    for axis in (0, 1):
        good = a.sum(axis=axis)
        assert check_sum_forward(good, a, axis, 'float32') <= 1.0
        bad = good.copy()
        # one output computed from all but the last 64 addends
        if axis == 1:
            bad[3] = a[3, :-64].sum()
        else:
            bad[3] = a[:-64, 3].sum()
        assert check_sum_forward(bad, a, axis, 'float32') > 1.0


def test_bound_follows_the_result_when_nothing_cancels():
    a = np.full((64, 1000), 0.1, np.float32)
    ref, bound = forward_sum_bound(a, 1, 'float32')
    assert np.allclose(bound, 1e-5 * np.abs(ref))


def test_square_sum_of_large_matrix_in_blocks():
    from helpers import _square_sum64
    rng = np.random.default_rng(5)
    a = rng.standard_normal((5000, 5000), dtype=np.float32)     # > 2**24 elements
    full = np.square(a, dtype=np.float64)
    assert np.allclose(_square_sum64(a, 1), full.sum(axis=1), rtol=1e-12)
    assert np.allclose(_square_sum64(a, 0), full.sum(axis=0), rtol=1e-12)
    assert np.allclose(_square_sum64(a, None), full.sum(), rtol=1e-12)
