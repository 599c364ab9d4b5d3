"""cumsum / cumprod and the statistics reductions (mean, var, std, ptp, the
nan-variants) against NumPy on the same seeded inputs.  Integer results are
bit-exact; floating-point results are compared within the reduction tolerance
(the evaluation order differs from NumPy's)."""
import warnings

import numpy as np
import pytest

import cupy_amd as cp
from helpers import assert_exact

pytestmark = pytest.mark.gpu

SHAPES = [(1,), (7,), (64,), (1000,), (4097,), (3, 5), (129, 33), (33, 129), (2, 3, 4),
          (5, 1, 7), (40, 50, 6), (1 << 16,), (300, 1000)]


def _rand(rng, shape, dtype):
    dtype = np.dtype(dtype)
    if dtype.kind == 'f':
        return rng.uniform(-1, 1, shape).astype(dtype)
    if dtype.kind == 'b':
        return rng.integers(0, 2, shape).astype(dtype)
    return rng.integers(-3 if dtype.kind == 'i' else 0, 4, shape).astype(dtype)


@pytest.mark.parametrize('dtype', [np.int8, np.uint8, np.int32, np.int64, np.bool_])
@pytest.mark.parametrize('shape', SHAPES)
def test_cumsum_integers_exact(shape, dtype):
    rng = np.random.default_rng(21)
    h = _rand(rng, shape, dtype)
    d = cp.asarray(h)
    for axis in [None] + list(range(len(shape))):
        assert_exact(d.cumsum(axis=axis).get(), h.cumsum(axis=axis))
    assert_exact(cp.cumsum(d, axis=-1, dtype=np.int32).get(), h.cumsum(axis=-1, dtype=np.int32))


@pytest.mark.parametrize('shape', [(7,), (1000,), (129, 33), (40, 50, 6)])
def test_cumprod_integers_exact(shape):
    rng = np.random.default_rng(22)
    h = rng.choice(np.array([-1, 1, 1, 1, 2], dtype=np.int64), size=shape)
    d = cp.asarray(h)
    for axis in [None] + list(range(len(shape))):
        assert_exact(d.cumprod(axis=axis).get(), h.cumprod(axis=axis))


@pytest.mark.parametrize('dtype,rtol', [(np.float32, 1e-5), (np.float64, 1e-12), (np.float16, 2e-3)])
@pytest.mark.parametrize('shape', SHAPES)
def test_cumsum_floats(shape, dtype, rtol):
    rng = np.random.default_rng(23)
    h = _rand(rng, shape, dtype)
    d = cp.asarray(h)
    for axis in [None] + list(range(len(shape))):
        got = d.cumsum(axis=axis).get()
        want = np.cumsum(h.astype(np.float64), axis=axis)
        bound = rtol * np.cumsum(np.abs(h).astype(np.float64), axis=axis) + 1e-300
        assert got.dtype == dtype and got.shape == want.shape
        assert np.all(np.abs(got.astype(np.float64) - want) <= bound)


@pytest.mark.parametrize('chain', [True, False])
def test_large_one_dimensional_scans_use_every_pass(chain):
    """Long rows: through the one-pass kernel and (with it switched off)
    through the three passes of the chunked kernels."""
    from cupy_amd._core import _tuning
    _tuning.set(scan_chain=chain)
    try:
        _large_scans()
    finally:
        _tuning.set(scan_chain=True)


def _large_scans():
    rng = np.random.default_rng(24)
    h = rng.integers(-5, 6, (1 << 23) + 12345).astype(np.int32)
    d = cp.asarray(h)
    assert_exact(d.cumsum().get(), h.cumsum())
    hf = rng.uniform(0, 1, 1 << 22).astype(np.float32)
    got = cp.asarray(hf).cumsum().get()
    want = np.cumsum(hf.astype(np.float64))
    assert np.all(np.abs(got - want) <= 1e-5 * want + 1e-6)
    # long columns, few of them: chunks along the strided axis
    hm = rng.integers(-5, 6, (70000, 24)).astype(np.int64)
    assert_exact(cp.asarray(hm).cumsum(axis=0).get(), hm.cumsum(axis=0))
    assert_exact(cp.asarray(hm.T.copy()).cumsum(axis=1).get(), hm.T.cumsum(axis=1))


def test_scan_views_out_and_nan_variants():
    rng = np.random.default_rng(25)
    h = rng.integers(-3, 4, (64, 48)).astype(np.int64)
    d = cp.asarray(h)
    assert_exact(d.T.cumsum(axis=0).get(), h.T.cumsum(axis=0))           # non-contiguous input
    assert_exact(d[::2, 1::3].cumsum(axis=1).get(), h[::2, 1::3].cumsum(axis=1))
    out = cp.empty((64, 48), np.int64)
    assert cp.cumsum(d, axis=1, out=out) is out
    assert_exact(out.get(), h.cumsum(axis=1))
    out_t = cp.empty((48, 64), np.int64).T                                # non-contiguous out
    cp.cumsum(d, axis=0, out=out_t)
    assert_exact(out_t.get(), h.cumsum(axis=0))
    d2 = cp.asarray(h)
    cp.cumsum(d2, axis=1, out=d2)                                         # in place
    assert_exact(d2.get(), h.cumsum(axis=1))
    with pytest.raises(ValueError):
        cp.cumsum(d, axis=0, out=cp.empty((3, 3), np.int64))
    with pytest.raises(np.exceptions.AxisError):
        d.cumsum(axis=2)
    f = rng.uniform(-1, 1, (50, 70))
    f[rng.uniform(size=f.shape) < 0.2] = np.nan
    df = cp.asarray(f)
    for axis in (None, 0, 1):
        np.testing.assert_allclose(cp.nancumsum(df, axis=axis).get(), np.nancumsum(f, axis=axis),
                                   rtol=1e-12, atol=1e-12)
        np.testing.assert_allclose(cp.nancumprod(df, axis=axis).get(), np.nancumprod(f, axis=axis),
                                   rtol=1e-10, atol=1e-300)
    got = cp.cumsum(df, axis=1).get()
    assert np.array_equal(np.isnan(got), np.isnan(np.cumsum(f, axis=1)))
    e = cp.asarray(np.zeros((0, 5)))
    assert e.cumsum(axis=0).shape == (0, 5) and e.cumsum().shape == (0,)


@pytest.mark.parametrize('dtype', [np.float32, np.float64, np.int32, np.float16, np.bool_])
@pytest.mark.parametrize('shape,axes', [((1000,), [None, 0]), ((129, 33), [None, 0, 1, (0, 1)]),
                                        ((40, 50, 6), [None, 0, 1, 2, (0, 2), (1, 2)]),
                                        ((300, 1000), [0, 1])])
def test_mean_var_std_ptp(shape, axes, dtype):
    rng = np.random.default_rng(26)
    h = _rand(rng, shape, dtype)
    d = cp.asarray(h)
    tol = {np.float16: 4e-3, np.float32: 2e-5}.get(dtype, 1e-11)
    for axis in axes:
        for keepdims in (False, True):
            got = d.mean(axis=axis, keepdims=keepdims).get()
            want = h.mean(axis=axis, keepdims=keepdims)
            assert got.dtype == want.dtype and got.shape == want.shape
            np.testing.assert_allclose(got.astype(np.float64), want.astype(np.float64),
                                       rtol=tol, atol=tol)
        if dtype is not np.bool_:
            for ddof in (0, 1):
                got = d.var(axis=axis, ddof=ddof).get()
                want = h.var(axis=axis, ddof=ddof)
                assert got.dtype == want.dtype and got.shape == want.shape
                np.testing.assert_allclose(got.astype(np.float64), want.astype(np.float64),
                                           rtol=20 * tol, atol=tol)
                got = cp.std(d, axis=axis, ddof=ddof).get()
                want = np.std(h, axis=axis, ddof=ddof)
                assert got.dtype == want.dtype
                np.testing.assert_allclose(got.astype(np.float64), want.astype(np.float64),
                                           rtol=20 * tol, atol=tol)
            assert_exact(d.ptp(axis=axis).get(), np.ptp(h, axis=axis))
    got = cp.mean(d, axis=0, dtype=np.float64).get()
    np.testing.assert_allclose(got, h.mean(axis=0, dtype=np.float64), rtol=1e-12, atol=1e-12)
    out = cp.empty(np.mean(h, axis=0).shape, np.float64)
    assert d.mean(axis=0, out=out) is out


def test_mean_of_nothing_is_nan():
    e = cp.asarray(np.zeros((0, 3), np.float32))
    with np.errstate(all='ignore'):
        assert np.isnan(e.mean().get())
        assert e.mean(axis=1).shape == (0,)
        assert np.isnan(e.mean(axis=0).get()).all()
        assert np.isnan(e.var().get())


@pytest.mark.parametrize('dtype', [np.float32, np.float64, np.float16])
def test_nan_reductions(dtype):
    rng = np.random.default_rng(27)
    h = rng.uniform(-1, 1, (60, 90)).astype(dtype)
    h[rng.uniform(size=h.shape) < 0.3] = np.nan
    h[5, :] = np.nan
    h[:, 7] = np.nan
    d = cp.asarray(h)
    tol = {np.float16: 4e-3, np.float32: 2e-5}.get(dtype, 1e-11)
    import warnings
    with np.errstate(all='ignore'):
        with warnings.catch_warnings():
            warnings.simplefilter('ignore')
            for axis in (None, 0, 1):
                assert_exact(cp.nanmin(d, axis=axis).get(), np.nanmin(h, axis=axis))
                assert_exact(cp.nanmax(d, axis=axis).get(), np.nanmax(h, axis=axis))
                got = cp.nanmean(d, axis=axis).get()
                want = np.nanmean(h, axis=axis)
                assert got.dtype == want.dtype
                np.testing.assert_allclose(got.astype(np.float64), want.astype(np.float64),
                                           rtol=tol, atol=tol)
                for ddof in (0, 1):
                    got = cp.nanvar(d, axis=axis, ddof=ddof).get()
                    want = np.nanvar(h, axis=axis, ddof=ddof)
                    assert got.dtype == want.dtype
                    np.testing.assert_allclose(got.astype(np.float64), want.astype(np.float64),
                                               rtol=20 * tol, atol=tol)
                    got = cp.nanstd(d, axis=axis, ddof=ddof).get()
                    np.testing.assert_allclose(got.astype(np.float64),
                                               np.nanstd(h, axis=axis, ddof=ddof).astype(np.float64),
                                               rtol=20 * tol, atol=tol)
                got = cp.nanprod(d, axis=axis).get()
                want = np.nanprod(h.astype(np.float64), axis=axis)
                # float16 products of many factors below one underflow
                np.testing.assert_allclose(got.astype(np.float64), want, rtol=50 * tol,
                                           atol=1e-4 if dtype is np.float16 else 1e-30)
    # arg-variants: slices of only NaNs give -1 (NumPy raises there)
    good = np.ones(h.shape[0], bool)
    good[5] = False
    got = cp.nanargmax(d, axis=1).get()
    assert got[5] == -1
    ref = np.array([np.nanargmax(r) for r in h[good]])
    assert np.array_equal(got[good], ref)
    got = cp.nanargmin(d, axis=1).get()
    assert got[5] == -1
    assert np.array_equal(got[good], np.array([np.nanargmin(r) for r in h[good]]))
    hi = rng.integers(0, 9, (20, 30)).astype(np.int32)
    assert_exact(cp.nanargmax(cp.asarray(hi), axis=1).get(), np.nanargmax(hi, axis=1))
    assert_exact(cp.count_nonzero(cp.asarray(hi), axis=0).get(), np.count_nonzero(hi, axis=0))
    assert int(cp.count_nonzero(cp.asarray(hi)).get()) == np.count_nonzero(hi)


@pytest.mark.parametrize('dtype', ['float32', 'float64'])
def test_one_pass_variance_is_stable_and_matches_numpy(dtype):
    """The variance is computed in one pass over the data, as sums of (x - k)
    and (x - k)**2 around pivots k that follow the data (see ``var_st``).  Data
    with a mean far above its spread is where a plain sum-of-squares formula
    cancels catastrophically; here it must not."""
    rng = np.random.default_rng(91)
    rtol = 2e-5 if dtype == 'float32' else 1e-11
    for offset in (0.0, 1.0e3, 1.0e4, -3.0e5):
        h = (rng.standard_normal((513, 1031)) + offset).astype(dtype)
        d = cp.asarray(h)
        for axis in (None, 0, 1):
            for ddof in (0, 1):
                want = h.astype(np.float64).var(axis=axis, ddof=ddof)
                got = d.var(axis=axis, ddof=ddof)
                assert got.dtype == np.dtype(dtype)
                np.testing.assert_allclose(got.get(), want, rtol=rtol)
    # outliers at the first and the last position of every row and column
    h = rng.standard_normal((513, 1031)).astype(dtype)
    h[0, :] = 1.0e6
    h[:, 1030] = -1.0e6
    d = cp.asarray(h)
    for axis in (0, 1):
        np.testing.assert_allclose(d.var(axis=axis).get(), h.astype(np.float64).var(axis=axis),
                                   rtol=rtol)
    # NaN and infinity propagate as in NumPy
    h = rng.standard_normal((40, 50)).astype(dtype)
    h[3, 4] = np.nan
    h[5, 6] = np.inf
    with np.errstate(all='ignore'):
        want = h.var(axis=0)
    got = cp.asarray(h).var(axis=0).get()
    assert np.array_equal(np.isnan(got), np.isnan(want))
    np.testing.assert_allclose(got[~np.isnan(want)], want[~np.isnan(want)], rtol=20 * rtol)
    # long reductions split over many blocks, and integers (computed in double)
    h = (rng.standard_normal((3, 400001)) * 3 + 100).astype(dtype)
    np.testing.assert_allclose(cp.asarray(h).var(axis=1).get(),
                               h.astype(np.float64).var(axis=1), rtol=20 * rtol)
    np.testing.assert_allclose(cp.asarray(h).var().get(), h.astype(np.float64).var(),
                               rtol=20 * rtol)
    i = rng.integers(-1000, 1000, (257, 129)).astype(np.int32)
    got = cp.asarray(i).var(axis=0, ddof=1)
    assert got.dtype == np.float64
    np.testing.assert_allclose(got.get(), i.var(axis=0, ddof=1), rtol=1e-12)
    # constant data: exactly zero
    c = np.full((100, 100), 7.25, dtype)
    assert np.array_equal(cp.asarray(c).var(axis=0).get(), np.zeros(100, dtype))
    # out= and std
    out = cp.empty((1031,), dtype)
    h = rng.standard_normal((513, 1031)).astype(dtype)
    r = cp.asarray(h).var(axis=0, out=out)
    assert r is out
    np.testing.assert_allclose(out.get(), h.var(axis=0), rtol=20 * rtol)
    np.testing.assert_allclose(cp.asarray(h).std(axis=1, ddof=1).get(), h.std(axis=1, ddof=1),
                               rtol=20 * rtol)


@pytest.mark.parametrize('shape,axis', [((1000, 8), 0), ((7, 1000, 2), 1), ((5000, 64), 0),
                                        ((100001, 16), 0), ((3, 70000, 4), 1), ((50, 32), 0),
                                        ((2, 3, 999, 8), 2),
                                        # rows that do not fill a power-of-two number of lanes
                                        ((100001, 3), 0), ((5000, 7), 0), ((3, 70000, 5), 1),
                                        ((40000, 12), 0), ((999, 20), 0), ((70001, 48), 0),
                                        ((6000, 100), 0), ((2, 9000, 31), 1), ((64, 6), 0),
                                        # whole rounds of the staged kernel, one row more, one less
                                        ((336 * 3, 3), 0), ((336 * 50 + 1, 3), 0), ((204 * 7 - 1, 5), 0),
                                        ((2000003, 3), 0), ((5, 64 * 9 + 1, 32), 1), ((300001, 2), 0)])
@pytest.mark.parametrize('dtype', ['float32', 'float64', 'int32', 'float16'])
def test_scans_along_an_axis_with_a_narrow_tail(shape, axis, dtype):
    """The axes after the scanned one span a few vectors only: rows sit in
    adjacent lanes and the scan runs across lanes (contiguous accesses), in one
    launch or split into chunks with carried totals."""
    rng = np.random.default_rng(93)
    if dtype == 'int32':
        h = rng.integers(-9, 10, shape).astype(dtype)
    else:
        h = rng.standard_normal(shape).astype(dtype)
    d = cp.asarray(h)
    got = cp.cumsum(d, axis=axis)
    want = np.cumsum(h, axis=axis)
    assert got.dtype == want.dtype and got.shape == want.shape
    if dtype == 'int32':
        assert np.array_equal(got.get(), want)
    else:
        tol = {'float16': 2e-2, 'float32': 1e-5, 'float64': 1e-12}[dtype]
        scale = np.cumsum(np.abs(h.astype(np.float64)), axis=axis)
        assert (np.abs(got.get().astype(np.float64) - np.cumsum(h.astype(np.float64), axis=axis))
                <= tol * scale + tol).all()
    if dtype in ('float32', 'int32') and h.shape[axis] <= 1000:
        small = np.sign(h).astype(dtype)
        small[small == 0] = 1
        assert np.array_equal(cp.cumprod(cp.asarray(small), axis=axis).get(),
                              np.cumprod(small, axis=axis))
    if dtype == 'float32':
        hn = h.copy()
        hn[..., ::3] = np.nan
        got = cp.nancumsum(cp.asarray(hn), axis=axis).get()
        want = np.nancumsum(hn.astype(np.float64), axis=axis)
        assert (np.abs(got - want) <= 1e-5 * np.cumsum(np.abs(np.nan_to_num(hn)), axis=axis) + 1e-5).all()
    # a view whose data is not aligned to the vector width takes another geometry
    flat = cp.asarray(np.concatenate([np.zeros(1, dtype), h.ravel()]))
    view = flat[1:].reshape(shape)
    got = cp.cumsum(view, axis=axis).get().astype(np.float64)
    want = np.cumsum(h.astype(np.float64), axis=axis)
    tol = {'float16': 2e-2, 'float32': 1e-5, 'float64': 1e-12, 'int32': 0}[dtype]
    scale = np.cumsum(np.abs(h.astype(np.float64)), axis=axis)
    assert (np.abs(got - want) <= tol * scale + tol).all()


@pytest.mark.parametrize('dtype', ['float32', 'float64'])
def test_variance_with_unrepresentative_edges_and_sentinels(dtype):
    """Tightly clustered data far from zero, with padding / sentinel values at
    the places a sampled pivot would look (first, middle, last element) and
    elsewhere: a one-pass formula around such a pivot is off by tens of
    percent; the result must stay within the tolerance of a two-pass one."""
    rng = np.random.default_rng(92)
    rtol = 2e-5 if dtype == 'float32' else 1e-11
    n = 1 << 22
    x = (rng.standard_normal(n) * 0.1 + 100).astype(dtype)
    for bad in ([0, n - 1], [0, n // 2, n - 1], [0, 1, 2, 3, n // 2, n - 2, n - 1],
                list(range(0, n, 65537))):
        h = x.copy()
        h[bad] = 0
        want = h.astype(np.float64).var()
        np.testing.assert_allclose(cp.asarray(h).var().get(), want, rtol=rtol)
        np.testing.assert_allclose(cp.asarray(h).std(ddof=1).get(),
                                   h.astype(np.float64).std(ddof=1), rtol=rtol)
    # the same along rows and columns of a matrix, whole leading rows / columns padded
    m = (rng.standard_normal((2048, 1500)) * 0.01 + 100).astype(dtype)
    m[:3, :] = 0
    m[-2:, :] = 0
    m[:, :5] = 0
    m[:, 749:751] = 0
    m[:, -1] = 0
    d = cp.asarray(m)
    for axis in (0, 1, None):
        np.testing.assert_allclose(d.var(axis=axis).get(), m.astype(np.float64).var(axis=axis),
                                   rtol=rtol)
    # short rows and narrow matrices (other kernels), mean far from the spread
    for shape in ((100000, 7), (30000, 33), (7, 100000), (64, 4096)):
        h = (rng.standard_normal(shape) * 0.05 - 3000).astype(dtype)
        h[0] = 0
        h[:, 0] = 0
        d = cp.asarray(h)
        for axis in (0, 1):
            np.testing.assert_allclose(d.var(axis=axis).get(),
                                       h.astype(np.float64).var(axis=axis), rtol=rtol)
    # constant data has variance exactly zero, whatever the constant
    c = np.full((1000, 300), 123456.7, dtype)
    assert not cp.asarray(c).var(axis=0).get().any()
    assert not cp.asarray(c).var(axis=1).get().any()
    assert float(cp.asarray(c).var().get()) == 0.0


def test_narrow_scans_of_other_types_and_operations():
    """int8 -> int64, complex and products through the kernel that stages
    narrow arrays in the LDS."""
    rng = np.random.default_rng(94)
    h8 = rng.integers(-100, 100, (150001, 3)).astype(np.int8)
    assert np.array_equal(cp.cumsum(cp.asarray(h8), axis=0).get(), np.cumsum(h8, axis=0))
    hu = rng.integers(0, 255, (4, 30011, 7)).astype(np.uint8)
    assert np.array_equal(cp.cumsum(cp.asarray(hu), axis=1).get(), np.cumsum(hu, axis=1))
    hc = (rng.standard_normal((70001, 5)) + 1j * rng.standard_normal((70001, 5))).astype(np.complex64)
    got = cp.cumsum(cp.asarray(hc), axis=0).get()
    want = np.cumsum(hc.astype(np.complex128), axis=0)
    scale = np.cumsum(np.abs(hc).astype(np.float64), axis=0)
    assert (np.abs(got - want) <= 1e-5 * scale + 1e-5).all()
    hp = rng.choice(np.array([-1, 1, 1, 2], dtype=np.int64), size=(40, 6))
    hp = np.concatenate([hp, np.ones((60000, 6), np.int64)])
    rng.shuffle(hp, axis=0)
    assert np.array_equal(cp.cumprod(cp.asarray(hp), axis=0).get(), np.cumprod(hp, axis=0))
    hb = rng.integers(0, 2, (100000, 12)).astype(bool)
    assert np.array_equal(cp.cumsum(cp.asarray(hb), axis=0).get(), np.cumsum(hb, axis=0))
    out = cp.empty((150001, 3), np.float64)
    r = cp.cumsum(cp.asarray(h8), axis=0, out=out)
    assert r is out and np.array_equal(out.get(), np.cumsum(h8, axis=0, dtype=np.float64))


@pytest.mark.parametrize('shape', [(40000, 4, 4), (30001, 16, 2), (5000, 2, 32), (20011, 5, 3),
                                   (7001, 9, 7), (3, 100, 2), (100000, 3, 2), (1500, 33, 8),
                                   (2, 7, 4, 5), (9000, 3, 33), (701, 100, 63), (40, 5000, 64),
                                   (3, 20000, 40),
                                   # two or three slices to a round
                                   (3001, 100, 3), (2000, 150, 3), (3000, 60, 5), (999, 70, 7),
                                   (4001, 12, 31), (3000, 10, 33), (2500, 6, 48),
                                   # slices of several rounds, a wave each
                                   (1100, 300, 36), (1030, 257, 100), (1025, 500, 16),
                                   # wide rows, slices that fit the LDS of a workgroup
                                   (700, 16, 257), (300, 3, 1000), (50, 33, 100), (9, 2, 4096),
                                   (1000, 81, 100), (5, 8, 65), (2100, 7, 129)])
def test_scans_of_many_short_slices_with_a_narrow_tail(shape):
    """Slices of few rows: a wave stages many of them per round and starts
    over at every slice."""
    rng = np.random.default_rng(sum(shape))
    axis = len(shape) - 2
    h = rng.integers(-9, 10, shape).astype(np.int32)
    d = cp.asarray(h)
    assert (d.cumsum(axis=axis).get() == h.cumsum(axis=axis)).all()
    h8 = h.astype(np.int8)
    assert (cp.cumsum(cp.asarray(h8), axis=axis, dtype=np.int8).get()
            == h8.cumsum(axis=axis, dtype=np.int8)).all()
    assert (cp.cumsum(cp.asarray(h8), axis=axis).get() == h8.cumsum(axis=axis)).all()
    hp = np.where(rng.uniform(size=shape) < 0.2, -1, 1).astype(np.int64)
    assert (cp.cumprod(cp.asarray(hp), axis=axis).get() == hp.cumprod(axis=axis)).all()
    hf = rng.standard_normal(shape)
    got = cp.cumsum(cp.asarray(hf), axis=axis).get()
    # (sums of up to 20000 values combined in another order than NumPy's)
    bound = 1e-13 * np.cumsum(np.abs(hf), axis=axis) + 1e-15
    assert (np.abs(got - hf.cumsum(axis=axis)) <= bound).all()
    hn = rng.uniform(0, 1, shape).astype(np.float32)
    hn[..., ::3, 1] = np.nan
    got = cp.nancumsum(cp.asarray(hn), axis=axis).get()
    assert np.allclose(got, np.nancumsum(hn.astype(np.float64), axis=axis), rtol=1e-5, atol=1e-6)
    hc = (hf + 1j * rng.standard_normal(shape)).astype(np.complex64)
    got = cp.cumsum(cp.asarray(hc), axis=axis).get()
    assert np.allclose(got, hc.astype(np.complex128).cumsum(axis=axis), rtol=1e-4, atol=1e-4)
    # a view that does not start on a 16-byte boundary
    flat = rng.integers(-9, 10, h.size + 1).astype(np.int32)
    assert (cp.asarray(flat)[1:].reshape(shape).cumsum(axis=axis).get()
            == flat[1:].reshape(shape).cumsum(axis=axis)).all()


@pytest.mark.parametrize('shape', [(2000, 100, 33), (50, 257, 257), (300, 1024, 33), (7, 9, 1001),
                                   (3, 40, 4099), (1, 70000, 37), (5, 3, 65537)])
def test_column_scans_with_odd_numbers_of_columns(shape):
    """Rows that are no whole number of vectors: the last vector of a row
    overlaps its neighbour; in place the kernel falls back to single elements."""
    rng = np.random.default_rng(sum(shape))
    h = rng.integers(-9, 10, shape).astype(np.int32)
    d = cp.asarray(h)
    assert (d.cumsum(axis=1).get() == h.cumsum(axis=1)).all()
    out = cp.empty(shape, np.int32)
    cp.cumsum(d, axis=1, out=out)
    assert (out.get() == h.cumsum(axis=1)).all()
    inplace = d.copy()
    cp.cumsum(inplace, axis=1, out=inplace)
    assert (inplace.get() == h.cumsum(axis=1)).all()
    h8 = h.astype(np.int8)
    assert (cp.cumsum(cp.asarray(h8), axis=1).get() == h8.cumsum(axis=1)).all()
    hf = rng.standard_normal(shape)
    got = cp.cumsum(cp.asarray(hf), axis=1).get()
    assert np.allclose(got, hf.cumsum(axis=1), rtol=1e-12, atol=1e-10)
    hh = rng.uniform(0, 1, shape).astype(np.float16)
    got = cp.cumsum(cp.asarray(hh), axis=1, dtype=np.float32).get()
    assert np.allclose(got, hh.astype(np.float32).cumsum(axis=1), rtol=1e-4, atol=1e-3)
    flat = rng.integers(-9, 10, h.size + 1).astype(np.int32)
    assert (cp.asarray(flat)[1:].reshape(shape).cumsum(axis=1).get()
            == flat[1:].reshape(shape).cumsum(axis=1)).all()


@pytest.mark.parametrize('shape', [(40, 300, 257), (7, 1000, 100), (3, 70, 500), (5, 80, 129),
                                   (600, 40, 321)])
def test_scans_of_long_slices_of_rows_that_are_no_whole_vectors(shape):
    """A workgroup per slice, a few rows per round, running values carried from
    round to round (taken from two slices per CU on; here from the first)."""
    from cupy_amd._core import _tuning
    rng = np.random.default_rng(sum(shape))
    _tuning.set(scan_slab_long_slices_per_cu=0)
    try:
        h = rng.integers(-9, 10, shape).astype(np.int32)
        assert (cp.asarray(h).cumsum(axis=1).get() == h.cumsum(axis=1)).all()
        h8 = h.astype(np.int8)
        assert (cp.cumsum(cp.asarray(h8), axis=1, dtype=np.int8).get()
                == h8.cumsum(axis=1, dtype=np.int8)).all()
        assert (cp.cumsum(cp.asarray(h8), axis=1).get() == h8.cumsum(axis=1)).all()
        hp = np.where(rng.uniform(size=shape) < 0.2, -1, 1).astype(np.int64)
        assert (cp.cumprod(cp.asarray(hp), axis=1).get() == hp.cumprod(axis=1)).all()
        hf = rng.standard_normal(shape)
        hf[:, 0, :3] = -0.0
        got = cp.cumsum(cp.asarray(hf), axis=1).get()
        bound = 1e-13 * np.cumsum(np.abs(hf), axis=1) + 1e-15
        assert (np.abs(got - hf.cumsum(axis=1)) <= bound).all()
        assert np.signbit(got[:, 0, :3]).all()
        hn = rng.uniform(0, 1, shape).astype(np.float32)
        hn[:, ::3, 1] = np.nan
        got = cp.nancumsum(cp.asarray(hn), axis=1).get()
        assert np.allclose(got, np.nancumsum(hn.astype(np.float64), axis=1), rtol=1e-5, atol=1e-6)
        hh = rng.uniform(0, 1, shape).astype(np.float16)
        got = cp.cumsum(cp.asarray(hh), axis=1).get()
        assert np.allclose(got, hh.astype(np.float64).cumsum(axis=1), rtol=2e-3, atol=1e-2)
        # in place, and from a view that does not start on a 16-byte boundary
        d = cp.asarray(h)
        r = cp.cumsum(d, axis=1, out=d)
        assert r is d and (d.get() == h.cumsum(axis=1)).all()
        flat = rng.integers(-9, 10, h.size + 1).astype(np.int32)
        assert (cp.asarray(flat)[1:].reshape(shape).cumsum(axis=1).get()
                == flat[1:].reshape(shape).cumsum(axis=1)).all()
        from test_gpu_scan_chain import launched
        if shape[2] % 4:      # (rows of 500 floats are whole vectors: a thread per vector)
            floats = cp.asarray(h.astype(np.float32))
            assert 'cupy_scan_slab_long' in launched(lambda: floats.cumsum(axis=1))
        bytes_ = cp.asarray(h8)
        assert 'cupy_scan_slab_long' in launched(lambda: cp.cumsum(bytes_, axis=1, dtype=np.int8))
    finally:
        _tuning.set(scan_slab_long_slices_per_cu=2)


@pytest.mark.parametrize('shape,axis', [((1 << 20,), 0), ((1000, 1000), 0), ((1000, 1000), 1),
                                        ((3000, 7, 5), 1), ((200, 100, 100), 1), ((64, 1 << 14), 0),
                                        ((64, 1 << 14), 1), ((100000, 3), 0), ((16, 257, 257), 1),
                                        ((40, 3, 1000), 1), ((5000, 2, 64), 1), ((1 << 16, 40), 0)])
@pytest.mark.parametrize('dtype', [np.float32, np.float64, np.complex64])
def test_sums_of_negative_zeros_stay_negative(shape, axis, dtype):
    """-0.0 + -0.0 is -0.0 and anything else added to a zero gives +0.0: the
    signs of a scan of signed zeros do not depend on the order of the additions
    -- only on what a scan starts from (NumPy and the reference's in-place scan,
    cupy/_core/_routines_math.pyx:160-751, start from the first element)."""
    rng = np.random.default_rng(len(shape) + axis)
    h = np.where(rng.uniform(size=shape) < 2.0 / shape[axis], 0.0, -0.0).astype(dtype)
    if dtype == np.complex64:
        h.imag = np.where(rng.uniform(size=shape) < 2.0 / shape[axis], 0.0, -0.0)
    want = np.cumsum(h, axis=axis)
    got = cp.cumsum(cp.asarray(h), axis=axis).get()
    assert (np.signbit(got.real) == np.signbit(want.real)).all()
    if dtype == np.complex64:
        assert (np.signbit(got.imag) == np.signbit(want.imag)).all()
    else:
        hn = h.copy()
        hn.reshape(-1)[::7] = np.nan
        # (a NaN that is skipped counts as +0.0)
        want = np.nancumsum(hn, axis=axis)
        got = cp.nancumsum(cp.asarray(hn), axis=axis).get()
        assert (np.signbit(got) == np.signbit(want)).all()


@pytest.mark.parametrize('dtype', ['complex64', 'complex128'])
def test_nan_statistics_of_complex_values(dtype):
    """nanmean / nanvar / nanstd over complex values: an element counts as NaN
    if either part is; the variance is the mean squared modulus of the
    deviations, a real number (reference: _routines_statistics.pyx:686-700,
    732-800)."""
    rng = np.random.default_rng(8)
    h = (rng.standard_normal((9, 11, 5)) + 1j * rng.standard_normal((9, 11, 5))).astype(dtype)
    h[0, 0, 0] = np.nan
    h[3, 4, 1] = complex(1.0, np.nan)
    h[:, 7, 2] = np.nan                     # a whole slice along axis 0
    d = cp.asarray(h)
    rtol = 2e-5 if dtype == 'complex64' else 1e-12
    for kwargs in ({}, {'axis': 0}, {'axis': (0, 2)}, {'axis': 1, 'keepdims': True}, {'axis': -1}):
        for name in ('nanmean', 'nanvar', 'nanstd'):
            with np.errstate(all='ignore'), warnings.catch_warnings():
                warnings.simplefilter('ignore')
                want = getattr(np, name)(h, **kwargs)
            got = getattr(cp, name)(d, **kwargs)
            assert got.dtype == want.dtype and got.shape == np.shape(want), (name, kwargs)
            np.testing.assert_allclose(got.get(), want, rtol=rtol, atol=rtol, equal_nan=True)
    for name in ('nanvar', 'nanstd'):
        with np.errstate(all='ignore'):
            want = getattr(np, name)(h, axis=1, ddof=1)
        np.testing.assert_allclose(getattr(cp, name)(d, axis=1, ddof=1).get(), want, rtol=rtol, atol=rtol,
                                   equal_nan=True)
    out = cp.empty((9, 5), want.dtype)
    assert cp.nanvar(d, axis=1, out=out) is out
    np.testing.assert_allclose(out.get(), np.nanvar(h, axis=1), rtol=rtol, atol=rtol, equal_nan=True)


def test_nanmean_of_real_values_with_a_complex_result_type():
    rng = np.random.default_rng(12)
    for dtype in ('float16', 'float32', 'float64'):
        h = rng.standard_normal((7, 9)).astype(dtype)
        h[2, 3] = np.nan
        d = cp.asarray(h)
        for out in ('complex64', 'complex128'):
            for kwargs in ({}, {'axis': 0}, {'axis': 1}):
                want = np.nanmean(h, dtype=out, **kwargs)
                got = cp.nanmean(d, dtype=out, **kwargs)
                assert got.dtype == want.dtype
                np.testing.assert_allclose(got.get(), want, rtol=2e-3 if dtype == 'float16' else 1e-5)
