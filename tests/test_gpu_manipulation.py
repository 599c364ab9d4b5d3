"""The functions either side of the generated kernels (views with other axes,
the Array-API scans, compositions of ufuncs and reductions, linspace,
isclose over complex values) against NumPy on the same inputs."""
import numpy as np
import pytest

import cupy_amd as cp

pytestmark = pytest.mark.gpu


def pair(shape, dtype='float32', seed=0):
    rng = np.random.default_rng(seed)
    h = rng.integers(-5, 6, size=shape).astype(dtype)
    return h, cp.asarray(h)


@pytest.mark.parametrize('src,dst', [(0, -1), (-1, 0), ((0, 1), (2, 0)), (1, 1), ((2, 0), (0, 1))])
def test_moveaxis_values(src, dst):
    h, d = pair((3, 4, 5))
    want = np.moveaxis(h, src, dst)
    got = cp.moveaxis(d, src, dst)
    assert got.strides == want.strides
    assert np.array_equal(got.get(), want)
    assert np.array_equal((got + 1).get(), want + 1)


def test_axis_views_compute_like_numpy():
    h, d = pair((3, 4, 5))
    assert np.array_equal(cp.rollaxis(d, 2, 0).get(), np.rollaxis(h, 2, 0))
    assert np.array_equal(cp.swapaxes(d, 0, 2).get(), np.swapaxes(h, 0, 2))
    assert np.array_equal(cp.expand_dims(d, (0, 3)).get(), np.expand_dims(h, (0, 3)))
    assert np.array_equal(cp.squeeze(cp.expand_dims(d, 1), 1).get(), h)
    assert np.array_equal(cp.flip(d).get(), np.flip(h))
    assert np.array_equal(cp.flip(d, (0, 2)).get(), np.flip(h, (0, 2)))
    assert np.array_equal(cp.fliplr(d).get(), np.fliplr(h))
    assert np.array_equal(cp.flipud(d).get(), np.flipud(h))
    assert np.array_equal(cp.flip(d, 1).sum(axis=1).get(), np.flip(h, 1).sum(axis=1))
    x, y = cp.broadcast_arrays(d[:, :1, :], d[:1, :, 0:1])
    hx, hy = np.broadcast_arrays(h[:, :1, :], h[:1, :, 0:1])
    assert np.array_equal(x.get(), hx) and np.array_equal(y.get(), hy)
    assert np.array_equal((x * y).get(), hx * hy)
    h1, d1 = pair((7,))
    for fn in ('atleast_1d', 'atleast_2d', 'atleast_3d'):
        assert np.array_equal(getattr(cp, fn)(d1).get(), getattr(np, fn)(h1))
        assert np.array_equal(getattr(cp, fn)(d).get(), getattr(np, fn)(h))
    with pytest.raises(np.exceptions.AxisError):
        cp.moveaxis(d, 3, 0)
    with pytest.raises(ValueError):
        cp.moveaxis(d, (0, 1), (0,))


@pytest.mark.parametrize('dtype', ['int8', 'uint16', 'int64', 'float32', 'float64', 'bool'])
@pytest.mark.parametrize('fn', ['cumulative_sum', 'cumulative_prod'])
def test_cumulative_scans(fn, dtype):
    rng = np.random.default_rng(3)
    if fn == 'cumulative_prod':
        h = np.where(rng.random((6, 37)) < 0.1, 2, 1).astype(dtype)
    else:
        h = rng.integers(0, 4, size=(6, 37)).astype(dtype)
    d = cp.asarray(h)
    for axis in (0, 1, -1):
        for initial in (False, True):
            want = getattr(np, fn)(h, axis=axis, include_initial=initial)
            got = getattr(cp, fn)(d, axis=axis, include_initial=initial)
            assert got.dtype == want.dtype and got.shape == want.shape
            assert np.array_equal(got.get(), want)
    want = getattr(np, fn)(h[0], include_initial=True, dtype=np.float64)
    got = getattr(cp, fn)(d[0], include_initial=True, dtype=np.float64)
    assert got.dtype == want.dtype and np.array_equal(got.get(), want)
    out = cp.empty((6, 38), np.float64)
    assert getattr(cp, fn)(d, axis=1, include_initial=True, out=out) is out
    assert np.array_equal(out.get(), getattr(np, fn)(h, axis=1, include_initial=True, dtype=np.float64))
    with pytest.raises(ValueError):
        getattr(cp, fn)(d)
    with pytest.raises(ValueError):
        getattr(cp, fn)(d, axis=0, out=cp.empty((6, 37), np.float64), include_initial=True)


def test_signed_infinities_and_equality():
    h = np.array([-np.inf, -4, np.nan, 0, 4, np.inf], np.float32)
    d = cp.asarray(h)
    assert np.array_equal(cp.isneginf(d).get(), np.isneginf(h))
    assert np.array_equal(cp.isposinf(d).get(), np.isposinf(h))
    with pytest.raises(TypeError):
        cp.isneginf(cp.asarray(np.array([1j], np.complex64)))
    assert bool(cp.array_equal(d, d)) is False           # NaN differs from itself
    assert bool(cp.array_equal(d, d, equal_nan=True)) is True
    assert bool(cp.array_equal(d[:3], d[3:])) is False
    assert bool(cp.array_equal(d[:2], d[:3])) is False
    i, di = pair((4, 5), 'int32')
    assert bool(cp.array_equal(di, di.copy(), equal_nan=True)) is True
    assert bool(cp.array_equiv(di, di[:1])) == np.array_equiv(i, i[:1])
    assert bool(cp.array_equiv(di[:1], cp.broadcast_to(di[:1], (4, 5)))) is True
    assert bool(cp.array_equiv(di, di[:, :3])) is False


def test_isclose_over_complex_values():
    a = np.array([1 + 1j, 1 + 1.00001j, np.nan + 0j, np.inf + 0j, 1e10 + 1e-7j, 2 - 3j], np.complex64)
    b = np.array([1 + 1j, 1 + 1j, np.nan + 0j, np.inf + 0j, 1.00001e10 + 0j, 2 + 3j], np.complex64)
    for equal_nan in (False, True):
        want = np.isclose(a, b, equal_nan=equal_nan)
        got = cp.isclose(cp.asarray(a), cp.asarray(b), equal_nan=equal_nan)
        assert np.array_equal(got.get(), want)
    a128, b128 = a.astype(np.complex128), b.astype(np.complex128)
    assert np.array_equal(cp.isclose(cp.asarray(a128), cp.asarray(b128), rtol=1e-3).get(),
                          np.isclose(a128, b128, rtol=1e-3))
    # a complex operand against a real one
    r = np.array([1, 1, 0, 1, 1e10, 2], np.float32)
    assert np.array_equal(cp.isclose(cp.asarray(a), cp.asarray(r)).get(), np.isclose(a, r))
    assert bool(cp.allclose(cp.asarray(a128[:2]), cp.asarray(b128[:2]), atol=1e-4))


def test_average():
    h, d = pair((5, 6, 7), 'float64')
    w = np.arange(1, 7, dtype=np.float64)
    dw = cp.asarray(w)
    np.testing.assert_allclose(cp.average(d).get(), np.average(h), rtol=1e-12)
    np.testing.assert_allclose(cp.average(d, axis=1).get(), np.average(h, axis=1), rtol=1e-12)
    np.testing.assert_allclose(cp.average(d, axis=1, weights=dw).get(),
                               np.average(h, axis=1, weights=w), rtol=1e-12)
    got, scl = cp.average(d, axis=1, weights=dw, returned=True, keepdims=True)
    want, hscl = np.average(h, axis=1, weights=w, returned=True, keepdims=True)
    np.testing.assert_allclose(got.get(), want, rtol=1e-12)
    assert scl.shape == hscl.shape and np.array_equal(scl.get(), hscl)
    i, di = pair((4, 9), 'int16')
    wi = np.arange(9, dtype=np.int32)
    got = cp.average(di, axis=1, weights=cp.asarray(wi))
    want = np.average(i, axis=1, weights=wi)
    assert got.dtype == want.dtype
    np.testing.assert_allclose(got.get(), want, rtol=1e-12)
    full = np.abs(h) + 1
    np.testing.assert_allclose(cp.average(d, weights=cp.asarray(full)).get(),
                               np.average(h, weights=full), rtol=1e-12)
    with pytest.raises(ZeroDivisionError):
        cp.average(d, axis=1, weights=cp.zeros(6))
    with pytest.raises(TypeError):
        cp.average(d, weights=dw)
    with pytest.raises(ValueError):
        cp.average(d, axis=0, weights=dw)


@pytest.mark.parametrize('args,kwargs', [
    ((0, 1, 11), {}), ((0, 10, 5), {'dtype': int}), ((2.5, -3, 50), {}),
    ((0, 1, 7), {'endpoint': False}), ((1, 1, 4), {}), ((0, 1, 1), {}), ((0, 1, 0), {}),
    ((0, 1, 1), {'endpoint': False}), ((0, 5e-324, 4), {}), ((-7, 7, 1000), {'dtype': np.float32}),
    ((0, 100, 13), {'dtype': np.int8}),
])
def test_linspace(args, kwargs):
    want, hstep = np.linspace(*args, retstep=True, **kwargs)
    got, step = cp.linspace(*args, retstep=True, **kwargs)
    assert got.dtype == want.dtype and got.shape == want.shape
    np.testing.assert_allclose(got.get(), want, rtol=1e-14 if want.dtype == np.float64 else 1e-6, atol=0)
    assert step == hstep or (np.isnan(step) and np.isnan(hstep))
    if want.size > 1 and kwargs.get('endpoint', True):
        assert got.get()[-1] == want[-1]
    assert np.array_equal(cp.linspace(*args, **kwargs).get(), got.get())


def test_linspace_refuses_what_numpy_refuses():
    with pytest.raises(ValueError):
        cp.linspace(0, 1, -1)


def test_conversions_and_type_names():
    h, d = pair((3, 4), 'int32')
    assert cp.astype(d, np.float32).dtype == np.float32
    assert cp.astype(d, np.int32, copy=False) is d
    with pytest.raises(TypeError):
        cp.astype(h, np.float32)
    f = cp.asfortranarray(d)
    assert f.flags.f_contiguous and np.array_equal(f.get(), h)
    assert cp.asanyarray(d) is d
    assert cp.size(d) == 12 and cp.size(d, 1) == 4 and cp.shape(d) == (3, 4) and cp.ndim(d) == 2
    assert cp.isscalar(3.0) and not cp.isscalar(d)
    assert cp.issubdtype(d.dtype, cp.integer) and cp.finfo(cp.float16).bits == 16
    assert cp.broadcast_shapes((3, 1), (4,)) == (3, 4)
