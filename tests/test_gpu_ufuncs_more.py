"""The rest of the real-valued ufunc catalogue against NumPy on the same seeded
inputs: integer and boolean results bit-exact, floating-point results within a
few ulp (the device's math library is not NumPy's libm: parity of those
functions is checked to the reference's own tolerance,
tests/cupy_tests/math_tests/*: ``numpy_cupy_allclose(atol=1e-5)``)."""
import warnings

import numpy as np
import pytest

import cupy_amd as cp
from helpers import assert_exact

pytestmark = pytest.mark.gpu

FLOATS = [np.float16, np.float32, np.float64]
INTS = [np.int8, np.uint8, np.int32, np.int64, np.uint64]


def _tol(dtype):
    return {np.float16: 2e-3, np.float32: 2e-6, np.float64: 1e-13}[dtype]


def _f(rng, dtype, n=4099, lo=-4, hi=4):
    return rng.uniform(lo, hi, n).astype(dtype)


@pytest.mark.parametrize('dtype', FLOATS)
def test_float_unary_and_binary(dtype):
    rng = np.random.default_rng(31)
    x = _f(rng, dtype)
    y = _f(rng, dtype)
    x[:7] = [0.0, -0.0, np.inf, -np.inf, np.nan, 1.0, -1.0]
    y[:7] = [1.0, 0.0, -np.inf, 2.0, 3.0, np.nan, -1.0]
    dx, dy = cp.asarray(x), cp.asarray(y)
    tol = _tol(dtype)
    with np.errstate(all='ignore'):
        assert_exact(cp.fabs(dx).get(), np.fabs(x))
        assert_exact(cp.heaviside(dx, dy).get(), np.heaviside(x, y))
        np.testing.assert_allclose(cp.fmod(dx, dy).get(), np.fmod(x, y), rtol=tol, atol=tol)
        nz = x != 0        # NumPy's float16 sinc(0) is NaN (its 1e-20 stand-in for 0 underflows)
        np.testing.assert_allclose(cp.sinc(dx).get()[nz], np.sinc(x)[nz], rtol=20 * tol, atol=20 * tol)
        assert np.all(cp.sinc(dx).get()[~nz] == 1)
        np.testing.assert_allclose(cp.logaddexp(dx, dy).get(), np.logaddexp(x, y), rtol=4 * tol, atol=4 * tol)
        np.testing.assert_allclose(cp.logaddexp2(dx, dy).get(), np.logaddexp2(x, y), rtol=4 * tol, atol=4 * tol)
        np.testing.assert_allclose(cp.deg2rad(dx).get(), np.deg2rad(x), rtol=2 * tol)
        np.testing.assert_allclose(cp.rad2deg(dx).get(), np.rad2deg(x), rtol=2 * tol)
        np.testing.assert_allclose(cp.radians(dx).get(), np.radians(x), rtol=2 * tol)
        np.testing.assert_allclose(cp.degrees(dx).get(), np.degrees(x), rtol=2 * tol)
        assert_exact(cp.nextafter(dx, dy).get(), np.nextafter(x, y))
        m, e = cp.frexp(dx)
        hm, he = np.frexp(x)
        fin = np.isfinite(x)
        assert_exact(m.get()[fin], hm[fin])
        assert_exact(e.get()[fin], he[fin])
        fr, ip = cp.modf(dx)
        hf, hi = np.modf(x)
        assert_exact(fr.get(), hf)
        assert_exact(ip.get(), hi)
        k = rng.integers(-20, 20, x.size).astype(np.int32)
        assert_exact(cp.ldexp(dx, cp.asarray(k)).get(), np.ldexp(x, k))
        assert_exact(cp.ldexp(dx, cp.asarray(k.astype(np.int64))).get(), np.ldexp(x, k.astype(np.int64)))
        assert_exact(cp.isclose(dx, dy).get(), np.isclose(x, y))
        assert_exact(cp.isclose(dx, dx + dtype(1e-3), rtol=1e-2, equal_nan=True).get(),
                     np.isclose(x, x + dtype(1e-3), rtol=1e-2, equal_nan=True))
        assert bool(cp.allclose(dx, dx, equal_nan=True).get())
        assert not bool(cp.allclose(dx, dy).get())
        assert_exact(cp.nan_to_num(dx).get(), np.nan_to_num(x))
        assert_exact(cp.nan_to_num(dx, nan=1.5, posinf=7.0, neginf=-7.0).get(),
                     np.nan_to_num(x, nan=1.5, posinf=7.0, neginf=-7.0))
        assert_exact(cp.clip(dx, -1, 1).get(), np.clip(x, -1, 1))
        assert_exact(cp.clip(dx, None, 0.5).get(), np.clip(x, None, 0.5))
        assert_exact(cp.clip(dx, dy, None).get(), np.clip(x, y, None))
        q, r = cp.divmod(dx, dy)
        hq, hr = np.divmod(x, y)
        np.testing.assert_allclose(q.get(), hq, rtol=tol, atol=tol)
        np.testing.assert_allclose(r.get(), hr, rtol=tol, atol=4 * tol)
    if dtype is not np.float16:
        xs = _f(rng, dtype, lo=-30, hi=30)
        np.testing.assert_allclose(cp.i0(cp.asarray(xs)).get(), np.i0(xs), rtol=1e-5 if dtype is np.float32 else 1e-12)
    np.testing.assert_allclose(cp.float_power(cp.asarray(np.abs(x[7:])), 1.5).get(),
                               np.float_power(np.abs(x[7:]), 1.5), rtol=1e-14)


@pytest.mark.parametrize('dtype', INTS)
def test_integer_functions_exact(dtype):
    rng = np.random.default_rng(32)
    info = np.iinfo(dtype)
    lo = max(info.min, -10 ** 6)
    hi = min(info.max, 10 ** 6)
    x = rng.integers(lo, hi, 5001, dtype=np.int64).astype(dtype)
    y = rng.integers(lo, hi, 5001, dtype=np.int64).astype(dtype)
    y[::17] = 0
    x[:3] = [0, info.max, info.min]
    dx, dy = cp.asarray(x), cp.asarray(y)
    with np.errstate(all='ignore'):
        assert_exact(cp.gcd(dx, dy).get(), np.gcd(x, y))
        m = 10 if info.max < 1000 else 1000          # keeps the products in range
        small = (x % dtype(m)).astype(dtype), (y % dtype(m)).astype(dtype)
        assert_exact(cp.lcm(cp.asarray(small[0]), cp.asarray(small[1])).get(), np.lcm(*small))
        assert_exact(cp.fmod(dx, dy).get(), np.fmod(x, y))
        if info.min < 0 and dtype is not np.int64:
            assert_exact(cp.bitwise_count(dx).get(), np.bitwise_count(x))
        elif info.min == 0:
            assert_exact(cp.bitwise_count(dx).get(), np.bitwise_count(x))
        q, r = cp.divmod(dx, dy)
        hq, hr = np.divmod(x, y)
        assert_exact(q.get(), hq)
        assert_exact(r.get(), hr)
        assert_exact(cp.clip(dx, 3, 77).get(), np.clip(x, 3, 77))
        assert_exact(cp.nan_to_num(dx).get(), x)
    cond = rng.integers(0, 2, x.size).astype(bool)
    assert_exact(cp.where(cp.asarray(cond), dx, dy).get(), np.where(cond, x, y))
    assert_exact(cp.where(dx, dx, 1).get(), np.where(x, x, 1))
    assert_exact(cp.isclose(dx, dy).get(), np.isclose(x, y))


def test_boolean_inputs_and_errors():
    b = cp.asarray(np.array([True, False, True]))
    with pytest.raises(TypeError):
        cp.gcd(b, b)
    with pytest.raises(TypeError):
        cp.lcm(b, b)
    assert_exact(cp.bitwise_count(b).get(), np.bitwise_count(np.array([True, False, True])))
    with pytest.raises(ValueError):
        cp.clip(b, None, None)
    with pytest.raises(NotImplementedError):
        cp.where(b)


def test_accumulate_follows_cumsum_and_cumprod():
    rng = np.random.default_rng(33)
    h = rng.integers(1, 4, (30, 40)).astype(np.int64)
    d = cp.asarray(h)
    assert_exact(cp.add.accumulate(d, axis=1).get(), np.add.accumulate(h, axis=1))
    assert_exact(cp.add.accumulate(d).get(), np.add.accumulate(h))
    small = rng.integers(1, 3, (6, 9)).astype(np.int64)
    assert_exact(cp.multiply.accumulate(cp.asarray(small), axis=1).get(),
                 np.multiply.accumulate(small, axis=1))
    with pytest.raises(NotImplementedError):
        cp.maximum.accumulate(d)


def test_int64_against_uint64_compares_values():
    a = np.array([-1, 0, 1, -2**63, 2**63 - 1, 5, 7], np.int64)
    b = np.array([2**64 - 1, 0, 1, 2**63, 2**63 - 1, 2**63 + 5, 6], np.uint64)
    da, db = cp.asarray(a), cp.asarray(b)
    for name in ('equal', 'not_equal', 'less', 'less_equal', 'greater', 'greater_equal'):
        assert_exact(getattr(cp, name)(da, db).get(), getattr(np, name)(a, b))
        assert_exact(getattr(cp, name)(db, da).get(), getattr(np, name)(b, a))
    # the array API names are the same objects
    assert cp.acos is cp.arccos and cp.atan2 is cp.arctan2 and cp.pow is cp.power
    assert cp.bitwise_invert is cp.invert and cp.bitwise_left_shift is cp.left_shift


def test_around_follows_numpy():
    rng = np.random.default_rng(77)
    for dtype in ('float16', 'float32', 'float64'):
        x = (rng.standard_normal(2000) * 100).astype(dtype)
        x[:8] = [0.5, 1.5, 2.5, -0.5, -1.5, 0.125, 0.375, 2.675]
        d = cp.asarray(x)
        for decimals in (0, 1, 2, -1):
            assert_exact(cp.around(d, decimals).get(), np.around(x, decimals))
        assert_exact(d.round(1).get(), x.round(1))
        assert_exact(cp.fix(d).get(), np.fix(x))
    i = rng.integers(-1000, 1000, 500).astype(np.int32)
    i[:6] = [15, 25, 35, -15, -25, 5]
    di = cp.asarray(i)
    for decimals in (0, 2, -1, -2):
        assert_exact(cp.around(di, decimals).get(), np.around(i, decimals))
    z = (rng.standard_normal(300) + 1j * rng.standard_normal(300)).astype(np.complex64) * 10
    assert_exact(cp.around(cp.asarray(z), 1).get(), np.around(z, 1))
    out = cp.zeros(2000, np.float64)
    r = cp.around(cp.asarray(x), 2, out=out)
    assert r is out
    assert_exact(out.get(), np.around(x, 2))

    @cp.fuse()
    def f(a):
        return cp.around(a * 3, 1) + cp.real(a)
    x32 = x.astype(np.float32)
    assert_exact(f(cp.asarray(x32)).get(), np.around(x32 * 3, 1) + np.real(x32))


def test_python_integers_outside_the_arrays_type():
    """A Python integer that does not fit the arrays' integer type: loops that
    answer in another kind (comparisons, true division, logical functions)
    compute with its value as NumPy does; loops with integer results raise as
    NumPy does."""
    for dtype in ('uint8', 'int8', 'uint64'):
        h = np.array([0, 1, 5, 100], dtype)
        d = cp.asarray(h)
        for value in (-1, 300, -(1 << 40)):
            for name in ('equal', 'not_equal', 'less', 'greater_equal', 'true_divide',
                         'logical_xor', 'logical_and'):
                with np.errstate(all='ignore'):
                    want = getattr(np, name)(h, value)
                    back = getattr(np, name)(value, h)
                got = getattr(cp, name)(d, value)
                assert got.dtype == want.dtype, (name, dtype, value)
                np.testing.assert_array_equal(got.get(), want)
                np.testing.assert_array_equal(getattr(cp, name)(value, d).get(), back)
            assert np.array_equal((d == value).get(), h == value)
            assert np.array_equal((value > d).get(), value > h)
            for name in ('add', 'maximum', 'floor_divide', 'bitwise_and'):
                info = np.iinfo(dtype)
                if info.min <= value <= info.max:
                    continue
                with pytest.raises(OverflowError):
                    getattr(np, name)(h, value)
                with pytest.raises(OverflowError):
                    getattr(cp, name)(d, value)


def test_where_keyword_and_input_casts_under_dtype():
    """``where=`` as NumPy spells it (elements it leaves out keep what ``out``
    held), and ``dtype=``: the arrays must be castable to the chosen loop's
    inputs under the casting rule."""
    rng = np.random.default_rng(2)
    h = rng.standard_normal((5, 7)).astype(np.float32)
    g = rng.standard_normal((5, 7)).astype(np.float32)
    mask = rng.integers(0, 2, (5, 7)).astype(bool)
    d, e, dm = cp.asarray(h), cp.asarray(g), cp.asarray(mask)
    want = np.full((5, 7), 9, np.float32)
    np.add(h, g, out=want, where=mask)
    out = cp.asarray(np.full((5, 7), 9, np.float32))
    assert cp.add(d, e, out=out, where=dm) is out
    np.testing.assert_array_equal(out.get(), want)
    np.testing.assert_array_equal(cp.add(d, e, where=True).get(), h + g)
    row = mask[0]
    want = np.full((5, 7), 3, np.float64)
    np.multiply(h, 2, out=want, where=row)
    out = cp.asarray(np.full((5, 7), 3, np.float64))
    cp.multiply(d, 2, out=out, where=cp.asarray(row))
    np.testing.assert_array_equal(out.get(), want)

    z = (rng.standard_normal(6) + 1j * rng.standard_normal(6)).astype(np.complex128)
    dz = cp.asarray(z)
    for casting in ('same_kind', 'safe'):
        with pytest.raises(TypeError):
            np.multiply(z, 2.0, dtype=np.float64, casting=casting)
        with pytest.raises(TypeError):
            cp.multiply(dz, 2.0, dtype=np.float64, casting=casting)
    with warnings.catch_warnings():
        warnings.simplefilter('ignore')
        want = np.multiply(z, 2.0, dtype=np.float64, casting='unsafe')
        got = cp.multiply(dz, 2.0, dtype=np.float64, casting='unsafe')
    np.testing.assert_array_equal(got.get(), want)
    i = np.arange(6, dtype=np.int64)
    with pytest.raises(TypeError):
        cp.negative(cp.asarray(i), dtype=np.uint8)
    with pytest.raises(TypeError):
        cp.true_divide(cp.asarray(i.astype(np.uint64)), cp.asarray(i.astype(np.uint32)), dtype=np.float32,
                       casting='safe')
    np.testing.assert_array_equal(cp.add(cp.asarray(i.astype(np.int16)), 1, dtype=np.float64).get(),
                                  np.add(i.astype(np.int16), 1, dtype=np.float64))


@pytest.mark.parametrize('out_dtype', ['uint64', 'bool', 'int8', 'float32', 'complex64'])
def test_where_into_an_output_of_another_type_keeps_the_skipped_elements(out_dtype):
    h = np.arange(0, 12, dtype=np.int8)          # (negative floats into unsigned types are undefined)
    g = np.full(12, 3, np.int64)
    mask = (np.arange(12) % 3 != 1)
    d, e, dm = cp.asarray(h), cp.asarray(g), cp.asarray(mask)
    for name, casting in (('less', 'same_kind'), ('logical_and', 'unsafe'), ('add', 'unsafe'),
                          ('true_divide', 'unsafe')):
        want = np.full(12, 7).astype(out_dtype)
        try:
            getattr(np, name)(h, g, out=want, where=mask, casting=casting)
        except TypeError:
            with pytest.raises(TypeError):
                getattr(cp, name)(d, e, out=cp.asarray(np.full(12, 7).astype(out_dtype)), where=dm,
                                  casting=casting)
            continue
        out = cp.asarray(np.full(12, 7).astype(out_dtype))
        assert getattr(cp, name)(d, e, out=out, where=dm, casting=casting) is out
        np.testing.assert_array_equal(out.get(), want)
