"""``ufunc.at`` and ``add.reduceat`` against NumPy (the behaviour the reference
has for add, subtract, maximum, minimum and the bitwise ufuncs,
cupy/_core/_kernel.pyx:1447-1456,1485-1493).  Integer and boolean results are
bit-exact whatever order the atomic updates land in; floating-point sums are
held to the tolerance of a sum (the order of the additions is not fixed)."""
import numpy as np
import pytest

import cupy_amd as cp

pytestmark = pytest.mark.gpu

INT_DTYPES = ['int8', 'int16', 'int32', 'int64', 'uint8', 'uint16', 'uint32', 'uint64']
FLOAT_DTYPES = ['float16', 'float32', 'float64']


def _names(dtype):
    kind = np.dtype(dtype).kind
    if kind == 'b':
        return ['add', 'maximum', 'minimum', 'bitwise_and', 'bitwise_or', 'bitwise_xor']
    if kind in 'iu':
        return ['add', 'subtract', 'maximum', 'minimum', 'bitwise_and', 'bitwise_or', 'bitwise_xor']
    if kind == 'f':
        return ['add', 'subtract', 'maximum', 'minimum']
    return ['add', 'subtract']


def _check(name, a, indices, b, exact):
    want = a.copy()
    with np.errstate(all='ignore'):
        getattr(np, name).at(want, indices, b)
    d = cp.asarray(a)
    dev_indices = indices
    getattr(cp, name).at(d, dev_indices, cp.asarray(b) if isinstance(b, np.ndarray) else b)
    got = d.get()
    assert got.dtype == want.dtype
    if exact:
        assert np.array_equal(got, want, equal_nan=True), (name, a.dtype)
    else:
        # the same addends in another order: bound by rtol * sum of |addends| per element
        mag = np.abs(a).astype(np.float64)
        np.add.at(mag, indices, np.abs(np.asarray(b, dtype=np.float64)))
        rtol = {2: 2e-2, 4: 1e-5, 8: 1e-12}[np.dtype(a.dtype).itemsize if a.dtype.kind == 'f'
                                          else a.dtype.itemsize // 2]
        err = np.abs(got.astype(np.complex128) - want.astype(np.complex128))
        assert np.all(err <= rtol * mag + 1e-300), (name, a.dtype, float(err.max()))


@pytest.mark.parametrize('dtype', INT_DTYPES + ['bool'])
def test_at_with_repeated_indices_is_exact_for_integers(dtype):
    rng = np.random.default_rng(60)
    n = 1000
    if dtype == 'bool':
        a = rng.integers(0, 2, n).astype(bool)
        b = rng.integers(0, 2, 50000).astype(bool)
    else:
        a = rng.integers(0, 100, n).astype(dtype)
        b = rng.integers(0, 100, 50000).astype(dtype)
    idx = rng.integers(0, n, 50000)            # every element is hit about 50 times
    for name in _names(dtype):
        _check(name, a, idx, b, True)
        # (a scalar of the array's own type: with a Python int NumPy's `at`
        # computes uint64 operands in float64)
        _check(name, a, idx, b[0], True)
    # device indices and negative indices
    d = cp.asarray(a)
    cp.add.at(d, cp.asarray(idx - n), cp.asarray(b))
    want = a.copy()
    np.add.at(want, idx - n, b)
    assert np.array_equal(d.get(), want)


@pytest.mark.parametrize('dtype', FLOAT_DTYPES + ['complex64', 'complex128'])
def test_at_floating_point(dtype):
    rng = np.random.default_rng(61)
    n = 500
    if np.dtype(dtype).kind == 'c':
        a = (rng.standard_normal(n) + 1j * rng.standard_normal(n)).astype(dtype)
        b = (rng.standard_normal(20000) + 1j * rng.standard_normal(20000)).astype(dtype)
    else:
        a = rng.standard_normal(n).astype(dtype)
        b = rng.standard_normal(20000).astype(dtype)
    idx = rng.integers(0, n, 20000)
    for name in _names(dtype):
        _check(name, a, idx, b, name in ('maximum', 'minimum'))
    if np.dtype(dtype).kind == 'f':
        # NaN wins a maximum / minimum, wherever it arrives
        b2 = b.copy()
        b2[::997] = np.nan
        _check('maximum', a, idx, b2, True)
        _check('minimum', a, idx, b2, True)
        # a sum that is exact in any order: small integers stored as floats
        ai = rng.integers(0, 8, n).astype(dtype)
        bi = rng.integers(0, 4, 2000).astype(dtype)
        ii = rng.integers(0, n, 2000)
        _check('add', ai, ii, bi, True)
        _check('subtract', ai, ii, bi, True)


def test_at_with_several_index_arrays_and_trailing_axes():
    rng = np.random.default_rng(62)
    a = rng.integers(0, 50, (6, 7, 5)).astype(np.int32)
    i0 = rng.integers(0, 6, 400)
    i1 = rng.integers(-7, 7, 400)
    i2 = rng.integers(0, 5, 400)
    _check('add', a, (i0, i1, i2), rng.integers(0, 9, 400).astype(np.int32), True)
    _check('add', a, (i0, i1), rng.integers(0, 9, (400, 5)).astype(np.int32), True)   # rows of 5
    _check('maximum', a, (i0,), rng.integers(0, 99, (400, 7, 5)).astype(np.int32), True)
    _check('add', a, 3, rng.integers(0, 9, (7, 5)).astype(np.int32), True)
    _check('add', a, (2, i1[:30]), 1, True)
    _check('bitwise_xor', a, (i0.reshape(20, 20), i1.reshape(20, 20)), 5, True)
    _check('add', a, (i0[:3, None], i1[None, :4]), np.arange(5, dtype=np.int32), True)   # broadcast
    # one element, and nothing at all
    _check('subtract', a, (1, 2, 3), 7, True)
    _check('add', a, np.zeros(0, np.int64), 1, True)
    # a view: only the view's elements change
    base = rng.integers(0, 50, (10, 12)).astype(np.int64)
    d = cp.asarray(base)
    cp.add.at(d[::2, 1::3], ([0, 0, 4], [1, 1, 3]), 10)
    want = base.copy()
    np.add.at(want[::2, 1::3], ([0, 0, 4], [1, 1, 3]), 10)
    assert np.array_equal(d.get(), want)


def test_at_errors():
    a = cp.asarray(np.zeros((4, 3), np.float32))
    with pytest.raises(IndexError):
        cp.add.at(a, [4], 1)
    with pytest.raises(IndexError):
        cp.add.at(a, ([0], [0], [0]), 1)
    with pytest.raises(NotImplementedError):
        cp.multiply.at(a, [0], 2)
    with pytest.raises(NotImplementedError):
        cp.add.at(a, (slice(None), [0]), 1)
    with pytest.raises(TypeError):
        cp.bitwise_and.at(a, [0], 1)
    with pytest.raises(TypeError):
        cp.subtract.at(cp.asarray(np.zeros(3, bool)), [0], True)
    with pytest.raises(ValueError):
        cp.add.at(a, [0])


@pytest.mark.parametrize('dtype', ['int8', 'uint16', 'int64', 'float16', 'float32', 'float64',
                                   'complex64', 'bool'])
def test_add_reduceat(dtype):
    rng = np.random.default_rng(63)
    if dtype == 'bool':
        a = rng.integers(0, 2, (9, 40)).astype(bool)
    elif np.dtype(dtype).kind == 'c':
        a = (rng.standard_normal((9, 40)) + 1j * rng.standard_normal((9, 40))).astype(dtype)
    else:
        a = (rng.standard_normal((9, 40)) * 10).astype(dtype)
    d = cp.asarray(a)
    for indices, axis in (([0, 10, 25], 1), ([0, 4, 2, 8, 8, 3], 0), ([39], 1), ([5, 1, 1, 0], -1),
                          ([0], 0)):
        want = np.add.reduceat(a, indices, axis=axis)
        got = cp.add.reduceat(d, indices, axis=axis)
        assert got.dtype == want.dtype and got.shape == want.shape
        if np.dtype(dtype).kind in 'biu':
            assert np.array_equal(got.get(), want)
        else:
            rtol = {'float16': 2e-2, 'float32': 1e-5, 'float64': 1e-12, 'complex64': 1e-5}[dtype]
            mag = np.add.reduceat(np.abs(a).astype(np.float64), indices, axis=axis)
            assert np.all(np.abs(got.get().astype(np.complex128) - want) <= rtol * mag + 1e-300)
        got2 = cp.add.reduceat(d, cp.asarray(np.array(indices)), axis=axis)
        assert np.array_equal(got2.get(), got.get(), equal_nan=True)
    # a transposed view, out= and dtype=
    want = np.add.reduceat(a.T, [3, 0, 20], axis=0)
    assert np.allclose(cp.add.reduceat(d.T, [3, 0, 20], axis=0).get(), want, rtol=2e-2)
    if dtype == 'float32':
        out = cp.empty((9, 2), np.float64)
        r = cp.add.reduceat(d, [0, 7], axis=1, out=out)
        assert r is out
        assert np.allclose(out.get(), np.add.reduceat(a.astype(np.float64), [0, 7], axis=1),
                           rtol=1e-12)
    with pytest.raises(IndexError):
        cp.add.reduceat(d, [40], axis=1)
    with pytest.raises(NotImplementedError):
        cp.multiply.reduceat(d, [0], axis=1)
