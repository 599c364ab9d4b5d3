"""Structured dtypes on the device against NumPy: field-wise casts, equality,
fills and field views.  The cases follow the reference's
tests/cupy_tests/core_tests/test_structured.py and
test_ndarray_copy_and_view.py:287-296."""
import operator

import numpy as np
import pytest

import cupy_amd as cp

pytestmark = pytest.mark.gpu


def both(fn):
    """fn(numpy) and fn(cupy) compared element for element (dtype included)."""
    want = fn(np)
    got = fn(cp)
    got = got.get() if isinstance(got, cp.ndarray) else np.asarray(got)
    assert got.dtype == want.dtype, (got.dtype, want.dtype)
    assert got.shape == want.shape
    assert np.array_equal(got, want), (got, want)


def test_zeros_and_round_trip():
    both(lambda xp: xp.zeros((2, 3, 4), dtype='i,i'))
    host = np.array([(1, 2.5), (3, -4.0), (7, 0.25)], dtype='i8,f8')
    assert np.array_equal(cp.asarray(host).get(), host)
    assert np.array_equal(cp.asarray(host)[::-1].get(), host[::-1])
    assert np.array_equal(cp.asarray(host).copy()[1:].get(), host[1:])


def test_casting_simple():
    both(lambda xp: xp.array([(1, 2.), (3, 4.)], dtype='i8,f8').astype('f8,i8'))


def test_casting_swapped_fields():
    both(lambda xp: xp.array([(1, 2.), (3, 4.)], dtype='i8,f8')[['f0', 'f1']].astype('f8,i8'))


def test_casting_nested():
    def f(xp):
        dtype = np.dtype([('a', 'f8'), ('b', np.dtype('i8,f8'))])
        a = xp.array(np.array([(1, (2, 3.)), (4, (5, 6.5))], dtype=dtype))
        return a.astype(np.dtype([('a', 'f4'), ('b', np.dtype('f4,i4'))]))
    both(f)


def test_casting_many_elements_and_views():
    rng = np.random.default_rng(3)
    host = np.zeros(10007, dtype=cp.make_aligned_dtype('i4,f4,i2'))
    host['f0'] = rng.integers(-1000, 1000, host.size)
    host['f1'] = rng.standard_normal(host.size)
    host['f2'] = rng.integers(-100, 100, host.size)
    dev = cp.asarray(host)
    target = cp.make_aligned_dtype('f8,f8,i8')
    assert np.array_equal(dev.astype(target).get(), host.astype(target))
    assert np.array_equal(dev[::3].astype(target).get(), host[::3].astype(target))
    m = host.reshape(-1, 1)[:10000].reshape(100, 100)
    dm = cp.asarray(m)
    assert np.array_equal(dm.T.astype(target).get(), m.T.astype(target))


@pytest.mark.parametrize('op', [operator.eq, operator.ne])
class TestComparison:
    def test_simple(self, op):
        both(lambda xp: op(xp.array(np.array([(1, 2)], dtype='i8,f8')),
                           xp.array(np.array([(1, 2.), (1, 3), (3, 2)], dtype='i8,f8'))))

    def test_with_cast(self, op):
        both(lambda xp: op(xp.array(np.array([(1, 2)], dtype='i8,f8')),
                           xp.array(np.array([(1, 2.), (1, 3), (3, 2)], dtype='f8,i8'))))

    def test_nested(self, op):
        adtype = np.dtype([('a', 'f8'), ('b', np.dtype('i8,f8'))])
        bdtype = np.dtype([('a', 'f4'), ('b', np.dtype('f4,i4'))])
        both(lambda xp: op(
            xp.array(np.array([(1, (2, 3))], dtype=adtype)),
            xp.array(np.array([(1, (2, 3)), (1, (2, 4)), (1, (3, 3))], dtype=bdtype))))

    def test_complex_field_promoted_and_aligned(self, op):
        a = cp.array(np.array([(1, 2)], dtype='f8,c8'))
        b = cp.array(np.array([(1, 2), (1, 3), (2, 3)], dtype='f8,f8'))
        assert np.array_equal(op(a, b).get(), op(a.get(), b.get()))

    def test_many_fields(self, op):
        dtype = np.dtype([('f%d' % i, 'i1') for i in range(256)])
        a = cp.zeros(3, dtype=dtype)
        b = cp.zeros(3, dtype=dtype)
        b['f200'] = cp.asarray(np.array([0, 1, 0], 'i1'))
        assert np.array_equal(op(a, b).get(), op(a.get(), b.get()))

    def test_large_and_broadcast(self, op):
        rng = np.random.default_rng(4)
        host = np.zeros((300, 70), dtype='i4,f4')
        host['f0'] = rng.integers(0, 3, host.shape)
        host['f1'] = rng.integers(0, 2, host.shape)
        row = host[5:6]
        got = op(cp.asarray(host), cp.asarray(row)).get()
        assert np.array_equal(got, op(host, row))


@pytest.mark.parametrize('value', [(42, 3.14), np.asarray((42, 3.14), dtype='i4,f4')])
def test_fill_structured_scalar_like(value):
    def f(xp):
        a = xp.zeros(3, dtype='i4,f4')
        a.fill(value)
        return a
    both(f)


def test_ones_and_full_of_structures():
    both(lambda xp: xp.ones(10, dtype='i,f,i'))
    both(lambda xp: xp.ones((3, 4), dtype=cp.make_aligned_dtype('?,q')))


@pytest.mark.parametrize('index', ['f0', 'f1'])
def test_getitem_field(index):
    both(lambda xp: xp.array(np.array([(1, 2), (3, 4)], dtype='i,i'))[index])


@pytest.mark.parametrize('index,value', [('f0', -1), ('f1', -2)])
def test_setitem_field(index, value):
    def f(xp):
        a = xp.array(np.array([(1, 2), (3, 4)], dtype='i,i'))
        a[index] = value
        return a
    both(f)


def test_nested_fields_in_place():
    def f(xp):
        dtype = np.dtype([('a', 'i,i'), ('b', 'i,i')])
        a = xp.array(np.array([((1, 2), (3, 4)), ((5, 6), (7, 8))], dtype=dtype))
        a['a']['f0'] += a['b']['f1']
        return a
    both(f)


def test_multiple_fields():
    def f(xp):
        a = xp.ones(10, 'i,f,i')
        a['f1'] = xp.arange(10)
        a['f2'] = -xp.arange(10)
        return a[['f2', 'f1']]
    both(f)


def test_fields_feed_the_other_kernels():
    rng = np.random.default_rng(5)
    host = np.zeros(70001, dtype=cp.make_aligned_dtype('f4,i4,f8'))
    host['f0'] = rng.standard_normal(host.size)
    host['f1'] = rng.integers(-9, 10, host.size)
    host['f2'] = rng.standard_normal(host.size)
    dev = cp.asarray(host)
    assert int(dev['f1'].sum().get()) == int(host['f1'].sum())
    assert int(dev['f1'].argmax().get()) == int(host['f1'].argmax())
    np.testing.assert_allclose(dev['f2'].sum().get(), host['f2'].sum(), rtol=1e-12)
    got = (dev['f0'] * dev['f1'] + dev['f2']).get()
    assert np.array_equal(got, host['f0'] * host['f1'] + host['f2'])
    assert np.array_equal(cp.cumsum(dev['f1']).get(), np.cumsum(host['f1']))


def test_user_kernel_over_structures():
    dt = cp.make_aligned_dtype('i4,f8')
    host = np.zeros(5000, dtype=dt)
    host['f0'] = np.arange(5000)
    host['f1'] = np.arange(5000) * 0.5
    dev = cp.asarray(host)
    k = cp.ElementwiseKernel('T x', 'float64 y', 'y = x.template at<0>() + x.template at<1>()',
                             'sum_of_fields')
    assert np.array_equal(k(dev).get(), host['f0'] + host['f1'])
    swap = cp.ElementwiseKernel(
        'T x', 'T y', 'y = x; y.template at<0>() = -x.template at<0>()', 'negate_first_field')
    got = swap(dev).get()
    want = host.copy()
    want['f0'] = -want['f0']
    assert np.array_equal(got, want)


def test_field_count_and_in_place_field_update_of_a_user_kernel():
    kernel = cp.ElementwiseKernel(
        'T in', 'T out',
        'static_assert(T::field_count == 2, "expected 2 fields"); out.at<1>() = -in.at<0>();',
        'test_struct_access')
    x = cp.array(np.array([(1, 0), (2, 0), (3, 0)], dtype='i,i'))
    y = cp.array(np.array([(4, 0), (5, 0), (6, 0)], dtype='i,i'))
    kernel(x, y)
    assert np.array_equal(y.get(), np.array([(4, -1), (5, -2), (6, -3)], dtype='i,i'))


def test_multifield_assignment_with_holes_and_casts():
    def f(xp):
        a = xp.ones(10, 'i,f,i,f,i,f')
        for i in range(6):
            a['f%d' % i] = xp.arange(i, 10 + i)
        a[['f1', 'f0', 'f4']] = a[['f2', 'f1', 'f5']].copy()
        return a
    both(f)


@pytest.mark.parametrize('scalar', [
    1.0, np.int32(-1),
    np.void((1, 2, 3, 4, 5, 6), dtype='q,q,q,q,i,i'),
    np.void((-1, 2, 3, 4, 5, -6), dtype='d,d,d,d,d,d')])
def test_scalars_into_structures(scalar):
    def full(xp):
        return xp.full(10, scalar, dtype='i,i,q,q,q,q')

    def assign(xp):
        a = xp.zeros(10, dtype='i,i,q,q,q,q')
        a[...] = scalar
        return a
    both(full)
    both(assign)


def test_raw_bytes():
    assert cp.empty(10, dtype='V10').dtype == np.dtype('V10')
    assert not cp.zeros(3, dtype='V10').get().view('uint8').any()
    host = np.array([b'1', b'2', b'3'], dtype='V10')
    dev = cp.array(host)
    assert np.array_equal(dev.get(), host) and np.array_equal(dev[::-1].copy().get(), host[::-1])
    a = np.array([b'87654321', b'12345678'], dtype='V8')
    b = np.array([b'87654321', b'1234567_'], dtype='V8')
    assert np.array_equal((cp.array(a) == cp.array(b)).get(), a == b)
    assert np.array_equal((cp.array(a) != cp.array(b)).get(), a != b)
    with pytest.raises(ValueError, match='Unsupported dtype'):
        cp.empty(3, dtype='3i')
    with pytest.raises(ValueError, match='Unsupported dtype'):
        cp.empty(3, dtype='V')
