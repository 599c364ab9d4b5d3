"""``order=`` of reshape / ravel / flatten / get and ``view(type=)``: the host
logic (which axes, which strides, which class) against NumPy arrays of the same
layout; the values are checked on the GPU in tests/test_gpu_elementwise.py."""
import itertools

import numpy as np
import pytest

import cupy_amd as cp


def twins(shape, perm=None, slicer=None):
    """A device array and a NumPy array with the same shape and strides."""
    h = np.arange(int(np.prod(shape)), dtype=np.float32).reshape(shape)
    d = cp.ndarray(shape, np.float32)
    if perm is not None:
        h, d = h.transpose(perm), d.transpose(perm)
    if slicer is not None:
        h, d = h[slicer], d[slicer]
    assert d.shape == h.shape and d.strides == h.strides
    return d, h


@pytest.mark.parametrize('perm', list(itertools.permutations(range(3))))
def test_memory_order_axes_reproduce_numpy_k_order(perm):
    d, h = twins((3, 4, 5), perm)
    axes = d._memory_order_axes()
    assert np.array_equal(h.transpose(axes).ravel(), h.ravel(order='K'))
    d, h = twins((4, 6, 5), perm, (slice(None, None, -1), slice(1, None, 2)))
    axes = d._memory_order_axes()
    assert np.array_equal(h.transpose(axes).ravel(), h.ravel(order='K'))


def test_memory_order_axes_with_broadcast_axes():
    h = np.broadcast_to(np.arange(12, dtype=np.float32).reshape(3, 1, 4), (3, 5, 4))
    d = cp.ndarray((3, 1, 4), np.float32)
    d = d._view((3, 5, 4), (d.strides[0], 0, d.strides[2]))
    assert d.strides == h.strides
    assert np.array_equal(h.transpose(d._memory_order_axes()).ravel(), h.ravel(order='K'))


def test_fortran_reshape_of_a_fortran_array_is_a_view():
    d, h = twins((4, 6), (1, 0))            # shape (6, 4), stored column after column
    r, want = d.reshape((3, 8), order='F'), h.reshape((3, 8), order='F')
    assert r.shape == want.shape and r.strides == want.strides
    assert r.base is not None
    r, want = d.reshape(2, -1, order='A'), h.reshape(2, -1, order='A')
    assert r.shape == want.shape and r.strides == want.strides
    with pytest.raises(ValueError):
        d.reshape((3, 8), order='Z')


def test_ravel_orders_give_views_where_numpy_does():
    d, h = twins((4, 6), (1, 0))
    for order in ('F', 'A', 'K'):
        r, want = d.ravel(order=order), h.ravel(order=order)
        assert r.shape == want.shape and r.strides == want.strides
        assert r.base is not None           # no copy


class _Tagged(cp.ndarray):
    def __array_finalize__(self, obj):
        self.tag = getattr(obj, 'tag', 'fresh')


def test_view_as_another_array_class():
    a = cp.ndarray((4, 6), np.float32)
    v = a.view(type=_Tagged)
    assert type(v) is _Tagged and v.tag == 'fresh' and v.data.ptr == a.data.ptr
    assert type(a.view(_Tagged)) is _Tagged             # the class in the dtype position
    w = v.view(np.int32, cp.ndarray)
    assert type(w) is cp.ndarray and w.dtype == np.int32 and w.shape == (4, 6)
    assert type(v.view(np.int16)) is _Tagged and v.view(np.int16).shape == (4, 12)
    with pytest.raises(ValueError, match='twice'):
        a.view(_Tagged, _Tagged)
    with pytest.raises(ValueError, match='sub-type'):
        a.view(type=np.ndarray)
