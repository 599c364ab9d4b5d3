"""Array creation routines needed around the kernel path (a small subset of
the reference's cupy/_creation)."""
import numpy

from cupy_amd._core._dtype import get_dtype
from cupy_amd._core._kernel import ElementwiseKernel
from cupy_amd._core.core import ndarray
from cupy_amd._core import internal


def empty(shape, dtype=float, order='C'):
    """Uninitialised array."""
    return ndarray(shape, dtype, order=order)


def empty_like(a, dtype=None, order='K', subok=None, shape=None):
    if dtype is None:
        dtype = a.dtype
    if shape is None:
        shape = a.shape
    if order in ('K', 'A', 'k', 'a'):
        order = 'F' if (a._f_contiguous and not a._c_contiguous) else 'C'
    return ndarray(shape, dtype, order=order)


def full(shape, fill_value, dtype=None, order='C'):
    if dtype is None:
        if isinstance(fill_value, ndarray):
            dtype = fill_value.dtype
        else:
            dtype = numpy.array(fill_value).dtype
    a = ndarray(shape, dtype, order=order)
    if a.size:
        a.fill(fill_value)
    return a


def zeros(shape, dtype=float, order='C'):
    a = ndarray(shape, dtype, order=order)
    if a.size:
        a.data.memset_async(0, a.nbytes)
    return a


def ones(shape, dtype=float, order='C'):
    return full(shape, 1, dtype, order)


def zeros_like(a, dtype=None, order='K', subok=None, shape=None):
    out = empty_like(a, dtype, order, subok, shape)
    if out.size:
        out.data.memset_async(0, out.nbytes)
    return out


def ones_like(a, dtype=None, order='K', subok=None, shape=None):
    out = empty_like(a, dtype, order, subok, shape)
    if out.size:
        out.fill(1)
    return out


def full_like(a, fill_value, dtype=None, order='K', subok=None, shape=None):
    out = empty_like(a, dtype, order, subok, shape)
    if out.size:
        out.fill(fill_value)
    return out


_arange_ufunc = ElementwiseKernel(
    'T start, T step', 'T y', 'y = start + i * step', 'cupy_arange')


def arange(start, stop=None, step=1, dtype=None):
    """Evenly spaced values in ``[start, stop)``."""
    if dtype is None:
        if any(numpy.dtype(type(v)).kind == 'f' for v in (start, stop, step)
               if v is not None):
            dtype = float
        else:
            dtype = int
    if stop is None:
        stop = start
        start = 0
    if step is None:
        step = 1
    size = int(numpy.ceil((stop - start) / step))
    dt = get_dtype(dtype)
    if size <= 0:
        return ndarray((0,), dt)
    if dt.kind == 'b':
        if size > 2:
            raise TypeError('arange() is only supported for booleans '
                            'when the result has at most length 2.')
        from cupy_amd._core.core import array
        return array(numpy.arange(start, stop, step, dtype=dt))
    ret = ndarray((size,), dt)
    typ = dt.type
    _arange_ufunc(typ(start), typ(step), ret)
    return ret


def _normalize_shape(shape):
    return internal.get_size(shape)
