"""Functions either side of the generated kernels that cost no kernel of
their own design: views with other axes, the Array-API spellings of the scans,
and compositions of ufuncs and reductions (each cites the reference function
whose arguments and errors it keeps)."""
import functools
import operator

import numpy

from cupy_amd._core import internal
from cupy_amd._core.core import ndarray, array, asarray
from cupy_amd._core import _ufuncs
from cupy_amd._core._kernel import create_ufunc
from cupy_amd._core import _scan


# ---------------------------------------------------------------------------------
# views
# ---------------------------------------------------------------------------------

def shape(a):
    return a.shape if isinstance(a, ndarray) else numpy.shape(a)


def ndim(a):
    return a.ndim if isinstance(a, ndarray) else numpy.ndim(a)


def size(a, axis=None):
    """Number of elements, or the extent of one axis
    (reference: cupy/_core/core.pyx `size`)."""
    if not isinstance(a, ndarray):
        raise ValueError('Only cupy.ndarray is supported for size, but got %s' % type(a))
    return a.size if axis is None else a.shape[axis]


def squeeze(a, axis=None):
    """reference: cupy/_manipulation/dims.py `squeeze`"""
    return a.squeeze(axis=axis)


def swapaxes(a, axis1, axis2):
    """reference: cupy/_manipulation/transpose.py `swapaxes`"""
    return a.swapaxes(axis1, axis2)


def moveaxis(a, source, destination):
    """View with the source axes at the destination positions, the others in
    their order (reference: cupy/_manipulation/transpose.py `moveaxis`,
    cupy/_core/_routines_manipulation.pyx `_move_single_axis`/`moveaxis`)."""
    nd = a.ndim
    src = internal._normalize_axis_indices(source, nd, sort_axes=False)
    dst = internal._normalize_axis_indices(destination, nd, sort_axes=False)
    if len(src) != len(dst):
        raise ValueError('`source` and `destination` arguments must have the '
                         'same number of elements')
    rest = [ax for ax in range(nd) if ax not in src]
    order = [None] * nd
    for s, d in zip(src, dst):
        order[d] = s
    it = iter(rest)
    order = [next(it) if o is None else o for o in order]
    return a.transpose(order)


def rollaxis(a, axis, start=0):
    """reference: cupy/_manipulation/transpose.py `rollaxis`"""
    nd = a.ndim
    axis = internal._normalize_axis_index(axis, nd)
    if not -nd <= start <= nd:
        raise numpy.exceptions.AxisError(
            "'start' arg requires %d <= start < %d, but %d was passed in" % (-nd, nd + 1, start))
    if start < 0:
        start += nd
    if start > axis:
        start -= 1
    if axis == start:
        return a
    axes = list(range(nd))
    axes.remove(axis)
    axes.insert(start, axis)
    return a.transpose(axes)


def expand_dims(a, axis):
    """View with axes of extent one inserted
    (reference: cupy/_manipulation/dims.py `expand_dims`)."""
    if not isinstance(axis, (tuple, list)):
        axis = (axis,)
    out_nd = a.ndim + len(axis)
    axis = internal._normalize_axis_indices(axis, out_nd)
    shp, std = list(a.shape), list(a.strides)
    for ax in axis:
        # the stride of an axis of one element never matters; the next
        # axis's span keeps the contiguity flags what NumPy reports
        st = (shp[ax] * std[ax]) if ax < len(shp) else a.itemsize
        shp.insert(ax, 1)
        std.insert(ax, st)
    return a._view(tuple(shp), tuple(std))


def _atleast(nd_wanted, arys):
    res = []
    for a in arys:
        if not isinstance(a, ndarray):
            raise TypeError('Only cupy arrays can be atleast_%dd' % nd_wanted)
        if a.ndim == 0:
            a = a.reshape((1,) * nd_wanted)
        elif a.ndim == 1 and nd_wanted >= 2:
            a = a[None, :] if nd_wanted == 2 else a[None, :, None]
        elif a.ndim == 2 and nd_wanted == 3:
            a = a[:, :, None]
        res.append(a)
    return res[0] if len(res) == 1 else res


def atleast_1d(*arys):
    """reference: cupy/_manipulation/dims.py `atleast_1d`"""
    return _atleast(1, arys)


def atleast_2d(*arys):
    """reference: cupy/_manipulation/dims.py `atleast_2d`"""
    return _atleast(2, arys)


def atleast_3d(*arys):
    """reference: cupy/_manipulation/dims.py `atleast_3d`"""
    return _atleast(3, arys)


def broadcast_arrays(*args):
    """Views of the arguments with their common shape
    (reference: cupy/_manipulation/dims.py `broadcast_arrays`)."""
    from cupy_amd import broadcast_to
    arrays = [asarray(a) for a in args]
    common = tuple(internal._broadcast_shapes([a.shape for a in arrays]))
    return [a if a.shape == common else broadcast_to(a, common) for a in arrays]


def flip(a, axis=None):
    """View with the elements of the given axes in reverse order
    (reference: cupy/_manipulation/rearrange.py `flip`)."""
    axes = internal._normalize_axis_indices(axis, a.ndim)
    return a[tuple(slice(None, None, -1) if ax in axes else slice(None) for ax in range(a.ndim))]


def fliplr(a):
    if a.ndim < 2:
        raise ValueError('Input must be >= 2-d')
    return a[:, ::-1]


def flipud(a):
    if a.ndim < 1:
        raise ValueError('Input must be >= 1-d')
    return a[::-1]


# ---------------------------------------------------------------------------------
# conversions
# ---------------------------------------------------------------------------------

def astype(x, dtype, /, *, copy=True):
    """Array-API spelling of ndarray.astype (reference: cupy/_manipulation/basic.py)."""
    if not isinstance(x, ndarray):
        raise TypeError('Input should be a CuPy array. It is a %s instead.' % type(x))
    return x.astype(dtype, copy=copy)


def asanyarray(a, dtype=None, order=None):
    return asarray(a, dtype) if order is None else array(a, dtype, copy=False, order=order)


def asfortranarray(a, dtype=None):
    """reference: cupy/_creation/from_data.py `asfortranarray`"""
    return array(a, dtype, copy=False, order='F', ndmin=1)


def isscalar(element):
    return numpy.isscalar(element)


# ---------------------------------------------------------------------------------
# scans, Array-API spelling
# ---------------------------------------------------------------------------------

def _cumulative(x, scan, identity, axis, dtype, out, include_initial):
    if not isinstance(x, ndarray):
        raise TypeError('`x` should be of type cupy.ndarray')
    if x.ndim == 0:
        x = x.reshape(1)
    if axis is None:
        if x.ndim >= 2:
            raise ValueError('For arrays which have more than one dimension '
                             '``axis`` argument is required.')
        axis = 0
    else:
        axis = internal._normalize_axis_index(axis, x.ndim)
    want = tuple(e + 1 if include_initial and ax == axis else e for ax, e in enumerate(x.shape))
    if out is not None and out.shape != want:
        raise ValueError('out.shape %s does not match expected shape %s' % (out.shape, want))
    if not include_initial:
        return scan(x, axis=axis, dtype=dtype, out=out)
    # the scan is written behind a leading slice that holds the identity
    if out is None:
        if dtype is not None:
            res_dtype = numpy.dtype(dtype)
        else:
            res_dtype = {'b': numpy.dtype('int64'), 'i': numpy.dtype('int64'),
                         'u': numpy.dtype('uint64')}.get(x.dtype.kind, x.dtype)
            if x.dtype.kind in 'iu' and x.dtype.itemsize == 8:
                res_dtype = x.dtype
        res = ndarray(want, res_dtype)
    else:
        res = out
    lead = tuple(slice(0, 1) if ax == axis else slice(None) for ax in range(x.ndim))
    rest = tuple(slice(1, None) if ax == axis else slice(None) for ax in range(x.ndim))
    res[lead] = identity
    if x.size:
        scan(x, axis=axis, dtype=dtype, out=res[rest])
    return res


def cumulative_sum(x, /, *, axis=None, dtype=None, out=None, include_initial=False):
    """reference: cupy/_math/sumprod.py:316-348"""
    return _cumulative(x, _scan.cumsum, 0, axis, dtype, out, include_initial)


def cumulative_prod(x, /, *, axis=None, dtype=None, out=None, include_initial=False):
    """reference: cupy/_math/sumprod.py `cumulative_prod`"""
    return _cumulative(x, _scan.cumprod, 1, axis, dtype, out, include_initial)


# ---------------------------------------------------------------------------------
# compositions of ufuncs and reductions
# ---------------------------------------------------------------------------------

def _signed_infinity(x, out, negative):
    is_inf = _ufuncs.isinf(x)
    try:
        sign = _ufuncs.signbit(x)
    except TypeError as e:
        raise TypeError('This operation is not supported for %s values '
                        'because it would be ambiguous.' % x.dtype) from e
    if not negative:
        sign = _ufuncs.logical_not(sign)
    return _ufuncs.logical_and(is_inf, sign, out=out)


def isneginf(x, out=None):
    """reference: cupy/_logic/content.py `isneginf`"""
    return _signed_infinity(x, out, True)


def isposinf(x, out=None):
    """reference: cupy/_logic/content.py `isposinf`"""
    return _signed_infinity(x, out, False)


def array_equal(a1, a2, equal_nan=False):
    """0-d boolean array: same shape and equal elements, no synchronisation
    (reference: cupy/_logic/comparison.py:44-77)."""
    if a1.shape != a2.shape:
        return array(False)
    if not equal_nan:
        return (a1 == a2).all()
    # NaNs compare equal where both arrays hold one
    both_nan = _ufuncs.logical_and(_ufuncs.isnan(a1), _ufuncs.isnan(a2)) \
        if a1.dtype.kind in 'fc' and a2.dtype.kind in 'fc' else None
    same = a1 == a2
    return (same if both_nan is None else _ufuncs.logical_or(same, both_nan)).all()


def array_equiv(a1, a2):
    """0-d boolean array: equal after broadcasting
    (reference: cupy/_logic/comparison.py `array_equiv`)."""
    try:
        internal._broadcast_shapes([a1.shape, a2.shape])
    except ValueError:
        return array(False)
    return (a1 == a2).all()


def average(a, axis=None, weights=None, returned=False, *, keepdims=False):
    """Weighted mean along the axes (reference: cupy/_statistics/meanvar.py `average`)."""
    a = asarray(a)
    if weights is None:
        avg = a.mean(axis=axis, keepdims=keepdims)
        scl = avg.dtype.type(a.size / avg.size)
    else:
        wgt = asarray(weights)
        if a.dtype.kind in 'iub':
            res_dtype = functools.reduce(numpy.promote_types, (a.dtype, wgt.dtype, 'f8'))
        else:
            res_dtype = numpy.promote_types(a.dtype, wgt.dtype)
        if a.shape != wgt.shape:
            if axis is None:
                raise TypeError('Axis must be specified when shapes of a and weights differ.')
            if wgt.ndim != 1:
                raise TypeError('1D weights expected when shapes of a and weights differ.')
            if wgt.shape[0] != a.shape[axis]:
                raise ValueError('Length of weights not compatible with specified axis.')
            from cupy_amd import broadcast_to
            wgt = broadcast_to(wgt, (a.ndim - 1) * (1,) + wgt.shape).swapaxes(-1, axis)
        scl = wgt.sum(axis=axis, dtype=res_dtype, keepdims=keepdims)
        if bool((scl == 0.0).any()):     # the one synchronisation of this function
            raise ZeroDivisionError("Weights sum to zero, can't be normalized")
        avg = _ufuncs.multiply(a, wgt, dtype=res_dtype).sum(axis, keepdims=keepdims) / scl
    if returned:
        if not isinstance(scl, ndarray) or scl.shape != avg.shape:
            from cupy_amd import broadcast_to
            scl = broadcast_to(array(scl), avg.shape).copy()
        return avg, scl
    return avg


# ---------------------------------------------------------------------------------
# linspace
# ---------------------------------------------------------------------------------

_linspace_ufunc = create_ufunc(
    'cupy_linspace', ('dd->d',), 'out0 = in0 + i * in1')

_linspace_ufunc_underflow = create_ufunc(
    'cupy_linspace', ('ddd->d',), 'out0 = in0 + i * in1 / in2')


def linspace(start, stop, num=50, endpoint=True, retstep=False, dtype=None, axis=0):
    """``num`` evenly spaced values from start to stop, scalar bounds
    (reference: cupy/_creation/ranges.py:63-125; the values come from one
    kernel, `start + i * step`, the last one is set to `stop`)."""
    num = operator.index(num)
    if num < 0:
        raise ValueError('linspace with num<0 is not supported')
    if not (numpy.isscalar(start) and numpy.isscalar(stop)):
        raise NotImplementedError('linspace over array bounds is not part of this build')
    dt = numpy.result_type(start, stop, float(num))
    if dtype is None:
        dtype = dt
    ret = ndarray((num,), dt)
    div = (num - 1) if endpoint else num
    if div <= 0:
        if num > 0:
            ret.fill(start)
        step = float('nan')
    else:
        step = float(stop - start) / div
        stop = float(stop)
        if step == 0.0:
            # the difference underflows once divided: divide last
            _linspace_ufunc_underflow(start, stop - start, div, ret)
        else:
            _linspace_ufunc(start, step, ret)
        if endpoint:
            ret[-1] = stop
    if numpy.issubdtype(dtype, numpy.integer):
        _ufuncs.floor(ret, out=ret)
    ret = ret.astype(dtype, copy=False)
    return (ret, step) if retstep else ret
