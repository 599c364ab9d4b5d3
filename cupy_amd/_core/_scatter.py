"""``ufunc.at`` and ``add.reduceat``.

``ufunc.at(a, indices, b)`` applies the operation in place at the indexed
elements, once per occurrence of an index (``a[indices] += b`` would count a
repeated index once).  Threads that hit the same element update it atomically
(``include/cupy/atomics.cuh``), so integer results are exact and
order-independent; floating-point sums depend on the order the hardware
serialises the updates in, as they do in the reference
(cupy/_core/_kernel.pyx:1447-1456 -> ``_scatter_op``,
cupy/_core/_routines_indexing.pyx:899-1120 with include/cupy/atomics.cuh).

Indices may be an integer, an integer array (device, NumPy or nested list), or
a tuple of those for the leading axes of ``a``; the remaining axes are taken
whole.  Slices and masks inside the index belong to the general indexing
routines, which this package does not build.

``add.reduceat(array, indices, axis)`` sums ``array[indices[i]:indices[i+1]]``
along ``axis`` (the element at ``indices[i]`` alone when the range is empty, the
rest of the axis for the last index), directly over each range instead of
through differences of a running sum as the reference does
(cupy/_core/_routines_indexing.pyx:1255-1270), so no cancellation is added.
"""
import numpy

from cupy_amd._core import _kernel
from cupy_amd._core import internal
from cupy_amd._core.core import ndarray, array as _array

_OPS = ('add', 'sub', 'max', 'min', 'and', 'or', 'xor')
_scatter_kernels = {}
_INDEX_TYPE_NAMES = 'IJKLMNPQRSUVWXYZ'     # type placeholders of the index arrays
_reduceat_kernels = {}


def _index_arrays(a, indices):
    """The index as a list of device integer arrays / Python ints for the
    leading axes of ``a``."""
    if not isinstance(indices, tuple):
        indices = (indices,)
    if len(indices) > len(_INDEX_TYPE_NAMES):
        raise NotImplementedError('ufunc.at with more than %d index arrays' % len(_INDEX_TYPE_NAMES))
    if len(indices) > a.ndim:
        raise IndexError('too many indices for array: array is %d-dimensional, but %d were '
                         'indexed' % (a.ndim, len(indices)))
    out = []
    for axis, ix in enumerate(indices):
        if isinstance(ix, (slice, type(Ellipsis), type(None))):
            raise NotImplementedError(
                'ufunc.at takes integers and integer arrays for the leading axes; '
                'slices, None and ... are not supported')
        if isinstance(ix, ndarray):
            arr = ix
        else:
            host = numpy.asarray(ix)
            if host.dtype.kind in 'iu' and host.size:
                # indices that come from the host are checked like NumPy checks them
                n = a.shape[axis]
                if host.min() < -n or host.max() >= n:
                    bad = host[(host < -n) | (host >= n)].flat[0]
                    raise IndexError('index %d is out of bounds for axis %d with size %d'
                                     % (bad, axis, n))
            if host.size == 0:
                host = host.astype(numpy.intp)
            arr = _array(host)
        if arr.dtype.kind == 'b':
            raise NotImplementedError('ufunc.at with a boolean mask is not supported')
        if arr.dtype.kind not in 'iu':
            raise IndexError('arrays used as indices must be of integer (or boolean) type')
        out.append(arr)
    return out


def _scatter_kernel(op, n_index, index_ndim, n_rest):
    key = (op, n_index, index_ndim, n_rest)
    ker = _scatter_kernels.get(key)
    if ker is None:
        lines = ['ptrdiff_t _off = 0;']
        for j in range(n_index):
            lines.append(
                '{ ptrdiff_t _k = static_cast<ptrdiff_t>(i%d); const ptrdiff_t _n = a.shape()[%d]; '
                '_k %%= _n; if (_k < 0) _k += _n; _off += _k * a.strides()[%d]; }' % (j, j, j))
        for r in range(n_rest):
            lines.append('_off += _ind.get()[%d] * a.strides()[%d];' % (index_ndim + r, n_index + r))
        lines.append('cupy::atomic_%s(reinterpret_cast<T*>(reinterpret_cast<char*>(a.data()) + _off), '
                     'static_cast<T>(v));' % op)
        in_params = ', '.join(['T v'] + ['%s i%d' % (_INDEX_TYPE_NAMES[j], j) for j in range(n_index)])
        ker = _kernel.ElementwiseKernel(
            in_params, 'raw T a', '\n'.join(lines), 'cupy_scatter_' + op, reduce_dims=False,
            preamble='#include <cupy/atomics.cuh>\n')
        _scatter_kernels[key] = ker
    return ker


def scatter_op(a, indices, b, op):
    """``a[indices] op= b`` with every occurrence of an index counted."""
    from cupy_amd import broadcast_to
    if op not in _OPS:
        raise ValueError('provided op is not supported')
    if not isinstance(a, ndarray):
        raise TypeError('the operand of ufunc.at must be a cupy.ndarray')
    if a.dtype.kind == 'c' and op not in ('add', 'sub'):
        raise NotImplementedError('ufunc.at with %s is not supported for complex arrays' % op)
    if a.dtype.kind == 'b' and op == 'sub':
        raise TypeError(
            'cupy boolean subtract, the `-` operator, is deprecated, use the '
            'bitwise_xor, the `^` operator, or the logical_xor function instead.')
    if a.dtype.kind in 'fc' and op in ('and', 'or', 'xor'):
        raise TypeError('ufunc \'bitwise_%s\' not supported for the input types' % op)
    if a.dtype.fields is not None or a.dtype.kind not in 'biufc':
        raise TypeError('ufunc.at is not supported for %s arrays' % a.dtype)
    idx = _index_arrays(a, indices)
    k = len(idx)
    index_shape = tuple(numpy.broadcast_shapes(*[ix.shape for ix in idx])) if idx else ()
    rest = tuple(a.shape[k:])
    full = index_shape + rest
    if internal.prod(full) == 0 or a.size == 0:
        return
    if isinstance(b, ndarray):
        v = b.astype(a.dtype, copy=False)
    else:
        v = _array(numpy.asarray(b).astype(a.dtype))
    v = broadcast_to(v, full)
    shaped = []
    for ix in idx:
        ix = ix.reshape((1,) * (len(index_shape) - ix.ndim) + tuple(ix.shape) + (1,) * len(rest))
        shaped.append(broadcast_to(ix, full))
    index_ndim = len(index_shape)
    if not full:
        # one element: give the loop one axis to run along
        v = v.reshape((1,))
        shaped = [ix.reshape((1,)) for ix in shaped]
        index_ndim = 1
    _scatter_kernel(op, k, index_ndim, len(rest))(v, *shaped, a)


def add_reduceat(array, indices, axis=0, dtype=None, out=None):
    from cupy_amd import broadcast_to
    if not isinstance(array, ndarray):
        raise TypeError('the operand of ufunc.reduceat must be a cupy.ndarray')
    axis = internal._normalize_axis_index(axis, array.ndim)
    n = array.shape[axis]
    if isinstance(indices, ndarray):
        lo = indices.astype(numpy.int64, copy=False).ravel()
    else:
        host = numpy.asarray(indices)
        if host.ndim != 1 or host.dtype.kind not in 'iu':
            raise ValueError('indices must be a one-dimensional array of integers')
        if host.size and (host.min() < 0 or host.max() >= n):
            bad = host[(host < 0) | (host >= n)][0]
            raise IndexError('index %d out-of-bounds in add.reduceat [0, %d)' % (bad, n))
        lo = _array(host.astype(numpy.int64))
    m = lo.size
    if dtype is not None:
        out_dtype = numpy.dtype(dtype)
    elif out is not None:
        out_dtype = out.dtype
    elif array.dtype.kind in 'bi':
        out_dtype = numpy.dtype(numpy.int64)
    elif array.dtype.kind == 'u':
        out_dtype = numpy.dtype(numpy.uint64)
    else:
        out_dtype = array.dtype
    out_shape = tuple(m if d == axis else s for d, s in enumerate(array.shape))
    if out is None:
        out = ndarray(out_shape, out_dtype)
    elif tuple(out.shape) != out_shape:
        raise ValueError('output parameter has the wrong shape: %r, expected %r'
                         % (tuple(out.shape), out_shape))
    if internal.prod(out_shape) == 0:
        return out
    # the end of every range: the next index, the length of the axis for the last
    from cupy_amd._core import _ufuncs
    hi = ndarray((m,), numpy.int64)
    if m > 1:
        _ufuncs.elementwise_copy(lo[1:], hi[:-1])
    hi[m - 1:].fill(n)
    bshape = tuple(m if d == axis else 1 for d in range(array.ndim))
    lo_b = broadcast_to(lo.reshape(bshape), out_shape)
    hi_b = broadcast_to(hi.reshape(bshape), out_shape)
    # accumulate in float for float16 (as sum does), in the output type otherwise
    from cupy_amd._core._scalar import get_typename
    acc_dtype = numpy.dtype(numpy.float32) if out_dtype == numpy.float16 else out_dtype
    key = (array.ndim, axis, acc_dtype)
    ker = _reduceat_kernels.get(key)
    if ker is None:
        lines = ['typedef %s A;' % get_typename(acc_dtype), 'ptrdiff_t _base = 0;']
        for d in range(array.ndim):
            if d != axis:
                lines.append('_base += _ind.get()[%d] * x.strides()[%d];' % (d, d))
        lines += [
            'const ptrdiff_t _n = x.shape()[%d], _sa = x.strides()[%d];' % (axis, axis),
            'ptrdiff_t _b = lo, _e = hi;',
            '_b = _b < 0 ? 0 : (_b >= _n ? _n - 1 : _b);',
            '_e = _e > _n ? _n : _e;',
            'if (_e <= _b) _e = _b + 1;',
            'const char* _p = reinterpret_cast<const char*>(x.data()) + _base;',
            'A _acc = static_cast<A>(*reinterpret_cast<const T*>(_p + _b * _sa));',
            'for (ptrdiff_t _j = _b + 1; _j < _e; ++_j) '
            '_acc = _acc + static_cast<A>(*reinterpret_cast<const T*>(_p + _j * _sa));',
            'y = static_cast<O>(_acc);']
        ker = _kernel.ElementwiseKernel(
            'raw T x, int64 lo, int64 hi', 'O y', '\n'.join(lines),
            'cupy_add_reduceat', reduce_dims=False)
        _reduceat_kernels[key] = ker
    ker(array, lo_b, hi_b, out)
    return out
