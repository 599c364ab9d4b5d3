"""Pure host helpers of the kernel generators: shape/stride arithmetic, axis
normalisation and broadcasting.

Counterpart of the reference's cupy/_core/internal.pyx (prod :32-51, clp2
:290-298, get_reduced_dims :86-116, get_c_contiguity :159-177,
complete_slice :179-249, infer_unknown_dimension :393-425, _broadcast_core
:320-376, _normalize_axis_index(es) :428-486).
"""
import operator

import numpy

from numpy.exceptions import AxisError


def prod(args):
    n = 1
    for x in args:
        n *= x
    return n


prod_sequence = prod


def is_in(args, x):
    return x in args


def vector_equal(x, y):
    return len(x) == len(y) and all(a == b for a, b in zip(x, y))


def get_size(size):
    """Normalises a shape argument to a tuple; booleans are rejected."""
    if size is None:
        return ()
    if isinstance(size, (bool, numpy.bool_)):
        raise TypeError('expected a sequence of integers or a single integer, '
                        'got %r' % (size,))
    if isinstance(size, numpy.ndarray):
        if size.dtype == numpy.bool_:
            raise TypeError('expected a sequence of integers or a single '
                            'integer, got %r' % (size,))
        if size.ndim == 0:
            return (size.item(),)
    if isinstance(size, (list, tuple)) or (
            isinstance(size, numpy.ndarray) and size.ndim > 0):
        out = []
        for x in size:
            if isinstance(x, (bool, numpy.bool_)) or (
                    isinstance(x, numpy.ndarray) and x.dtype == numpy.bool_):
                raise TypeError('expected a sequence of integers or a single '
                                'integer, got %r' % (size,))
            out.append(x.item() if isinstance(x, numpy.ndarray) else x)
        return tuple(out)
    if isinstance(size, (int, float, numpy.integer, numpy.floating)):
        return (size,)
    raise TypeError('expected a sequence of integers or a single integer, '
                    'got %r' % (size,))


def clp2(x):
    """Smallest power of two >= x (0 -> 0)."""
    if x <= 0:
        return 0
    return 1 << (int(x) - 1).bit_length()


def flp2(x):
    """Largest power of two <= x (0 -> 0)."""
    if x <= 0:
        return 0
    return 1 << (int(x).bit_length() - 1)


def get_contiguous_strides(shape, itemsize, is_c_contiguous=True):
    strides = [0] * len(shape)
    st = itemsize
    order = range(len(shape) - 1, -1, -1) if is_c_contiguous else range(len(shape))
    for i in order:
        strides[i] = st
        st *= max(shape[i], 1)
    return tuple(strides)


def get_reduced_dims(shape, strides, itemsize):
    """Merges adjacent axes that are laid out back to back and drops axes of
    extent 1.  Returns (shape, strides) of an equivalent view with the fewest
    axes; a zero-size array reduces to ((0,), (itemsize,))."""
    ndim = len(shape)
    if ndim == 0:
        return (), ()
    if 0 in shape:
        return (0,), (itemsize,)
    out_shape = []
    out_strides = []
    for sh, st in zip(shape, strides):
        if sh == 1:
            continue
        if out_shape and out_strides[-1] == sh * st:
            out_shape[-1] *= sh
            out_strides[-1] = st
        else:
            out_shape.append(sh)
            out_strides.append(st)
    return tuple(out_shape), tuple(out_strides)


def get_c_contiguity(shape, strides, itemsize):
    if 0 in shape:
        return True
    rshape, rstrides = get_reduced_dims(shape, strides, itemsize)
    return len(rshape) == 0 or (len(rshape) == 1 and rstrides[0] == itemsize)


def get_f_contiguity(shape, strides, itemsize):
    return get_c_contiguity(shape[::-1], strides[::-1], itemsize)


def infer_unknown_dimension(shape, size):
    shape = list(shape)
    unknown = [i for i, s in enumerate(shape) if s < 0]
    if len(unknown) > 1:
        raise ValueError('can only specify one unknown dimension')
    if unknown:
        known = prod(s for s in shape if s >= 0)
        shape[unknown[0]] = size // known if known != 0 else 0
    return shape


def complete_slice(slc, dim):
    """Fills in start/stop/step of a slice for an axis of extent ``dim`` (the
    result addresses the same elements as NumPy would)."""
    step = slc.step
    if step is None:
        step = 1
    else:
        try:
            step = operator.index(step)
        except TypeError:
            raise TypeError('slice.step must be int or None or have __index__ '
                            'method: {}'.format(slc))
    if step == 0:
        raise ValueError('Slice step must be nonzero.')
    start_none = slc.start is None
    stop_none = slc.stop is None
    try:
        start = 0 if start_none else operator.index(slc.start)
    except TypeError:
        raise TypeError('slice.start must be int or None or have __index__ '
                        'method: {}'.format(slc))
    try:
        stop = 0 if stop_none else operator.index(slc.stop)
    except TypeError:
        raise TypeError('slice.stop must be int or None or have __index__ '
                        'method: {}'.format(slc))
    if step > 0:
        start = 0 if start_none else max(0, min(dim, start + dim if start < 0 else start))
        stop = dim if stop_none else max(start, min(dim, stop + dim if stop < 0 else stop))
    else:
        start = dim - 1 if start_none else max(-1, min(dim - 1, start + dim if start < 0 else start))
        stop = -1 if stop_none else max(-1, min(start, stop + dim if stop < 0 else stop))
    return slice(start, stop, step)


def _normalize_axis_index(axis, ndim):
    if not -ndim <= axis < ndim:
        raise AxisError(axis, ndim)
    return axis + ndim if axis < 0 else axis


def _normalize_axis_indices(axes, ndim, sort_axes=True):
    if axes is None:
        axes = tuple(range(ndim))
    elif not isinstance(axes, (tuple, list)):
        axes = (axes,)
    res = []
    for axis in axes:
        axis = _normalize_axis_index(operator.index(axis), ndim)
        if axis in res:
            raise ValueError('Duplicate value in \'axis\'')
        res.append(axis)
    return tuple(sorted(res) if sort_axes else res)


def _broadcast_shapes(shapes):
    """NumPy broadcasting of a list of shapes -> result shape."""
    ndim = max((len(s) for s in shapes), default=0)
    out = [1] * ndim
    for s in shapes:
        off = ndim - len(s)
        for i, ext in enumerate(s):
            cur = out[off + i]
            if cur == ext or ext == 1:
                continue
            if cur == 1:
                out[off + i] = ext
            else:
                raise ValueError(
                    'operands could not be broadcast together with shapes {}'
                    .format(' '.join(str(tuple(x)) for x in shapes)))
    return tuple(out)


def _broadcast_core(arrays):
    """Broadcasts the ndarrays in ``arrays`` (entries that are not arrays are
    left alone) against each other.  Returns the broadcast shape and replaces
    each array in place by a zero-stride view of that shape."""
    from cupy_amd._core.core import ndarray
    idx = [i for i, a in enumerate(arrays) if isinstance(a, ndarray)]
    if not idx:
        return ()
    first = arrays[idx[0]]._shape
    if all(arrays[i]._shape == first for i in idx):
        return first
    shape = _broadcast_shapes([arrays[i]._shape for i in idx])
    ndim = len(shape)
    for i in idx:
        a = arrays[i]
        if a._shape == shape:
            continue
        off = ndim - a.ndim
        strides = [0] * ndim
        for d, (ext, st) in enumerate(zip(a._shape, a._strides)):
            if ext != 1:
                strides[off + d] = st
        arrays[i] = a._view(shape, tuple(strides))
    return shape
