"""``ndarray``: the strided N-d device array the kernel generators operate on.

Only the slice of the reference's ndarray that the generated-kernel path
consumes is here (cupy/_core/core.pyx:134-301 construction and flags,
:1298-1400 reductions, :1564-1674 operators, :1969-2026 ``__array_ufunc__``,
:2098-2244 get/set, :2246-2366 views, :303-340 ``__cuda_array_interface__``).
"""
import ctypes
import operator
import pickle

builtins_type = type

import numpy

from cupy_amd import _dryrun
from cupy_amd import _rt
from cupy_amd._core import _dtype
from cupy_amd._core import _tuning
from cupy_amd._core import internal
from cupy_amd.cuda import device as _device
from cupy_amd.cuda import memory as _memory
from cupy_amd.cuda import stream as _stream

MAX_NDIM = 64
_INT32_SPAN = 1 << 31


class _Flags:
    __slots__ = ('c_contiguous', 'f_contiguous', 'owndata')

    def __init__(self, c, f, own):
        self.c_contiguous, self.f_contiguous, self.owndata = c, f, own

    def __getitem__(self, name):
        key = name.lower()
        if key in ('c_contiguous', 'c'):
            return self.c_contiguous
        if key in ('f_contiguous', 'f'):
            return self.f_contiguous
        if key in ('owndata', 'o'):
            return self.owndata
        raise KeyError('%s is not defined for cupy.ndarray.flags' % name)

    def __repr__(self):
        return ('  C_CONTIGUOUS : %s\n  F_CONTIGUOUS : %s\n  OWNDATA : %s'
                % (self.c_contiguous, self.f_contiguous, self.owndata))


def _byte_extent(shape, strides, itemsize):
    """(lowest, one-past-highest) byte offsets touched by a view."""
    lo = 0
    hi = itemsize
    for sh, st in zip(shape, strides):
        if sh == 0:
            return 0, 0
        if st >= 0:
            hi += (sh - 1) * st
        else:
            lo += (sh - 1) * st
    return lo, hi


class ndarray:
    """Multi-dimensional array in device memory.

    Args:
        shape (tuple of ints): Length of axes.
        dtype: Data type.
        memptr (cupy.cuda.MemoryPointer): Pointer to the first element; new
            memory is allocated from the current allocator if omitted.
        strides (tuple of ints or None): Byte strides.
        order ({'C', 'F'}): Layout of a newly allocated array.
    """

    __array_priority__ = 100
    __hash__ = None

    def __init__(self, shape, dtype=float, memptr=None, strides=None, order='C'):
        shape = internal.get_size(shape)
        if len(shape) > MAX_NDIM:
            raise ValueError('maximum supported dimension for an ndarray is '
                             '%d, found %d' % (MAX_NDIM, len(shape)))
        for x in shape:
            if x < 0:
                raise ValueError('Negative dimensions are not allowed')
        shape = tuple(int(x) for x in shape)
        dt = _dtype.get_dtype(dtype)
        if memptr is None:
            _dtype.check_supported_dtype(dt)
        itemsize = dt.itemsize
        if order is None:
            order = 'C'
        if order not in ('C', 'F', 'c', 'f'):
            raise ValueError('order not understood: %r' % (order,))
        size = internal.prod(shape)
        if strides is not None:
            strides = tuple(int(s) for s in strides)
            if len(strides) != len(shape):
                raise ValueError('strides must have the same length as shape')
            lo, hi = _byte_extent(shape, strides, itemsize)
            if memptr is None:
                if lo != 0:
                    raise ValueError('ndarray() with strides currently does not '
                                     'allow negative strides')
                if hi > size * itemsize:
                    raise ValueError(
                        'ndarray() with strides must stay within a contiguous '
                        'size of %d but got %d.' % (size * itemsize, hi))
                alloc = hi
            else:
                alloc = hi - lo
        else:
            strides = internal.get_contiguous_strides(
                shape, itemsize, order in ('C', 'c'))
            alloc = size * itemsize
        self.dtype = dt
        self._shape = shape
        self._strides = strides
        self.size = size
        self.base = None
        self._update_contiguity()
        self._index_32_bits = max(alloc, size * itemsize) <= _INT32_SPAN
        self.data = _memory.alloc(alloc) if memptr is None else memptr

    # -- fast internal construction ---------------------------------------------
    @classmethod
    def _new_contiguous(cls, shape, dtype, c_order=True):
        """Freshly allocated C (or F) contiguous array; no argument checks."""
        self = object.__new__(cls)
        dt = _dtype.get_dtype(dtype)
        itemsize = dt.itemsize
        size = 1
        for x in shape:
            size *= x
        self.dtype = dt
        self._shape = shape
        self._strides = internal.get_contiguous_strides(shape, itemsize, c_order)
        self.size = size
        self.base = None
        if len(shape) <= 1 or size == 0:
            self._c_contiguous = self._f_contiguous = True
        elif c_order:
            self._c_contiguous = True
            self._f_contiguous = sum(1 for x in shape if x != 1) <= 1
        else:
            self._f_contiguous = True
            self._c_contiguous = sum(1 for x in shape if x != 1) <= 1
        self._index_32_bits = size * itemsize <= _INT32_SPAN
        self.data = _memory.alloc(size * itemsize)
        return self

    def _view(self, shape, strides, dtype=None):
        """View of the same memory with another shape/strides (and dtype)."""
        v = object.__new__(type(self))
        v.dtype = self.dtype if dtype is None else dtype
        v._shape = shape
        v._strides = strides
        size = 1
        for x in shape:
            size *= x
        v.size = size
        v.base = self if self.base is None else self.base
        v.data = self.data
        v._update_contiguity()
        v._index_32_bits = self._index_32_bits
        if type(v) is not ndarray:
            v.__array_finalize__(self)
        return v

    def __array_finalize__(self, obj):
        pass

    def _update_contiguity(self):
        shape, strides, itemsize = self._shape, self._strides, self.dtype.itemsize
        self._c_contiguous = internal.get_c_contiguity(shape, strides, itemsize)
        self._f_contiguous = internal.get_f_contiguity(shape, strides, itemsize)

    # -- attributes ----------------------------------------------------------------
    @property
    def shape(self):
        return self._shape

    @shape.setter
    def shape(self, newshape):
        v = self.reshape(newshape)
        if v.data.ptr != self.data.ptr or (v.base is None and v is not self):
            raise AttributeError('Incompatible shape for in-place modification. '
                                 'Use `.reshape()` to make a copy with the '
                                 'desired shape.')
        self._shape, self._strides = v._shape, v._strides
        self._update_contiguity()

    @property
    def strides(self):
        return self._strides

    @property
    def ndim(self):
        return len(self._shape)

    @property
    def itemsize(self):
        return self.dtype.itemsize

    @property
    def nbytes(self):
        return self.size * self.dtype.itemsize

    @property
    def flags(self):
        return _Flags(self._c_contiguous, self._f_contiguous, self.base is None)

    @property
    def device(self):
        return _device.Device(self.data.device_id)

    @property
    def T(self):
        if len(self._shape) < 2:
            return self
        return self.transpose()

    @property
    def __cuda_array_interface__(self):
        desc = {
            'shape': self._shape,
            'typestr': self.dtype.str,
            'descr': self.dtype.descr,
            'version': 3,
            'strides': None if self._c_contiguous else self._strides,
            'data': (self.data.ptr if self.size > 0 else 0, False),
        }
        sptr = _stream.get_current_stream_ptr()
        desc['stream'] = sptr if sptr != 0 else 1
        return desc

    def __len__(self):
        if not self._shape:
            raise TypeError('len() of unsized object')
        return self._shape[0]

    # -- kernel argument (CArray struct: data, size, shape[nd], strides[nd]) -------
    def _kernel_arg_bytes(self):
        nd = len(self._shape)
        return (ctypes.c_int64 * (2 + 2 * nd))(
            self.data.ptr, self.size, *self._shape, *self._strides)

    # -- views -------------------------------------------------------------------
    def transpose(self, *axes):
        nd = len(self._shape)
        if len(axes) == 1 and (axes[0] is None or isinstance(axes[0], (tuple, list))):
            axes = axes[0]
        if axes is None or len(axes) == 0:
            if nd < 2:
                return self._view(self._shape, self._strides)
            axes = tuple(range(nd - 1, -1, -1))
        else:
            if len(axes) != nd:
                raise ValueError('axes don\'t match array')
            norm = []
            for ax in axes:
                ax = internal._normalize_axis_index(operator.index(ax), nd)
                if ax in norm:
                    raise ValueError('repeated axis in transpose')
                norm.append(ax)
            axes = tuple(norm)
        return self._view(tuple(self._shape[a] for a in axes),
                          tuple(self._strides[a] for a in axes))

    def swapaxes(self, axis1, axis2):
        nd = len(self._shape)
        a = internal._normalize_axis_index(axis1, nd)
        b = internal._normalize_axis_index(axis2, nd)
        axes = list(range(nd))
        axes[a], axes[b] = axes[b], axes[a]
        return self.transpose(axes)

    def _index_order(self, order, allow_k=False):
        """'C' or 'F' (or 'K') for an ``order=`` argument; 'A' means Fortran
        order exactly for arrays stored that way and not in C order."""
        letter = 'C' if order is None else str(order).upper()
        if letter == 'A':
            letter = 'F' if (self._f_contiguous and not self._c_contiguous) else 'C'
        if letter not in ('C', 'F') and not (allow_k and letter == 'K'):
            raise ValueError('order not understood: %r' % (order,))
        return letter

    def _memory_order_axes(self):
        """Axes from the one with the largest step in memory to the one with
        the smallest, as NumPy's iterator orders them for ``order='K'``: an
        axis moves in front of those with smaller steps; axes without a step
        (broadcast) stay where they are met, and ties keep the axis order."""
        steps = [abs(s) for s in self._strides]
        axes = []
        for axis in reversed(range(len(steps))):
            pos = 0
            if steps[axis]:
                for k, other in enumerate(axes):
                    if steps[other] == 0:
                        continue
                    if steps[other] <= steps[axis]:
                        break
                    pos = k + 1
            axes.insert(pos, axis)
        return axes

    def reshape(self, *shape, order='C'):
        if len(shape) == 1 and isinstance(shape[0], (tuple, list)):
            shape = tuple(shape[0])
        if self._index_order(order) == 'F':
            # elements taken and placed with the first index changing fastest:
            # the C-order reshape of the transposed array, transposed back
            return self.transpose().reshape(*tuple(shape)[::-1]).transpose()
        shape = internal.infer_unknown_dimension(
            [operator.index(s) for s in shape], self.size)
        if internal.prod(shape) != self.size:
            raise ValueError('cannot reshape array of size %d into shape %s'
                             % (self.size, tuple(shape)))
        shape = tuple(shape)
        strides = _reshape_strides(self._shape, self._strides, shape,
                                   self.dtype.itemsize)
        if strides is None:
            src = self.copy()
            return src._view(shape, internal.get_contiguous_strides(
                shape, self.dtype.itemsize))
        return self._view(shape, strides)

    def ravel(self, order='C'):
        """1-d array of the elements in C, Fortran ('F'), stored ('A') or
        memory ('K') order; a view where memory allows (reference:
        cupy/_core/_routines_manipulation.pyx:190-208)."""
        letter = self._index_order(order, allow_k=True)
        if letter == 'F':
            return self.transpose().reshape(-1)
        if letter == 'K':
            return self.transpose(self._memory_order_axes()).reshape(-1)
        return self.reshape(-1)

    def flatten(self, order='C'):
        """Like ``ravel`` but always a copy."""
        letter = self._index_order(order, allow_k=True)
        src = self
        if letter == 'F':
            src = self.transpose()
        elif letter == 'K':
            src = self.transpose(self._memory_order_axes())
        return src.copy().reshape(-1) if src._c_contiguous else \
            _ascontiguous(src).reshape(-1)

    def squeeze(self, axis=None):
        nd = len(self._shape)
        if axis is None:
            keep = [i for i in range(nd) if self._shape[i] != 1]
        else:
            axes = internal._normalize_axis_indices(axis, nd)
            for a in axes:
                if self._shape[a] != 1:
                    raise ValueError('Cannot select an axis to squeeze out which '
                                     'has size not equal to one')
            keep = [i for i in range(nd) if i not in axes]
        return self._view(tuple(self._shape[i] for i in keep),
                          tuple(self._strides[i] for i in keep))

    def view(self, dtype=None, type=None):
        """View of the same memory as another dtype and / or another array
        class (reference: cupy/_core/core.pyx:926-990)."""
        cls = type
        if isinstance(dtype, builtins_type) and issubclass(dtype, ndarray):
            if cls is not None:
                raise ValueError('Cannot specify output type twice.')
            cls, dtype = dtype, None
        if cls is not None:
            if not isinstance(cls, builtins_type) or not issubclass(cls, ndarray):
                raise ValueError('Type must be a sub-type of ndarray type')
            plain = self.view(dtype)
            return plain if builtins_type(plain) is cls else plain._retype(cls, self)
        if dtype is None or _dtype.get_dtype(dtype) == self.dtype:
            return self._view(self._shape, self._strides)
        dt = _dtype.get_dtype(dtype)
        if dt.itemsize == self.dtype.itemsize:
            return self._view(self._shape, self._strides, dt)
        if not self._shape or self._strides[-1] != self.dtype.itemsize:
            raise ValueError('To change to a dtype of a different size, the last '
                             'axis must be contiguous')
        nbytes = self._shape[-1] * self.dtype.itemsize
        if nbytes % dt.itemsize:
            raise ValueError('When changing to a larger dtype, its size must be '
                             'a divisor of the total size in bytes of the last '
                             'axis of the array.')
        return self._view(self._shape[:-1] + (nbytes // dt.itemsize,),
                          self._strides[:-1] + (dt.itemsize,), dt)

    def reduced_view(self, dtype=None):
        """View with the fewest axes that addresses the same elements in the
        same order (adjacent axes merged where memory allows)."""
        shape, strides = internal.get_reduced_dims(
            self._shape, self._strides, self.dtype.itemsize)
        if len(shape) == len(self._shape) and dtype is None:
            return self
        return self._view(shape, strides, dtype)

    def __getitem__(self, key):
        if self.dtype.fields is not None and (
                isinstance(key, str) or (isinstance(key, list) and key
                                         and all(isinstance(k, str) for k in key))):
            return self._field_view(key)
        shape, strides, offset = _basic_index(self._shape, self._strides, key)
        v = self._view(shape, strides)
        if offset:
            v.data = self.data + offset
        return v

    def _field_view(self, key):
        """View of one field, or of several fields at their places in the
        element (as NumPy does it)."""
        fields = self.dtype.fields
        if isinstance(key, str):
            if key not in fields:
                raise ValueError('no field of name %s' % key)
            sub, offset = fields[key][0], fields[key][1]
            if sub.subdtype is not None:
                raise ValueError('CuPy does not yet support accessing nested subarrays')
        else:
            for k in key:
                if k not in fields:
                    raise ValueError('no field of name %s' % k)
            if len(set(key)) != len(key):
                raise ValueError('duplicate field of name %s' % key)
            sub = numpy.dtype(dict(names=list(key), formats=[fields[k][0] for k in key],
                                   offsets=[fields[k][1] for k in key],
                                   itemsize=self.dtype.itemsize))
            offset = 0
        v = ndarray(self._shape, sub, memptr=self.data + offset, strides=self._strides)
        v.base = self.base if self.base is not None else self
        if sub.fields is None and v.size:
            # every element of a plain field must sit at a multiple of its size
            # (cupy/_core/internal.pyx:532-562)
            mask = sub.itemsize - 1
            if v.data.ptr & mask or any(st & mask for st in v._strides):
                raise ValueError(
                    f'result array with dtype {sub} would not be sufficiently aligned for GPU '
                    'operations. When using structured dtypes you must manually align the '
                    'dtype and its fields; CuPy may provide utilities for this in the future.')
        return v

    def __setitem__(self, key, value):
        from cupy_amd._core._ufuncs import elementwise_copy
        if key is Ellipsis or (isinstance(key, slice) and key == slice(None)):
            dst = self
        else:
            dst = self[key]
        if isinstance(value, numpy.ndarray):
            value = array(value)
        elementwise_copy(value, dst, casting='unsafe')

    # -- data movement -------------------------------------------------------------
    def get(self, stream=None, order='C', out=None, blocking=True):
        """Copies the array to host memory and returns a ``numpy.ndarray``."""
        if _dryrun.enabled():
            _dryrun.forbid('ndarray.get()')
        if out is None:
            letter = self._index_order(order)
        else:
            if not isinstance(out, numpy.ndarray):
                raise TypeError('Only numpy.ndarray can be obtained from cupy.ndarray')
            if out.shape != self._shape or out.dtype != self.dtype:
                raise ValueError('out must be a numpy.ndarray of the same shape and dtype')
            if out.flags.c_contiguous:
                letter = 'C'
            elif out.flags.f_contiguous:
                letter = 'F'
            else:
                raise ValueError('out must be a C- or Fortran-contiguous numpy.ndarray')
        if letter == 'F' and len(self._shape) > 1:
            # a Fortran-ordered host array is the C-ordered array of the
            # transposed data: fetch that into the transposed host array
            if out is None:
                out = numpy.empty(self._shape, dtype=self.dtype, order='F')
            self.transpose().get(stream=stream, order='C', out=out.T, blocking=blocking)
            return out
        src = self if self._c_contiguous else _ascontiguous(self)
        if out is None:
            out = numpy.empty(self._shape, dtype=self.dtype)
        if self.size == 0:
            return out
        if stream is None:
            stream = _stream.get_current_stream()
        if stream.ptr == 0:
            src.data.copy_to_host(out.ctypes.data, src.nbytes)
        else:
            src.data.copy_to_host_async(out.ctypes.data, src.nbytes, stream)
            if blocking:
                stream.synchronize()
        return out

    def set(self, arr, stream=None):
        """Copies a ``numpy.ndarray`` of the same shape and dtype into the array."""
        if not isinstance(arr, numpy.ndarray):
            raise TypeError('Only numpy.ndarray can be set to cupy.ndarray')
        if arr.dtype != self.dtype:
            raise TypeError('{} array cannot be set to {} array'.format(
                arr.dtype, self.dtype))
        if arr.shape != self._shape:
            raise ValueError('Shape mismatch. Old shape: {}, new shape: {}'.format(
                self._shape, arr.shape))
        if self.size == 0:
            return
        if not self._c_contiguous:
            tmp = ndarray._new_contiguous(self._shape, self.dtype)
            tmp.set(arr, stream)
            from cupy_amd._core._ufuncs import elementwise_copy
            elementwise_copy(tmp, self)
            return
        host = numpy.ascontiguousarray(arr)
        if stream is None or stream.ptr == 0:
            cur = _stream.get_current_stream_ptr()
            if cur == 0:
                self.data.copy_from_host(host.ctypes.data, self.nbytes)
            else:
                self.data.copy_from_host_async(host.ctypes.data, self.nbytes)
                _stream.get_current_stream().synchronize()
        else:
            self.data.copy_from_host_async(host.ctypes.data, self.nbytes, stream)
            stream.synchronize()

    def copy(self, order='C'):
        if order in ('K', 'k', 'A', 'a'):
            order = 'F' if (self._f_contiguous and not self._c_contiguous) else 'C'
        if order in ('C', 'c'):
            out = ndarray._new_contiguous(self._shape, self.dtype)
            if type(self) is not ndarray:
                out = out._retype(type(self), self)
            if self.size == 0:
                return out
            if self._c_contiguous and (self.nbytes < _tuning.get('copy_kernel_min_bytes')
                                       or self.dtype.fields is not None):
                out.data.copy_from_device_async(self.data, self.nbytes)
            else:
                from cupy_amd._core._ufuncs import elementwise_copy
                elementwise_copy(self, out)
            return out
        if order in ('F', 'f'):
            out = ndarray._new_contiguous(self._shape, self.dtype, c_order=False)
            if self.size:
                from cupy_amd._core._ufuncs import elementwise_copy
                elementwise_copy(self, out)
            return out
        raise ValueError('order not understood: %r' % (order,))

    def _retype(self, cls, template):
        v = object.__new__(cls)
        v.__dict__.update(self.__dict__)
        v.__array_finalize__(template)
        return v

    def astype(self, dtype, order='K', casting=None, subok=None, copy=True):
        dt = _dtype.get_dtype(dtype)
        if casting is not None:
            _dtype._raise_if_invalid_cast(self.dtype, dt, casting)
        if (dt.fields is not None or self.dtype.fields is not None) and \
                not numpy.can_cast(self.dtype, dt, 'unsafe'):
            raise TypeError(f'Cannot cast array data from {self.dtype!r} to {dt!r}')
        if dt == self.dtype and not copy:
            return self
        if order in ('K', 'k', 'A', 'a'):
            c_order = not (self._f_contiguous and not self._c_contiguous)
        else:
            c_order = order in ('C', 'c')
        out = ndarray._new_contiguous(self._shape, dt, c_order)
        if self.size:
            from cupy_amd._core._ufuncs import elementwise_copy
            elementwise_copy(self, out, casting='unsafe')
        return out

    def fill(self, value):
        from cupy_amd._core._ufuncs import elementwise_copy
        if isinstance(value, ndarray) and value.ndim != 0:
            raise ValueError('non-scalar cupy.ndarray cannot be used for fill')
        if self.dtype.fields is not None and not isinstance(value, ndarray):
            # a structured value travels as a one-element array of this dtype
            value = array(numpy.asarray(value, dtype=self.dtype).reshape(()))
        elementwise_copy(value, self, casting='unsafe')

    def item(self):
        if self.size != 1:
            raise ValueError('can only convert an array of size 1 to a Python scalar')
        return self.get().item()

    def tolist(self):
        return self.get().tolist()

    def tobytes(self, order='C'):
        """The elements as a Python bytes object (reference: core.pyx:708-710)."""
        return self.get().tobytes(order)

    def tofile(self, fid, sep='', format='%s'):
        """Writes the array to a file as numpy.ndarray.tofile does
        (reference: core.pyx:712-718)."""
        self.get().tofile(fid, sep, format)

    def dump(self, file):
        """Pickles the array into an open file (reference: core.pyx:720-727)."""
        pickle.dump(self, file, -1)

    def dumps(self):
        """The array's pickle as bytes (reference: core.pyx:729-731)."""
        return pickle.dumps(self, -1)

    # a pickle holds the host copy; loading it uploads to the current device
    # (reference: core.pyx:1796-1797)
    def __reduce__(self):
        return array, (self.get(order='A'),)

    def __copy__(self):
        return self.copy()

    def __deepcopy__(self, memo):
        # the copy is made on the array's own device (reference: core.pyx:1787-1794)
        with self.device:
            return self.copy()

    def __iter__(self):
        if not self._shape:
            raise TypeError('iteration over a 0-d array')
        return (self[i] for i in range(self._shape[0]))

    def __complex__(self):
        return complex(self.get().reshape(()))

    def __bool__(self):
        if self.size != 1:
            raise ValueError('The truth value of an array with more than one '
                             'element is ambiguous. Use a.any() or a.all()')
        return bool(self.get().reshape(()))

    def __int__(self):
        return int(self.get().reshape(()))

    def __float__(self):
        return float(self.get().reshape(()))

    def __index__(self):
        return operator.index(self.get().reshape(()))

    def __repr__(self):
        if _dryrun.enabled():
            return '<cupy.ndarray %s %s (dry run)>' % (self._shape, self.dtype)
        return repr(self.get())

    def __str__(self):
        if _dryrun.enabled():
            return repr(self)
        return str(self.get())

    def __array__(self, dtype=None, copy=None):
        raise TypeError(
            'Implicit conversion to a NumPy array is not allowed. '
            'Please use `.get()` to construct a NumPy array explicitly.')

    # -- NumPy dispatch ------------------------------------------------------------
    def __array_ufunc__(self, ufunc, method, *inputs, **kwargs):
        import cupy_amd
        name = ufunc.__name__
        cp_ufunc = getattr(cupy_amd, name, None)
        if cp_ufunc is None:
            return NotImplemented
        if method == '__call__':
            if 'where' in kwargs:
                kwargs['_where'] = kwargs.pop('where')
            return cp_ufunc(*inputs, **kwargs)
        if method == 'reduce' and hasattr(cp_ufunc, 'reduce'):
            return cp_ufunc.reduce(*inputs, **kwargs)
        return NotImplemented

    # -- operators -------------------------------------------------------------------
    def _binary(self, name, other, reflected=False):
        if isinstance(other, numpy.ndarray) and other.ndim != 0:
            return NotImplemented
        prio = getattr(other, '__array_priority__', None)
        if prio is not None and not isinstance(other, ndarray) and \
                prio > self.__array_priority__ and hasattr(other, '__array_ufunc__') is False:
            return NotImplemented
        from cupy_amd._core import _ufuncs
        fn = getattr(_ufuncs, name)
        return fn(other, self) if reflected else fn(self, other)

    def __add__(self, other):
        return self._binary('add', other)

    def __radd__(self, other):
        return self._binary('add', other, True)

    def __iadd__(self, other):
        from cupy_amd._core import _ufuncs
        return _ufuncs.add(self, other, self)

    def __sub__(self, other):
        return self._binary('subtract', other)

    def __rsub__(self, other):
        return self._binary('subtract', other, True)

    def __isub__(self, other):
        from cupy_amd._core import _ufuncs
        return _ufuncs.subtract(self, other, self)

    def __mul__(self, other):
        return self._binary('multiply', other)

    def __rmul__(self, other):
        return self._binary('multiply', other, True)

    def __imul__(self, other):
        from cupy_amd._core import _ufuncs
        return _ufuncs.multiply(self, other, self)

    def __truediv__(self, other):
        return self._binary('true_divide', other)

    def __rtruediv__(self, other):
        return self._binary('true_divide', other, True)

    def __itruediv__(self, other):
        from cupy_amd._core import _ufuncs
        return _ufuncs.true_divide(self, other, self)

    def __floordiv__(self, other):
        return self._binary('floor_divide', other)

    def __rfloordiv__(self, other):
        return self._binary('floor_divide', other, True)

    def __ifloordiv__(self, other):
        from cupy_amd._core import _ufuncs
        return _ufuncs.floor_divide(self, other, self)

    def __mod__(self, other):
        return self._binary('remainder', other)

    def __rmod__(self, other):
        return self._binary('remainder', other, True)

    def __imod__(self, other):
        from cupy_amd._core import _ufuncs
        return _ufuncs.remainder(self, other, self)

    def __divmod__(self, other):
        return self._binary('divmod', other)

    def __rdivmod__(self, other):
        return self._binary('divmod', other, True)

    def __pow__(self, other, modulo=None):
        if modulo is not None:
            return NotImplemented
        from cupy_amd._core import _ufuncs
        # Python-scalar exponents with a dedicated loop (NumPy takes the same
        # short cuts, so results stay bit-identical with it).
        if type(other) in (int, float) and self.dtype.kind in 'fc':
            if other == 2:
                return _ufuncs.square(self)
            if other == 0.5:
                return _ufuncs.sqrt(self)
            if other == -1:
                return _ufuncs.reciprocal(self)
            if other == 1:
                return _ufuncs.positive(self)
        elif type(other) is int and other == 2 and self.dtype.kind in 'iub':
            return _ufuncs.square(self)
        return self._binary('power', other)

    def __rpow__(self, other):
        return self._binary('power', other, True)

    def __ipow__(self, other):
        from cupy_amd._core import _ufuncs
        return _ufuncs.power(self, other, self)

    def __neg__(self):
        from cupy_amd._core import _ufuncs
        return _ufuncs.negative(self)

    def __pos__(self):
        from cupy_amd._core import _ufuncs
        return _ufuncs.positive(self)

    def __abs__(self):
        from cupy_amd._core import _ufuncs
        return _ufuncs.absolute(self)

    def __invert__(self):
        from cupy_amd._core import _ufuncs
        return _ufuncs.invert(self)

    def __and__(self, other):
        return self._binary('bitwise_and', other)

    def __rand__(self, other):
        return self._binary('bitwise_and', other, True)

    def __iand__(self, other):
        from cupy_amd._core import _ufuncs
        return _ufuncs.bitwise_and(self, other, self)

    def __or__(self, other):
        return self._binary('bitwise_or', other)

    def __ror__(self, other):
        return self._binary('bitwise_or', other, True)

    def __ior__(self, other):
        from cupy_amd._core import _ufuncs
        return _ufuncs.bitwise_or(self, other, self)

    def __xor__(self, other):
        return self._binary('bitwise_xor', other)

    def __rxor__(self, other):
        return self._binary('bitwise_xor', other, True)

    def __ixor__(self, other):
        from cupy_amd._core import _ufuncs
        return _ufuncs.bitwise_xor(self, other, self)

    def __lshift__(self, other):
        return self._binary('left_shift', other)

    def __rlshift__(self, other):
        return self._binary('left_shift', other, True)

    def __ilshift__(self, other):
        from cupy_amd._core import _ufuncs
        return _ufuncs.left_shift(self, other, self)

    def __rshift__(self, other):
        return self._binary('right_shift', other)

    def __rrshift__(self, other):
        return self._binary('right_shift', other, True)

    def __irshift__(self, other):
        from cupy_amd._core import _ufuncs
        return _ufuncs.right_shift(self, other, self)

    def __lt__(self, other):
        return self._binary('less', other)

    def __le__(self, other):
        return self._binary('less_equal', other)

    def __gt__(self, other):
        return self._binary('greater', other)

    def __ge__(self, other):
        return self._binary('greater_equal', other)

    def __eq__(self, other):
        return self._binary('equal', other)

    def __ne__(self, other):
        return self._binary('not_equal', other)

    # -- reductions ---------------------------------------------------------------
    def sum(self, axis=None, dtype=None, out=None, keepdims=False):
        from cupy_amd._core import _routines_math
        return _routines_math._ndarray_sum(self, axis, dtype, out, keepdims)

    def prod(self, axis=None, dtype=None, out=None, keepdims=False):
        from cupy_amd._core import _routines_math
        return _routines_math._ndarray_prod(self, axis, dtype, out, keepdims)

    def max(self, axis=None, out=None, keepdims=False):
        from cupy_amd._core import _routines_statistics
        return _routines_statistics._ndarray_max(self, axis, out, None, keepdims)

    def min(self, axis=None, out=None, keepdims=False):
        from cupy_amd._core import _routines_statistics
        return _routines_statistics._ndarray_min(self, axis, out, None, keepdims)

    def argmax(self, axis=None, out=None, dtype=None, keepdims=False):
        from cupy_amd._core import _routines_statistics
        return _routines_statistics._ndarray_argmax(self, axis, out, dtype, keepdims)

    def argmin(self, axis=None, out=None, dtype=None, keepdims=False):
        from cupy_amd._core import _routines_statistics
        return _routines_statistics._ndarray_argmin(self, axis, out, dtype, keepdims)

    def mean(self, axis=None, dtype=None, out=None, keepdims=False):
        from cupy_amd._core import _routines_statistics
        return _routines_statistics._ndarray_mean(self, axis, dtype, out, keepdims)

    def var(self, axis=None, dtype=None, out=None, ddof=0, keepdims=False):
        from cupy_amd._core import _routines_statistics
        return _routines_statistics._ndarray_var(
            self, axis=axis, dtype=dtype, out=out, ddof=ddof, keepdims=keepdims)

    def std(self, axis=None, dtype=None, out=None, ddof=0, keepdims=False):
        from cupy_amd._core import _routines_statistics
        return _routines_statistics._ndarray_std(
            self, axis=axis, dtype=dtype, out=out, ddof=ddof, keepdims=keepdims)

    def ptp(self, axis=None, out=None, keepdims=False):
        from cupy_amd._core import _routines_statistics
        return _routines_statistics._ndarray_ptp(self, axis, out, keepdims)

    def clip(self, min=None, max=None, out=None):
        """Values limited to ``[min, max]`` (reference: cupy/_core/core.pyx
        ``ndarray.clip`` -> ``_routines_math._ndarray_clip``)."""
        from cupy_amd._core import _ufuncs
        return _ufuncs.clip(self, min, max, out=out)

    def cumsum(self, axis=None, dtype=None, out=None):
        from cupy_amd._core import _scan
        return _scan.cumsum(self, axis, dtype, out)

    def cumprod(self, axis=None, dtype=None, out=None):
        from cupy_amd._core import _scan
        return _scan.cumprod(self, axis, dtype, out)

    # -- complex numbers (reference: cupy/_core/core.pyx real/imag/conj) ----------------
    def _complex_part(self, second):
        part = numpy.dtype('float32' if self.dtype.itemsize == 8 else 'float64')
        v = self._view(self._shape, self._strides, part)
        if second:
            v.data = self.data + part.itemsize
        return v

    @property
    def real(self):
        """Real part: a view of the same memory for complex arrays, the array
        itself otherwise."""
        if self.dtype.kind == 'c':
            return self._complex_part(False)
        return self

    @real.setter
    def real(self, value):
        from cupy_amd._core._ufuncs import elementwise_copy
        elementwise_copy(value, self.real, casting='unsafe')

    @property
    def imag(self):
        """Imaginary part: a view of the same memory for complex arrays, a new
        array of zeros otherwise."""
        if self.dtype.kind == 'c':
            return self._complex_part(True)
        out = ndarray._new_contiguous(self._shape, self.dtype)
        out.fill(0)
        return out

    @imag.setter
    def imag(self, value):
        if self.dtype.kind != 'c':
            raise TypeError('cupy.ndarray does not have imaginary part to set')
        from cupy_amd._core._ufuncs import elementwise_copy
        elementwise_copy(value, self.imag, casting='unsafe')

    def conj(self):
        """Complex conjugate; the array itself when it is not complex."""
        if self.dtype.kind != 'c':
            return self
        from cupy_amd._core._ufuncs import conjugate
        return conjugate(self)

    conjugate = conj

    def round(self, decimals=0, out=None):
        from cupy_amd._core._ufuncs import around
        return around(self, decimals, out)

    def any(self, axis=None, out=None, keepdims=False):
        from cupy_amd._core import _routines_logic
        return _routines_logic._ndarray_any(self, axis, out, keepdims)

    def all(self, axis=None, out=None, keepdims=False):
        from cupy_amd._core import _routines_logic
        return _routines_logic._ndarray_all(self, axis, out, keepdims)


# ---------------------------------------------------------------------------------
# helpers
# ---------------------------------------------------------------------------------

def _reshape_strides(old_shape, old_strides, new_shape, itemsize):
    """Strides that present the same elements under ``new_shape`` without a
    copy, or None when the layout does not allow it."""
    size = internal.prod(new_shape)
    if size == 0:
        return internal.get_contiguous_strides(new_shape, itemsize)
    old = [(sh, st) for sh, st in zip(old_shape, old_strides) if sh != 1]
    new_strides = [0] * len(new_shape)
    oi = 0
    ni = 0
    n_old = len(old)
    n_new = len(new_shape)
    while ni < n_new:
        if new_shape[ni] == 1:
            # any stride will do; use the one a C-contiguous array would have
            new_strides[ni] = itemsize
            ni += 1
            continue
        if oi >= n_old:
            return None
        # Grow a group of old axes and a group of new axes until their
        # element counts agree.
        o_end = oi + 1
        n_end = ni + 1
        o_count = old[oi][0]
        n_count = new_shape[ni]
        while o_count != n_count:
            if n_count < o_count:
                if n_end >= n_new:
                    return None
                n_count *= new_shape[n_end]
                n_end += 1
            else:
                if o_end >= n_old:
                    return None
                o_count *= old[o_end][0]
                o_end += 1
        # The old axes of the group must lie back to back in memory.
        for k in range(oi, o_end - 1):
            if old[k][1] != old[k + 1][1] * old[k + 1][0]:
                return None
        st = old[o_end - 1][1]
        for k in range(n_end - 1, ni - 1, -1):
            new_strides[k] = st
            st *= new_shape[k]
        oi, ni = o_end, n_end
    # fix up strides of unit axes so that a contiguous result is recognised
    st = itemsize
    for k in range(n_new - 1, -1, -1):
        if new_shape[k] == 1:
            new_strides[k] = st
        else:
            st = new_strides[k] * new_shape[k]
    return tuple(new_strides)


def _basic_index(shape, strides, key):
    """Applies ints / slices / None / Ellipsis; returns (shape, strides,
    byte offset)."""
    if not isinstance(key, tuple):
        key = (key,)
    n_ellipsis = sum(1 for k in key if k is Ellipsis)
    if n_ellipsis > 1:
        raise IndexError('an index can only have a single ellipsis (\'...\')')
    n_consume = sum(1 for k in key if k is not None and k is not Ellipsis)
    nd = len(shape)
    if n_consume > nd:
        raise IndexError('too many indices for array: array is %d-dimensional, '
                         'but %d were indexed' % (nd, n_consume))
    if n_ellipsis == 0:
        key = key + (Ellipsis,)
    out_shape = []
    out_strides = []
    offset = 0
    ax = 0
    for k in key:
        if k is Ellipsis:
            n = nd - n_consume
            out_shape.extend(shape[ax:ax + n])
            out_strides.extend(strides[ax:ax + n])
            ax += n
        elif k is None:
            out_shape.append(1)
            out_strides.append(0)
        elif isinstance(k, slice):
            s = internal.complete_slice(k, shape[ax])
            if s.step > 0:
                n = max(0, (s.stop - s.start + s.step - 1) // s.step)
            else:
                n = max(0, (s.stop - s.start + s.step + 1) // s.step)
            out_shape.append(n)
            out_strides.append(strides[ax] * s.step)
            if n > 0:
                offset += s.start * strides[ax]
            ax += 1
        elif isinstance(k, (ndarray, numpy.ndarray, list)) and not (
                isinstance(k, (ndarray, numpy.ndarray)) and k.ndim == 0
                and k.dtype.kind in 'iu'):
            raise NotImplementedError(
                'indexing with arrays is outside the generated-kernel path of '
                'this package; only ints, slices, None and Ellipsis are supported')
        else:
            try:
                i = operator.index(k)
            except TypeError:
                raise IndexError(
                    'only integers, slices (`:`), ellipsis (`...`) and '
                    'numpy.newaxis (`None`) are valid indices')
            ext = shape[ax]
            if not -ext <= i < ext:
                raise IndexError('index %d is out of bounds for axis %d with '
                                 'size %d' % (i, ax, ext))
            if i < 0:
                i += ext
            offset += i * strides[ax]
            ax += 1
    return tuple(out_shape), tuple(out_strides), offset


def _ascontiguous(a):
    out = ndarray._new_contiguous(a._shape, a.dtype)
    if a.size:
        from cupy_amd._core._ufuncs import elementwise_copy
        elementwise_copy(a, out)
    return out


def ascontiguousarray(a, dtype=None):
    a = array(a, dtype=dtype, copy=False)
    return a if a._c_contiguous else _ascontiguous(a)


def _from_cuda_array_interface(obj):
    desc = obj.__cuda_array_interface__
    shape = tuple(desc['shape'])
    dt = numpy.dtype(desc['typestr'])
    strides = desc.get('strides')
    ptr = desc['data'][0] or 0
    nbytes = _byte_extent(
        shape, strides or internal.get_contiguous_strides(shape, dt.itemsize),
        dt.itemsize)[1]
    mem = _memory.UnownedMemory(ptr, nbytes, obj)
    return ndarray(shape, dt, _memory.MemoryPointer(mem, 0), strides)


def _convert_from_cupy_like(obj, error=False):
    """ndarray for ndarrays and foreign device arrays; None (or a TypeError
    naming ``error``) otherwise."""
    if isinstance(obj, ndarray):
        return obj
    getter = getattr(obj, '__cupy_get_ndarray__', None)
    if getter is not None:
        return getter()
    if hasattr(obj, '__cuda_array_interface__'):
        return _from_cuda_array_interface(obj)
    if error:
        raise TypeError(
            f"{error} has incorrect type (expected cupy.ndarray or an object "
            f"exposing __cuda_array_interface__, got {type(obj).__name__})")
    return None


def array(obj, dtype=None, copy=True, order='K', subok=False, ndmin=0):
    """Creates a device array from an array-like (host data is uploaded)."""
    if isinstance(obj, ndarray) or hasattr(obj, '__cuda_array_interface__') \
            or hasattr(obj, '__cupy_get_ndarray__'):
        src = _convert_from_cupy_like(obj)
        want = (order or 'K').upper()
        if dtype is not None and _dtype.get_dtype(dtype) != src.dtype:
            out = src.astype(dtype, order=want)
        elif copy or (want == 'C' and not src._c_contiguous) \
                or (want == 'F' and not src._f_contiguous):
            out = src.copy(order=want)
        else:
            out = src
    else:
        host = numpy.asarray(obj, dtype=dtype)
        _dtype.check_supported_dtype(host.dtype)
        keep_f = (order in ('K', 'A', 'F', 'k', 'a', 'f') and host.ndim > 1
                  and host.flags.f_contiguous and not host.flags.c_contiguous) \
            or (order in ('F', 'f') and host.ndim > 1)
        out = ndarray._new_contiguous(host.shape, host.dtype, c_order=not keep_f)
        if out.size:
            # the bytes of an F-ordered array are those of its C-ordered transpose
            buf = numpy.require(host.T if keep_f else host, requirements='C')
            # synchronous copy: the data is on the device when it returns,
            # whichever stream uses it next
            out.data.copy_from_host(buf.ctypes.data, out.nbytes)
    if out.ndim < ndmin:
        out = out.reshape((1,) * (ndmin - out.ndim) + out._shape)
    return out


def asarray(a, dtype=None, order=None):
    return array(a, dtype=dtype, copy=False, order=order or 'K')


def asnumpy(a, stream=None, order='C', out=None, blocking=True):
    """Host copy of a device array (host arrays pass through)."""
    if isinstance(a, ndarray):
        return a.get(stream=stream, order=order, out=out, blocking=blocking)
    if hasattr(a, '__cuda_array_interface__'):
        return _from_cuda_array_interface(a).get(stream=stream, out=out)
    return numpy.asarray(a, order=order)


# the extension module recognises this package's arrays and NumPy's scalars by type
_rt.hot.setup(ndarray, numpy.generic)
