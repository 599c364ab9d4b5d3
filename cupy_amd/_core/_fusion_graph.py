"""Recording of a fused function as a graph of values.

``cupy.fuse`` runs the decorated function once on stand-ins for its arguments
(``Proxy``).  Every ufunc call and reduction made on them is noted by the
``Recorder`` as a node of a value graph (``Value``) with its loop, dtype and
shape already resolved; nothing is computed.  ``fusion.py`` then decides how
many kernels the graph needs and ``_fusion_emit.py`` writes them.

The reference records with two tracers (cupy/_core/fusion.pyx:370-785 for the
one-kernel case, cupy/_core/_fusion_trace.pyx:26-624 for everything else); here
one recorder serves every back end.

What a proxy can do while recording:

* arithmetic, comparisons and every ``cupy`` ufunc, with ``out=`` and the
  in-place operators (the proxy then stands for the new value, and if it is
  bound to an argument array that array receives the value at the end);
* ``astype``, ``copy``, ``x[...] = v``, ``sum / prod / max / min / any / all``;
* ``x[index]`` with integers, slices, ``None`` and ``...`` on an argument or a
  captured array (a view of it becomes one more input of the kernels);
* ``shape``, ``ndim``, ``size``, ``dtype``.

Anything else raises ``NotImplementedError`` and the caller runs the function
as written.
"""
import numpy

from cupy_amd._core import internal
from cupy_amd._core import _kernel
from cupy_amd._core._dtype import get_dtype, _raise_if_invalid_cast
from cupy_amd._core.core import ndarray

_SCALAR_TYPES = (int, float, complex, bool, numpy.generic)


class Value:
    """One value of the recorded function.

    kind      fields
    'array'   source: ('arg', position) | ('captured', ndarray) |
              ('view', base Value, index); an input array of the kernels
    'scalar'  source: ('arg', position); weak: Python type or False
    'const'   const: the Python / NumPy scalar; weak as above
    'apply'   call: the ``Apply`` this value is output ``index`` of
    'reduce'  func, src, axes, loop: a reduction of ``src`` over ``axes``
    'keepdims' src: a reduced value with the reduced axes put back as 1
    """
    __slots__ = ('kind', 'order', 'dtype', 'shape', 'source', 'weak', 'const', 'call',
                 'index', 'func', 'src', 'axes', 'axis_arg', 'loop')

    def __init__(self, kind, order, dtype, shape):
        self.kind = kind
        self.order = order
        self.dtype = dtype
        self.shape = shape          # None for scalars
        self.source = self.const = self.call = self.func = self.src = None
        self.axes = self.axis_arg = self.loop = None
        self.weak = False
        self.index = 0

    @property
    def inputs(self):
        if self.kind == 'apply':
            return self.call.inputs
        if self.kind in ('reduce', 'keepdims'):
            return (self.src,)
        return ()

    def __repr__(self):
        return '<%s #%d %s %s>' % (self.kind, self.order, self.dtype, self.shape)


class Apply:
    """One ufunc call: the loop that was selected and the values it reads."""
    __slots__ = ('ufunc', 'loop', 'inputs', 'in_dtypes', 'out_dtypes')

    def __init__(self, ufunc, loop, inputs):
        self.ufunc = ufunc
        self.loop = loop
        self.inputs = tuple(inputs)
        self.in_dtypes = tuple(numpy.dtype(t) for t in loop.in_types)
        self.out_dtypes = tuple(numpy.dtype(t) for t in loop.out_types)


def _u(name):
    from cupy_amd._core import _ufuncs
    return getattr(_ufuncs, name)


def _binary(name, reflected=False):
    def op(self, other):
        return _u(name)(other, self) if reflected else _u(name)(self, other)
    return op


def _inplace(name):
    def op(self, other):
        return _u(name)(self, other, self)
    return op


def _unary(name):
    def op(self):
        return _u(name)(self)
    return op


class Proxy:
    """Stand-in for an argument or an intermediate value while the function is
    recorded.  ``_value`` is what the proxy stands for right now; it changes
    when the proxy is written to (``x += y``, ``out=x``, ``x[...] = v``)."""
    __slots__ = ('_rec', '_value', '_home')
    __array_priority__ = 1000

    def __init__(self, rec, value, home=None):
        self._rec = rec
        self._value = value
        self._home = home           # the argument array's Value this proxy writes back to

    # -- what the function may ask about a value --------------------------------------
    @property
    def dtype(self):
        return self._value.dtype

    @property
    def shape(self):
        self._rec.shape_dependent = True
        if self._value.shape is None:
            return ()
        return self._value.shape

    @property
    def ndim(self):
        return 0 if self._value.shape is None else len(self._value.shape)

    @property
    def size(self):
        return internal.prod(self.shape)

    def __len__(self):
        shape = self.shape
        if not shape:
            raise TypeError('len() of unsized object')
        return shape[0]

    def __repr__(self):
        return '<fused value %s %s>' % (self._value.dtype, self._value.shape)

    __hash__ = None

    def __bool__(self):
        raise TypeError('the truth value of an array is not known while a fused '
                        'function is recorded')

    # -- operators are ufunc calls, which report to the recorder ----------------------
    for _name, _uf in (
            ('add', 'add'), ('sub', 'subtract'), ('mul', 'multiply'),
            ('truediv', 'true_divide'), ('floordiv', 'floor_divide'), ('mod', 'remainder'),
            ('lshift', 'left_shift'), ('rshift', 'right_shift'),
            ('and', 'bitwise_and'), ('or', 'bitwise_or'), ('xor', 'bitwise_xor')):
        locals()['__%s__' % _name] = _binary(_uf)
        locals()['__r%s__' % _name] = _binary(_uf, True)
        locals()['__i%s__' % _name] = _inplace(_uf)
    for _name, _uf in (('lt', 'less'), ('le', 'less_equal'), ('gt', 'greater'),
                       ('ge', 'greater_equal'), ('eq', 'equal'), ('ne', 'not_equal')):
        locals()['__%s__' % _name] = _binary(_uf)
    __neg__ = _unary('negative')
    __pos__ = _unary('positive')
    __abs__ = _unary('absolute')
    __invert__ = _unary('invert')
    __rpow__ = _binary('power', True)
    __ipow__ = _inplace('power')
    del _name, _uf

    def __pow__(self, other):
        # the short cuts ndarray.__pow__ (and NumPy) take for Python exponents:
        # squaring is a multiply, not a call to pow()
        if type(other) in (int, float):
            kind = self._value.dtype.kind
            if other == 2 and (kind in 'fc' or (kind in 'iub' and type(other) is int)):
                return _u('square')(self)
            if kind == 'f' and other == 0.5:
                return _u('sqrt')(self)
            if kind == 'f' and other == -1:
                return _u('reciprocal')(self)
        return _u('power')(self, other)

    # -- methods ----------------------------------------------------------------------
    def copy(self):
        return _u('elementwise_copy')(self)

    def astype(self, dtype, order=None, casting=None, subok=None, copy=True):
        for name, given in (('order', order), ('casting', casting), ('subok', subok)):
            if given is not None:
                raise TypeError('%s is not supported yet' % name)
        dtype = get_dtype(dtype)
        if not copy and self._value.dtype == dtype:
            return self
        from cupy_amd._core import fusion
        return fusion._dtype_to_astype(dtype)(self)

    def __setitem__(self, key, value):
        if key is Ellipsis or (isinstance(key, slice) and key == slice(None)):
            _u('elementwise_copy')(value, self)
        else:
            raise ValueError('The fusion supports `[...]` or `[:]`.')

    def __getitem__(self, key):
        return self._rec.index(self, key)

    def sum(self, axis=None, dtype=None, out=None, keepdims=False):
        from cupy_amd._core import _routines_math
        return _routines_math.sum(self, axis, dtype, out, keepdims)

    def prod(self, axis=None, dtype=None, out=None, keepdims=False):
        from cupy_amd._core import _routines_math
        return _routines_math.prod(self, axis, dtype, out, keepdims)

    def max(self, axis=None, out=None, keepdims=False):
        from cupy_amd._core import _routines_statistics
        return _routines_statistics.amax(self, axis, out, keepdims)

    def min(self, axis=None, out=None, keepdims=False):
        from cupy_amd._core import _routines_statistics
        return _routines_statistics.amin(self, axis, out, keepdims)

    def any(self, axis=None, out=None, keepdims=False):
        from cupy_amd._core import _routines_logic
        return _routines_logic.any(self, axis, out, keepdims)

    def all(self, axis=None, out=None, keepdims=False):
        from cupy_amd._core import _routines_logic
        return _routines_logic.all(self, axis, out, keepdims)


class Recorder:
    """Collects the values of one run of the function.  Installed as the
    thread's fusion history, so ufuncs and reductions report here
    (``call_ufunc`` / ``call_reduction``)."""
    split = True        # reductions may keep their axes (``records_keepdims``)

    def __init__(self):
        self.values = []
        self.shape_dependent = False     # the function looked at a shape
        self.stores = {}                 # order of an argument's Value -> its Proxy
        self.viewed = set()              # orders of argument Values indexed by the function
        self._captured = {}

    # -- creation of values -------------------------------------------------------------
    def _new(self, kind, dtype, shape):
        v = Value(kind, len(self.values), dtype, shape)
        self.values.append(v)
        return v

    def argument(self, position, a):
        """Proxy for argument ``a`` of the fused function (None stays None)."""
        if a is None:
            return None
        if isinstance(a, ndarray):
            v = self._new('array', a.dtype, tuple(a.shape))
            v.source = ('arg', position)
            return Proxy(self, v, home=v)
        v = self._new('scalar', *self._scalar_type(a))
        v.source = ('arg', position)
        v.weak = self._weak(a)
        return Proxy(self, v)

    @staticmethod
    def _scalar_type(a):
        if isinstance(a, numpy.generic):
            return a.dtype, None
        return numpy.dtype(type(a)), None

    @staticmethod
    def _weak(a):
        t = type(a)
        return t if t in (int, float, complex) else False

    def _operand(self, a):
        """The Value behind anything a ufunc may be called with."""
        if isinstance(a, Proxy):
            if a._rec is not self:
                raise NotImplementedError('value of another recording')
            return a._value
        if isinstance(a, ndarray):
            # an array the function captured from its surroundings: one more input
            v = self._captured.get(id(a))
            if v is None:
                v = self._new('array', a.dtype, tuple(a.shape))
                v.source = ('captured', a)
                self._captured[id(a)] = v
            return v
        if isinstance(a, _SCALAR_TYPES):
            v = self._new('const', *self._scalar_type(a))
            v.const = a
            v.weak = self._weak(a)
            return v
        raise TypeError('Unsupported type {}'.format(type(a)))

    # -- indexing ---------------------------------------------------------------------
    def index(self, proxy, key):
        """``x[key]`` for an argument (or captured) array: the view becomes an
        input of its own.  Only what yields a view is recorded."""
        base = proxy._value
        if base.kind != 'array':
            raise NotImplementedError('indexing of an intermediate value is not recorded')
        return self._index_view(base, key)

    def _index_view(self, base, key):
        keys = key if isinstance(key, tuple) else (key,)
        for k in keys:
            if not (k is None or k is Ellipsis or isinstance(k, (int, slice, numpy.integer))):
                raise NotImplementedError('only basic indexing is recorded')
        root = base
        chain = [key]
        while root.source[0] == 'view':
            chain.append(root.source[2])
            root = root.source[1]
        if root.order in self.stores:
            raise NotImplementedError('a view of an array that was written before')
        # the shape comes from indexing a stand-in of the same shape (raises
        # IndexError exactly where the array would)
        stand_in = numpy.lib.stride_tricks.as_strided(
            numpy.empty((), numpy.int8), base.shape, (0,) * len(base.shape))
        shape = stand_in[key].shape
        v = self._new('array', base.dtype, tuple(shape))
        v.source = ('view', base, key)
        self.viewed.add(root.order)
        self.shape_dependent = True      # integer indices and slice bounds met real extents
        return Proxy(self, v)

    # -- ufuncs -----------------------------------------------------------------------
    def call_ufunc(self, ufunc, *args, **kwargs):
        nin, nout = ufunc.nin, ufunc.nout
        args = list(args)
        outs = args[nin:]
        args = args[:nin]
        out = kwargs.pop('out', None)
        if out is not None:
            if outs:
                raise ValueError('cannot specify \'out\' as both a positional '
                                 'and keyword argument')
            outs = list(out) if isinstance(out, tuple) else [out]
        dtype = kwargs.pop('dtype', None)
        casting = kwargs.pop('casting', None) or 'same_kind'
        kwargs = {k: v for k, v in kwargs.items() if v is not None}
        if kwargs:
            raise TypeError('Wrong arguments {}'.format(kwargs))
        if len(args) != nin or len(outs) > nout:
            raise ValueError('invalid number of arguments')
        for o in outs:
            if o is not None and not (isinstance(o, Proxy) and o._value.shape is not None):
                raise TypeError('return arrays must be of ArrayType')

        operands = [self._operand(a) for a in args]
        in_dtypes = tuple(v.dtype for v in operands)
        if dtype is not None:
            loop = ufunc._ops._guess_routine_from_dtype(get_dtype(dtype))
        else:
            weaks = tuple(v.weak for v in operands)
            if not _kernel._check_should_use_weak_scalar(
                    in_dtypes, weaks if any(weaks) else None):
                weaks = (False,) * nin
            loop = ufunc._ops._guess_routine_from_in_types(in_dtypes, weaks)
        if loop is None:
            raise TypeError('Invalid type cast in \'{}\': {} -> {}'.format(
                ufunc.name, [str(t) for t in in_dtypes],
                [str(o._value.dtype) for o in outs if o is not None]))
        loop.check_valid()

        shapes = [v.shape for v in operands if v.shape is not None]
        shape = tuple(numpy.broadcast_shapes(*shapes)) if shapes else None
        call = Apply(ufunc, loop, operands)
        results = []
        for i in range(nout):
            v = self._new('apply', call.out_dtypes[i], shape)
            v.call = call
            v.index = i
            target = outs[i] if i < len(outs) else None
            if target is None:
                results.append(Proxy(self, v))
            else:
                results.append(self._assign(target, v, casting, i))
        return results[0] if nout == 1 else tuple(results)

    def _assign(self, target, value, casting, i=0):
        """``target`` (a proxy) now stands for ``value``, converted to the
        target's dtype and shape."""
        t = target._value
        _raise_if_invalid_cast(value.dtype, t.dtype, casting, lambda: f'output {i}')
        if value.shape is not None:
            if tuple(numpy.broadcast_shapes(value.shape, t.shape)) != tuple(t.shape):
                raise ValueError('non-broadcastable output operand with shape %s doesn\'t '
                                 'match the broadcast shape %s' % (t.shape, value.shape))
        if value.dtype != t.dtype:
            from cupy_amd._core import fusion
            cast = fusion._dtype_to_astype(t.dtype)
            loop = cast._ops._guess_routine_from_in_types((value.dtype,), None)
            if loop is None:
                raise TypeError('cannot convert %s to %s' % (value.dtype, t.dtype))
            call = Apply(cast, loop, [value])
            value = self._new('apply', t.dtype, value.shape)
            value.call = call
        if value.shape != t.shape:
            # written into a larger array: every element of the target receives a value
            spread = self._new('apply', t.dtype, tuple(t.shape))
            spread.call = Apply(_u('elementwise_copy'),
                                _u('elementwise_copy')._ops._guess_routine_from_in_types(
                                    (value.dtype,), None), [value])
            value = spread
        home = target._home
        if home is not None:
            if home.order in self.viewed:
                raise NotImplementedError('writing to an array the function also indexes')
            self.stores[home.order] = target
        target._value = value
        return target

    # -- reductions ----------------------------------------------------------------------
    def call_reduction(self, func, a, axis=None, dtype=None, out=None, keepdims=False):
        if out is not None:
            raise NotImplementedError('out= of a reduction is not recorded')
        src = self._operand(a)
        if src.shape is None:
            raise NotImplementedError('reduction of a scalar')
        ndim = len(src.shape)
        if axis is None:
            axes = tuple(range(ndim))
        elif isinstance(axis, (tuple, list)):
            axes = tuple(sorted(internal._normalize_axis_index(ax, ndim) for ax in axis))
        else:
            axes = (internal._normalize_axis_index(axis, ndim),)
        if len(set(axes)) != len(axes):
            raise ValueError('duplicate value in \'axis\'')
        loop = None
        if dtype is not None:
            loop = func._ops._guess_routine_from_dtype(get_dtype(dtype))
        else:
            for candidate in func._ops.ops:
                if numpy.can_cast(src.dtype, candidate.in_types[0]):
                    loop = candidate
                    break
        if loop is None:
            raise TypeError('Type is mismatched. {}(...), {}'.format(func.name, src.dtype.type))
        shape = tuple(s for i, s in enumerate(src.shape) if i not in axes)
        v = self._new('reduce', numpy.dtype(loop.out_types[0]), shape)
        v.func, v.src, v.axes, v.axis_arg, v.loop = func, src, axes, axis, loop
        if keepdims:
            kept = tuple(1 if i in axes else s for i, s in enumerate(src.shape))
            k = self._new('keepdims', v.dtype, kept)
            k.src, k.axes = v, axes
            v = k
        return Proxy(self, v)
