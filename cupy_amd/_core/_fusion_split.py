"""Fused functions that need more than one kernel.

A function with several reductions, or one that combines a reduced value with
an array again, is not a single elementwise or map-reduce kernel.  The
reference hands such functions to its general tracer
(cupy/_core/_fusion_trace.pyx:26-624, _fusion_kernel.pyx:57-381), which emits
one kernel with grid-wide barriers between the passes -- a cooperative launch
that HIP does not offer for run-time compiled code.

Here the function is recorded once as a graph of ufunc and reduction calls and
cut at the reductions: every reduction, together with all elementwise work that
feeds it, becomes one map-reduce kernel; what remains after the last reduction
becomes one elementwise kernel per output shape.  Intermediate elementwise
values are never written to memory (a value needed by two kernels is computed
in both); only reduction results are, in pool memory, and the kernels run in
order on the current stream.  Each piece is compiled by the single-kernel
tracer of ``fusion.py``.

Not recorded (the caller then runs the function as written): in-place
operators and ``out=``, indexing, reshaping, functions that look at the dtype
of an intermediate value, ufuncs with several outputs.
"""
import numpy

from cupy_amd._core import _fusion_thread_local
from cupy_amd._core import internal
from cupy_amd._core.core import ndarray

_thread_local = _fusion_thread_local.thread_local


class _Node:
    """A value of the recorded graph."""
    __slots__ = ('kind', 'fn', 'args', 'kwargs', 'shape', 'order', 'dtype')

    def __init__(self, kind, fn, args, kwargs, shape, order, dtype=None):
        self.kind = kind        # 'leaf' | 'ufunc' | 'reduce' | 'keepdims'
        self.fn = fn            # ufunc / reduction function; leaf: position or array
        self.args = args
        self.kwargs = kwargs
        self.shape = shape      # None for scalars
        self.order = order      # creation order
        self.dtype = dtype      # known for leaves only


def _binary(name, reflected=False):
    def op(self, other):
        from cupy_amd._core import _ufuncs
        fn = getattr(_ufuncs, name)
        return fn(other, self) if reflected else fn(self, other)
    return op


def _unary(name):
    def op(self):
        from cupy_amd._core import _ufuncs
        return getattr(_ufuncs, name)(self)
    return op


def _inplace(self, other):
    raise NotImplementedError('in-place operators are not recorded')


class _Lazy:
    """Stand-in for an array (or scalar argument) while the function is
    recorded."""
    __slots__ = ('_tracer', '_node')
    __array_priority__ = 1000

    def __init__(self, tracer, node):
        self._tracer = tracer
        self._node = node

    @property
    def shape(self):
        if self._node.shape is None:
            raise AttributeError('shape')
        return self._node.shape

    @property
    def ndim(self):
        return 0 if self._node.shape is None else len(self._node.shape)

    @property
    def size(self):
        return internal.prod(self.shape)

    @property
    def dtype(self):
        if self._node.dtype is None:
            raise NotImplementedError('dtype of an intermediate value is not recorded')
        return self._node.dtype

    for _name, _uf in (
            ('add', 'add'), ('sub', 'subtract'), ('mul', 'multiply'),
            ('truediv', 'true_divide'), ('floordiv', 'floor_divide'), ('mod', 'remainder'),
            ('pow', 'power'), ('lshift', 'left_shift'), ('rshift', 'right_shift'),
            ('and', 'bitwise_and'), ('or', 'bitwise_or'), ('xor', 'bitwise_xor')):
        locals()['__%s__' % _name] = _binary(_uf)
        locals()['__r%s__' % _name] = _binary(_uf, True)
        locals()['__i%s__' % _name] = _inplace
    for _name, _uf in (('lt', 'less'), ('le', 'less_equal'), ('gt', 'greater'),
                       ('ge', 'greater_equal'), ('eq', 'equal'), ('ne', 'not_equal')):
        locals()['__%s__' % _name] = _binary(_uf)
    __neg__ = _unary('negative')
    __pos__ = _unary('positive')
    __abs__ = _unary('absolute')
    __invert__ = _unary('invert')
    del _name, _uf
    __hash__ = None

    def __bool__(self):
        raise TypeError('the truth value of an array is not known while a fused '
                        'function is recorded')

    def __setitem__(self, key, value):
        raise NotImplementedError('assignment is not recorded')

    def __getitem__(self, key):
        raise NotImplementedError('indexing is not recorded')

    def copy(self):
        from cupy_amd._core import _ufuncs
        return _ufuncs.elementwise_copy(self)

    def astype(self, dtype, order=None, casting=None, subok=None, copy=True):
        from cupy_amd._core import fusion
        return fusion._dtype_to_astype(numpy.dtype(dtype))(self)

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


def _apply_reduction(func, value, axis, dtype):
    """The reduction ``func`` inside a piece: traced by the single-kernel
    tracer, or run directly when the piece is evaluated with real arrays."""
    if _fusion_thread_local.is_fusing():
        return _fusion_thread_local.call_reduction(func, value, axis=axis, dtype=dtype)
    return func(value, axis, dtype, None, False)


class _Tracer:
    """Records the calls of one run of the function (installed as the thread's
    fusion history, so ufuncs and reductions report here)."""
    split = True

    def __init__(self):
        self.nodes = []

    def _node(self, *args, **kwargs):
        n = _Node(*args, order=len(self.nodes), **kwargs)
        self.nodes.append(n)
        return n

    def leaf(self, position, value):
        if isinstance(value, ndarray):
            return self._node('leaf', position, (), {}, value.shape, dtype=value.dtype)
        return self._node('leaf', position, (), {}, None,
                          dtype=getattr(value, 'dtype', None))

    def _operand(self, a):
        """Graph node, or the value itself for constants."""
        if isinstance(a, _Lazy):
            if a._tracer is not self:
                raise NotImplementedError('value of another recording')
            return a._node
        if isinstance(a, ndarray):
            # an array captured by the function: a leaf that is not an argument
            return self._node('leaf', a, (), {}, a.shape, dtype=a.dtype)
        if isinstance(a, (int, float, complex, bool, numpy.generic)):
            return a
        raise NotImplementedError('operand of type %s is not recorded' % type(a))

    def call_ufunc(self, ufunc, *args, **kwargs):
        if getattr(ufunc, 'nout', 1) != 1 or len(args) != ufunc.nin:
            raise NotImplementedError('only ufunc(inputs...) -> one output is recorded')
        kwargs = {k: v for k, v in kwargs.items() if v is not None}
        if 'out' in kwargs or '_where' in kwargs or 'where' in kwargs:
            raise NotImplementedError('out= / where= are not recorded')
        operands = [self._operand(a) for a in args]
        shapes = [o.shape for o in operands if isinstance(o, _Node) and o.shape is not None]
        shape = numpy.broadcast_shapes(*shapes) if shapes else None
        return _Lazy(self, self._node('ufunc', ufunc, tuple(operands), kwargs, shape))

    def call_reduction(self, func, a, axis=None, dtype=None, out=None, keepdims=False):
        if out is not None:
            raise NotImplementedError('out= is not recorded')
        src = self._operand(a)
        if not isinstance(src, _Node) or src.shape is None:
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
        shape = tuple(s for i, s in enumerate(src.shape) if i not in axes)
        node = self._node('reduce', func, (src,),
                          {'axis': axis, 'dtype': dtype, 'axes': axes}, shape)
        if keepdims:
            kept = tuple(1 if i in axes else s for i, s in enumerate(src.shape))
            node = self._node('keepdims', None, (node,), {'axes': axes}, kept)
        return _Lazy(self, node)


class _Piece:
    """One kernel of the plan: ``targets`` computed from ``leaves``."""
    __slots__ = ('fused', 'func', 'leaves', 'targets')

    def __init__(self, targets, leaves, stored, name):
        from cupy_amd._core import fusion
        self.targets = targets
        self.leaves = leaves
        stored_ids = frozenset(id(n) for n in stored)

        def piece(*values):
            env = {id(n): v for n, v in zip(leaves, values)}

            def value_of(n):
                if not isinstance(n, _Node):
                    return n
                v = env.get(id(n))
                if v is None:
                    assert id(n) not in stored_ids
                    if n.kind == 'ufunc':
                        v = n.fn(*[value_of(a) for a in n.args], **n.kwargs)
                    else:
                        v = _apply_reduction(n.fn, value_of(n.args[0]),
                                             n.kwargs['axis'], n.kwargs['dtype'])
                    env[id(n)] = v
                return v

            outs = tuple(value_of(t) for t in targets)
            return outs[0] if len(outs) == 1 else outs

        piece.__name__ = name
        self.func = piece
        self.fused = fusion.Fusion(piece, name, split=False)


class Plan:
    """The kernels of one recorded function, in launch order."""

    def __init__(self, steps, n_nodes, arg_leaves, const_leaves, returns, single):
        self.steps = steps
        self.n_nodes = n_nodes
        self.arg_leaves = arg_leaves        # (node order, argument position)
        self.const_leaves = const_leaves    # (node order, captured array)
        self.returns = returns              # node order, or ('const', value)
        self.single = single

    def run(self, *args):
        vals = [None] * self.n_nodes
        for order, pos in self.arg_leaves:
            vals[order] = args[pos]
        for order, value in self.const_leaves:
            vals[order] = value
        for step in self.steps:
            if step[0] == 'kernel':
                _, piece = step
                out = piece.fused(*[vals[n.order] for n in piece.leaves])
                if len(piece.targets) == 1:
                    vals[piece.targets[0].order] = out
                else:
                    for t, o in zip(piece.targets, out):
                        vals[t.order] = o
            else:
                _, node, axes = step
                base = vals[node.args[0].order]
                shape = list(base.shape)
                for ax in axes:
                    shape.insert(ax, 1)
                vals[node.order] = base.reshape(tuple(shape))
        outs = tuple(r[1] if isinstance(r, tuple) else vals[r] for r in self.returns)
        return outs[0] if self.single else outs


def _leaves_of(targets, stored):
    """Stored nodes that ``targets`` are computed from, in creation order."""
    seen = set()
    found = {}
    stack = list(targets)
    while stack:
        n = stack.pop()
        if not isinstance(n, _Node) or id(n) in seen:
            continue
        seen.add(id(n))
        if id(n) in stored and not any(n is t for t in targets):
            found[n.order] = n
            continue
        if n.kind == 'leaf':
            found[n.order] = n
            continue
        stack.extend(n.args)
    return [found[k] for k in sorted(found)]


def trace(func, args, name):
    """Records ``func(*args)`` and cuts it into kernels.  Raises whatever the
    function raises on stand-in arguments, or NotImplementedError for what is
    not recorded."""
    tracer = _Tracer()
    lazy_args = []
    arg_leaves = []
    for pos, a in enumerate(args):
        if a is None:
            lazy_args.append(None)
            continue
        node = tracer.leaf(pos, a)
        arg_leaves.append((node.order, pos))
        lazy_args.append(_Lazy(tracer, node))
    _thread_local.history = tracer
    _thread_local.is_old_fusing = True
    try:
        ret = func(*lazy_args)
    finally:
        _thread_local.history = None
        _thread_local.is_old_fusing = False

    single = not isinstance(ret, tuple)
    rets = (ret,) if single else ret
    nodes = tracer.nodes
    stored = {id(n): n for n in nodes if n.kind == 'leaf'}
    steps = []
    n_kernels = 0
    for n in nodes:
        if n.kind == 'reduce':
            leaves = _leaves_of([n], stored)
            steps.append(('kernel', _Piece(
                [n], leaves, list(stored.values()), '%s_part%d' % (name, n_kernels))))
            n_kernels += 1
            stored[id(n)] = n
        elif n.kind == 'keepdims':
            steps.append(('view', n, n.kwargs['axes']))
            stored[id(n)] = n
    # what is left: elementwise results, one kernel per shape
    returns = []
    pending = {}
    for r in rets:
        if isinstance(r, _Lazy):
            if r._tracer is not tracer:
                raise NotImplementedError('value of another recording')
            n = r._node
            returns.append(n.order)
            if id(n) not in stored:
                if n.shape is None:
                    raise NotImplementedError('scalar result')
                group = pending.setdefault(n.shape, [])
                if not any(n is m for m in group):
                    group.append(n)
        elif isinstance(r, ndarray) or r is None or isinstance(
                r, (int, float, complex, bool, numpy.generic)):
            returns.append(('const', r))
        else:
            raise NotImplementedError('return value of type %s' % type(r))
    for shape, group in pending.items():
        leaves = _leaves_of(group, stored)
        steps.append(('kernel', _Piece(
            group, leaves, list(stored.values()), '%s_part%d' % (name, n_kernels))))
        n_kernels += 1
    const_leaves = [(n.order, n.fn) for n in nodes
                    if n.kind == 'leaf' and isinstance(n.fn, ndarray)]
    # all reductions along the rows of one matrix, rows short enough for the
    # registers of a workgroup: one kernel that reads the matrix once
    from cupy_amd._core import _fusion_rows
    pieces = [st[1] for st in steps if st[0] == 'kernel']
    sequence = Plan(steps, len(nodes), arg_leaves, const_leaves, returns, single)
    row_plan = _fusion_rows.build(nodes, pieces, returns, single, args, name)
    if row_plan is not None:
        # for calls whose arrays are laid out differently from those the
        # kernel was built for
        row_plan.fallback = sequence
        return row_plan
    return sequence
