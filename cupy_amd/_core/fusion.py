"""``cupy.fuse``: run a Python function of array operations as few kernels as
possible.

The decorated function is recorded once per kind of arguments as a graph of
values (``_fusion_graph``).  What the graph needs decides the back end:

* no reduction                        one elementwise kernel;
* one reduction whose result is only
  combined with scalars afterwards    one map-reduce kernel;
* anything else (several reductions,
  a reduced value meeting an array
  again, results of several shapes)   one kernel that keeps rows in registers
                                      (``_fusion_rows``) when all reductions run
                                      along the rows of one matrix, else a
                                      sequence of map-reduce and elementwise
                                      kernels cut at the reductions
                                      (``_fusion_split``).

The kernels themselves are written by ``_fusion_emit`` and run on the same
emitters as hand-written ``ElementwiseKernel`` / ``ReductionKernel`` objects.

Call surface and caching follow the reference (cupy/_core/fusion.pyx:788-919:
``fuse``, ``Fusion``, ``clear_cache``; one specialisation per dtype and number
of dimensions of the array arguments and per Python type of the scalars, :833-858),
which needs two tracers and a cooperative launch for what is one recorder and
stream-ordered kernels here.  A function that cannot be recorded runs as
written: every operation launches its own kernel.
"""
import functools
import re

import numpy

from cupy_amd._core import _fusion_thread_local
from cupy_amd._core import _kernel
from cupy_amd._core import _launch_plan
from cupy_amd._core._scalar import get_typename
from cupy_amd._core.core import ndarray
from cupy_amd.cuda import device as _device

_thread_local = _fusion_thread_local.thread_local

_acceptable_types = (
    ndarray, numpy.ndarray, numpy.generic, int, float, complex, bool, type(None))

_EAGER = 'eager'            # memo entry: run the function as written
_BY_SHAPE = 'by shape'      # memo entry: plans are kept per argument shapes


def _types_key(args):
    """What a specialisation depends on: dtype and ndim of arrays, the Python
    type of scalars (cupy/_core/fusion.pyx:833-858)."""
    key = []
    for a in args:
        if isinstance(a, ndarray):
            key.append((a.dtype.char, a.ndim))
        elif isinstance(a, numpy.generic):
            key.append(a.dtype.char)
        elif a is None:
            key.append(None)
        else:
            key.append(type(a))
    return tuple(key)


class Recording:
    """One run of the function on proxies: the graph, what it returned and
    which argument arrays it wrote to."""

    def __init__(self, func, args):
        from cupy_amd._core import _fusion_graph
        rec = _fusion_graph.Recorder()
        proxies = [rec.argument(i, a) for i, a in enumerate(args)]
        saved = (getattr(_thread_local, 'history', None),
                 getattr(_thread_local, 'is_old_fusing', False))
        _fusion_thread_local.begin_recording()
        _thread_local.history = rec
        _thread_local.is_old_fusing = True
        try:
            ret = func(*proxies)
        finally:
            _thread_local.history, _thread_local.is_old_fusing = saved
            _fusion_thread_local.end_recording()
        self.recorder = rec
        self.single = not isinstance(ret, tuple)
        # every returned item: ('value', Value) | ('arg', position) | ('const', object)
        self.returns = []
        for r in ((ret,) if self.single else ret):
            if isinstance(r, _fusion_graph.Proxy):
                if r._rec is not rec:
                    raise NotImplementedError('value of another recording')
                home = r._home
                if home is not None and (r._value is home or rec.stores.get(home.order) is r):
                    # the argument itself, as it is after the call
                    self.returns.append(('arg', home.source[1]))
                elif r._value.kind == 'scalar':
                    self.returns.append(('arg', r._value.source[1]))
                elif r._value.kind == 'array':
                    # a captured array or a view, handed back as it is
                    self.returns.append(('leaf', _leaf_reader(r._value)))
                else:
                    self.returns.append(('value', r._value))
            elif r is None or isinstance(r, (ndarray, int, float, complex, bool, numpy.generic)):
                self.returns.append(('const', r))
            else:
                raise TypeError('Fusion function can\'t return {}'.format(type(r)))
        # argument arrays that end up with a new value
        self.stores = [(p._home, p._value) for p in rec.stores.values()]
        self.values = rec.values

    def roots(self):
        return [v for kind, v in self.returns if kind == 'value'] + [v for _, v in self.stores]


def _reachable(roots):
    seen = {}
    stack = list(roots)
    while stack:
        v = stack.pop()
        if v.order in seen:
            continue
        seen[v.order] = v
        stack.extend(v.inputs)
    return [seen[k] for k in sorted(seen)]


def _leaf_reader(v):
    """Function of the call's arguments that yields the array or scalar an
    input Value stands for."""
    what = v.source[0]
    if what == 'arg':
        pos = v.source[1]
        return lambda args: args[pos]
    if what == 'captured':
        arr = v.source[1]
        return lambda args: arr
    base = _leaf_reader(v.source[1])
    key = v.source[2]
    return lambda args: base(args)[key]


class _KernelPlan:
    """The whole function as one ElementwiseKernel or ReductionKernel call."""

    def __init__(self, kernel, leaves, kwargs, returns, n_targets, single, store_positions):
        self.kernel = kernel
        self.readers = [_leaf_reader(v) for v in leaves]
        self.kwargs = kwargs
        # ('out', k) | ('arg', position) | ('leaf', reader) | ('const', object)
        self.returns = returns
        self.n_targets = n_targets
        self.single = single
        self.store_positions = store_positions
        self.steps = (('kernel', self),)

    def run(self, *args):
        out = self.kernel(*[r(args) for r in self.readers], **self.kwargs)
        if self.n_targets == 1:
            out = (out,)
        return _collect(self.returns, out, args, self.single)

    def replay_runner(self, args):
        """After ``run(*args)``: a callable that goes straight to the launch
        record the kernel made for arguments of this signature (skipping the
        kernel object's own argument checks and signature lookup), or None."""
        kargs = [r(args) for r in self.readers]
        key = _launch_plan.call_signature(kargs, _device.get_device_id())
        if key is None:
            return None
        if 'axis' in self.kwargs or hasattr(self.kernel, 'map_expr'):
            key = key + ((self.kwargs.get('axis'), False),)
        fast = getattr(self.kernel, '_fast_calls', {}).get(key)
        if fast is None:
            return None
        readers, returns, single, one = self.readers, self.returns, self.single, self.n_targets == 1
        slow = self.run

        def run(*a):
            out = fast.run([r(a) for r in readers])
            if out is NotImplemented:       # an output overlaps an input this time
                return slow(*a)
            return _collect(returns, (out,) if one else out, a, single)
        return run


def _collect(returns, outs, args, single):
    """The call's return value from the kernels' outputs and the arguments."""
    res = tuple(outs[ref] if kind == 'out' else args[ref] if kind == 'arg' else
                ref(args) if kind == 'leaf' else ref for kind, ref in returns)
    return res[0] if single else res


class _PassThroughPlan:
    """A function that computes nothing: arguments, views of them and
    constants are handed back."""
    store_positions = ()
    steps = ()

    def __init__(self, returns, single):
        self.returns = returns
        self.single = single

    def run(self, *args):
        return _collect(self.returns, (), args, self.single)


def _plan_single_kernel(recording, name):
    """``_KernelPlan`` when the recorded function is one elementwise or one
    map-reduce kernel, else None."""
    from cupy_amd._core import _fusion_emit
    roots = recording.roots()
    if not roots:
        return None
    reach = _reachable(roots)
    reduces = [v for v in reach if v.kind == 'reduce']
    if any(v.kind == 'keepdims' for v in reach) or len(reduces) > 1:
        return None
    leaves = [v for v in reach if v.kind in ('array', 'scalar')]
    for leaf, _ in recording.stores:          # arrays that are written but never read
        if not any(leaf is m for m in leaves):
            leaves.append(leaf)
    targets = []
    returns = []
    for kind, ref in recording.returns:
        if kind != 'value':
            returns.append((kind, ref))
            continue
        if not any(ref is t for t in targets):
            targets.append(ref)
        returns.append(('out', [t.order for t in targets].index(ref.order)))
    store_positions = [leaf.source[1] for leaf, _ in recording.stores]
    if not reduces:
        shapes = set(r.shape for r in roots)
        if len(shapes) != 1 or None in shapes:
            return None
        shape, = shapes
        arrays = [v.shape for v in leaves if v.kind == 'array']
        if not arrays or tuple(numpy.broadcast_shapes(*arrays)) != tuple(shape):
            return None
        kernel = _fusion_emit.elementwise_kernel(name, leaves, targets, recording.stores)
        return _KernelPlan(kernel, leaves, {}, returns, len(targets), recording.single,
                           store_positions)
    if recording.stores or not targets:
        return None
    red, = reduces
    # after the reduction only the reduced value and scalars may be combined
    for t in targets:
        stack = [t]
        while stack:
            v = stack.pop()
            if v is red or v.kind in ('const', 'scalar'):
                continue
            if v.kind != 'apply':
                return None
            stack.extend(v.inputs)
        if t.shape != red.shape:
            return None
    before = [v for v in _reachable([red.src]) if v.kind in ('array', 'scalar')]
    after_scalars = [v for v in leaves if v.kind == 'scalar' and
                     not any(v is b for b in before)]
    kernel = _fusion_emit.reduction_kernel(name, red, before + after_scalars, targets)
    kwargs = {} if red.axis_arg is None else {'axis': red.axis_arg}
    return _KernelPlan(kernel, before + after_scalars, kwargs, returns, len(targets),
                       recording.single, store_positions)


class Fusion:
    """Callable returned by :func:`fuse`."""

    def __init__(self, func, name=None):
        self.func = func
        name = name or getattr(func, '__name__', 'fused')
        # '<lambda>' and the like are not C identifiers
        name = re.sub(r'[^a-zA-Z0-9_]', '_', name)
        if not name or name[0].isdigit():
            name = '_' + name
        self.name = name
        self._memo = {}         # types key -> plan | _EAGER | _BY_SHAPE
        self._plans = {}        # (types key, shapes) -> plan | False
        self._fast = {}         # call signature -> plan.run

    def __repr__(self):
        return '<Fusion \'{}\'>'.format(self.name)

    def clear_cache(self):
        self._memo = {}
        self._plans = {}
        self._fast = {}

    def __call__(self, *args):
        # called while another fused function is recorded: part of that one
        if _fusion_thread_local.is_old_fusing():
            return self.func(*args)
        # same argument types and layouts as an earlier call: same launches
        sig = _launch_plan.call_signature(args, _device.get_device_id())
        if sig is not None:
            run = self._fast.get(sig)
            if run is not None:
                return run(*args)
        if not any(isinstance(a, ndarray) for a in args):
            return self.func(*args)
        for arg in args:
            if not isinstance(arg, _acceptable_types):
                mes = 'Invalid argument type for \'{}\': ({})'
                arg_types = ', '.join(repr(type(a)) for a in args)
                raise TypeError(mes.format(self.name, arg_types))
        if any(isinstance(a, numpy.ndarray) for a in args):
            raise TypeError(
                'numpy.ndarray arguments cannot be mixed with cupy.ndarray '
                'arguments in a fused function')
        key = _types_key(args)
        plan = self._memo.get(key)
        if plan is None:
            plan = self._memo[key] = self._make_plan(args, key)
        if plan is _BY_SHAPE:
            plan_key = (key, tuple(a.shape for a in args if isinstance(a, ndarray)))
            plan = self._plans.get(plan_key)
            if plan is None:
                plan = self._make_plan(args, key, by_shape=True)
                if plan is _EAGER or plan is _BY_SHAPE:
                    plan = False
                if len(self._plans) >= 64:
                    self._plans.clear()
                self._plans[plan_key] = plan
            if plan is False:
                plan = _EAGER
        if plan is _EAGER:
            return self.func(*args)
        run = plan.run
        first = None
        if type(plan) is _KernelPlan and not plan.store_positions:
            # the first call makes the kernel's launch record; later calls with
            # this signature replay it directly
            first = plan.run(*args)
            run = plan.replay_runner(args) or plan.run
        if getattr(plan, 'store_positions', None):
            def run(*a, _plan=plan):
                if self._writes_overlap(_plan, a):
                    return self.func(*a)
                return _plan.run(*a)
        if sig is not None:
            if len(self._fast) >= 256:
                self._fast.clear()
            self._fast[sig] = run
        if type(plan) is _KernelPlan and not plan.store_positions:
            return first
        return run(*args)

    @staticmethod
    def _writes_overlap(plan, args):
        """True if an array the plan writes to shares memory with another
        argument: the recorded order of reads and writes then no longer
        describes what the function does."""
        positions = getattr(plan, 'store_positions', None)
        if not positions:
            return False
        for p in positions:
            for q, other in enumerate(args):
                if q != p and isinstance(other, ndarray) and \
                        _launch_plan.ranges_overlap(args[p], other):
                    return True
        return False

    def _make_plan(self, args, key, by_shape=False):
        try:
            recording = Recording(self.func, args)
        except Exception:
            # Not recordable (or the function itself fails): run it as written;
            # its own errors surface from that run.
            return _EAGER
        try:
            if not recording.roots():
                plan = _PassThroughPlan(recording.returns, recording.single)
                return _BY_SHAPE if recording.recorder.shape_dependent and not by_shape else plan
            plan = _plan_single_kernel(recording, self.name)
            if plan is not None:
                if recording.recorder.shape_dependent and not by_shape:
                    return _BY_SHAPE
                return plan
            if not by_shape:
                return _BY_SHAPE
            from cupy_amd._core import _fusion_split
            return _fusion_split.plan(recording, args, self.name)
        except Exception:
            return _EAGER


def fuse(*args, **kwargs):
    """Decorator that fuses a function of array operations.

    Args:
        kernel_name (str): Name of the fused kernel function.  Defaults to the
            name of the decorated function.

    Example:

        >>> @cupy.fuse(kernel_name='squared_diff')
        ... def squared_diff(x, y):
        ...     return (x - y) * (x - y)
    """
    if len(args) == 1 and not kwargs and callable(args[0]):
        return functools.update_wrapper(Fusion(args[0]), args[0])

    def decorate(f, kernel_name=None):
        return functools.update_wrapper(Fusion(f, kernel_name), f)
    return lambda f: decorate(f, *args, **kwargs)


# -- hooks: ufuncs and reductions called on proxies report to the recorder ------------------

def _call_ufunc(ufunc, *args, **kwargs):
    return _thread_local.history.call_ufunc(ufunc, *args, **kwargs)


def _call_reduction(func, *args, **kwargs):
    return _thread_local.history.call_reduction(func, *args, **kwargs)


# -- astype inside fused functions: a ufunc per target type -----------------------------------

_cast_sources = [numpy.dtype(c) for c in '?bhilqBHILQefdFD']
_astype_ufuncs = {}


def _dtype_to_astype(dtype):
    dtype = numpy.dtype(dtype)
    fn = _astype_ufuncs.get(dtype)
    if fn is None:
        loops = tuple('%s->%s' % (src.char, dtype.char) for src in _cast_sources
                      if not (src.kind == 'c' and dtype.kind != 'c'))
        fn = _astype_ufuncs[dtype] = _kernel.create_ufunc(
            'astype_%s' % dtype, loops, 'out0 = static_cast< %s >(in0)' % get_typename(dtype))
    return fn
