"""``cupy.fuse``: trace a Python function over proxy variables and emit one
elementwise kernel, or one map-reduce kernel, for the whole function.

Capability and call surface of the reference's legacy fusion
(cupy/_core/fusion.pyx: proxies :166-367, trace history :370-785, ``Fusion``
:788-880, ``fuse`` :886-919, reduction hook :926-961).  The trace is lowered to
straight-line code inside an ``ElementwiseKernel`` body or a ``ReductionKernel``
pre-map function, so the fused function runs on the same emitters (vectorised
loads, wave64 reductions) as hand-written kernels.
"""
import functools
import re

import numpy

from cupy_amd._core import _fusion_thread_local
from cupy_amd._core import _kernel
from cupy_amd._core import _launch_plan
from cupy_amd._core import _reduction
from cupy_amd._core._dtype import get_dtype, _raise_if_invalid_cast
from cupy_amd._core._scalar import get_typename, get_scalar_literal
from cupy_amd._core.core import ndarray
from cupy_amd.cuda import device as _device
from numpy.exceptions import AxisError

_thread_local = _fusion_thread_local.thread_local

_dtype_list = [numpy.dtype(c) for c in '?bhilqBHILQefd']

_acceptable_types = (
    ndarray, numpy.ndarray, numpy.generic, int, float, complex, bool, type(None))


class _FusionVarCUDA:
    """A variable of the generated code: ``v<index>`` of ``dtype``; constants
    carry their value."""

    def __init__(self, index, dtype, const_value=None):
        self.index = index
        self.dtype = dtype
        self.const_value = const_value
        self.mutable = False

    def __repr__(self):
        return 'v{}'.format(self.index)

    def mutate(self):
        self.mutable = True

    def declaration(self):
        ctype = get_typename(self.dtype)
        if self.const_value is None:
            return '{} v{};\n'.format(ctype, self.index)
        c = self.const_value
        val = c.item() if hasattr(c, 'dtype') else c
        return 'const {} v{} = {};\n'.format(
            ctype, self.index, get_scalar_literal(val, self.dtype))

    def declaration_in_param(self):
        non_const = '_non_const ' if self.mutable else ''
        return '{}{} v{}'.format(non_const, self.dtype, self.index)

    def declaration_out_param(self):
        return '{} v{}'.format(self.dtype, self.index)


class _FusionOp:
    """One traced ufunc call: loop types, routine and the variables bound to
    its inputs and outputs."""

    def __init__(self, index, ufunc, op, in_dtypes, out_dtypes, args):
        self.index = index
        self.name = ufunc.name
        self.routine = op.routine
        self.preamble = ufunc._preamble
        self.in_dtypes = in_dtypes
        self.out_dtypes = out_dtypes
        self.args = args
        self.nin = len(in_dtypes)

    def code(self):
        lines = ['{ // %s' % self.name]
        for i, t in enumerate(self.in_dtypes):
            lines.append('typedef %s in%d_type;' % (get_typename(t), i))
        for i, t in enumerate(self.out_dtypes):
            lines.append('typedef %s out%d_type;' % (get_typename(t), i))
        for i, v in enumerate(self.args[:self.nin]):
            lines.append('const in%d_type in%d = static_cast<in%d_type>(v%d);' % (
                i, i, i, v.index))
        for i, v in enumerate(self.args[self.nin:]):
            lines.append('out%d_type out%d;' % (i, i))
        lines.append('%s;' % self.routine)
        for i, v in enumerate(self.args[self.nin:]):
            lines.append('v%d = static_cast< %s >(out%d);' % (
                v.index, get_typename(v.dtype), i))
        lines.append('}')
        return '\n'.join(lines) + '\n'


class _FusionVarScalar:
    """Proxy handed to the traced function for a scalar value."""

    def __init__(self, var, ndim, is_postmap, is_weak):
        self._var = var
        self.dtype = var.dtype
        self.ndim = ndim
        self._is_postmap = is_postmap
        self.is_weak = is_weak
        assert ndim == -1

    def __repr__(self):
        return '<_FusionVar {} scalar ({})>'.format(self.dtype, self.is_weak)

    # every operator is the corresponding ufunc, which the trace intercepts
    def _u(self, name, *args):
        from cupy_amd._core import _ufuncs
        return getattr(_ufuncs, name)(*args)

    def __neg__(self):
        return self._u('negative', self)

    def __add__(self, other):
        return self._u('add', self, other)

    def __radd__(self, other):
        return self._u('add', other, self)

    def __sub__(self, other):
        return self._u('subtract', self, other)

    def __rsub__(self, other):
        return self._u('subtract', other, self)

    def __mul__(self, other):
        return self._u('multiply', self, other)

    def __rmul__(self, other):
        return self._u('multiply', other, self)

    def __truediv__(self, other):
        return self._u('true_divide', self, other)

    def __rtruediv__(self, other):
        return self._u('true_divide', other, self)

    def __floordiv__(self, other):
        return self._u('floor_divide', self, other)

    def __rfloordiv__(self, other):
        return self._u('floor_divide', other, self)

    def __mod__(self, other):
        return self._u('remainder', self, other)

    def __rmod__(self, other):
        return self._u('remainder', other, self)

    def __pow__(self, other):
        # The same short cuts ndarray.__pow__ (and NumPy) take for Python
        # exponents: squaring is a multiply, not a call to pow().
        if type(other) in (int, float) and other == 2 and self.dtype.kind in 'iuf':
            return self._u('square', self)
        if type(other) in (int, float) and self.dtype.kind == 'f':
            if other == 0.5:
                return self._u('sqrt', self)
            if other == -1:
                return self._u('reciprocal', self)
        return self._u('power', self, other)

    def __rpow__(self, other):
        return self._u('power', other, self)

    def __lshift__(self, other):
        return self._u('left_shift', self, other)

    def __rlshift__(self, other):
        return self._u('left_shift', other, self)

    def __rshift__(self, other):
        return self._u('right_shift', self, other)

    def __rrshift__(self, other):
        return self._u('right_shift', other, self)

    def __and__(self, other):
        return self._u('bitwise_and', self, other)

    def __rand__(self, other):
        return self._u('bitwise_and', other, self)

    def __or__(self, other):
        return self._u('bitwise_or', self, other)

    def __ror__(self, other):
        return self._u('bitwise_or', other, self)

    def __xor__(self, other):
        return self._u('bitwise_xor', self, other)

    def __rxor__(self, other):
        return self._u('bitwise_xor', other, self)

    def __invert__(self):
        return self._u('invert', self)

    def __abs__(self):
        return self._u('absolute', self)

    def __lt__(self, other):
        return self._u('less', self, other)

    def __le__(self, other):
        return self._u('less_equal', self, other)

    def __eq__(self, other):
        return self._u('equal', self, other)

    def __ne__(self, other):
        return self._u('not_equal', self, other)

    def __gt__(self, other):
        return self._u('greater', self, other)

    def __ge__(self, other):
        return self._u('greater_equal', self, other)

    __hash__ = None

    def __bool__(self):
        raise Exception('Can\'t cast to bool')

    def __setitem__(self, slices, value):
        if slices is Ellipsis or (isinstance(slices, slice) and
                                  slices == slice(None)):
            from cupy_amd._core import _ufuncs
            _call_ufunc(_ufuncs.elementwise_copy, value, out=self)
        else:
            raise ValueError('The fusion supports `[...]` or `[:]`.')

    def copy(self):
        from cupy_amd._core import _ufuncs
        return _ufuncs.elementwise_copy(self)

    def astype(self, dtype, order=None, casting=None, subok=None, copy=True):
        dtype = get_dtype(dtype)
        if order is not None:
            raise TypeError('order is not supported yet')
        if casting is not None:
            raise TypeError('casting is not supported yet')
        if subok is not None:
            raise TypeError('subok is not supported yet')
        if not copy and self.dtype == dtype:
            return self
        return _dtype_to_astype(dtype)(self)

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


class _FusionVarArray(_FusionVarScalar):
    """Proxy for an array value (``ndim`` known, shape abstract)."""

    def __init__(self, var, ndim, is_postmap):
        self._var = var
        self.dtype = var.dtype
        self.ndim = ndim
        self._is_postmap = is_postmap
        self.is_weak = False
        assert ndim >= 0

    def __repr__(self):
        return '<_FusionVar {} {}-dim array>'.format(self.dtype, self.ndim)

    def __iadd__(self, other):
        return self._u('add', self, other, self)

    def __isub__(self, other):
        return self._u('subtract', self, other, self)

    def __imul__(self, other):
        return self._u('multiply', self, other, self)

    def __itruediv__(self, other):
        return self._u('true_divide', self, other, self)

    def __ifloordiv__(self, other):
        return self._u('floor_divide', self, other, self)

    def __imod__(self, other):
        return self._u('remainder', self, other, self)

    def __ipow__(self, other):
        return self._u('power', self, other, self)

    def __ilshift__(self, other):
        return self._u('left_shift', self, other, self)

    def __irshift__(self, other):
        return self._u('right_shift', self, other, self)

    def __iand__(self, other):
        return self._u('bitwise_and', self, other, self)

    def __ior__(self, other):
        return self._u('bitwise_or', self, other, self)

    def __ixor__(self, other):
        return self._u('bitwise_xor', self, other, self)


class _FusionHistory:
    """Everything recorded while the function runs on proxies: parameters,
    local variables and operations, split into the part before the (single)
    reduction ("pre-map") and the part after it ("post-map")."""

    def __init__(self):
        self.preamble_set = []
        self.count = 0
        self.op_list = []
        self.param_list = []
        self.local_list = []
        self.reduce_op = None
        self.reduce_identity = None
        self.reduce_kwargs = None
        self.reduce_name = None
        self.postmap_op_list = []
        self.premap_ret = None
        self.postmap_param = None
        self.postmap_local_list = []
        self.ndim = 0

    def _has_reduction(self):
        return self.reduce_op is not None

    def _fresh_index(self):
        res = self.count
        self.count += 1
        return res

    def _new_var(self, *args, **kwargs):
        return _FusionVarCUDA(self._fresh_index(), *args, **kwargs)

    def _fresh_premap_param(self, *args, **kwargs):
        var = self._new_var(*args, **kwargs)
        self.param_list.append(var)
        return var

    def _fresh_postmap_param(self, *args, **kwargs):
        assert self.postmap_param is None
        var = self._new_var(*args, **kwargs)
        self.postmap_param = var
        return var

    def _fresh_local(self, *args, **kwargs):
        var = self._new_var(*args, **kwargs)
        if self._has_reduction():
            self.postmap_local_list.append(var)
        else:
            self.local_list.append(var)
        return var

    def _add_preamble(self, preamble):
        if preamble and preamble not in self.preamble_set:
            self.preamble_set.append(preamble)

    def add_op(self, ufunc, op, in_dtypes, out_dtypes, args):
        target = self.postmap_op_list if self._has_reduction() else self.op_list
        fop = _FusionOp(len(target), ufunc, op, in_dtypes, out_dtypes, args)
        target.append(fop)
        self._add_preamble(ufunc._preamble)
        return fop

    def set_reduce_op(self, raw, arg, kwargs):
        if self.reduce_op is not None:
            raise NotImplementedError('Multiple reduction is not implemented yet')
        for op in raw._ops.ops:
            input_type, = op.in_types
            output_type, = op.out_types
            if numpy.can_cast(arg.dtype, input_type):
                return_dtype = numpy.dtype(output_type)
                self.premap_ret = self._get_fusion_var(arg)._var
                self.reduce_op = op
                self.reduce_identity = raw.identity
                self.reduce_kwargs = kwargs
                self.reduce_name = raw.name
                self._add_preamble(raw.preamble)
                return self._fresh_postmap_param(return_dtype)
        raise TypeError('Type is mismatched. {}(...), {}'.format(
            raw.name, arg.dtype.type))

    def _get_fusion_var(self, arg):
        """Proxy for a proxy (checked to live on the right side of the
        reduction) or for a Python/NumPy scalar (becomes a constant)."""
        if isinstance(arg, _FusionVarScalar):
            if arg._is_postmap == self._has_reduction():
                return arg
            raise Exception('Shape mismatch')
        if isinstance(arg, (int, float, bool, complex, numpy.generic)):
            pytype = type(arg)
            is_weak = pytype if pytype in (int, float, complex) else False
            if isinstance(arg, numpy.generic):
                dtype = arg.dtype
            else:
                dtype = numpy.dtype(pytype)
            var = self._fresh_local(dtype, const_value=arg)
            return _FusionVarScalar(var, -1, self._has_reduction(), is_weak)
        raise TypeError('Unsupported type {}'.format(type(arg)))

    def call_ufunc(self, ufunc, *args, **kwargs):
        nin = ufunc.nin
        nout = ufunc.nout

        def make_fusion_var(var, ndim, is_weak):
            if ndim == -1:
                return _FusionVarScalar(var, ndim, self._has_reduction(), is_weak)
            return _FusionVarArray(var, ndim, self._has_reduction())

        var_list = [self._get_fusion_var(arg) for arg in args]
        in_vars = var_list[:nin]
        out_vars = var_list[nin:]
        if 'out' in kwargs:
            out = kwargs.pop('out')
            if out_vars:
                raise ValueError('cannot specify \'out\' as both a positional '
                                 'and keyword argument')
            if isinstance(out, _FusionVarArray):
                out_vars.append(self._get_fusion_var(out))
            elif out is not None:
                raise ValueError('The \'out\' tuple must have exactly one '
                                 'entry per ufunc output')
        kwargs.pop('casting', None)
        if kwargs:
            raise TypeError('Wrong arguments {}'.format(kwargs))
        if len(in_vars) != nin or len(out_vars) > nout:
            raise ValueError('invalid number of arguments')
        if not all(isinstance(v, _FusionVarArray) for v in out_vars):
            raise TypeError('return arrays must be of ArrayType')

        ndim = max(v.ndim for v in in_vars)
        if any(v.ndim < ndim for v in out_vars):
            raise ValueError('non-broadcastable output operand')

        in_dtypes = tuple(a.dtype for a in in_vars)
        weaks = tuple(getattr(a, 'is_weak', False) for a in in_vars)
        if not _kernel._check_should_use_weak_scalar(
                in_dtypes, weaks if any(weaks) else None):
            weaks = (False,) * nin
        op = ufunc._ops._guess_routine_from_in_types(in_dtypes, weaks)
        if op is None:
            raise TypeError('Invalid type cast in \'{}\': {} -> {}'.format(
                ufunc.name, [v.dtype for v in in_vars],
                [v.dtype for v in out_vars]))
        op.check_valid()
        op_in = [numpy.dtype(t) for t in op.in_types]
        op_out = [numpy.dtype(t) for t in op.out_types]
        ret = []
        for i in range(nout):
            if i >= len(out_vars):
                out_var = make_fusion_var(self._fresh_local(op_out[i]), ndim, False)
                out_vars.append(out_var)
            else:
                _raise_if_invalid_cast(
                    op_out[i], out_vars[i].dtype, 'same_kind', lambda: f'output {i}')
                out_var = out_vars[i]
            out_var._var.mutate()
            ret.append(out_var)
        self.add_op(ufunc, op, op_in, op_out, [v._var for v in in_vars + out_vars])
        return ret[0] if len(ret) == 1 else tuple(ret)

    # -- code emission -------------------------------------------------------------------
    @staticmethod
    def _emit_ops(local_list, op_list):
        res = '// {} operations\n'.format(len(op_list))
        res += ''.join(v.declaration() for v in local_list)
        res += ''.join(op.code() for op in op_list)
        return res

    def _gen_abstracted_args(self, a):
        if isinstance(a, ndarray):
            cuda_var = self._fresh_premap_param(a.dtype)
            python_var = _FusionVarArray(cuda_var, a.ndim, False)
        elif a is None:
            cuda_var = None
            python_var = None
        else:
            pytype = type(a)
            if isinstance(a, numpy.generic):
                dtype = a.dtype
                is_weak = False
            else:
                dtype = numpy.dtype(pytype)
                is_weak = pytype if pytype in (int, float, complex) else False
            cuda_var = self._fresh_premap_param(dtype)
            python_var = _FusionVarScalar(cuda_var, -1, False, is_weak)
        return cuda_var, python_var

    def get_fusion(self, func, args, name, describe_only=False):
        """Runs ``func`` on proxies and returns (kernel, kwargs for its call).
        With ``describe_only`` no kernel object is made: the return value is a
        dict of the generated pieces (parameter variables, the body of an
        elementwise function, or the device functions, combine expression,
        accumulator type and identity of a map-reduce function) for emitters
        that compose several traced functions into one kernel."""
        self.ndim = max(a.ndim for a in args if isinstance(a, ndarray))
        in_params = []
        function_args = []
        for a in args:
            cuda_var, python_var = self._gen_abstracted_args(a)
            if cuda_var is not None:
                in_params.append(cuda_var)
            function_args.append(python_var)

        return_value = func(*function_args)

        if isinstance(return_value, tuple):
            return_tuple = True
            no_return = False
            out_pvars = return_value
        elif isinstance(return_value, _FusionVarScalar):
            return_tuple = False
            no_return = False
            out_pvars = [return_value]
        elif return_value is None:
            return_tuple = False
            no_return = True
            out_pvars = []
        else:
            raise TypeError(
                'Fusion function can\'t return {}'.format(type(return_value)))

        out_pvars = [v for v in out_pvars if v is not None]
        out_cvars = [self._get_fusion_var(v)._var for v in out_pvars]
        out_dtypes = [v.dtype for v in out_pvars]
        out_params = [self._fresh_premap_param(t) for t in out_dtypes]

        in_params_code = ', '.join(v.declaration_in_param() for v in in_params)
        out_params_code = ', '.join(v.declaration_out_param() for v in out_params)
        operation = self._emit_ops(self.local_list, self.op_list)
        preamble = '\n'.join(self.preamble_set) + '\n'

        if self.reduce_op is None:
            operation += ' '.join('{} = {};'.format(t, s)
                                  for s, t in zip(out_cvars, out_params))
            if describe_only:
                return dict(kind='elementwise', in_params=in_params, out_params=out_params,
                            operation=operation, preambles=list(self.preamble_set),
                            return_tuple=return_tuple)
            kernel = _kernel.ElementwiseKernel(
                in_params_code, out_params_code, operation, preamble=preamble,
                return_tuple=return_tuple, no_return=no_return, name=name)
            return kernel, {}

        map_expr, reduce_expr, postmap_expr, reduce_ctype = self.reduce_op.routine
        if reduce_ctype is None:
            reduce_ctype = 'type_out0_raw'
        postmap_type, = self.reduce_op.out_types
        postmap_dtype = numpy.dtype(postmap_type)
        postmap_ctype = get_typename(postmap_dtype)
        premap_in_type, = self.reduce_op.in_types
        premap_ctype = get_typename(numpy.dtype(premap_in_type))

        postmap_code = self._emit_ops(self.postmap_local_list, self.postmap_op_list)
        postmap_code += ' '.join('{} = {};'.format(t, s)
                                 for s, t in zip(out_cvars, out_params))

        ret = self.premap_ret
        shared_preambles = list(self.preamble_set)
        defs_start = len(preamble)
        # the reduction's own element map (identity for sum/prod/min/max)
        preamble += 'typedef %s type_in0_raw;\n' % premap_ctype
        preamble += 'typedef %s type_out0_raw;\n' % postmap_ctype
        preamble += '''
__device__ __forceinline__ %s _pre_map(%s) {
%s
const type_in0_raw in0 = static_cast<type_in0_raw>(%s);
return static_cast<%s>(%s);
}
''' % (reduce_ctype if reduce_ctype != 'type_out0_raw' else postmap_ctype,
            ', '.join('{} v{}'.format(get_typename(v.dtype), v.index)
                      for v in in_params),
            operation, ret,
            reduce_ctype if reduce_ctype != 'type_out0_raw' else postmap_ctype,
            map_expr)
        preamble += '''
__device__ __forceinline__ %s _postmap_cast(%s a) {
%s out0;
%s;
return out0;
}
''' % (postmap_ctype, reduce_ctype, postmap_ctype, postmap_expr)
        in_ctype = get_typename(self.postmap_param.dtype)
        preamble += '''
__device__ __forceinline__ void _post_map(%s in, %s) {
%s v%d = in;
%s;
}
''' % (in_ctype,
            ', '.join('{} &v{}'.format(get_typename(v.dtype), v.index)
                      for v in out_params),
            in_ctype, self.postmap_param.index, postmap_code)

        if describe_only:
            return dict(kind='reduce', in_params=in_params, out_params=out_params,
                        preambles=shared_preambles, defs=preamble[defs_start:],
                        reduce_expr=reduce_expr,
                        reduce_ctype=(reduce_ctype if reduce_ctype != 'type_out0_raw'
                                      else postmap_ctype),
                        identity=self.reduce_identity, kwargs=self.reduce_kwargs,
                        return_tuple=return_tuple)
        kernel = _reduction.ReductionKernel(
            in_params_code, out_params_code,
            '_pre_map({})'.format(', '.join(repr(p) for p in in_params)),
            reduce_expr,
            '_post_map(_postmap_cast(a), {})'.format(
                ', '.join(repr(p) for p in out_params)),
            self.reduce_identity, name=name, reduce_type=reduce_ctype,
            preamble=preamble)
        return kernel, self.reduce_kwargs


class Fusion:
    """Callable returned by :func:`fuse`; behaves like an ElementwiseKernel or
    ReductionKernel specialised per argument types."""

    def __init__(self, func, name=None, split=True):
        self.func = func
        self._may_split = split
        self._plans = {}
        name = name or getattr(func, '__name__', 'fused')
        # '<lambda>' and the like are not C identifiers
        name = re.sub(r'[^a-zA-Z0-9_]', '_', name)
        if not name or name[0].isdigit():
            name = '_' + name
        self.name = name
        self._memo = {}
        self._fast = {}

    def __repr__(self):
        return '<Fusion \'{}\'>'.format(self.name)

    def __call__(self, *args):
        # a fused function called from inside another trace is just inlined
        if _fusion_thread_local.is_old_fusing():
            return self.func(*args)
        # Same argument types and layouts as an earlier call: same kernel.
        sig = _launch_plan.call_signature(args, _device.get_device_id())
        if sig is not None:
            hit = self._fast.get(sig)
            if hit is not None:
                return hit[0](*args, **hit[1])
        if not any(isinstance(a, ndarray) for a in args):
            return self.func(*args)
        for arg in args:
            if not isinstance(arg, _acceptable_types):
                mes = 'Invalid argument type for \'{}\': ({})'
                arg_types = ', '.join(repr(type(a)) for a in args)
                raise TypeError(mes.format(self.name, arg_types))

        params_info = []
        for arg in args:
            if isinstance(arg, ndarray):
                params_info.append(arg.dtype.char)
                params_info.append(arg.ndim)
            elif isinstance(arg, numpy.generic):
                params_info.append(arg.dtype.char)
            elif arg is None:
                params_info.append(None)
            elif isinstance(arg, bool):
                params_info.append('?')
                params_info.append(bool)
            elif isinstance(arg, float):
                params_info.append('d')
                params_info.append(float)
            elif isinstance(arg, int):
                params_info.append('l')
                params_info.append(int)
            elif isinstance(arg, complex):
                params_info.append('D')
                params_info.append(complex)
            else:
                params_info.append(type(arg))
        key = tuple(params_info)

        if key not in self._memo:
            history = _FusionHistory()
            _thread_local.history = history
            _thread_local.is_old_fusing = True
            try:
                self._memo[key] = history.get_fusion(self.func, args, self.name)
            except Exception:
                # Not expressible as ONE elementwise or map-reduce kernel
                # (several reductions, arrays combined with a reduced value,
                # ...).  The reference hands such functions to its second
                # tracer (cupy/_core/fusion.pyx:860-871), whose multi-pass
                # kernels need a grid-wide barrier.  Here the function is cut
                # into a sequence of fused kernels (_fusion_split), or, if it
                # cannot be recorded either, runs as written: every step
                # launches its own generated kernel on the current stream,
                # temporaries come from the pool.  Errors of the function
                # itself surface from that run.
                self._memo[key] = None
            finally:
                _thread_local.history = None
                _thread_local.is_old_fusing = False
        if self._memo[key] is None:
            return self._call_sequence(args, key, sig)
        kernel, kwargs = self._memo[key]
        call_args = []
        for a in args:
            if a is None:
                continue
            if isinstance(a, numpy.ndarray):
                raise TypeError(
                    'numpy.ndarray arguments cannot be mixed with cupy.ndarray '
                    'arguments in a fused function')
            call_args.append(a)
        if sig is not None and len(call_args) == len(args):
            if len(self._fast) >= 256:
                self._fast.clear()
            self._fast[sig] = (kernel, kwargs)
        return kernel(*call_args, **kwargs)

    def _call_sequence(self, args, key, sig):
        """The function as a sequence of fused kernels, planned once per
        argument types and shapes; as written if it cannot be recorded."""
        if not self._may_split:
            return self.func(*args)
        plan_key = (key, tuple(a.shape for a in args if isinstance(a, ndarray)))
        plan = self._plans.get(plan_key)
        if plan is None:
            from cupy_amd._core import _fusion_split
            try:
                plan = _fusion_split.trace(self.func, args, self.name)
            except Exception:
                plan = False
            if len(self._plans) >= 64:
                self._plans.clear()
            self._plans[plan_key] = plan
        if plan is False:
            return self.func(*args)
        if sig is not None:
            if len(self._fast) >= 256:
                self._fast.clear()
            self._fast[sig] = (plan.run, {})
        return plan.run(*args)

    def clear_cache(self):
        self._memo = {}
        self._fast = {}
        self._plans = {}


def describe(func, args, name):
    """Traces ``func`` on stand-ins of ``args`` with the single-kernel tracer
    and returns the generated pieces instead of a kernel (see
    ``_FusionHistory.get_fusion``)."""
    history = _FusionHistory()
    saved = (getattr(_thread_local, 'history', None),
             getattr(_thread_local, 'is_old_fusing', False))
    _thread_local.history = history
    _thread_local.is_old_fusing = True
    try:
        return history.get_fusion(func, args, name, describe_only=True)
    finally:
        _thread_local.history, _thread_local.is_old_fusing = saved


def fuse(*args, **kwargs):
    """Decorator that fuses a function of ufunc calls (optionally ending in one
    reduction) into a single kernel.

    Args:
        kernel_name (str): Name of the fused kernel function.  Defaults to the
            name of the decorated function.

    Example:

        >>> @cupy.fuse(kernel_name='squared_diff')
        ... def squared_diff(x, y):
        ...     return (x - y) * (x - y)
    """
    def wrapper(f, kernel_name=None):
        return Fusion(f, kernel_name)

    if len(args) == 1 and len(kwargs) == 0 and callable(args[0]):
        return functools.update_wrapper(wrapper(args[0]), args[0])
    return lambda f: functools.update_wrapper(wrapper(f, *args, **kwargs), f)


def _call_ufunc(fusion_op, *args, **kwargs):
    return _thread_local.history.call_ufunc(fusion_op, *args, **kwargs)


def _call_reduction(fusion_op, *args, **kwargs):
    if len(args) != 1:
        mes = '{}() takes 1 positional argument but {} were given'
        raise TypeError(mes.format(fusion_op.name, len(args)))
    arg = args[0]
    kwargs = {key: value for key, value in kwargs.items()
              if key in ('axis', 'out') and value is not None}
    if arg._is_postmap:
        raise NotImplementedError('Multiple reduction is not implemented yet')
    history = _thread_local.history
    var = history.set_reduce_op(fusion_op, arg, kwargs)
    src_ndim = max(0, arg.ndim)
    if 'axis' in kwargs:
        axis = kwargs['axis']
        if isinstance(axis, (tuple, list)):
            ndim = src_ndim - len(axis)
        else:
            ndim = src_ndim - 1
    else:
        axis = None
        ndim = 0
    if ndim < 0:
        raise AxisError(axis, src_ndim)
    history.ndim = ndim
    if ndim >= 1:
        return _FusionVarArray(var, ndim, True)
    return _FusionVarScalar(var, -1, True, False)


def _create_astype_ufunc(dtype):
    name = 'astype_{}'.format(dtype)
    rules = tuple('{}->{}'.format(cast_from.char, dtype.char)
                  for cast_from in _dtype_list)
    command = 'out0 = static_cast< {} >(in0)'.format(get_typename(dtype))
    return _kernel.create_ufunc(name, rules, command)


_dtype_to_astype_dict = {}


def _dtype_to_astype(dtype):
    fn = _dtype_to_astype_dict.get(dtype)
    if fn is None:
        fn = _dtype_to_astype_dict[dtype] = _create_astype_ufunc(dtype)
    return fn
