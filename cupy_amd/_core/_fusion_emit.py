"""Kernel text for pieces of a recorded fused function.

A piece is a set of target values of the graph of ``_fusion_graph`` together
with the values it starts from (its leaves: argument arrays, scalars, values an
earlier kernel stored).  Everything between leaves and targets is elementwise
and becomes straight-line code: one local variable per value, one call of a
small device function per ufunc application.  Every distinct (ufunc, loop) gets
one such function, whose body is the loop's routine with the names it expects
(``in0``, ``out0``, ``in0_type`` ...) bound by the function's signature.

Three products:

* ``elementwise_kernel``   an ``ElementwiseKernel`` computing the targets
* ``reduction_kernel``     a ``ReductionKernel``: elementwise work feeding one
                           reduction, the reduction, elementwise work on the
                           reduced value
* ``describe_*``           the same pieces as bare device functions, for the
                           row kernel of ``_fusion_rows`` which composes several
                           pieces in one kernel

The reference writes its fused kernels in cupy/_core/fusion.pyx:35-163,668-785
(single kernel) and cupy/_core/_fusion_kernel.pyx:57-381 (general tracer).
"""
import numpy

from cupy_amd._core import _kernel
from cupy_amd._core import _reduction
from cupy_amd._core._scalar import get_typename, get_scalar_literal


class Code:
    """Accumulates the device functions and preambles one kernel needs."""

    def __init__(self):
        self.preambles = []          # ufunc / reduction preambles, in first-use order
        self._functions = {}         # (ufunc name, loop types, routine) -> function name
        self.definitions = []        # text of the op functions

    def preamble(self, text):
        if text and text not in self.preambles:
            self.preambles.append(text)

    def function_for(self, call):
        """Name of the device function of one ufunc loop (defined on first use)."""
        loop = call.loop
        key = (call.ufunc.name, tuple(loop.in_types), tuple(loop.out_types), loop.routine)
        name = self._functions.get(key)
        if name is None:
            name = '_fz%d_%s' % (len(self._functions), call.ufunc.name)
            self._functions[key] = name
            self.preamble(call.ufunc._preamble)
            sig = ['const %s in%d' % (get_typename(t), i) for i, t in enumerate(call.in_dtypes)]
            sig += ['%s& out%d' % (get_typename(t), i) for i, t in enumerate(call.out_dtypes)]
            body = ['typedef %s in%d_type;' % (get_typename(t), i)
                    for i, t in enumerate(call.in_dtypes)]
            body += ['typedef %s out%d_type;' % (get_typename(t), i)
                     for i, t in enumerate(call.out_dtypes)]
            self.definitions.append(
                '__device__ __forceinline__ void %s(%s) {\n  %s\n  %s;\n}\n' % (
                    name, ', '.join(sig), ' '.join(body), loop.routine))
        return name

    def text(self):
        return '\n'.join(self.preambles) + '\n' + ''.join(self.definitions)


def _name(v):
    return 'v%d' % v.order


def _read(v, as_dtype):
    """Expression of value ``v`` converted to ``as_dtype``."""
    if v.kind == 'const':
        c = v.const
        c = c.item() if hasattr(c, 'dtype') else c
        lit = get_scalar_literal(c, v.dtype)
        if v.dtype == as_dtype:
            return lit
        return 'static_cast<%s>(%s)' % (get_typename(as_dtype), lit)
    if v.dtype == as_dtype:
        return _name(v)
    return 'static_cast<%s>(%s)' % (get_typename(as_dtype), _name(v))


def straight_line(code, targets, leaves):
    """Statements computing ``targets`` from ``leaves`` (Values whose variables
    are taken as given), in the order the function made the calls."""
    given = set(v.order for v in leaves)
    needed = {}
    stack = list(targets)
    while stack:
        v = stack.pop()
        if v.order in given or v.order in needed or v.kind == 'const':
            continue
        if v.kind != 'apply':
            raise ValueError('value %r cannot be computed inside one piece' % (v,))
        needed[v.order] = v
        stack.extend(v.call.inputs)
    lines = []
    done = set()
    for order in sorted(needed):
        call = needed[order].call
        if id(call) in done:
            continue
        done.add(id(call))
        fn = code.function_for(call)
        outs = []
        for i, t in enumerate(call.out_dtypes):
            # every output of the call that the recording gave a Value
            mate = _output_of(needed, call, i)
            if mate is None:
                outs.append('_unused%d_%d' % (order, i))
                lines.append('%s _unused%d_%d;' % (get_typename(t), order, i))
            else:
                outs.append(_name(mate))
                lines.append('%s %s;' % (get_typename(t), _name(mate)))
        ins = [_read(v, t) for v, t in zip(call.inputs, call.in_dtypes)]
        lines.append('%s(%s);' % (fn, ', '.join(ins + outs)))
    return lines


def _output_of(needed, call, i):
    for v in needed.values():
        if v.call is call and v.index == i:
            return v
    return None


def _param(v, non_const=False):
    return '%s%s %s' % ('_non_const ' if non_const else '', v.dtype, _name(v))


# ---------------------------------------------------------------------------------------
# one elementwise kernel
# ---------------------------------------------------------------------------------------

def elementwise_kernel(name, leaves, targets, stores=()):
    """``ElementwiseKernel`` with the leaves as inputs, one fresh output per
    target and, for every ``(leaf, value)`` of ``stores``, the value written
    into that input array at the end.  Call it with the leaves' arrays and
    scalars in order; it returns the outputs (a tuple when ``targets`` is one)."""
    code = Code()
    stored = dict((leaf.order, value) for leaf, value in stores)
    lines = straight_line(code, list(targets) + [v for _, v in stores], leaves)
    in_params = ', '.join(_param(v, v.order in stored) for v in leaves)
    out_params = ', '.join('%s o%d' % (t.dtype, i) for i, t in enumerate(targets))
    for i, t in enumerate(targets):
        lines.append('o%d = %s;' % (i, _read(t, t.dtype)))
    for leaf, value in stores:
        lines.append('%s = %s;' % (_name(leaf), _read(value, leaf.dtype)))
    return _kernel.ElementwiseKernel(
        in_params, out_params, '\n'.join(lines), name=name, preamble=code.text(),
        return_tuple=len(targets) != 1, no_return=not targets)


def describe_elementwise(leaves, targets):
    """The same computation as a device function
    ``void elementwise(leaf values..., target references...)``."""
    code = Code()
    lines = straight_line(code, targets, leaves)
    sig = ['%s %s' % (get_typename(v.dtype), _name(v)) for v in leaves]
    sig += ['%s& o%d' % (get_typename(t.dtype), i) for i, t in enumerate(targets)]
    for i, t in enumerate(targets):
        lines.append('o%d = %s;' % (i, _read(t, t.dtype)))
    function = '__device__ __forceinline__ void elementwise(%s) {\n%s\n}\n' % (
        ', '.join(sig), '\n'.join(lines))
    return dict(kind='elementwise', preambles=code.preambles,
                functions=''.join(code.definitions) + function,
                out_dtypes=[t.dtype for t in targets])


# ---------------------------------------------------------------------------------------
# elementwise work, one reduction, elementwise work on the reduced value
# ---------------------------------------------------------------------------------------

def _reduction_parts(code, reduce_value, leaves, targets, scalar_leaves):
    """Text of the two device functions around a reduction: ``_fz_map`` (leaf
    values of one element -> the reduction's accumulator type) and
    ``_fz_finish`` (accumulated value -> the targets)."""
    loop = reduce_value.loop
    map_expr, reduce_expr, post_expr, reduce_ctype = loop.routine
    in_ctype = get_typename(numpy.dtype(loop.in_types[0]))
    out_ctype = get_typename(numpy.dtype(loop.out_types[0]))
    if reduce_ctype is None:
        reduce_ctype = out_ctype
    reduce_ctype = reduce_ctype.replace('type_out0_raw', out_ctype).replace(
        'type_in0_raw', in_ctype)
    code.preamble(reduce_value.func.preamble)
    src = reduce_value.src
    before = straight_line(code, [src], leaves)
    sig = ', '.join('%s %s' % (get_typename(v.dtype), _name(v)) for v in leaves)
    text = ['typedef %s type_in0_raw;' % in_ctype, 'typedef %s type_out0_raw;' % out_ctype,
            '__device__ __forceinline__ %s _fz_map(%s) {' % (reduce_ctype, sig)]
    text += before
    text += ['const type_in0_raw in0 = %s;' % _read(src, numpy.dtype(loop.in_types[0])),
             'return static_cast<%s>(%s);' % (reduce_ctype, map_expr), '}']
    # after the reduction: the loop's own post-map gives the reduced value, then
    # whatever the function did with it
    after = straight_line(code, targets, [reduce_value] + list(scalar_leaves))
    sig = ['%s a' % reduce_ctype]
    sig += ['%s %s' % (get_typename(v.dtype), _name(v)) for v in scalar_leaves]
    sig += ['%s& o%d' % (get_typename(t.dtype), i) for i, t in enumerate(targets)]
    text += ['__device__ __forceinline__ void _fz_finish(%s) {' % ', '.join(sig),
             'type_out0_raw out0;', '%s;' % post_expr,
             'const %s %s = out0;' % (out_ctype, _name(reduce_value))]
    text += after
    for i, t in enumerate(targets):
        text.append('o%d = %s;' % (i, _read(t, t.dtype)))
    text.append('}')
    return '\n'.join(text) + '\n', reduce_expr, reduce_ctype


def _scalars_after(reduce_value, targets, leaves):
    """Leaves that the work after the reduction reads (scalars only)."""
    given = set(v.order for v in leaves)
    found = {}
    stack = list(targets)
    seen = set()
    while stack:
        v = stack.pop()
        if v.order in seen or v is reduce_value or v.kind == 'const':
            continue
        seen.add(v.order)
        if v.order in given:
            found[v.order] = v
            continue
        stack.extend(v.inputs)
    return [found[k] for k in sorted(found)]


def reduction_kernel(name, reduce_value, leaves, targets):
    """``ReductionKernel`` whose map is everything elementwise that feeds
    ``reduce_value`` and whose post-map computes ``targets`` from the reduced
    value.  Call it with the leaves in order and ``axis=``."""
    code = Code()
    after_leaves = _scalars_after(reduce_value, targets, leaves)
    functions, reduce_expr, reduce_ctype = _reduction_parts(
        code, reduce_value, leaves, targets, after_leaves)
    in_params = ', '.join(_param(v) for v in leaves)
    out_params = ', '.join('%s o%d' % (t.dtype, i) for i, t in enumerate(targets))
    map_call = '_fz_map(%s)' % ', '.join(_name(v) for v in leaves)
    finish = '_fz_finish(%s)' % ', '.join(
        ['a'] + [_name(v) for v in after_leaves] + ['o%d' % i for i in range(len(targets))])
    return _reduction.ReductionKernel(
        in_params, out_params, map_call, reduce_expr, finish,
        reduce_value.func.identity, name=name, reduce_type=reduce_ctype,
        preamble=code.text() + functions)


def describe_reduction(reduce_value, leaves):
    """The reduction as device functions for a kernel that runs the combine
    itself: ``_fz_map(leaf values...)`` and ``_fz_finish(accumulated, result&)``."""
    code = Code()
    functions, reduce_expr, reduce_ctype = _reduction_parts(
        code, reduce_value, leaves, [reduce_value], ())
    return dict(kind='reduce', preambles=code.preambles,
                functions=''.join(code.definitions) + functions,
                reduce_expr=reduce_expr, reduce_ctype=reduce_ctype,
                identity=reduce_value.func.identity, out_dtype=reduce_value.dtype)
