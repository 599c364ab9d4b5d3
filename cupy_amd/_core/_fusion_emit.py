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

    def divide_by_row_value(self):
        """Name of the float32 division by a value that many elements share,
        given the value's reciprocal (defined on first use)."""
        name = '_fz_divide_by_shared'
        if name not in self._functions.values():
            self._functions[name] = name
            self.definitions.append(_DIVIDE_BY_SHARED % name)
        return name

    def text(self):
        return '\n'.join(self.preambles) + '\n' + ''.join(self.definitions)


# x / d for a divisor that a whole row shares, from r = 1 / d (correctly rounded,
# computed once per row): the product x * r is within an ulp or so of the
# quotient; its residual x - q * d is exact in one fused multiply-add, and adding
# residual * r gives the correctly rounded quotient except in rare cases that
# end one ulp away (Markstein's correction step).  Four instructions against the
# ten to thirteen of the division's full expansion.  Where that reasoning does not hold
# the division itself is carried out: a quotient that is infinite or NaN (an
# infinite or NaN dividend, overflow), and every quotient of a row whose
# reciprocal is zero, subnormal, infinite or NaN -- the caller hands NaN in for
# such a reciprocal (`shared_reciprocal`), which makes every quotient NaN here.
_DIVIDE_BY_SHARED = '''__device__ __forceinline__ void %s(
    const float x, const float d, const float r, float& out) {
  const float p = x * r;
  const float e = __builtin_fmaf(-p, d, x);
  const float q = __builtin_fmaf(e, r, p);
  // one test of the quotient's class sorts out what the three operations
  // above do not settle: zeros (0x60), infinities (0x204), NaN (0x3)
  if (__builtin_expect(!__builtin_amdgcn_classf(q, 0x267), 1)) {
    out = q;
  } else if (q == 0.0f) {
    // (a zero quotient takes its sign from the product: the correction step
    // turns -0 into +0)
    out = p;
  } else {
    // (the empty statement keeps the division on this side of the branch: as a
    // plain conditional expression it is evaluated for every element)
    float dd = d;
    asm volatile("" : "+v"(dd));
    out = x / dd;
  }
}
'''

# the reciprocal such a division takes: NaN unless it is a normal number well
# inside the range (so that neither it nor the products with it lose bits)
SHARED_RECIPROCAL = '''__device__ __forceinline__ float shared_reciprocal(const float d) {
  const float r = 1.0f / d;
  const float a = __builtin_fabsf(r);
  return (a > 1.0e-30f && a < 1.0e30f) ? r : __builtin_nanf("");
}
'''


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


def _is_float32_divide(call):
    f32 = numpy.dtype('float32')
    return (call.ufunc.name == 'cupy_true_divide' and len(call.inputs) == 2
            and all(numpy.dtype(t) == f32 for t in tuple(call.in_dtypes) + tuple(call.out_dtypes)))


def shared_divisors(targets, leaves, shared):
    """Orders of the leaves among ``shared`` (values that many elements have
    in common) by which a float32 value is divided on the way to ``targets``."""
    given = set(v.order for v in leaves)
    found = []
    stack = list(targets)
    seen = set()
    while stack:
        v = stack.pop()
        if v.order in seen or v.order in given or v.kind != 'apply':
            continue
        seen.add(v.order)
        call = v.call
        d = call.inputs[1] if _is_float32_divide(call) else None
        if d is not None and d.order in shared and d.order in given and d.order not in found \
                and d.dtype == numpy.dtype('float32'):
            found.append(d.order)
        stack.extend(call.inputs)
    return sorted(found)


def straight_line(code, targets, leaves, reciprocals=None):
    """Statements computing ``targets`` from ``leaves`` (Values whose variables
    are taken as given), in the order the function made the calls.
    ``reciprocals``: order of a float32 leaf -> name of a variable that holds
    its reciprocal; divisions by such a leaf use it."""
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
        if reciprocals and _is_float32_divide(call) and call.inputs[1].order in reciprocals:
            fn = code.divide_by_row_value()
            ins.append(reciprocals[call.inputs[1].order])
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


def describe_elementwise(leaves, targets, shared=()):
    """The same computation as a device function
    ``void elementwise(leaf values..., reciprocals..., target references...)``.
    ``shared``: orders of leaves whose value many elements have in common (one
    per row); for those among them that float32 values are divided by, the
    function takes the reciprocal as one more argument each (``reciprocals``
    of the result lists their orders) and divides through it."""
    code = Code()
    divisors = shared_divisors(targets, leaves, set(shared)) if shared else []
    lines = straight_line(code, targets, leaves,
                          dict((o, '_rcp%d' % o) for o in divisors))
    sig = ['%s %s' % (get_typename(v.dtype), _name(v)) for v in leaves]
    sig += ['float _rcp%d' % o for o in divisors]
    sig += ['%s& o%d' % (get_typename(t.dtype), i) for i, t in enumerate(targets)]
    for i, t in enumerate(targets):
        lines.append('o%d = %s;' % (i, _read(t, t.dtype)))
    function = '__device__ __forceinline__ void elementwise(%s) {\n%s\n}\n' % (
        ', '.join(sig), '\n'.join(lines))
    return dict(kind='elementwise', preambles=code.preambles,
                functions=''.join(code.definitions) + function,
                out_dtypes=[t.dtype for t in targets], reciprocals=divisors)


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
