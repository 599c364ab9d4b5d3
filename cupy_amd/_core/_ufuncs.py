"""ufunc definitions: loop tables in NumPy's order (first match reproduces
NumPy's promotion) and the HIP routine of each loop.

The arithmetic tables correspond to the reference's
cupy/_core/_routines_math.pyx:878-1060 (add, subtract, multiply, power, ...),
cupy/_core/_ufuncs.py:7-13 (elementwise_copy) and cupy/_math/misc.py:197-206
(square); the rest of the catalogue follows NumPy's ``ufunc.types``.  Complex loops
('F', 'D') compute with ``complex<float>`` / ``complex<double>`` of
cupy/complex.cuh.
"""
from cupy_amd._core import _fusion_thread_local
from cupy_amd._core._kernel import create_ufunc

_INTS = 'bBhHiIlLqQ'
_FLOATS = 'efd'
_COMPLEX = 'FD'


def _sig(chars, nin, out=None):
    return tuple('%s->%s' % (c * nin, out or c) for c in chars)


elementwise_copy = create_ufunc(
    'cupy_copy',
    _sig('?' + _INTS + _FLOATS + _COMPLEX, 1),
    'out0 = in0',
    default_casting='unsafe')


def _create_arithmetic(name, op, boolop, doc):
    if isinstance(boolop, str):
        boolop = 'out0 = in0 %s in1' % boolop
    return create_ufunc(
        'cupy_' + name,
        (('??->?', boolop),) + _sig(_INTS + _FLOATS + _COMPLEX, 2),
        'out0 = in0 %s in1' % op,
        doc=doc)


def _subtract_boolean_error():
    raise TypeError(
        'cupy boolean subtract, the `-` operator, is deprecated, use the '
        'bitwise_xor, the `^` operator, or the logical_xor function instead.')


def _negative_boolean_error():
    raise TypeError(
        'The cupy boolean negative, the `-` operator, is not supported, '
        'use the `~` operator or the logical_not function instead.')


def _positive_boolean_error():
    raise TypeError(
        'The cupy boolean positive, the `+` operator, is not supported.')


add = _create_arithmetic(
    'add', '+', '|', 'Adds two arrays elementwise.\n\n.. seealso:: :data:`numpy.add`')
subtract = _create_arithmetic(
    'subtract', '-', _subtract_boolean_error,
    'Subtracts arguments elementwise.\n\n.. seealso:: :data:`numpy.subtract`')
multiply = _create_arithmetic(
    'multiply', '*', '&',
    'Multiplies two arrays elementwise.\n\n.. seealso:: :data:`numpy.multiply`')

true_divide = create_ufunc(
    'cupy_true_divide',
    _sig(_INTS, 2, 'd') + _sig(_FLOATS + _COMPLEX, 2),
    'out0 = (out0_type)in0 / (out0_type)in1',
    doc='Elementwise true division.\n\n.. seealso:: :data:`numpy.true_divide`')
divide = true_divide

_float_floor_divide = '''
template <typename T> __device__ __forceinline__ T _cupy_fdiv(T a, T b) {
  // floor(a / b) computed from the exact remainder so that the result does not
  // jump when a / b rounds up to an integer.
  if (b == T(0)) return a / b;
  T mod = fmod(a, b);
  T div = (a - mod) / b;
  if (mod != T(0) && ((b < T(0)) != (mod < T(0)))) div -= T(1);
  if (div != T(0)) {
    T fl = floor(div);
    if (div - fl > T(0.5)) fl += T(1);
    return fl;
  }
  return copysign(T(0), a / b);
}
template <typename T> __device__ __forceinline__ T _cupy_fmod_py(T a, T b) {
  if (b == T(0)) return fmod(a, b);
  T mod = fmod(a, b);
  if (mod != T(0)) { if ((b < T(0)) != (mod < T(0))) mod += b; }
  else mod = copysign(T(0), b);
  return mod;
}
'''

floor_divide = create_ufunc(
    'cupy_floor_divide',
    _sig(_INTS, 2) + (
        ('ee->e', 'out0 = _cupy_fdiv<float>(in0, in1)'),
        ('ff->f', 'out0 = _cupy_fdiv<float>(in0, in1)'),
        ('dd->d', 'out0 = _cupy_fdiv<double>(in0, in1)')),
    'out0 = _floor_divide(in0, in1)',
    preamble=_float_floor_divide,
    doc='Elementwise floor division.\n\n.. seealso:: :data:`numpy.floor_divide`')

remainder = create_ufunc(
    'cupy_remainder',
    _sig(_INTS, 2) + (
        ('ee->e', 'out0 = _cupy_fmod_py<float>(in0, in1)'),
        ('ff->f', 'out0 = _cupy_fmod_py<float>(in0, in1)'),
        ('dd->d', 'out0 = _cupy_fmod_py<double>(in0, in1)')),
    'out0 = in1 == 0 ? (out0_type)0 : (out0_type)(in0 - _floor_divide(in0, in1) * in1)',
    preamble=_float_floor_divide,
    doc='Elementwise remainder with the sign of the divisor.\n\n'
        '.. seealso:: :data:`numpy.remainder`')
mod = remainder

_power_preamble = '''
template <typename T>
__device__ __forceinline__ T integral_power(T in0, T in1) {
  if (in1 < 0) {
    if (in0 == -1) return (in1 & 1) ? -1 : 1;
    return (in0 == 1) ? 1 : 0;
  }
  T out0 = 1;
  while (in1 > 0) {
    if (in1 & 1) out0 *= in0;
    in0 *= in0;
    in1 >>= 1;
  }
  return out0;
}
'''

power = create_ufunc(
    'cupy_power',
    ('??->b',) + _sig(_INTS, 2) + (
        ('ee->e', 'out0 = powf(in0, in1)'),
        ('ff->f', 'out0 = powf(in0, in1)'),
        ('dd->d', 'out0 = pow(in0, in1)'),
        ('FF->F', 'out0 = pow(in0, in1)'),
        ('DD->D', 'out0 = pow(in0, in1)')),
    'out0 = integral_power(in0, in1)',
    preamble=_power_preamble,
    doc='Computes ``x1 ** x2`` elementwise.\n\n.. seealso:: :data:`numpy.power`')

negative = create_ufunc(
    'cupy_negative',
    (('?->?', _negative_boolean_error),) + _sig(_INTS + _FLOATS + _COMPLEX, 1),
    'out0 = -in0',
    doc='Takes numerical negative elementwise.\n\n.. seealso:: :data:`numpy.negative`')

positive = create_ufunc(
    'cupy_positive',
    (('?->?', _positive_boolean_error),) + _sig(_INTS + _FLOATS + _COMPLEX, 1),
    'out0 = +in0',
    doc='Takes numerical positive elementwise.\n\n.. seealso:: :data:`numpy.positive`')

square = create_ufunc(
    'cupy_square',
    _sig(_INTS + _FLOATS + _COMPLEX, 1),
    'out0 = in0 * in0',
    doc='Elementwise square of the input.\n\n.. seealso:: :data:`numpy.square`')

absolute = create_ufunc(
    'cupy_absolute',
    (('?->?', 'out0 = in0'),
     'b->b', ('B->B', 'out0 = in0'), 'h->h', ('H->H', 'out0 = in0'),
     'i->i', ('I->I', 'out0 = in0'), 'l->l', ('L->L', 'out0 = in0'),
     'q->q', ('Q->Q', 'out0 = in0'),
     ('e->e', 'out0 = fabsf(in0)'),
     ('f->f', 'out0 = fabsf(in0)'),
     ('d->d', 'out0 = fabs(in0)'),
     ('F->f', 'out0 = abs(in0)'),
     ('D->d', 'out0 = abs(in0)')),
    'out0 = in0 > 0 ? in0 : -in0',
    doc='Elementwise absolute value.\n\n.. seealso:: :data:`numpy.absolute`')
abs = absolute

sign = create_ufunc(
    'cupy_sign',
    ('b->b', ('B->B', 'out0 = in0 > 0'), 'h->h', ('H->H', 'out0 = in0 > 0'),
     'i->i', ('I->I', 'out0 = in0 > 0'), 'l->l', ('L->L', 'out0 = in0 > 0'),
     'q->q', ('Q->Q', 'out0 = in0 > 0'),
     ('e->e', 'out0 = isnan(in0) ? in0 : (out0_type)((in0 > 0) - (in0 < 0))'),
     ('f->f', 'out0 = isnan(in0) ? in0 : (out0_type)((in0 > 0) - (in0 < 0))'),
     ('d->d', 'out0 = isnan(in0) ? in0 : (out0_type)((in0 > 0) - (in0 < 0))'),
     ('F->F', 'out0 = _cupy_csign(in0)'),
     ('D->D', 'out0 = _cupy_csign(in0)')),
    'out0 = (in0 > 0) - (in0 < 0)',
    preamble='''
// z / |z|; 0 for 0, NaN for what has no direction (NumPy >= 2)
template <typename T> __device__ __forceinline__ complex<T> _cupy_csign(const complex<T>& z) {
  const T a = abs(z);
  if (a == 0) return complex<T>(0, 0);
  if (isnan(a)) return complex<T>(CUDART_NAN, CUDART_NAN);
  if (isinf(a)) {
    if (isinf(z.re) && isinf(z.im)) return complex<T>(CUDART_NAN, CUDART_NAN);
    if (isinf(z.re)) return complex<T>(z.re > 0 ? 1 : -1, 0);
    return complex<T>(0, z.im > 0 ? 1 : -1);
  }
  return complex<T>(z.re / a, z.im / a);
}
''',
    doc='Elementwise sign.\n\n.. seealso:: :data:`numpy.sign`')

reciprocal = create_ufunc(
    'cupy_reciprocal',
    _sig(_INTS, 1) + (
        ('e->e', 'out0 = 1 / in0'), ('f->f', 'out0 = 1 / in0'),
        ('d->d', 'out0 = 1 / in0'),
        ('F->F', 'out0 = in0_type(1) / in0'),
        ('D->D', 'out0 = in0_type(1) / in0')),
    'out0 = in0 == 0 ? 0 : (1 / in0)',
    doc='Elementwise reciprocal.\n\n.. seealso:: :data:`numpy.reciprocal`')


def _float_unary(name, f32, f64, doc, cplx=None):
    loops = (('e->e', 'out0 = %s(in0)' % f32),
             ('f->f', 'out0 = %s(in0)' % f32),
             ('d->d', 'out0 = %s(in0)' % f64))
    if cplx:
        loops += (('F->F', 'out0 = %s(in0)' % cplx), ('D->D', 'out0 = %s(in0)' % cplx))
    return create_ufunc('cupy_' + name, loops, doc=doc)


sqrt = _float_unary('sqrt', 'sqrtf', 'sqrt', 'Elementwise square root.', 'sqrt')
cbrt = _float_unary('cbrt', 'cbrtf', 'cbrt', 'Elementwise cube root.')
exp = _float_unary('exp', 'expf', 'exp', 'Elementwise exponential.', 'exp')
exp2 = _float_unary('exp2', 'exp2f', 'exp2', 'Elementwise 2**x.', 'exp2')
expm1 = _float_unary('expm1', 'expm1f', 'expm1', 'Elementwise exp(x) - 1.', 'expm1')
log = _float_unary('log', 'logf', 'log', 'Elementwise natural logarithm.', 'log')
log2 = _float_unary('log2', 'log2f', 'log2', 'Elementwise base-2 logarithm.', 'log2')
log10 = _float_unary('log10', 'log10f', 'log10', 'Elementwise base-10 logarithm.', 'log10')
log1p = _float_unary('log1p', 'log1pf', 'log1p', 'Elementwise log(1 + x).', 'log1p')
sin = _float_unary('sin', 'sinf', 'sin', 'Elementwise sine.', 'sin')
cos = _float_unary('cos', 'cosf', 'cos', 'Elementwise cosine.', 'cos')
tan = _float_unary('tan', 'tanf', 'tan', 'Elementwise tangent.', 'tan')
arcsin = _float_unary('arcsin', 'asinf', 'asin', 'Elementwise inverse sine.', 'asin')
arccos = _float_unary('arccos', 'acosf', 'acos', 'Elementwise inverse cosine.', 'acos')
arctan = _float_unary('arctan', 'atanf', 'atan', 'Elementwise inverse tangent.', 'atan')
sinh = _float_unary('sinh', 'sinhf', 'sinh', 'Elementwise hyperbolic sine.', 'sinh')
cosh = _float_unary('cosh', 'coshf', 'cosh', 'Elementwise hyperbolic cosine.', 'cosh')
tanh = _float_unary('tanh', 'tanhf', 'tanh', 'Elementwise hyperbolic tangent.', 'tanh')
arcsinh = _float_unary('arcsinh', 'asinhf', 'asinh', 'Elementwise inverse sinh.', 'asinh')
arccosh = _float_unary('arccosh', 'acoshf', 'acosh', 'Elementwise inverse cosh.', 'acosh')
arctanh = _float_unary('arctanh', 'atanhf', 'atanh', 'Elementwise inverse tanh.', 'atanh')


def _rounding(name, f32, f64, doc):
    # NumPy >= 2.1 returns integers unchanged from floor/ceil/trunc.
    return create_ufunc(
        'cupy_' + name,
        tuple(('%s->%s' % (c, c), 'out0 = in0') for c in '?' + _INTS) + (
            ('e->e', 'out0 = %s(in0)' % f32),
            ('f->f', 'out0 = %s(in0)' % f32),
            ('d->d', 'out0 = %s(in0)' % f64)),
        doc=doc)


floor = _rounding('floor', 'floorf', 'floor', 'Elementwise floor.')
ceil = _rounding('ceil', 'ceilf', 'ceil', 'Elementwise ceiling.')
trunc = _rounding('trunc', 'truncf', 'trunc', 'Elementwise truncation.')
rint = _float_unary('rint', 'rintf', 'rint', 'Elementwise round half to even.', 'rint')

arctan2 = create_ufunc(
    'cupy_arctan2',
    (('ee->e', 'out0 = atan2f(in0, in1)'),
     ('ff->f', 'out0 = atan2f(in0, in1)'),
     ('dd->d', 'out0 = atan2(in0, in1)')),
    doc='Elementwise arc tangent of x1/x2 choosing the quadrant correctly.')

hypot = create_ufunc(
    'cupy_hypot',
    (('ee->e', 'out0 = hypotf(in0, in1)'),
     ('ff->f', 'out0 = hypotf(in0, in1)'),
     ('dd->d', 'out0 = hypot(in0, in1)')),
    doc='Elementwise hypotenuse.')

copysign = create_ufunc(
    'cupy_copysign',
    (('ee->e', 'out0 = copysignf(in0, in1)'),
     ('ff->f', 'out0 = copysignf(in0, in1)'),
     ('dd->d', 'out0 = copysign(in0, in1)')),
    doc='Elementwise copysign.')

maximum = create_ufunc(
    'cupy_maximum',
    ('??->?',) + _sig(_INTS, 2) + (
        ('ee->e', 'out0 = (isnan(in0) | isnan(in1)) ? (isnan(in0) ? in0 : in1) : (in0 > in1 ? in0 : in1)'),
        ('ff->f', 'out0 = (isnan(in0) | isnan(in1)) ? (isnan(in0) ? in0 : in1) : (in0 > in1 ? in0 : in1)'),
        ('dd->d', 'out0 = (isnan(in0) | isnan(in1)) ? (isnan(in0) ? in0 : in1) : (in0 > in1 ? in0 : in1)'),
        ('FF->F', 'out0 = (in0 >= in1 || isnan(in0)) ? in0 : in1'),
        ('DD->D', 'out0 = (in0 >= in1 || isnan(in0)) ? in0 : in1')),
    'out0 = in0 > in1 ? in0 : in1',
    doc='Elementwise maximum; NaNs propagate.\n\n.. seealso:: :data:`numpy.maximum`')

minimum = create_ufunc(
    'cupy_minimum',
    ('??->?',) + _sig(_INTS, 2) + (
        ('ee->e', 'out0 = (isnan(in0) | isnan(in1)) ? (isnan(in0) ? in0 : in1) : (in0 < in1 ? in0 : in1)'),
        ('ff->f', 'out0 = (isnan(in0) | isnan(in1)) ? (isnan(in0) ? in0 : in1) : (in0 < in1 ? in0 : in1)'),
        ('dd->d', 'out0 = (isnan(in0) | isnan(in1)) ? (isnan(in0) ? in0 : in1) : (in0 < in1 ? in0 : in1)'),
        ('FF->F', 'out0 = (in0 <= in1 || isnan(in0)) ? in0 : in1'),
        ('DD->D', 'out0 = (in0 <= in1 || isnan(in0)) ? in0 : in1')),
    'out0 = in0 < in1 ? in0 : in1',
    doc='Elementwise minimum; NaNs propagate.\n\n.. seealso:: :data:`numpy.minimum`')

fmax = create_ufunc(
    'cupy_fmax',
    ('??->?',) + _sig(_INTS, 2) + (
        ('ee->e', 'out0 = fmaxf(in0, in1)'),
        ('ff->f', 'out0 = fmaxf(in0, in1)'),
        ('dd->d', 'out0 = fmax(in0, in1)'),
        ('FF->F', 'out0 = (in0 >= in1 || isnan(in1)) ? in0 : in1'),
        ('DD->D', 'out0 = (in0 >= in1 || isnan(in1)) ? in0 : in1')),
    'out0 = in0 > in1 ? in0 : in1',
    doc='Elementwise maximum ignoring NaNs.')

fmin = create_ufunc(
    'cupy_fmin',
    ('??->?',) + _sig(_INTS, 2) + (
        ('ee->e', 'out0 = fminf(in0, in1)'),
        ('ff->f', 'out0 = fminf(in0, in1)'),
        ('dd->d', 'out0 = fmin(in0, in1)'),
        ('FF->F', 'out0 = (in0 <= in1 || isnan(in1)) ? in0 : in1'),
        ('DD->D', 'out0 = (in0 <= in1 || isnan(in1)) ? in0 : in1')),
    'out0 = in0 < in1 ? in0 : in1',
    doc='Elementwise minimum ignoring NaNs.')


def _comparison(name, op, doc):
    # int64 against uint64 compares the values, not their common C type: a
    # negative number is below every unsigned one
    signed_first = 'out0 = in0 < 0 ? (-1 %s 0) : ((unsigned long long)in0 %s in1)' % (op, op)
    unsigned_first = 'out0 = in1 < 0 ? (0 %s -1) : (in0 %s (unsigned long long)in1)' % (op, op)
    return create_ufunc(
        'cupy_' + name,
        _sig('?' + _INTS, 2, '?') + (('qQ->?', signed_first), ('Qq->?', unsigned_first))
        + _sig(_FLOATS + _COMPLEX, 2, '?'),
        'out0 = in0 %s in1' % op,
        doc=doc)


less = _comparison('less', '<', 'Tests elementwise ``x1 < x2``.')
less_equal = _comparison('less_equal', '<=', 'Tests elementwise ``x1 <= x2``.')
greater = _comparison('greater', '>', 'Tests elementwise ``x1 > x2``.')
greater_equal = _comparison('greater_equal', '>=', 'Tests elementwise ``x1 >= x2``.')
equal = _comparison('equal', '==', 'Tests elementwise ``x1 == x2``.')
not_equal = _comparison('not_equal', '!=', 'Tests elementwise ``x1 != x2``.')

logical_and = create_ufunc(
    'cupy_logical_and', _sig('?' + _INTS + _FLOATS + _COMPLEX, 2, '?'),
    'out0 = in0 && in1', doc='Elementwise logical AND.')
logical_or = create_ufunc(
    'cupy_logical_or', _sig('?' + _INTS + _FLOATS + _COMPLEX, 2, '?'),
    'out0 = in0 || in1', doc='Elementwise logical OR.')
logical_xor = create_ufunc(
    'cupy_logical_xor', _sig('?' + _INTS + _FLOATS + _COMPLEX, 2, '?'),
    'out0 = !in0 != !in1', doc='Elementwise logical XOR.')
logical_not = create_ufunc(
    'cupy_logical_not', _sig('?' + _INTS + _FLOATS + _COMPLEX, 1, '?'),
    'out0 = !in0', doc='Elementwise logical NOT.')

bitwise_and = create_ufunc(
    'cupy_bitwise_and', ('??->?',) + _sig(_INTS, 2),
    'out0 = in0 & in1', doc='Elementwise bitwise AND.')
bitwise_or = create_ufunc(
    'cupy_bitwise_or', ('??->?',) + _sig(_INTS, 2),
    'out0 = in0 | in1', doc='Elementwise bitwise OR.')
bitwise_xor = create_ufunc(
    'cupy_bitwise_xor', ('??->?',) + _sig(_INTS, 2),
    'out0 = in0 ^ in1', doc='Elementwise bitwise XOR.')
invert = create_ufunc(
    'cupy_invert', (('?->?', 'out0 = !in0'),) + _sig(_INTS, 1),
    'out0 = ~in0', doc='Elementwise bitwise NOT.')
bitwise_not = invert

# in-place application at indices (ufunc.at): the operation each of these
# applies atomically (cupy/_core/_routines_math.pyx:905,1060,
# cupy/_core/_routines_binary.pyx:23-47 pass the same names as scatter_op=)
for _uf, _op in ((add, 'add'), (subtract, 'sub'), (maximum, 'max'), (minimum, 'min'),
                 (bitwise_and, 'and'), (bitwise_or, 'or'), (bitwise_xor, 'xor')):
    _uf._scatter_op = _op
del _uf, _op
left_shift = create_ufunc(
    'cupy_left_shift', _sig(_INTS, 2),
    'out0 = (in1 < 0 || in1 >= (int)(sizeof(in0_type) * 8)) ? (out0_type)0 : (out0_type)(in0 << in1)',
    doc='Elementwise left shift.')
right_shift = create_ufunc(
    'cupy_right_shift', _sig(_INTS, 2),
    'out0 = (in1 < 0 || in1 >= (int)(sizeof(in0_type) * 8)) ? (out0_type)(in0 < 0 ? -1 : 0) : (out0_type)(in0 >> in1)',
    doc='Elementwise right shift.')

isnan = create_ufunc(
    'cupy_isnan',
    tuple(('%s->?' % c, 'out0 = false') for c in '?' + _INTS) + _sig(_FLOATS + _COMPLEX, 1, '?'),
    'out0 = isnan(in0)', doc='Tests elementwise for NaN.')
isinf = create_ufunc(
    'cupy_isinf',
    tuple(('%s->?' % c, 'out0 = false') for c in '?' + _INTS) + _sig(_FLOATS + _COMPLEX, 1, '?'),
    'out0 = isinf(in0)', doc='Tests elementwise for +/- infinity.')
isfinite = create_ufunc(
    'cupy_isfinite',
    tuple(('%s->?' % c, 'out0 = true') for c in '?' + _INTS) + _sig(_FLOATS + _COMPLEX, 1, '?'),
    'out0 = isfinite(in0)', doc='Tests elementwise for finiteness.')
signbit = create_ufunc(
    'cupy_signbit', _sig(_FLOATS, 1, '?'),
    'out0 = signbit(in0)', doc='Tests elementwise whether the sign bit is set.')

_where_ufunc = create_ufunc(
    'cupy_where',
    tuple('?%s%s->%s' % (c, c, c) for c in '?' + _INTS + _FLOATS + _COMPLEX),
    'out0 = in0 ? in1 : in2')

_clip = create_ufunc(
    'cupy_clip',
    tuple('%s%s%s->%s' % (c, c, c, c) for c in '?' + _INTS + _FLOATS + _COMPLEX),
    'out0 = in0 < in1 ? in1 : (in0 > in2 ? in2 : in0)')


# ---------------------------------------------------------------------------------
# The rest of NumPy's real-valued catalogue (reference: cupy/_math/arithmetic.py,
# floating.py, rational.py, trigonometric.py, explog.py, misc.py, special.py,
# cupy/_binary/elementwise.py, cupy/_logic/comparison.py).
# ---------------------------------------------------------------------------------

fabs = create_ufunc(
    'cupy_fabs',
    (('e->e', 'out0 = fabsf(in0)'), ('f->f', 'out0 = fabsf(in0)'), ('d->d', 'out0 = fabs(in0)')),
    doc='Absolute value of floating-point elements.\n\n.. seealso:: :data:`numpy.fabs`')

fmod = create_ufunc(
    'cupy_fmod',
    tuple(('%s%s->%s' % (c, c, c), 'out0 = in1 == 0 ? (out0_type)0 : (out0_type)(in0 % in1)')
          for c in _INTS) + (
        ('ee->e', 'out0 = fmodf(in0, in1)'), ('ff->f', 'out0 = fmodf(in0, in1)'),
        ('dd->d', 'out0 = fmod(in0, in1)')),
    doc='Remainder of C division (sign of the dividend).\n\n.. seealso:: :data:`numpy.fmod`')

float_power = create_ufunc(
    'cupy_float_power', (('dd->d', 'out0 = pow(in0, in1)'), ('DD->D', 'out0 = pow(in0, in1)')),
    doc='Power computed in float64 whatever the inputs.\n\n.. seealso:: :data:`numpy.float_power`')

_gcd_preamble = '''
template <typename T> __device__ __forceinline__ T _cupy_gcd(T a, T b) {
  while (b != 0) { const T r = a % b; a = b; b = r; }
  return a < 0 ? (T)(-a) : a;
}
template <typename T> __device__ __forceinline__ T _cupy_lcm(T a, T b) {
  const T g = _cupy_gcd(a, b);
  if (g == 0) return 0;
  const T r = a / g * b;
  return r < 0 ? (T)(-r) : r;
}
'''


def _no_bool(name):
    def raiser():
        raise TypeError('%s cannot be computed with boolean arrays' % name)
    return raiser


gcd = create_ufunc(
    'cupy_gcd', (('??->?', _no_bool('gcd')),) + _sig(_INTS, 2),
    'out0 = _cupy_gcd(in0, in1)', preamble=_gcd_preamble,
    doc='Greatest common divisor.\n\n.. seealso:: :data:`numpy.gcd`')
lcm = create_ufunc(
    'cupy_lcm', (('??->?', _no_bool('lcm')),) + _sig(_INTS, 2),
    'out0 = _cupy_lcm(in0, in1)', preamble=_gcd_preamble,
    doc='Least common multiple.\n\n.. seealso:: :data:`numpy.lcm`')

heaviside = create_ufunc(
    'cupy_heaviside', _sig(_FLOATS, 2),
    'out0 = (in0 != in0) ? in0 : (in0 == 0 ? in1 : (out0_type)(in0 > 0 ? 1 : 0))',
    doc='Heaviside step function.\n\n.. seealso:: :data:`numpy.heaviside`')

_sinc_preamble = '''
template <typename T> __device__ __forceinline__ T _cupy_sinc(T x) {
  if (x == 0) return 1;
  const T px = x * (T)3.14159265358979323846;
  return sin(px) / px;
}
'''
sinc = create_ufunc(
    'cupy_sinc',
    (('e->e', 'out0 = _cupy_sinc((float)in0)'), ('f->f', 'out0 = _cupy_sinc(in0)'),
     ('d->d', 'out0 = _cupy_sinc(in0)')),
    preamble=_sinc_preamble,
    doc='Normalised sinc: sin(pi x) / (pi x).\n\n.. seealso:: :func:`numpy.sinc`')

ldexp = create_ufunc(
    'cupy_ldexp',
    (('ei->e', 'out0 = ldexpf(in0, in1)'), ('fi->f', 'out0 = ldexpf(in0, in1)'),
     ('el->e', 'out0 = ldexpf(in0, (int)(in1 > 65536 ? 65536 : (in1 < -65536 ? -65536 : in1)))'),
     ('fl->f', 'out0 = ldexpf(in0, (int)(in1 > 65536 ? 65536 : (in1 < -65536 ? -65536 : in1)))'),
     ('di->d', 'out0 = ldexp(in0, in1)'),
     ('dl->d', 'out0 = ldexp(in0, (int)(in1 > 65536 ? 65536 : (in1 < -65536 ? -65536 : in1)))')),
    doc='x1 * 2**x2.\n\n.. seealso:: :data:`numpy.ldexp`')

frexp = create_ufunc(
    'cupy_frexp',
    (('e->ei', 'int _e; out0 = frexpf(in0, &_e); out1 = _e'),
     ('f->fi', 'int _e; out0 = frexpf(in0, &_e); out1 = _e'),
     ('d->di', 'int _e; out0 = frexp(in0, &_e); out1 = _e')),
    doc='Mantissa and exponent of two.\n\n.. seealso:: :data:`numpy.frexp`')

modf = create_ufunc(
    'cupy_modf',
    (('e->ee', 'float _i; out0 = modff(in0, &_i); out1 = _i'),
     ('f->ff', 'float _i; out0 = modff(in0, &_i); out1 = _i'),
     ('d->dd', 'double _i; out0 = modf(in0, &_i); out1 = _i')),
    doc='Fractional and integral parts.\n\n.. seealso:: :data:`numpy.modf`')

nextafter = create_ufunc(
    'cupy_nextafter',
    (('ee->e', 'out0 = _cupy_nextafter_half(in0, in1)'),
     ('ff->f', 'out0 = nextafterf(in0, in1)'), ('dd->d', 'out0 = nextafter(in0, in1)')),
    preamble='''
__device__ __forceinline__ float16 _cupy_nextafter_half(float16 x, float16 y) {
  // one step in the ordered integer image of the half's bits
  unsigned short xb, yb;
  __builtin_memcpy(&xb, &x, 2);
  __builtin_memcpy(&yb, &y, 2);
  const float xf = x, yf = y;
  if (xf != xf || yf != yf) { unsigned short q = 0x7e00; float16 r; __builtin_memcpy(&r, &q, 2); return r; }
  if (xf == yf) return y;
  unsigned short rb;
  if ((xb & 0x7fff) == 0) rb = (unsigned short)((yb & 0x8000) | 1);
  else if ((xf < yf) == ((xb & 0x8000) == 0)) rb = (unsigned short)(xb + 1);
  else rb = (unsigned short)(xb - 1);
  float16 r; __builtin_memcpy(&r, &rb, 2); return r;
}
''',
    doc='Next representable value towards x2.\n\n.. seealso:: :data:`numpy.nextafter`')

_logaddexp_preamble = '''
template <typename T> __device__ __forceinline__ T _cupy_logaddexp(T x, T y) {
  if (x == y) return x + (T)0.693147180559945309417;       // also +-inf
  const T d = x - y;
  if (d > 0) return x + log1p(exp(-d));
  if (d <= 0) return y + log1p(exp(d));
  return x + y;                                            // NaN
}
template <typename T> __device__ __forceinline__ T _cupy_logaddexp2(T x, T y) {
  const T k = (T)1.442695040888963407359924681;            // 1 / ln 2
  if (x == y) return x + (T)1;
  const T d = x - y;
  if (d > 0) return x + log1p(exp2(-d)) * k;
  if (d <= 0) return y + log1p(exp2(d)) * k;
  return x + y;
}
'''
logaddexp = create_ufunc(
    'cupy_logaddexp',
    (('ee->e', 'out0 = _cupy_logaddexp((float)in0, (float)in1)'),
     ('ff->f', 'out0 = _cupy_logaddexp(in0, in1)'), ('dd->d', 'out0 = _cupy_logaddexp(in0, in1)')),
    preamble=_logaddexp_preamble,
    doc='log(exp(x1) + exp(x2)).\n\n.. seealso:: :data:`numpy.logaddexp`')
logaddexp2 = create_ufunc(
    'cupy_logaddexp2',
    (('ee->e', 'out0 = _cupy_logaddexp2((float)in0, (float)in1)'),
     ('ff->f', 'out0 = _cupy_logaddexp2(in0, in1)'), ('dd->d', 'out0 = _cupy_logaddexp2(in0, in1)')),
    preamble=_logaddexp_preamble,
    doc='log2(2**x1 + 2**x2).\n\n.. seealso:: :data:`numpy.logaddexp2`')

deg2rad = create_ufunc(
    'cupy_deg2rad',
    (('e->e', 'out0 = (float)in0 * 0.017453292519943295f'),
     ('f->f', 'out0 = in0 * 0.017453292519943295f'),
     ('d->d', 'out0 = in0 * 0.017453292519943295')),
    doc='Degrees to radians.\n\n.. seealso:: :data:`numpy.deg2rad`')
rad2deg = create_ufunc(
    'cupy_rad2deg',
    (('e->e', 'out0 = (float)in0 * 57.29577951308232f'),
     ('f->f', 'out0 = in0 * 57.29577951308232f'),
     ('d->d', 'out0 = in0 * 57.29577951308232')),
    doc='Radians to degrees.\n\n.. seealso:: :data:`numpy.rad2deg`')
radians = deg2rad
degrees = rad2deg

bitwise_count = create_ufunc(
    'cupy_bitwise_count',
    tuple(('%s->B' % c,
           'out0 = __popcll((unsigned long long)(in0 < 0 ? -in0 : in0))' if c.islower()
           else 'out0 = __popcll((unsigned long long)in0)') for c in _INTS),
    doc='Number of set bits of the absolute value.\n\n.. seealso:: :data:`numpy.bitwise_count`')

i0 = create_ufunc(
    'cupy_i0',
    (('e->e', 'out0 = cyl_bessel_i0f((float)in0)'), ('f->f', 'out0 = cyl_bessel_i0f(in0)'),
     ('d->d', 'out0 = cyl_bessel_i0(in0)')),
    doc='Modified Bessel function of the first kind, order 0.\n\n.. seealso:: :func:`numpy.i0`')

_is_close = create_ufunc(
    'cupy_is_close',
    (('eeee?->?', None), ('ffff?->?', None), ('dddd?->?', None)),
    '''
    bool equal_nan = in4;
    if (isfinite(in0) && isfinite(in1)) {
      out0 = fabs(in0 - in1) <= in3 + in2 * fabs(in1);
    } else if (equal_nan) {
      out0 = (in0 == in1) || (isnan(in0) && isnan(in1));
    } else {
      out0 = (in0 == in1);
    }
    ''')

# complex operands: the same test with the modulus in place of fabs
# (reference: cupy/_logic/comparison.py:24-41)
_is_close_complex = create_ufunc(
    'cupy_is_close_complex',
    (('FFff?->?', None), ('DDdd?->?', None)),
    '''
    bool equal_nan = in4;
    if (isfinite(in0) && isfinite(in1)) {
      out0 = abs(in0 - in1) <= in3 + in2 * abs(in1);
    } else if (equal_nan) {
      out0 = (in0 == in1) || (isnan(in0) && isnan(in1));
    } else {
      out0 = (in0 == in1);
    }
    ''')

_nan_to_num = create_ufunc(
    'cupy_nan_to_num_',
    tuple(('%s%s%s%s->%s' % (c, c, c, c, c), 'out0 = in0') for c in '?' + _INTS) +
    tuple(('%s%s%s%s->%s' % (c, c, c, c, c), None) for c in _FLOATS),
    'out0 = isnan(in0) ? in1 : (isinf(in0) ? (in0 > 0 ? in2 : in3) : in0)')


def isclose(a, b, rtol=1.e-5, atol=1.e-8, equal_nan=False):
    """Elementwise ``|a - b| <= atol + rtol * |b|`` as a boolean array.

    .. seealso:: :func:`numpy.isclose`
    """
    import numpy
    from cupy_amd._core.core import array
    a = array(a, copy=False)
    b = array(b, copy=False)
    dt = numpy.result_type(a.dtype, b.dtype)
    if dt.kind == 'c':
        real = numpy.dtype('float32' if dt == numpy.complex64 else 'float64').type
        return _is_close_complex(a.astype(dt, copy=False), b.astype(dt, copy=False),
                                 real(rtol), real(atol), bool(equal_nan))
    if dt.kind != 'f':
        dt = numpy.dtype('float64')
    return _is_close(a.astype(dt, copy=False), b.astype(dt, copy=False),
                     dt.type(rtol), dt.type(atol), bool(equal_nan))


def allclose(a, b, rtol=1.e-5, atol=1.e-8, equal_nan=False):
    """0-d boolean array: all elements close (no synchronisation).

    .. seealso:: :func:`numpy.allclose`
    """
    return isclose(a, b, rtol, atol, equal_nan).all()


def nan_to_num(x, copy=True, nan=0.0, posinf=None, neginf=None):
    """Replaces NaN and infinities with finite numbers.

    .. seealso:: :func:`numpy.nan_to_num`
    """
    import numpy
    from cupy_amd._core.core import array
    x = array(x, copy=False)
    if x.dtype.kind != 'f':
        return x.copy() if copy else x
    info = numpy.finfo(x.dtype)
    posinf = info.max if posinf is None else posinf
    neginf = info.min if neginf is None else neginf
    t = x.dtype.type
    with numpy.errstate(all='ignore'):
        args = (x, t(nan), t(posinf), t(neginf))
    return _nan_to_num(*args, out=None if copy else x)


def clip(a, a_min=None, a_max=None, out=None):
    """Limits the values to ``[a_min, a_max]``.

    .. seealso:: :func:`numpy.clip`
    """
    if a_min is None and a_max is None:
        raise ValueError('array_clip: must set either max or min')
    if _fusion_thread_local.is_fusing() and a_min is not None and a_max is not None:
        return _fusion_thread_local.call_ufunc(_clip, a, a_min, a_max, out=out)
    if a_min is None:
        return minimum(a, a_max, out=out)
    if a_max is None:
        return maximum(a, a_min, out=out)
    return _clip(a, a_min, a_max, out=out)


def where(condition, x=None, y=None):
    """Elements of ``x`` where ``condition`` holds, of ``y`` elsewhere.

    .. seealso:: :func:`numpy.where`
    """
    if x is None or y is None:
        raise NotImplementedError(
            'where(condition) alone returns indices, which needs a stream '
            'compaction that is not part of this package')
    if _fusion_thread_local.is_fusing():
        return _fusion_thread_local.call_ufunc(_where_ufunc, condition, x, y)
    from cupy_amd._core.core import array
    condition = array(condition, copy=False)
    if condition.dtype != bool:
        condition = condition.astype(bool)
    return _where_ufunc(condition, x, y)


divmod = create_ufunc(
    'cupy_divmod',
    tuple('%s%s->%s%s' % (c, c, c, c) for c in _INTS) + (
        ('ee->ee', 'out0 = _cupy_fdiv<float>(in0, in1); out1 = _cupy_fmod_py<float>(in0, in1)'),
        ('ff->ff', 'out0 = _cupy_fdiv<float>(in0, in1); out1 = _cupy_fmod_py<float>(in0, in1)'),
        ('dd->dd', 'out0 = _cupy_fdiv<double>(in0, in1); out1 = _cupy_fmod_py<double>(in0, in1)')),
    'out0 = _floor_divide(in0, in1); '
    'out1 = in1 == 0 ? (out1_type)0 : (out1_type)(in0 - out0 * in1)',
    preamble=_float_floor_divide,
    doc='Quotient and remainder of floor division, as two arrays.\n\n'
        '.. seealso:: :data:`numpy.divmod`')


# ---------------------------------------------------------------------------------
# Complex-number helpers (reference: cupy/_core/_routines_math.pyx:908-949,
# cupy/_math/misc.py real/imag/angle).
# ---------------------------------------------------------------------------------

conjugate = create_ufunc(
    'cupy_conjugate',
    _sig(_INTS + _FLOATS, 1) + (
        ('F->F', 'out0 = conj(in0)'), ('D->D', 'out0 = conj(in0)')),
    'out0 = in0',
    doc='Complex conjugate, elementwise.\n\n.. seealso:: :data:`numpy.conjugate`')
conj = conjugate

# names of the array API standard, as in NumPy 2
acos, acosh, asin, asinh, atan, atanh, atan2 = (
    arccos, arccosh, arcsin, arcsinh, arctan, arctanh, arctan2)
bitwise_invert, bitwise_left_shift, bitwise_right_shift = invert, left_shift, right_shift
pow = power

_real_ufunc = create_ufunc(
    'cupy_real',
    _sig('?' + _INTS + _FLOATS, 1) + (
        ('F->f', 'out0 = in0.real()'), ('D->d', 'out0 = in0.real()')),
    'out0 = in0')
_imag_ufunc = create_ufunc(
    'cupy_imag',
    _sig('?' + _INTS + _FLOATS, 1) + (
        ('F->f', 'out0 = in0.imag()'), ('D->d', 'out0 = in0.imag()')),
    'out0 = 0')

_angle_ufunc = create_ufunc(
    'cupy_angle',
    tuple(('%s->d' % c, 'out0 = in0 >= 0 ? 0.0 : M_PI') for c in '?' + _INTS) + (
        ('e->e', 'out0 = atan2f(0.0f, in0)'),
        ('f->f', 'out0 = atan2f(0.0f, in0)'),
        ('d->d', 'out0 = atan2(0.0, in0)'),
        ('F->f', 'out0 = arg(in0)'),
        ('D->d', 'out0 = arg(in0)')))
_angle_deg_ufunc = create_ufunc(
    'cupy_angle_deg',
    tuple(('%s->d' % c, 'out0 = in0 >= 0 ? 0.0 : 180.0') for c in '?' + _INTS) + (
        ('e->e', 'out0 = atan2f(0.0f, in0) * (float)(180.0 / M_PI)'),
        ('f->f', 'out0 = atan2f(0.0f, in0) * (float)(180.0 / M_PI)'),
        ('d->d', 'out0 = atan2(0.0, in0) * (180.0 / M_PI)'),
        ('F->f', 'out0 = arg(in0) * (float)(180.0 / M_PI)'),
        ('D->d', 'out0 = arg(in0) * (180.0 / M_PI)')))


def angle(z, deg=False):
    """Angle of the complex argument, in radians or degrees.

    .. seealso:: :func:`numpy.angle`
    """
    if _fusion_thread_local.is_fusing():
        return _fusion_thread_local.call_ufunc(_angle_deg_ufunc if deg else _angle_ufunc, z)
    if deg:
        return _angle_deg_ufunc(z)
    return _angle_ufunc(z)


def real(val):
    """Real part of the elements (a view for complex arrays).

    .. seealso:: :func:`numpy.real`
    """
    if _fusion_thread_local.is_fusing():
        return _fusion_thread_local.call_ufunc(_real_ufunc, val)
    from cupy_amd._core.core import array
    return array(val, copy=False).real


def imag(val):
    """Imaginary part of the elements (a view for complex arrays).

    .. seealso:: :func:`numpy.imag`
    """
    if _fusion_thread_local.is_fusing():
        return _fusion_thread_local.call_ufunc(_imag_ufunc, val)
    from cupy_amd._core.core import array
    return array(val, copy=False).imag


def iscomplexobj(x):
    """True if the argument's type is complex.

    .. seealso:: :func:`numpy.iscomplexobj`
    """
    import numpy
    dtype = getattr(x, 'dtype', None)
    if dtype is None:
        return numpy.iscomplexobj(x)
    return numpy.dtype(dtype).kind == 'c'


def isrealobj(x):
    """True if the argument's type is not complex.

    .. seealso:: :func:`numpy.isrealobj`
    """
    return not iscomplexobj(x)


def iscomplex(x):
    """Tests elementwise for a non-zero imaginary part.

    .. seealso:: :func:`numpy.iscomplex`
    """
    from cupy_amd._core.core import array
    x = array(x, copy=False)
    if x.dtype.kind == 'c':
        return x.imag != 0
    from cupy_amd import zeros
    return zeros(x.shape, bool)


def isreal(x):
    """Tests elementwise for a zero imaginary part.

    .. seealso:: :func:`numpy.isreal`
    """
    from cupy_amd._core.core import array
    x = array(x, copy=False)
    if x.dtype.kind == 'c':
        return x.imag == 0
    from cupy_amd import ones
    return ones(x.shape, bool)


# ---------------------------------------------------------------------------------
# Rounding to decimals (reference: cupy/_math/rounding.py:11-40 and the
# `_round_ufunc` of cupy/_core/_routines_math.pyx); the order of operations is
# NumPy's: scale by the power of ten in the array's own type, round half to
# even, scale back.  Integers go through double, as in NumPy.
# ---------------------------------------------------------------------------------

_round_preamble = '''
template <typename T> __device__ __forceinline__ T _cupy_round_real(T v, long long d) {
  if (d == 0) return T(rint(v));
  if (d > 0) { const T x = T(pow(10.0, (double)d)); return T(rint(v * x)) / x; }
  const T x = T(pow(10.0, (double)(-d)));
  return T(rint(v / x)) * x;
}
__device__ __forceinline__ float16 _cupy_round_half(float16 v, long long d) {
  if (d == 0) return float16(rintf(float(v)));
  const float16 x = float16(pow(10.0, (double)(d > 0 ? d : -d)));
  if (d > 0) return float16(rintf(float(float16(float(v) * float(x))))) / x;
  return float16(rintf(float(float16(float(v) / float(x))))) * x;
}
template <typename T> __device__ __forceinline__ T _cupy_round_int(T v, long long d) {
  if (d >= 0) return v;
  const double x = pow(10.0, (double)(-d));
  return (T)(rint((double)v / x) * x);
}
template <typename T> __device__ __forceinline__ complex<T> _cupy_round_complex(
    const complex<T>& v, long long d) {
  return complex<T>(_cupy_round_real(v.re, d), _cupy_round_real(v.im, d));
}
'''

_round_ufunc = create_ufunc(
    'cupy_round',
    (('?q->e', 'out0 = _cupy_round_half(float16(in0 ? 1.0f : 0.0f), in1)'),)
    + tuple(('%sq->%s' % (c, c), 'out0 = _cupy_round_int(in0, in1)') for c in _INTS)
    + (('eq->e', 'out0 = _cupy_round_half(in0, in1)'),
       ('fq->f', 'out0 = _cupy_round_real(in0, in1)'),
       ('dq->d', 'out0 = _cupy_round_real(in0, in1)'),
       ('Fq->F', 'out0 = _cupy_round_complex(in0, in1)'),
       ('Dq->D', 'out0 = _cupy_round_complex(in0, in1)')),
    preamble=_round_preamble)


def around(a, decimals=0, out=None):
    """Rounds to the given number of decimals (half to even).

    .. seealso:: :func:`numpy.around`
    """
    import operator
    decimals = operator.index(decimals)
    if _fusion_thread_local.is_fusing():
        return _fusion_thread_local.call_ufunc(_round_ufunc, a, decimals, out=out)
    from cupy_amd._core.core import array
    import numpy
    return _round_ufunc(array(a, copy=False), numpy.int64(decimals), out=out)


round = around


def round_(a, decimals=0, out=None):
    import warnings
    warnings.warn('Please use `round` instead.', DeprecationWarning)
    return around(a, decimals, out=out)


fix = create_ufunc(
    'cupy_fix',
    tuple(('%s->%s' % (c, c), 'out0 = in0') for c in '?' + _INTS) + (
        ('e->e', 'out0 = truncf(in0)'), ('f->f', 'out0 = truncf(in0)'),
        ('d->d', 'out0 = trunc(in0)')),
    doc='Rounds towards zero.\n\n.. seealso:: :func:`numpy.fix`')
