"""ufunc definitions: loop tables in NumPy's order (first match reproduces
NumPy's promotion) and the HIP routine of each loop.

The arithmetic tables correspond to the reference's
cupy/_core/_routines_math.pyx:878-1060 (add, subtract, multiply, power, ...),
cupy/_core/_ufuncs.py:7-13 (elementwise_copy) and cupy/_math/misc.py:197-206
(square); the rest of the catalogue follows NumPy's ``ufunc.types``.  Complex
loops are left out: the emitters have no complex type.
"""
from cupy_amd._core._kernel import create_ufunc

_INTS = 'bBhHiIlLqQ'
_FLOATS = 'efd'


def _sig(chars, nin, out=None):
    return tuple('%s->%s' % (c * nin, out or c) for c in chars)


elementwise_copy = create_ufunc(
    'cupy_copy',
    _sig('?' + _INTS + _FLOATS, 1),
    'out0 = in0',
    default_casting='unsafe')


def _create_arithmetic(name, op, boolop, doc):
    if isinstance(boolop, str):
        boolop = 'out0 = in0 %s in1' % boolop
    return create_ufunc(
        'cupy_' + name,
        (('??->?', boolop),) + _sig(_INTS + _FLOATS, 2),
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
    _sig(_INTS, 2, 'd') + _sig(_FLOATS, 2),
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
        ('dd->d', 'out0 = pow(in0, in1)')),
    'out0 = integral_power(in0, in1)',
    preamble=_power_preamble,
    doc='Computes ``x1 ** x2`` elementwise.\n\n.. seealso:: :data:`numpy.power`')

negative = create_ufunc(
    'cupy_negative',
    (('?->?', _negative_boolean_error),) + _sig(_INTS + _FLOATS, 1),
    'out0 = -in0',
    doc='Takes numerical negative elementwise.\n\n.. seealso:: :data:`numpy.negative`')

positive = create_ufunc(
    'cupy_positive',
    (('?->?', _positive_boolean_error),) + _sig(_INTS + _FLOATS, 1),
    'out0 = +in0',
    doc='Takes numerical positive elementwise.\n\n.. seealso:: :data:`numpy.positive`')

square = create_ufunc(
    'cupy_square',
    _sig(_INTS + _FLOATS, 1),
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
     ('d->d', 'out0 = fabs(in0)')),
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
     ('d->d', 'out0 = isnan(in0) ? in0 : (out0_type)((in0 > 0) - (in0 < 0))')),
    'out0 = (in0 > 0) - (in0 < 0)',
    doc='Elementwise sign.\n\n.. seealso:: :data:`numpy.sign`')

reciprocal = create_ufunc(
    'cupy_reciprocal',
    _sig(_INTS, 1) + (
        ('e->e', 'out0 = 1 / in0'), ('f->f', 'out0 = 1 / in0'),
        ('d->d', 'out0 = 1 / in0')),
    'out0 = in0 == 0 ? 0 : (1 / in0)',
    doc='Elementwise reciprocal.\n\n.. seealso:: :data:`numpy.reciprocal`')


def _float_unary(name, f32, f64, doc):
    return create_ufunc(
        'cupy_' + name,
        (('e->e', 'out0 = %s(in0)' % f32),
         ('f->f', 'out0 = %s(in0)' % f32),
         ('d->d', 'out0 = %s(in0)' % f64)),
        doc=doc)


sqrt = _float_unary('sqrt', 'sqrtf', 'sqrt', 'Elementwise square root.')
cbrt = _float_unary('cbrt', 'cbrtf', 'cbrt', 'Elementwise cube root.')
exp = _float_unary('exp', 'expf', 'exp', 'Elementwise exponential.')
exp2 = _float_unary('exp2', 'exp2f', 'exp2', 'Elementwise 2**x.')
expm1 = _float_unary('expm1', 'expm1f', 'expm1', 'Elementwise exp(x) - 1.')
log = _float_unary('log', 'logf', 'log', 'Elementwise natural logarithm.')
log2 = _float_unary('log2', 'log2f', 'log2', 'Elementwise base-2 logarithm.')
log10 = _float_unary('log10', 'log10f', 'log10', 'Elementwise base-10 logarithm.')
log1p = _float_unary('log1p', 'log1pf', 'log1p', 'Elementwise log(1 + x).')
sin = _float_unary('sin', 'sinf', 'sin', 'Elementwise sine.')
cos = _float_unary('cos', 'cosf', 'cos', 'Elementwise cosine.')
tan = _float_unary('tan', 'tanf', 'tan', 'Elementwise tangent.')
arcsin = _float_unary('arcsin', 'asinf', 'asin', 'Elementwise inverse sine.')
arccos = _float_unary('arccos', 'acosf', 'acos', 'Elementwise inverse cosine.')
arctan = _float_unary('arctan', 'atanf', 'atan', 'Elementwise inverse tangent.')
sinh = _float_unary('sinh', 'sinhf', 'sinh', 'Elementwise hyperbolic sine.')
cosh = _float_unary('cosh', 'coshf', 'cosh', 'Elementwise hyperbolic cosine.')
tanh = _float_unary('tanh', 'tanhf', 'tanh', 'Elementwise hyperbolic tangent.')
arcsinh = _float_unary('arcsinh', 'asinhf', 'asinh', 'Elementwise inverse sinh.')
arccosh = _float_unary('arccosh', 'acoshf', 'acosh', 'Elementwise inverse cosh.')
arctanh = _float_unary('arctanh', 'atanhf', 'atanh', 'Elementwise inverse tanh.')


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
rint = _float_unary('rint', 'rintf', 'rint', 'Elementwise round half to even.')

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
        ('dd->d', 'out0 = (isnan(in0) | isnan(in1)) ? (isnan(in0) ? in0 : in1) : (in0 > in1 ? in0 : in1)')),
    'out0 = in0 > in1 ? in0 : in1',
    doc='Elementwise maximum; NaNs propagate.\n\n.. seealso:: :data:`numpy.maximum`')

minimum = create_ufunc(
    'cupy_minimum',
    ('??->?',) + _sig(_INTS, 2) + (
        ('ee->e', 'out0 = (isnan(in0) | isnan(in1)) ? (isnan(in0) ? in0 : in1) : (in0 < in1 ? in0 : in1)'),
        ('ff->f', 'out0 = (isnan(in0) | isnan(in1)) ? (isnan(in0) ? in0 : in1) : (in0 < in1 ? in0 : in1)'),
        ('dd->d', 'out0 = (isnan(in0) | isnan(in1)) ? (isnan(in0) ? in0 : in1) : (in0 < in1 ? in0 : in1)')),
    'out0 = in0 < in1 ? in0 : in1',
    doc='Elementwise minimum; NaNs propagate.\n\n.. seealso:: :data:`numpy.minimum`')

fmax = create_ufunc(
    'cupy_fmax',
    ('??->?',) + _sig(_INTS, 2) + (
        ('ee->e', 'out0 = fmaxf(in0, in1)'),
        ('ff->f', 'out0 = fmaxf(in0, in1)'),
        ('dd->d', 'out0 = fmax(in0, in1)')),
    'out0 = in0 > in1 ? in0 : in1',
    doc='Elementwise maximum ignoring NaNs.')

fmin = create_ufunc(
    'cupy_fmin',
    ('??->?',) + _sig(_INTS, 2) + (
        ('ee->e', 'out0 = fminf(in0, in1)'),
        ('ff->f', 'out0 = fminf(in0, in1)'),
        ('dd->d', 'out0 = fmin(in0, in1)')),
    'out0 = in0 < in1 ? in0 : in1',
    doc='Elementwise minimum ignoring NaNs.')


def _comparison(name, op, doc):
    return create_ufunc(
        'cupy_' + name,
        _sig('?' + _INTS + _FLOATS, 2, '?'),
        'out0 = in0 %s in1' % op,
        doc=doc)


less = _comparison('less', '<', 'Tests elementwise ``x1 < x2``.')
less_equal = _comparison('less_equal', '<=', 'Tests elementwise ``x1 <= x2``.')
greater = _comparison('greater', '>', 'Tests elementwise ``x1 > x2``.')
greater_equal = _comparison('greater_equal', '>=', 'Tests elementwise ``x1 >= x2``.')
equal = _comparison('equal', '==', 'Tests elementwise ``x1 == x2``.')
not_equal = _comparison('not_equal', '!=', 'Tests elementwise ``x1 != x2``.')

logical_and = create_ufunc(
    'cupy_logical_and', _sig('?' + _INTS + _FLOATS, 2, '?'),
    'out0 = in0 && in1', doc='Elementwise logical AND.')
logical_or = create_ufunc(
    'cupy_logical_or', _sig('?' + _INTS + _FLOATS, 2, '?'),
    'out0 = in0 || in1', doc='Elementwise logical OR.')
logical_xor = create_ufunc(
    'cupy_logical_xor', _sig('?' + _INTS + _FLOATS, 2, '?'),
    'out0 = !in0 != !in1', doc='Elementwise logical XOR.')
logical_not = create_ufunc(
    'cupy_logical_not', _sig('?' + _INTS + _FLOATS, 1, '?'),
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
    tuple(('%s->?' % c, 'out0 = false') for c in '?' + _INTS) + _sig(_FLOATS, 1, '?'),
    'out0 = isnan(in0)', doc='Tests elementwise for NaN.')
isinf = create_ufunc(
    'cupy_isinf',
    tuple(('%s->?' % c, 'out0 = false') for c in '?' + _INTS) + _sig(_FLOATS, 1, '?'),
    'out0 = isinf(in0)', doc='Tests elementwise for +/- infinity.')
isfinite = create_ufunc(
    'cupy_isfinite',
    tuple(('%s->?' % c, 'out0 = true') for c in '?' + _INTS) + _sig(_FLOATS, 1, '?'),
    'out0 = isfinite(in0)', doc='Tests elementwise for finiteness.')
signbit = create_ufunc(
    'cupy_signbit', _sig(_FLOATS, 1, '?'),
    'out0 = signbit(in0)', doc='Tests elementwise whether the sign bit is set.')

_where_ufunc = create_ufunc(
    'cupy_where',
    tuple('?%s%s->%s' % (c, c, c) for c in '?' + _INTS + _FLOATS),
    'out0 = in0 ? in1 : in2')

_clip = create_ufunc(
    'cupy_clip',
    tuple('%s%s%s->%s' % (c, c, c, c) for c in '?' + _INTS + _FLOATS),
    'out0 = in0 < in1 ? in1 : (in0 > in2 ? in2 : in0)')
