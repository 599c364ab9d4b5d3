"""min / max / argmin / argmax / mean reductions (reference:
cupy/_core/_routines_statistics.pyx:27-125 dispatch, :190-353 definitions).

The combiner carries ``(value, index)``.  It is written to be commutative and
associative for every input, NaNs included, so the result does not depend on
the shape of the reduction tree: a better value wins, NaN beats every number,
and among equals (or among NaNs) the smaller index wins -- which is NumPy's
first-occurrence rule.
"""
from cupy_amd._core import _fusion_thread_local
from cupy_amd._core._reduction import create_reduction_func

_min_max_preamble = '''
template <typename T>
struct min_max_st {
  T value;
  IndexT index;
  __device__ min_max_st() : value(), index(-1) {}
  __device__ min_max_st(T v) : value(v), index(0) {}
  __device__ min_max_st(T v, IndexT i) : value(v), index(i) {}
};

template <typename T> __device__ __forceinline__ bool _mm_isnan(T) { return false; }
template <> __device__ __forceinline__ bool _mm_isnan<float>(float x) { return x != x; }
template <> __device__ __forceinline__ bool _mm_isnan<double>(double x) { return x != x; }
template <> __device__ __forceinline__ bool _mm_isnan<float16>(float16 x) { return x.isnan(); }

// kMax: larger values win, otherwise smaller ones; kNan: NaN wins over numbers.
// `index == -1` marks "no element yet".  Written with selects on the members
// (no control flow, operands by value) so that everything stays in registers.
template <bool kMax, bool kNan, typename T>
__device__ __forceinline__ min_max_st<T> _mm_pick(min_max_st<T> a, min_max_st<T> b) {
  const bool a_valid = a.index != -1;
  const bool b_valid = b.index != -1;
  bool a_better = kMax ? (a.value > b.value) : (a.value < b.value);
  bool tie = a.value == b.value;
  if (kNan) {
    const bool an = _mm_isnan(a.value), bn = _mm_isnan(b.value);
    a_better = (an & !bn) | (!an & !bn & a_better);
    tie = tie | (an & bn);
  }
  bool take_a = a_better | (tie & (a.index <= b.index));
  take_a = (take_a & a_valid) | !b_valid;
  min_max_st<T> r;
  r.value = take_a ? a.value : b.value;
  r.index = take_a ? a.index : b.index;
  return r;
}

// ---- argmin / argmax state ---------------------------------------------------
// For element types of at most 32 bits (and 32-bit reduce indices) value and
// index are packed into one signed 64-bit key: the high word is an
// order-preserving image of the value (NaN mapped to the winning extreme), the
// low word orders equal values by index so that the smallest index wins.  The
// whole combine is then a 64-bit max or min.  Wider types use (value, index).
template <typename T> struct _arg_small { static const bool value = false; };
template <> struct _arg_small<bool> { static const bool value = true; };
template <> struct _arg_small<signed char> { static const bool value = true; };
template <> struct _arg_small<unsigned char> { static const bool value = true; };
template <> struct _arg_small<short> { static const bool value = true; };
template <> struct _arg_small<unsigned short> { static const bool value = true; };
template <> struct _arg_small<int> { static const bool value = true; };
template <> struct _arg_small<unsigned int> { static const bool value = true; };
template <> struct _arg_small<float> { static const bool value = true; };
template <> struct _arg_small<float16> { static const bool value = true; };

template <bool kMax> __device__ __forceinline__ int _arg_ord(bool v) { return v ? 1 : 0; }
template <bool kMax> __device__ __forceinline__ int _arg_ord(signed char v) { return v; }
template <bool kMax> __device__ __forceinline__ int _arg_ord(unsigned char v) { return v; }
template <bool kMax> __device__ __forceinline__ int _arg_ord(short v) { return v; }
template <bool kMax> __device__ __forceinline__ int _arg_ord(unsigned short v) { return v; }
template <bool kMax> __device__ __forceinline__ int _arg_ord(int v) { return v; }
template <bool kMax> __device__ __forceinline__ int _arg_ord(unsigned int v) {
  return static_cast<int>(v ^ 0x80000000u);
}
template <bool kMax> __device__ __forceinline__ int _arg_ord(float v) {
  if (v != v) return kMax ? 0x7fffffff : (-0x7fffffff - 1);
  v = v + 0.0f;                                  // -0 and +0 must tie
  const int b = __builtin_bit_cast(int, v);
  return b ^ ((b >> 31) & 0x7fffffff);
}
template <bool kMax> __device__ __forceinline__ int _arg_ord(float16 v) {
  return _arg_ord<kMax>(static_cast<float>(v));
}

template <typename T, bool kMax>
struct arg_key32 {
  long long k;
  __device__ arg_key32() : k(kMax ? (-9223372036854775807LL - 1) : 9223372036854775807LL) {}
  __device__ arg_key32(T v, IndexT i) {
    const unsigned int low = kMax ? static_cast<unsigned int>(0x7fffffff - static_cast<int>(i))
                                  : static_cast<unsigned int>(i);
    k = static_cast<long long>(
        (static_cast<unsigned long long>(static_cast<unsigned int>(_arg_ord<kMax>(v))) << 32) | low);
  }
  __device__ __forceinline__ IndexT index() const {
    const int low = static_cast<int>(static_cast<unsigned int>(k & 0xffffffffLL));
    return kMax ? (0x7fffffff - low) : low;
  }
};
template <typename T, bool kMax>
__device__ __forceinline__ arg_key32<T, kMax> arg_pick(arg_key32<T, kMax> a, arg_key32<T, kMax> b) {
  arg_key32<T, kMax> r;
  r.k = kMax ? (a.k > b.k ? a.k : b.k) : (a.k < b.k ? a.k : b.k);
  return r;
}

template <typename T, bool kMax>
struct arg_wide {
  min_max_st<T> s;
  __device__ arg_wide() {}
  __device__ arg_wide(T v, IndexT i) : s(v, i) {}
  __device__ __forceinline__ IndexT index() const { return s.index; }
};
template <typename T, bool kMax>
__device__ __forceinline__ arg_wide<T, kMax> arg_pick(arg_wide<T, kMax> a, arg_wide<T, kMax> b) {
  arg_wide<T, kMax> r;
  r.s = _mm_pick<kMax, true>(a.s, b.s);
  return r;
}

template <typename T, bool kMax>
struct arg_state {
  typedef typename cupy::conditional<(_arg_small<T>::value && sizeof(IndexT) == 4),
                                     arg_key32<T, kMax>, arg_wide<T, kMax> >::type type;
};

template <typename T> __device__ __forceinline__ min_max_st<T> my_min(
    const min_max_st<T>& a, const min_max_st<T>& b) { return _mm_pick<false, false>(a, b); }
template <typename T> __device__ __forceinline__ min_max_st<T> my_min_float(
    const min_max_st<T>& a, const min_max_st<T>& b) { return _mm_pick<false, true>(a, b); }
template <typename T> __device__ __forceinline__ min_max_st<T> my_max(
    const min_max_st<T>& a, const min_max_st<T>& b) { return _mm_pick<true, false>(a, b); }
template <typename T> __device__ __forceinline__ min_max_st<T> my_max_float(
    const min_max_st<T>& a, const min_max_st<T>& b) { return _mm_pick<true, true>(a, b); }
template <typename T> __device__ __forceinline__ min_max_st<T> my_argmin(
    const min_max_st<T>& a, const min_max_st<T>& b) { return _mm_pick<false, false>(a, b); }
template <typename T> __device__ __forceinline__ min_max_st<T> my_argmin_float(
    const min_max_st<T>& a, const min_max_st<T>& b) { return _mm_pick<false, true>(a, b); }
template <typename T> __device__ __forceinline__ min_max_st<T> my_argmax(
    const min_max_st<T>& a, const min_max_st<T>& b) { return _mm_pick<true, false>(a, b); }
template <typename T> __device__ __forceinline__ min_max_st<T> my_argmax_float(
    const min_max_st<T>& a, const min_max_st<T>& b) { return _mm_pick<true, true>(a, b); }
'''

_int_sigs = ('?->?', 'b->b', 'B->B', 'h->h', 'H->H', 'i->i', 'I->I', 'l->l',
             'L->L', 'q->q', 'Q->Q')

_amin = create_reduction_func(
    'cupy_min',
    _int_sigs + (
        ('e->e', (None, 'my_min_float(a, b)', None, None)),
        ('f->f', (None, 'my_min_float(a, b)', None, None)),
        ('d->d', (None, 'my_min_float(a, b)', None, None))),
    ('min_max_st<type_in0_raw>(in0)', 'my_min(a, b)', 'out0 = a.value',
     'min_max_st<type_in0_raw>'),
    None, _min_max_preamble)

_amax = create_reduction_func(
    'cupy_max',
    _int_sigs + (
        ('e->e', (None, 'my_max_float(a, b)', None, None)),
        ('f->f', (None, 'my_max_float(a, b)', None, None)),
        ('d->d', (None, 'my_max_float(a, b)', None, None))),
    ('min_max_st<type_in0_raw>(in0)', 'my_max(a, b)', 'out0 = a.value',
     'min_max_st<type_in0_raw>'),
    None, _min_max_preamble)

_arg_sigs = tuple('{}->{}'.format(d, r) for r in 'qlihb' for d in '?bBhHiIlLqQ') + (
    'e->q', 'f->q', 'd->q')

_argmin = create_reduction_func(
    'cupy_argmin', _arg_sigs,
    ('arg_state<type_in0_raw, false>::type(in0, _J)', 'arg_pick(a, b)',
     'out0 = a.index()', 'arg_state<type_in0_raw, false>::type'),
    None, _min_max_preamble, sort_reduce_axis=False)

_argmax = create_reduction_func(
    'cupy_argmax', _arg_sigs,
    ('arg_state<type_in0_raw, true>::type(in0, _J)', 'arg_pick(a, b)',
     'out0 = a.index()', 'arg_state<type_in0_raw, true>::type'),
    None, _min_max_preamble, sort_reduce_axis=False)


def _ndarray_max(self, axis, out, dtype, keepdims):
    return _amax(self, axis=axis, out=out, dtype=dtype, keepdims=keepdims)


def _ndarray_min(self, axis, out, dtype, keepdims):
    return _amin(self, axis=axis, out=out, dtype=dtype, keepdims=keepdims)


def _ndarray_argmax(self, axis, out, dtype, keepdims):
    return _argmax(self, axis=axis, out=out, dtype=dtype, keepdims=keepdims)


def _ndarray_argmin(self, axis, out, dtype, keepdims):
    return _argmin(self, axis=axis, out=out, dtype=dtype, keepdims=keepdims)


def _ndarray_mean(self, axis, dtype, out, keepdims):
    from cupy_amd._core import _ufuncs
    import numpy
    if dtype is None:
        dtype = self.dtype if self.dtype.kind == 'f' else numpy.dtype('float64')
    total = self.sum(axis=axis, dtype=dtype if numpy.dtype(dtype).kind == 'f'
                     else None, keepdims=keepdims)
    count = max(self.size // max(total.size, 1), 1) if self.size else 0
    if count == 0:
        count = float('nan')
    res = _ufuncs.true_divide(total, total.dtype.type(count) if count == count
                              else float('nan'))
    if out is not None:
        _ufuncs.elementwise_copy(res, out, casting='unsafe')
        return out
    return res.astype(dtype, copy=False)


def amax(a, axis=None, out=None, keepdims=False):
    """Maximum along the given axes; NaNs propagate.

    .. seealso:: :func:`numpy.amax`
    """
    if _fusion_thread_local.is_fusing():
        if keepdims:
            raise NotImplementedError(
                'cupy.amax does not support `keepdims` in fusion yet.')
        return _fusion_thread_local.call_reduction(_amax, a, axis=axis, out=out)
    return a.max(axis=axis, out=out, keepdims=keepdims)


def amin(a, axis=None, out=None, keepdims=False):
    """Minimum along the given axes; NaNs propagate.

    .. seealso:: :func:`numpy.amin`
    """
    if _fusion_thread_local.is_fusing():
        if keepdims:
            raise NotImplementedError(
                'cupy.amin does not support `keepdims` in fusion yet.')
        return _fusion_thread_local.call_reduction(_amin, a, axis=axis, out=out)
    return a.min(axis=axis, out=out, keepdims=keepdims)


def argmax(a, axis=None, dtype=None, out=None, keepdims=False):
    """Index of the (first) maximum along an axis.

    .. seealso:: :func:`numpy.argmax`
    """
    return a.argmax(axis=axis, dtype=dtype, out=out, keepdims=keepdims)


def argmin(a, axis=None, dtype=None, out=None, keepdims=False):
    """Index of the (first) minimum along an axis.

    .. seealso:: :func:`numpy.argmin`
    """
    return a.argmin(axis=axis, dtype=dtype, out=out, keepdims=keepdims)
