"""min / max / argmin / argmax / mean reductions (reference:
cupy/_core/_routines_statistics.pyx:27-125 dispatch, :190-353 definitions).

The combiner carries ``(value, index)``.  It is written to be commutative and
associative for every input, NaNs included, so the result does not depend on
the shape of the reduction tree: a better value wins, NaN beats every number,
and among equals (or among NaNs) the smaller index wins -- which is NumPy's
first-occurrence rule.
"""
from cupy_amd._core import _fusion_thread_local
from cupy_amd._core import internal
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
template <> __device__ __forceinline__ bool _mm_isnan<complex<float> >(complex<float> x) {
  return (x.re != x.re) | (x.im != x.im);
}
template <> __device__ __forceinline__ bool _mm_isnan<complex<double> >(complex<double> x) {
  return (x.re != x.re) | (x.im != x.im);
}

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

// NaN-ignoring variant: a number beats NaN; NaN survives only among NaNs.
template <bool kMax, typename T>
__device__ __forceinline__ min_max_st<T> _mm_pick_nanlast(min_max_st<T> a, min_max_st<T> b) {
  const bool a_valid = a.index != -1;
  const bool b_valid = b.index != -1;
  const bool an = _mm_isnan(a.value), bn = _mm_isnan(b.value);
  const bool cmp = kMax ? (a.value > b.value) : (a.value < b.value);
  const bool a_better = (!an & bn) | (!an & !bn & cmp);
  const bool tie = (a.value == b.value) | (an & bn);
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

// All-reduces of packed keys over lanes go word by word: first the high words
// (a 32-bit max or min, whose lane exchange folds into the instruction itself),
// then the low words of the lanes that hold the winning high word.  A step
// costs two instructions instead of seven for the 64-bit compare-and-select.
struct _arg_imax { __device__ __forceinline__ int operator()(int a, int b) const { return a > b ? a : b; } };
struct _arg_imin { __device__ __forceinline__ int operator()(int a, int b) const { return a < b ? a : b; } };
struct _arg_umax { __device__ __forceinline__ unsigned int operator()(unsigned int a, unsigned int b) const { return a > b ? a : b; } };
struct _arg_umin { __device__ __forceinline__ unsigned int operator()(unsigned int a, unsigned int b) const { return a < b ? a : b; } };
template <bool kMax> struct _arg_word_ops {
  typedef typename cupy::conditional<kMax, _arg_imax, _arg_imin>::type high;
  typedef typename cupy::conditional<kMax, _arg_umax, _arg_umin>::type low;
};
namespace cupy {
template <int kFirst, int kTop, bool kKeepLow, typename T, bool kMax, int kBatch>
__device__ __forceinline__ void _arg_key_allreduce(arg_key32<T, kMax> (&s)[kBatch]) {
  int hi[kBatch], best[kBatch];
  unsigned int lo[kBatch];
#pragma unroll
  for (int r = 0; r < kBatch; ++r) {
    hi[r] = static_cast<int>(s[r].k >> 32);
    best[r] = _AllReduce<kFirst, kTop, kKeepLow>::run(hi[r], typename _arg_word_ops<kMax>::high());
  }
#pragma unroll
  for (int r = 0; r < kBatch; ++r) {
    lo[r] = (hi[r] == best[r]) ? static_cast<unsigned int>(s[r].k) : (kMax ? 0u : 0xffffffffu);
    lo[r] = _AllReduce<kFirst, kTop, kKeepLow>::run(lo[r], typename _arg_word_ops<kMax>::low());
    s[r].k = static_cast<long long>(
        (static_cast<unsigned long long>(static_cast<unsigned int>(best[r])) << 32) | lo[r]);
  }
}
template <int kGroup, typename T, bool kMax, typename Op>
__device__ __forceinline__ arg_key32<T, kMax> group_allreduce(arg_key32<T, kMax> v, Op) {
  arg_key32<T, kMax> s[1] = {v};
  _arg_key_allreduce<1, kGroup, false>(s);
  return s[0];
}
template <int kStride, typename T, bool kMax, typename Op>
__device__ __forceinline__ arg_key32<T, kMax> strided_allreduce(arg_key32<T, kMax> v, Op) {
  arg_key32<T, kMax> s[1] = {v};
  _arg_key_allreduce<kStride, 64, true>(s);
  return s[0];
}
template <int kGroup, typename T, bool kMax, int kBatch, typename Op>
__device__ __forceinline__ void batch_allreduce(arg_key32<T, kMax> (&s)[kBatch], Op) {
  _arg_key_allreduce<1, kGroup, false>(s);
}
}  // namespace cupy

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
template <typename T> __device__ __forceinline__ min_max_st<T> my_nanmin(
    const min_max_st<T>& a, const min_max_st<T>& b) { return _mm_pick_nanlast<false>(a, b); }
template <typename T> __device__ __forceinline__ min_max_st<T> my_nanmax(
    const min_max_st<T>& a, const min_max_st<T>& b) { return _mm_pick_nanlast<true>(a, b); }
'''

_int_sigs = ('?->?', 'b->b', 'B->B', 'h->h', 'H->H', 'i->i', 'I->I', 'l->l',
             'L->L', 'q->q', 'Q->Q')

# min / max keep a bare value (arg-reductions need the index beside it): the
# state starts from the type's extreme, which any element replaces, so that
# lanes without elements drop out of the combine.  NaN wins for floats.
_extremum_preamble = '''
template <typename T> struct _mm_is_float { static const bool value = false; };
template <> struct _mm_is_float<float> { static const bool value = true; };
template <> struct _mm_is_float<double> { static const bool value = true; };
template <> struct _mm_is_float<float16> { static const bool value = true; };
template <typename T> struct _mm_limits {
  static __device__ __forceinline__ T get(bool lowest) {
    if (_mm_is_float<T>::value) return lowest ? T(-CUDART_INF_F) : T(CUDART_INF_F);
    if (cupy::is_same<T, bool>::value) return T(!lowest);
    if (T(-1) < T(0)) {
      const unsigned long long top = 1ull << (8 * sizeof(T) - 1);
      return static_cast<T>(lowest ? top : ~top);
    }
    return lowest ? T(0) : static_cast<T>(~0ull);
  }
};
// complex numbers are ordered by real part, then by imaginary part
template <typename U> struct _mm_limits<complex<U> > {
  static __device__ __forceinline__ complex<U> get(bool lowest) {
    const U inf = lowest ? U(-CUDART_INF_F) : U(CUDART_INF_F);
    return complex<U>(inf, inf);
  }
};
template <typename T, bool kMax>
struct mm_val {
  T v;
  __device__ __forceinline__ mm_val() : v(_mm_limits<T>::get(kMax)) {}
  __device__ __forceinline__ explicit mm_val(T x) : v(x) {}
};
template <bool kNan, typename T, bool kMax>
__device__ __forceinline__ mm_val<T, kMax> mm_pick(const mm_val<T, kMax>& a,
                                                   const mm_val<T, kMax>& b) {
  bool take_b = kMax ? (b.v > a.v) : (b.v < a.v);
  if (kNan) {
    // NaN wins and stays.  For real floating types "b beats a, or b is NaN"
    // is one comparison: the negation of an ordered one is true for NaN
    // (and for NaN in a, which the second test takes out again).
    if (_mm_is_float<T>::value) take_b = kMax ? !(b.v <= a.v) : !(b.v >= a.v);
    else take_b = take_b | (b.v != b.v);
    take_b = take_b & !(a.v != a.v);
  }
  mm_val<T, kMax> r;
  r.v = take_b ? b.v : a.v;
  return r;
}
'''

_amin = create_reduction_func(
    'cupy_min',
    _int_sigs + (
        ('e->e', (None, 'mm_pick<true>(a, b)', None, None)),
        ('f->f', (None, 'mm_pick<true>(a, b)', None, None)),
        ('d->d', (None, 'mm_pick<true>(a, b)', None, None)),
        ('F->F', (None, 'mm_pick<true>(a, b)', None, None)),
        ('D->D', (None, 'mm_pick<true>(a, b)', None, None))),
    ('mm_val<type_in0_raw, false>(in0)', 'mm_pick<false>(a, b)', 'out0 = a.v',
     'mm_val<type_in0_raw, false>'),
    None, _extremum_preamble)

_amax = create_reduction_func(
    'cupy_max',
    _int_sigs + (
        ('e->e', (None, 'mm_pick<true>(a, b)', None, None)),
        ('f->f', (None, 'mm_pick<true>(a, b)', None, None)),
        ('d->d', (None, 'mm_pick<true>(a, b)', None, None)),
        ('F->F', (None, 'mm_pick<true>(a, b)', None, None)),
        ('D->D', (None, 'mm_pick<true>(a, b)', None, None))),
    ('mm_val<type_in0_raw, true>(in0)', 'mm_pick<false>(a, b)', 'out0 = a.v',
     'mm_val<type_in0_raw, true>'),
    None, _extremum_preamble)

_arg_sigs = tuple('{}->{}'.format(d, r) for r in 'qlihb' for d in '?bBhHiIlLqQ') + (
    'e->q', 'f->q', 'd->q', 'F->q', 'D->q')

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


_float_sigs = ('e->e', 'f->f', 'd->d', 'F->F', 'D->D')

# NaNs are skipped; a slice of NaNs only gives NaN
# (cupy/_core/_routines_statistics.pyx:307-326)
nanmin = create_reduction_func(
    'cupy_nanmin', _int_sigs + _float_sigs,
    ('min_max_st<type_in0_raw>(in0)', 'my_nanmin(a, b)', 'out0 = a.value',
     'min_max_st<type_in0_raw>'),
    None, _min_max_preamble)

nanmax = create_reduction_func(
    'cupy_nanmax', _int_sigs + _float_sigs,
    ('min_max_st<type_in0_raw>(in0)', 'my_nanmax(a, b)', 'out0 = a.value',
     'min_max_st<type_in0_raw>'),
    None, _min_max_preamble)

# index -1 = "no element": NaNs never take part; a slice of NaNs only gives -1
# (:365-391)
_nanarg_sigs = tuple('%s->q' % c for c in '?BhHiIlLqQefdFD')

_nanargmin_func = create_reduction_func(
    'cupy_nanargmin', _nanarg_sigs,
    ('min_max_st<type_in0_raw>(in0, _mm_isnan(in0) ? (IndexT)-1 : (IndexT)_J)',
     'my_argmin(a, b)', 'out0 = a.index', 'min_max_st<type_in0_raw>'),
    None, _min_max_preamble, sort_reduce_axis=False)

_nanargmax_func = create_reduction_func(
    'cupy_nanargmax', _nanarg_sigs,
    ('min_max_st<type_in0_raw>(in0, _mm_isnan(in0) ? (IndexT)-1 : (IndexT)_J)',
     'my_argmax(a, b)', 'out0 = a.index', 'min_max_st<type_in0_raw>'),
    None, _min_max_preamble, sort_reduce_axis=False)

# mean = sum / count, the count taken from the problem's size (:647-666)
_mean_sigs = ('?->d', 'B->d', 'h->d', 'H->d', 'i->d', 'I->d', 'l->d', 'L->d',
              'q->d', 'Q->d', ('e->e', (None, None, None, 'float')), 'f->f', 'd->d',
              'F->F', 'D->D')

_mean_core = create_reduction_func(
    'cupy_mean', _mean_sigs,
    ('in0', 'a + b',
     'out0 = a / _type_reduce(_in_ind.size() / _out_ind.size())', None))

_mean_core_empty = create_reduction_func(
    'cupy_mean_empty', _mean_sigs,
    ('in0', 'a + b',
     'out0 = a / _type_reduce(_in_ind.size() / _out_ind.size())', None), 0)

_nanmean_preamble = '''
template <typename T>
struct nanmean_st {
  typedef long long ll;
  T value;
  ll count;
  __device__ nanmean_st() : value(0), count(0) {}
  __device__ nanmean_st(T v) : value(v != v ? T(0) : v), count(v != v ? 0 : 1) {}
  __device__ nanmean_st(T v, ll c) : value(v), count(c) {}
};
template <typename T>
__device__ nanmean_st<T> my_nanmean(const nanmean_st<T>& a, const nanmean_st<T>& b) {
  return nanmean_st<T>(a.value + b.value, a.count + b.count);
}
'''

_nanmean_func = create_reduction_func(
    'cupy_nanmean',
    (('e->e', ('nanmean_st<float>(static_cast<float>(in0))', None,
               'out0 = a.value / float(a.count)', 'nanmean_st<float>')),
     'f->f', 'd->d',
     # (the input may be real when ``dtype=`` asked for a complex mean)
     ('F->F', ('nanmean_st<type_out0_raw>(type_out0_raw(in0))', None,
               'out0 = a.value / float(a.count)', None)),
     ('D->D', ('nanmean_st<type_out0_raw>(type_out0_raw(in0))', None,
               'out0 = a.value / double(a.count)', None))),
    ('nanmean_st<type_out0_raw>(in0)', 'my_nanmean(a, b)',
     'out0 = a.value / type_out0_raw(a.count)', 'nanmean_st<type_out0_raw>'),
    None, _nanmean_preamble)

_count_non_nan = create_reduction_func(
    'cupy_count_non_nan', ('e->q', 'f->q', 'd->q', 'F->q', 'D->q'),
    ('(in0 == in0) ? 1 : 0', 'a + b', 'out0 = a', None), 0)


def _ndarray_mean(self, axis, dtype, out, keepdims):
    if self.size == 0:
        # NaN (and no error): numpy/numpy#13582
        return _mean_core_empty(self, axis, dtype, out, keepdims)
    return _mean_core(self, axis, dtype, out, keepdims)


def _ndarray_ptp(self, axis, out, keepdims):
    result = _amax(self, axis=axis, out=out, keepdims=keepdims)
    result -= _amin(self, axis=axis, out=None, keepdims=keepdims)
    return result


_norm_preamble = '''
template <typename T> __device__ T my_norm(T x) { return x * x; }
__device__ float my_norm(const complex<float>& x) { return norm(x); }
__device__ double my_norm(const complex<double>& x) { return norm(x); }
'''

_var_cores = {}


def _var_core(out_type):
    """ReductionKernel ``out = alpha * sum((x - mean)**2)`` with ``out_type``
    output (``None``: the type of the given output array); built on first use
    (cupy/_core/_routines_statistics.pyx:611-643)."""
    from cupy_amd._core._reduction import ReductionKernel
    ker = _var_cores.get(out_type)
    if ker is None:
        if out_type is None:
            ker = ReductionKernel(
                'S x, T mean, U alpha', 'U out', 'my_norm(x - mean)', 'a + b',
                'out = alpha * a', '0', 'cupy_var_core_out', preamble=_norm_preamble)
        else:
            alpha_t = 'float64' if out_type == 'float64' else 'float32'
            ker = ReductionKernel(
                'S x, T mean, %s alpha' % alpha_t, '%s out' % out_type,
                'my_norm(x - mean)', 'a + b', 'out = alpha * a', '0',
                'cupy_var_core_' + out_type, preamble=_norm_preamble)
        _var_cores[out_type] = ker
    return ker


_var_onepass_preamble = '''
// One-pass variance that no input can make cancel.  State of a set of values:
// their number n, a pivot k (the first value that joined), and -- of the values
// counted from the pivot, y = x - k -- the mean m and the sum of squared
// deviations from that mean, M2.
//  * A value joins the set by Welford's update, d = y - m, m += d / n,
//    M2 += d * (y - m): the mean the deviations are taken from follows the data
//    with every value, so nothing large is ever subtracted from something
//    large.  Counting from the pivot keeps m small next to the data (data at
//    3e5 with a spread of 1 has |m| of order 1), so that rounding m costs
//    nothing; a pivot far from the rest of the set is a member of the set whose
//    distance is part of the true variance.  1 / n is the hardware's
//    reciprocal (one more Newton step for double): the update needs a mean
//    that is close, not one that is correctly rounded, because what m misses
//    enters the result squared.
//  * Two sets merge by M2 = M2a + M2b + delta^2 na nb / n (Chan, Golub,
//    LeVeque 1983) with delta, the difference of the means, formed as
//    (kb - ka) + (mb - ma).
// The reference takes two passes instead (mean, then squared deviations:
// cupy/_core/_routines_statistics.pyx:553-598).
__device__ __forceinline__ float var_rcp(float n) { return __builtin_amdgcn_rcpf(n); }
__device__ __forceinline__ double var_rcp(double n) {
  const double r = __builtin_amdgcn_rcp(n);
  return r * (2.0 - n * r);
}
// The count is kept in T: exact far beyond what one thread folds (2^24 values
// in float), and where it saturates the update degrades into a moving average
// with a very long window instead of overflowing; merged counts only serve as
// weights.
template <typename T>
struct var_st {
  T n, k, m, m2;
  __device__ __forceinline__ var_st() : n(0), k(0), m(0), m2(0) {}
  __device__ __forceinline__ explicit var_st(T x) : n(1), k(x), m(0), m2(0) {}
};
template <typename T>
__device__ __forceinline__ var_st<T> operator+(const var_st<T>& a, const var_st<T>& b) {
  var_st<T> r;
  if (b.n == 1) {                       // a value joins a set (also an empty one)
    r.n = a.n + 1;
    r.k = a.n == 0 ? b.k : a.k;
    const T y = b.k - r.k;
    const T d = y - a.m;
    r.m = a.m + d * var_rcp(r.n);
    r.m2 = a.m2 + d * (y - r.m);
    return r;
  }
  if (a.n == 0) return b;
  if (b.n == 0) return a;
  const T delta = (b.k - a.k) + (b.m - a.m);
  r.n = a.n + b.n;
  const T w = b.n / r.n;
  r.k = a.k;
  r.m = a.m + delta * w;
  r.m2 = a.m2 + b.m2 + delta * delta * (a.n * w);
  return r;
}
template <typename T>
__device__ __forceinline__ T var_finish(const var_st<T>& a, T alpha) {
  return alpha * (a.m2 < 0 ? T(0) : a.m2);          // NaN stays NaN
}
'''

_var_onepass_cores = {}
_FLOAT_NAMES = {'e': 'float16', 'f': 'float32', 'd': 'float64'}


def _var_onepass(out_name):
    """ReductionKernel of the one-pass variance, accumulating in double for a
    float64 result and in float otherwise (as the sums of those types do)."""
    from cupy_amd._core._reduction import ReductionKernel
    ker = _var_onepass_cores.get(out_name)
    if ker is None:
        work, scalar_t = ('double', 'float64') if out_name == 'float64' else ('float', 'float32')
        ker = ReductionKernel(
            'S x, %s alpha' % scalar_t, '%s out' % out_name,
            'var_st<%s>(static_cast<%s>(x))' % (work, work),
            'a + b', 'out = var_finish<%s>(a, alpha)' % work, 'var_st<%s>()' % work,
            'cupy_var_%s' % out_name, reduce_type='var_st<%s>' % work,
            preamble=_var_onepass_preamble)
        _var_onepass_cores[out_name] = ker
    return ker


def _ndarray_var(a, axis=None, dtype=None, out=None, ddof=0, keepdims=False):
    """Variance.  Real inputs take one pass over the data (``var_st`` above;
    the reference reads them twice: the mean first, then the squared
    deviations, cupy/_core/_routines_statistics.pyx:553-598); complex inputs
    keep that two-pass form."""
    import numpy
    if axis is None:
        axis = tuple(range(a.ndim))
    if not isinstance(axis, tuple):
        axis = (axis,)
    if dtype is None:
        if a.dtype.kind in 'biu':
            dtype_mean = dtype_out = numpy.dtype('float64')
        else:
            dtype_mean = dtype_out = a.dtype
            if a.dtype.kind == 'c':
                # |x - mean|**2 is real
                dtype_out = numpy.dtype(a.dtype.char.lower())
    else:
        dtype_mean = a.dtype
        dtype_out = numpy.dtype(dtype)
    items = 1
    for ax in axis:
        items *= a.shape[ax]
    div = max(items - ddof, 0)
    alpha = 1. / div if div != 0 else float('nan')
    if (a.dtype.kind in 'biuf' and dtype_out.kind == 'f' and dtype_out.itemsize <= 8
            and items > 0 and (out is None or out.dtype == dtype_out)):
        axis = tuple(internal._normalize_axis_index(ax, a.ndim) for ax in axis)
        args = (a, alpha) + (() if out is None else (out,))
        # (numpy's dtype.name is computed on every access)
        out_name = _FLOAT_NAMES[dtype_out.char]
        return _var_onepass(out_name)(*args, axis=axis, keepdims=keepdims)
    arrmean = a.mean(axis=axis, dtype=dtype_mean, out=None, keepdims=True)
    if out is None:
        name = dtype_out.name if dtype_out.name in ('float16', 'float32') else 'float64'
        return _var_core(name)(a, arrmean, alpha, axis=axis, keepdims=keepdims)
    out = _var_core(None)(a, arrmean, alpha, out, axis=axis, keepdims=keepdims)
    return out.astype(dtype_out, copy=False)


def _ndarray_std(a, axis=None, dtype=None, out=None, ddof=0, keepdims=False):
    from cupy_amd._core import _ufuncs
    ret = _ndarray_var(a, axis=axis, dtype=dtype, out=None, ddof=ddof, keepdims=keepdims)
    return _ufuncs.sqrt(ret, dtype=dtype, out=out)


_nanvar_preamble = '''
template <typename S, typename T>
__device__ T nanvar_impl(S x, T mean, long long alpha) {
  return ((x != x) ? T(0) : T((x - mean) * (x - mean))) / alpha;
}
template <typename S, typename T>
__device__ T nanvar_impl(complex<S> x, complex<T> mean, long long alpha) {
  return ((x != x) ? T(0) : T(norm(x - mean))) / alpha;
}
'''

_nanvar_cores = {}


def _nanvar(a, axis, dtype, out, ddof, keepdims):
    """Variance ignoring NaNs (cupy/_core/_routines_statistics.pyx:699-760)."""
    from cupy_amd._core._reduction import ReductionKernel
    from cupy_amd._core import _routines_math
    if not _nanvar_cores:
        _nanvar_cores['new'] = ReductionKernel(
            'S x, T sum, int64 _count, int64 ddof', 'S out',
            'nanvar_impl(x, sum / _count, max(_count - ddof, 0LL))',
            'a + b', 'out = a', '0', '_nanvar_core', preamble=_nanvar_preamble)
        _nanvar_cores['out'] = ReductionKernel(
            'S x, T sum, int64 _count, int64 ddof', 'U out',
            'nanvar_impl(x, sum / _count, max(_count - ddof, 0LL))',
            'a + b', 'out = a', '0', '_nanvar_core', preamble=_nanvar_preamble)
    count = _count_non_nan(a, axis=axis, keepdims=True)
    arrsum = _routines_math.nansum(a, axis=axis, dtype=dtype, out=None, keepdims=True)
    if a.dtype.kind == 'c':
        # the squared modulus of the deviations: a real result
        # (cupy/_core/_routines_statistics.pyx:751-762, 790-800)
        real = 'float32' if a.dtype.itemsize == 8 else 'float64'
        key = 'complex:' + real
        if key not in _nanvar_cores:
            ctype = 'float' if real == 'float32' else 'double'
            _nanvar_cores[key] = ReductionKernel(
                '%s x, %s sum, int64 _count, int64 ddof' % (a.dtype.name, a.dtype.name),
                '%s out' % real,
                'nanvar_impl(x, sum / static_cast<%s>(_count), max(_count - ddof, 0LL))' % ctype,
                'a + b', 'out = a', '0', '_nanvar_core_' + a.dtype.name, preamble=_nanvar_preamble)
        var = _nanvar_cores[key](a, arrsum.astype(a.dtype, copy=False), count, ddof,
                                 axis=axis, keepdims=keepdims)
        if out is None:
            return var
        from cupy_amd._core._ufuncs import elementwise_copy
        elementwise_copy(var, out)
        return out
    if out is None:
        return _nanvar_cores['new'](a, arrsum, count, ddof, axis=axis, keepdims=keepdims)
    _nanvar_cores['out'](a, arrsum, count, ddof, out, axis=axis, keepdims=keepdims)
    return out


def _nanstd(a, axis, dtype, out, ddof, keepdims):
    from cupy_amd._core import _ufuncs
    var = _nanvar(a, axis, dtype, None, ddof, keepdims)
    return _ufuncs.sqrt(var, dtype=dtype, out=out)


def mean(a, axis=None, dtype=None, out=None, keepdims=False):
    """Arithmetic mean along the given axes.

    .. seealso:: :func:`numpy.mean`
    """
    return a.mean(axis=axis, dtype=dtype, out=out, keepdims=keepdims)


def var(a, axis=None, dtype=None, out=None, ddof=0, keepdims=False):
    """Variance along the given axes.

    .. seealso:: :func:`numpy.var`
    """
    return a.var(axis=axis, dtype=dtype, out=out, ddof=ddof, keepdims=keepdims)


def std(a, axis=None, dtype=None, out=None, ddof=0, keepdims=False):
    """Standard deviation along the given axes.

    .. seealso:: :func:`numpy.std`
    """
    return a.std(axis=axis, dtype=dtype, out=out, ddof=ddof, keepdims=keepdims)


def ptp(a, axis=None, out=None, keepdims=False):
    """Range (maximum - minimum) along the given axes.

    .. seealso:: :func:`numpy.ptp`
    """
    return _ndarray_ptp(a, axis, out, keepdims)


def nanmean(a, axis=None, dtype=None, out=None, keepdims=False):
    """Mean ignoring NaNs.

    .. seealso:: :func:`numpy.nanmean`
    """
    if a.dtype.kind in 'biu':
        return a.mean(axis=axis, dtype=dtype, out=out, keepdims=keepdims)
    return _nanmean_func(a, axis=axis, dtype=dtype, out=out, keepdims=keepdims)


def nanvar(a, axis=None, dtype=None, out=None, ddof=0, keepdims=False):
    """Variance ignoring NaNs.

    .. seealso:: :func:`numpy.nanvar`
    """
    if a.dtype.kind in 'biu':
        return a.var(axis=axis, dtype=dtype, out=out, ddof=ddof, keepdims=keepdims)
    return _nanvar(a, axis, dtype, out, ddof, keepdims)


def nanstd(a, axis=None, dtype=None, out=None, ddof=0, keepdims=False):
    """Standard deviation ignoring NaNs.

    .. seealso:: :func:`numpy.nanstd`
    """
    if a.dtype.kind in 'biu':
        return a.std(axis=axis, dtype=dtype, out=out, ddof=ddof, keepdims=keepdims)
    return _nanstd(a, axis, dtype, out, ddof, keepdims)


def nanargmax(a, axis=None, dtype=None, out=None, keepdims=False):
    """Index of the maximum ignoring NaNs (-1 where a slice holds only NaNs).

    .. seealso:: :func:`numpy.nanargmax`
    """
    if a.dtype.kind in 'biu':
        return a.argmax(axis=axis, dtype=dtype, out=out, keepdims=keepdims)
    return _nanargmax_func(a, axis=axis, out=out, dtype=dtype, keepdims=keepdims)


def nanargmin(a, axis=None, dtype=None, out=None, keepdims=False):
    """Index of the minimum ignoring NaNs (-1 where a slice holds only NaNs).

    .. seealso:: :func:`numpy.nanargmin`
    """
    if a.dtype.kind in 'biu':
        return a.argmin(axis=axis, dtype=dtype, out=out, keepdims=keepdims)
    return _nanargmin_func(a, axis=axis, out=out, dtype=dtype, keepdims=keepdims)


def amax(a, axis=None, out=None, keepdims=False):
    """Maximum along the given axes; NaNs propagate.

    .. seealso:: :func:`numpy.amax`
    """
    if _fusion_thread_local.is_fusing():
        if keepdims and not _fusion_thread_local.records_keepdims():
            raise NotImplementedError(
                'cupy.amax does not support `keepdims` in fusion yet.')
        return _fusion_thread_local.call_reduction(_amax, a, axis=axis, out=out, keepdims=keepdims)
    return a.max(axis=axis, out=out, keepdims=keepdims)


def amin(a, axis=None, out=None, keepdims=False):
    """Minimum along the given axes; NaNs propagate.

    .. seealso:: :func:`numpy.amin`
    """
    if _fusion_thread_local.is_fusing():
        if keepdims and not _fusion_thread_local.records_keepdims():
            raise NotImplementedError(
                'cupy.amin does not support `keepdims` in fusion yet.')
        return _fusion_thread_local.call_reduction(_amin, a, axis=axis, out=out, keepdims=keepdims)
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
