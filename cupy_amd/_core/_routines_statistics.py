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
  __device__ min_max_st() : index(-1) {}
  __device__ min_max_st(T v) : value(v), index(0) {}
  __device__ min_max_st(T v, IndexT i) : value(v), index(i) {}
};

template <typename T> __device__ __forceinline__ bool _mm_isnan(T) { return false; }
template <> __device__ __forceinline__ bool _mm_isnan<float>(float x) { return x != x; }
template <> __device__ __forceinline__ bool _mm_isnan<double>(double x) { return x != x; }
template <> __device__ __forceinline__ bool _mm_isnan<float16>(float16 x) { return x.isnan(); }

// kMax: larger values win, otherwise smaller ones; kNan: NaN wins over numbers.
// `index == -1` marks "no element yet".
template <bool kMax, bool kNan, typename T>
__device__ __forceinline__ min_max_st<T> _mm_pick(
    const min_max_st<T>& a, const min_max_st<T>& b) {
  if (a.index == -1) return b;
  if (b.index == -1) return a;
  bool a_first;   // a strictly better than b
  bool tie;
  if (kNan) {
    const bool an = _mm_isnan(a.value), bn = _mm_isnan(b.value);
    if (an | bn) {
      a_first = an & !bn;
      tie = an & bn;
    } else {
      a_first = kMax ? (a.value > b.value) : (a.value < b.value);
      tie = a.value == b.value;
    }
  } else {
    a_first = kMax ? (a.value > b.value) : (a.value < b.value);
    tie = a.value == b.value;
  }
  if (tie) return (a.index <= b.index) ? a : b;
  return a_first ? a : b;
}

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

_arg_sigs = tuple('{}->{}'.format(d, r) for r in 'qlihb' for d in '?bBhHiIlLqQ')

_argmin = create_reduction_func(
    'cupy_argmin',
    _arg_sigs + (
        ('e->q', (None, 'my_argmin_float(a, b)', None, None)),
        ('f->q', (None, 'my_argmin_float(a, b)', None, None)),
        ('d->q', (None, 'my_argmin_float(a, b)', None, None))),
    ('min_max_st<type_in0_raw>(in0, _J)', 'my_argmin(a, b)', 'out0 = a.index',
     'min_max_st<type_in0_raw>'),
    None, _min_max_preamble, sort_reduce_axis=False)

_argmax = create_reduction_func(
    'cupy_argmax',
    _arg_sigs + (
        ('e->q', (None, 'my_argmax_float(a, b)', None, None)),
        ('f->q', (None, 'my_argmax_float(a, b)', None, None)),
        ('d->q', (None, 'my_argmax_float(a, b)', None, None))),
    ('min_max_st<type_in0_raw>(in0, _J)', 'my_argmax(a, b)', 'out0 = a.index',
     'min_max_st<type_in0_raw>'),
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
