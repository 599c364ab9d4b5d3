"""sum / prod reductions (reference: cupy/_core/_routines_math.pyx:109-157
dispatch, :777-876 loop tables)."""
from cupy_amd._core import _fusion_thread_local
from cupy_amd._core._reduction import create_reduction_func

# NumPy's result types: bool and signed ints widen to int64, unsigned to uint64,
# float16 accumulates in float.
_sumprod_types = (
    '?->l', 'b->l', 'B->L', 'h->l', 'H->L', 'i->l', 'I->L', 'l->l', 'L->L',
    'q->q', 'Q->Q',
    ('e->e', (None, None, None, 'float')),
    'f->f', 'd->d', 'F->F', 'D->D')

_keep_types = (
    '?->?', 'b->b', 'B->B', 'h->h', 'H->H', 'i->i', 'I->I', 'l->l', 'L->L',
    'q->q', 'Q->Q',
    ('e->e', (None, None, None, 'float')),
    'f->f', 'd->d', 'F->F', 'D->D')

_sum_auto_dtype = create_reduction_func(
    'cupy_sum', _sumprod_types,
    ('in0', 'a + b', 'out0 = type_out0_raw(a)', None), 0)

_sum_keep_dtype = create_reduction_func(
    'cupy_sum_with_dtype', _keep_types,
    ('in0', 'a + b', 'out0 = type_out0_raw(a)', None), 0)

_prod_auto_dtype = create_reduction_func(
    'cupy_prod', _sumprod_types,
    ('in0', 'a * b', 'out0 = type_out0_raw(a)', None), 1)

_prod_keep_dtype = create_reduction_func(
    'cupy_prod_with_dtype', _keep_types,
    ('in0', 'a * b', 'out0 = type_out0_raw(a)', None), 1)

_nansum_auto_dtype = create_reduction_func(
    'cupy_nansum', _sumprod_types,
    ('(in0 == in0) ? in0 : type_in0_raw(0)', 'a + b',
     'out0 = type_out0_raw(a)', None), 0)

_nansum_keep_dtype = create_reduction_func(
    'cupy_nansum_with_dtype', _keep_types,
    ('(in0 == in0) ? in0 : type_in0_raw(0)', 'a + b',
     'out0 = type_out0_raw(a)', None), 0)


_nanprod_auto_dtype = create_reduction_func(
    'cupy_nanprod', _sumprod_types,
    ('(in0 == in0) ? in0 : type_in0_raw(1)', 'a * b',
     'out0 = type_out0_raw(a)', None), 1)

_nanprod_keep_dtype = create_reduction_func(
    'cupy_nanprod_with_dtype', _keep_types,
    ('(in0 == in0) ? in0 : type_in0_raw(1)', 'a * b',
     'out0 = type_out0_raw(a)', None), 1)

_count_nonzero = create_reduction_func(
    'cupy_count_nonzero', tuple('%s->q' % c for c in '?bBhHiIlLqQefdFD'),
    ('(in0 != type_in0_raw(0)) ? 1 : 0', 'a + b', 'out0 = a', None), 0)


def _ndarray_sum(self, axis, dtype, out, keepdims):
    if dtype is None:
        return _sum_auto_dtype(self, axis, dtype, out, keepdims)
    return _sum_keep_dtype(self, axis, dtype, out, keepdims)


def _ndarray_prod(self, axis, dtype, out, keepdims):
    if dtype is None:
        return _prod_auto_dtype(self, axis, dtype, out, keepdims)
    return _prod_keep_dtype(self, axis, dtype, out, keepdims)


def sum(a, axis=None, dtype=None, out=None, keepdims=False):
    """Sum of array elements over the given axes.

    .. seealso:: :func:`numpy.sum`
    """
    if _fusion_thread_local.is_fusing():
        if keepdims and not _fusion_thread_local.records_keepdims():
            raise NotImplementedError(
                'cupy.sum does not support `keepdims` in fusion yet.')
        func = _sum_auto_dtype if dtype is None else _sum_keep_dtype
        return _fusion_thread_local.call_reduction(
            func, a, axis=axis, dtype=dtype, out=out, keepdims=keepdims)
    return a.sum(axis, dtype, out, keepdims)


def prod(a, axis=None, dtype=None, out=None, keepdims=False):
    """Product of array elements over the given axes.

    .. seealso:: :func:`numpy.prod`
    """
    if _fusion_thread_local.is_fusing():
        if keepdims and not _fusion_thread_local.records_keepdims():
            raise NotImplementedError(
                'cupy.prod does not support `keepdims` in fusion yet.')
        func = _prod_auto_dtype if dtype is None else _prod_keep_dtype
        return _fusion_thread_local.call_reduction(
            func, a, axis=axis, dtype=dtype, out=out, keepdims=keepdims)
    return a.prod(axis, dtype, out, keepdims)


def nansum(a, axis=None, dtype=None, out=None, keepdims=False):
    """Sum treating NaNs as zero.

    .. seealso:: :func:`numpy.nansum`
    """
    func = _nansum_auto_dtype if dtype is None else _nansum_keep_dtype
    if _fusion_thread_local.is_fusing():
        if keepdims and not _fusion_thread_local.records_keepdims():
            raise NotImplementedError(
                'cupy.nansum does not support `keepdims` in fusion yet.')
        return _fusion_thread_local.call_reduction(
            func, a, axis=axis, dtype=dtype, out=out, keepdims=keepdims)
    return func(a, axis, dtype, out, keepdims)


def nanprod(a, axis=None, dtype=None, out=None, keepdims=False):
    """Product of array elements over the given axes, NaNs counted as one.

    .. seealso:: :func:`numpy.nanprod`
    """
    func = _nanprod_auto_dtype if dtype is None else _nanprod_keep_dtype
    if _fusion_thread_local.is_fusing():
        if keepdims and not _fusion_thread_local.records_keepdims():
            raise NotImplementedError(
                'cupy.nanprod does not support `keepdims` in fusion yet.')
        return _fusion_thread_local.call_reduction(
            func, a, axis=axis, dtype=dtype, out=out, keepdims=keepdims)
    return func(a, axis, dtype, out, keepdims)


def count_nonzero(a, axis=None):
    """Number of non-zero elements, as an array (no synchronisation).

    .. seealso:: :func:`numpy.count_nonzero`
    """
    return _count_nonzero(a, axis=axis)
