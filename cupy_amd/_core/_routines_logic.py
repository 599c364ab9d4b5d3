"""any / all reductions (reference: cupy/_core/_routines_logic.pyx)."""
from cupy_amd._core import _fusion_thread_local
from cupy_amd._core._reduction import create_reduction_func

_all_sigs = tuple('%s->?' % c for c in '?bBhHiIlLqQefdFD')

_all = create_reduction_func(
    'cupy_all', _all_sigs,
    ('in0 != type_in0_raw(0)', 'a & b', 'out0 = a', 'bool'), 'true')

_any = create_reduction_func(
    'cupy_any', _all_sigs,
    ('in0 != type_in0_raw(0)', 'a | b', 'out0 = a', 'bool'), 'false')


def _ndarray_all(self, axis, out, keepdims):
    return _all(self, axis=axis, out=out, keepdims=keepdims)


def _ndarray_any(self, axis, out, keepdims):
    return _any(self, axis=axis, out=out, keepdims=keepdims)


def all(a, axis=None, out=None, keepdims=False):
    """Tests whether all elements along the given axes are true."""
    if _fusion_thread_local.is_fusing():
        if keepdims and not _fusion_thread_local.records_keepdims():
            raise NotImplementedError(
                'cupy.all does not support `keepdims` in fusion yet.')
        return _fusion_thread_local.call_reduction(_all, a, axis=axis, out=out, keepdims=keepdims)
    return a.all(axis=axis, out=out, keepdims=keepdims)


def any(a, axis=None, out=None, keepdims=False):
    """Tests whether any element along the given axes is true."""
    if _fusion_thread_local.is_fusing():
        if keepdims and not _fusion_thread_local.records_keepdims():
            raise NotImplementedError(
                'cupy.any does not support `keepdims` in fusion yet.')
        return _fusion_thread_local.call_reduction(_any, a, axis=axis, out=out, keepdims=keepdims)
    return a.any(axis=axis, out=out, keepdims=keepdims)
