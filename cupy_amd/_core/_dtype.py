"""dtype lookup and cast checks (reference: cupy/_core/_dtype.pyx:97-101 get_dtype,
:149-182 _raise_if_invalid_cast)."""
import warnings

import numpy
from numpy.exceptions import ComplexWarning

_dtype_memo = {}

# dtypes the generated kernels can address
SUPPORTED_CHARS = '?bhilqBHILQefdFD'


def get_dtype(t):
    try:
        dt = _dtype_memo.get(t)
    except TypeError:          # unhashable specifier
        return numpy.dtype(t)
    if dt is None:
        dt = numpy.dtype(t)
        _dtype_memo[t] = dt
    return dt


def check_supported_dtype(dtype, error=True):
    if dtype.char in SUPPORTED_CHARS and dtype.isnative:
        return True
    if dtype.kind == 'V' and dtype.fields is None and dtype.subdtype is None \
            and dtype.itemsize > 0:
        return True                      # raw bytes
    if dtype.kind == 'V' and dtype.fields is not None:
        # structured: any layout can be stored and moved; kernels check the
        # alignment of the fields when one is built for it
        from cupy_amd._core import _structured
        if not _structured.has_references(dtype):
            return True
        if error:
            raise ValueError('dtypes that hold Python objects cannot live in device memory: %s'
                             % dtype)
        return False
    if error:
        raise ValueError('Unsupported dtype %s' % dtype)
    return False


def _raise_if_invalid_cast(from_dt, to_dt, casting, argname='array data'):
    """TypeError unless ``from_dt`` may be cast to ``to_dt`` under ``casting``."""
    if from_dt is to_dt:
        return
    to_dt = get_dtype(to_dt)
    from_dt = get_dtype(from_dt)
    if casting == 'same_kind' and from_dt.kind == to_dt.kind:
        return
    if numpy.can_cast(from_dt, to_dt, casting):
        if casting == 'unsafe' and from_dt.kind == 'c' and to_dt.kind in 'iuf':
            warnings.warn(
                'Casting complex values to real discards the imaginary part',
                ComplexWarning)
        return
    if not isinstance(argname, str):
        argname = argname()
    raise TypeError(
        f'Cannot cast {argname} from {from_dt!r} to {to_dt!r} '
        f'according to the rule \'{casting}\'')
