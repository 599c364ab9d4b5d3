"""Scalars as kernel arguments, and the dtype -> C type-name table.

Counterpart of the reference's cupy/_core/_scalar.pyx (type names :14-29,
numpy_dtype_from_pyscalar :302-317, CScalar :320-407, literal formatting
:410-454).
"""
import math

import numpy

from cupy_amd._core._dtype import get_dtype

_typenames = {
    numpy.dtype('complex128'): 'complex<double>',
    numpy.dtype('complex64'): 'complex<float>',
    numpy.dtype('float64'): 'double',
    numpy.dtype('float32'): 'float',
    numpy.dtype('float16'): 'float16',
    numpy.dtype('int64'): 'long long',
    numpy.dtype('int32'): 'int',
    numpy.dtype('int16'): 'short',
    numpy.dtype('int8'): 'signed char',
    numpy.dtype('uint64'): 'unsigned long long',
    numpy.dtype('uint32'): 'unsigned int',
    numpy.dtype('uint16'): 'unsigned short',
    numpy.dtype('uint8'): 'unsigned char',
    numpy.dtype('bool'): 'bool',
}
_typenames_by_key = {}


def get_typename(dtype, type_decls=None):
    """C type used for ``dtype`` inside generated kernels."""
    if dtype is None:
        raise TypeError('dtype is None')
    try:
        name = _typenames_by_key.get(dtype)
    except TypeError:
        name = None
    if name is None:
        dt = get_dtype(dtype)
        name = _typenames.get(dt)
        if name is None:
            if dt.kind == 'V' and dt.fields is not None:
                # a struct written out for this dtype; not memoised here: the
                # registry of definitions keeps its own table
                from cupy_amd._core import _structured
                return _structured.struct_typename(dt)[0]
            if dt.kind == 'V' and dt.subdtype is None and dt.itemsize > 0:
                from cupy_amd._core import _structured
                return _structured.void_typename(dt.itemsize)       # a blob of bytes
            raise ValueError(f'Unsupported dtype {dtype}')
        try:
            _typenames_by_key[dtype] = name
        except TypeError:
            pass
    return name


_numpy_bool = numpy.dtype(numpy.bool_)
_numpy_int64 = numpy.dtype(numpy.int64)
_numpy_uint64 = numpy.dtype(numpy.uint64)
_numpy_float64 = numpy.dtype(numpy.float64)
_numpy_complex128 = numpy.dtype(numpy.complex128)


def numpy_dtype_from_pyscalar(x):
    """(dtype, weak type) for a Python scalar; (None, False) otherwise.
    ``bool`` is never weak."""
    typ = type(x)
    if typ is bool:
        return _numpy_bool, False
    if typ is float:
        return _numpy_float64, float
    if typ is complex:
        return _numpy_complex128, complex
    if typ is int:
        if x >= 0x8000000000000000:
            return _numpy_uint64, int
        return _numpy_int64, int
    return None, False


class CScalar:
    """A Python or NumPy scalar on its way into a kernel.

    ``descr`` is the dtype it will be passed as, ``weak_t`` the Python type if
    the value is a "weak" Python scalar (NEP 50) else ``False``.
    """
    ndim = 0
    __slots__ = ('value', 'descr', 'weak_t', '_bytes', '_pyval')

    def __init__(self, value, dtype=None):
        self.value = value
        self._bytes = None
        self._pyval = None
        if dtype is not None:
            self.descr = numpy.dtype(dtype)
            self.weak_t = False
        else:
            self.descr, self.weak_t = numpy_dtype_from_pyscalar(value)
            if self.descr is None:
                if isinstance(value, numpy.generic):
                    self.descr = value.dtype
                else:
                    raise TypeError(f'Unsupported type {type(value)}')

    @property
    def dtype(self):
        return self.descr

    def get_numpy_type(self):
        return self.descr.type

    def apply_dtype(self, dtype):
        descr = get_dtype(dtype)
        if descr != self.descr:
            self.descr = descr
            self._bytes = None
            self._pyval = None

    def _as_array(self):
        v = self.value
        with numpy.errstate(all='ignore'):
            if isinstance(v, numpy.generic):
                return numpy.asarray(v).astype(self.descr)
            return numpy.array(v, dtype=self.descr)

    def _struct_value(self):
        """The value as the Python object ``struct.pack`` takes for ``descr``
        (already rounded / wrapped to that type)."""
        v = self._pyval
        if v is None:
            v = self._pyval = self._as_array().item()
        return v

    def _kernel_arg_bytes(self):
        """Value converted to ``descr`` with NumPy's assignment rules: Python
        ints out of range raise OverflowError, NumPy scalars are cast."""
        b = self._bytes
        if b is None:
            v = self.value
            if isinstance(v, numpy.generic):
                with numpy.errstate(all='ignore'):
                    b = numpy.asarray(v).astype(self.descr).tobytes()
            else:
                with numpy.errstate(all='ignore'):
                    b = numpy.array(v, dtype=self.descr).tobytes()
            self._bytes = b
        return b


def get_scalar_literal(obj, dtype):
    """C literal for a constant of ``dtype``."""
    dtype = get_dtype(dtype)
    kind = dtype.kind
    if kind == 'b':
        return 'true' if bool(obj) else 'false'
    if kind == 'i':
        v = int(obj)
        if dtype.itemsize < 8:
            return str(v)
        if v == -(1 << 63):
            return '(-9223372036854775807ll - 1)'
        return str(v) + 'll'
    if kind == 'u':
        return str(int(obj)) + ('u' if dtype.itemsize < 8 else 'ull')
    if kind == 'f':
        v = float(obj)
        single = dtype.itemsize < 8
        if math.isnan(v):
            return 'CUDART_NAN_F' if single else 'CUDART_NAN'
        if math.isinf(v):
            lit = 'CUDART_INF_F' if single else 'CUDART_INF'
            return lit if v > 0 else '-' + lit
        if single:
            # Round to the target precision first: the decimal text of that
            # value parses back to exactly the same single (or half).
            with numpy.errstate(all='ignore'):
                v = float(dtype.type(v))
            if math.isinf(v):
                return 'CUDART_INF_F' if v > 0 else '-CUDART_INF_F'
            return repr(v) + 'f'
        return repr(v)
    if kind == 'c':
        v = complex(obj)
        part = numpy.dtype('float32' if dtype.itemsize == 8 else 'float64')
        return '%s(%s, %s)' % (get_typename(dtype), get_scalar_literal(v.real, part),
                               get_scalar_literal(v.imag, part))
    raise TypeError(f'Unsupported dtype: {dtype}')
