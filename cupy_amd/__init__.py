"""cupy_amd: the generated-kernel hot path of CuPy (ElementwiseKernel,
ReductionKernel, ufuncs, ``fuse`` and the device memory pool) built natively
for AMD Instinct MI355X (gfx950).  ``import cupy_amd as cupy`` keeps existing
call sites of that path working."""
import numpy as _numpy

from cupy_amd import _rt  # noqa: loads the native shim or fails loudly
from cupy_amd import cuda  # noqa
from cupy_amd._core.core import (  # noqa
    ndarray, array, asarray, asnumpy, ascontiguousarray)
from cupy_amd._core._kernel import (  # noqa
    ElementwiseKernel, ufunc, create_ufunc)
from cupy_amd._core._ufuncs import *  # noqa
from cupy_amd._core import _ufuncs as _ufuncs_module

__version__ = '0.1.0'

# dtypes and constants re-exported from NumPy
from numpy import (  # noqa
    bool_, int8, int16, int32, int64, uint8, uint16, uint32, uint64,
    float16, float32, float64, dtype, newaxis, inf, nan, pi, e)
from numpy import result_type, can_cast, promote_types  # noqa
from numpy.exceptions import AxisError, ComplexWarning  # noqa

# -- memory pool -------------------------------------------------------------------
_default_memory_pool = cuda.MemoryPool()
cuda.set_allocator(_default_memory_pool.malloc)


def get_default_memory_pool():
    """The pool that backs every ``ndarray`` allocation by default."""
    return _default_memory_pool
