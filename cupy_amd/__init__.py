"""cupy_amd: the generated-kernel hot path of CuPy (ElementwiseKernel,
ReductionKernel, ufuncs, ``fuse`` and the device memory pool) built natively
for AMD Instinct MI355X (gfx950).  ``import cupy_amd as cupy`` keeps existing
call sites of that path working."""
import numpy as _numpy
from cupy_amd._core._structured import make_aligned_dtype  # noqa: F401

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
    float16, float32, float64, complex64, complex128, dtype, newaxis, inf, nan, pi, e)
from numpy import (  # noqa
    result_type, can_cast, promote_types, broadcast_shapes, issubdtype, finfo, iinfo,
    min_scalar_type, isdtype,
    generic, number, integer, signedinteger, unsignedinteger, inexact, floating,
    complexfloating, byte, ubyte, short, ushort, intc, uintc, int_, uint, intp, uintp,
    longlong, ulonglong, half, single, double, csingle, cdouble, euler_gamma)
from numpy.exceptions import AxisError, ComplexWarning  # noqa

# -- memory pool -------------------------------------------------------------------
_default_memory_pool = cuda.MemoryPool()
cuda.set_allocator(_default_memory_pool.malloc)


def get_default_memory_pool():
    """The pool that backs every ``ndarray`` allocation by default."""
    return _default_memory_pool


def _runtime_records():
    """(label, value) pairs describing the installation, in display order."""
    import os
    import platform
    import shutil
    from cupy_amd import _dryrun
    from cupy_amd.cuda import compiler as _compiler
    from cupy_amd.cuda import _compiler_cache
    records = [
        ('OS', platform.platform()),
        ('Python Version', platform.python_version()),
        ('CuPy Version', __version__),
        ('CuPy Platform', 'AMD ROCm (MI355X-native build, gfx950)'),
        ('NumPy Version', _numpy.__version__),
        ('ROCm Include Dir', _compiler.rocm_include_dir()),
        ('HIPCC PATH', shutil.which('hipcc')),
        ('Runtime Library', _rt.LIB_PATH),
        ('Kernel Cache Dir', _compiler_cache.get_cache_dir()),
    ]
    if _dryrun.enabled():
        records.append(('Mode', 'compile check only (CUPY_AMD_DRYRUN): nothing runs on a device'))
        return records
    records += [
        ('HIP Driver Version', cuda.runtime.driverGetVersion()),
        ('HIP Runtime Version', cuda.runtime.runtimeGetVersion()),
        ('hipRTC Version', '%d.%d' % _compiler.get_rtc_version()),
        ('Per-Thread Default Stream', cuda.stream.is_ptds_enabled()),
    ]
    for device_id in range(cuda.runtime.getDeviceCount()):
        props = cuda.device.get_device_properties(device_id)
        label = 'Device %d ' % device_id
        records += [
            (label + 'Name', props['name']),
            (label + 'Arch', props['arch']),
            (label + 'Compute Units', props['compute_units']),
            (label + 'Memory', '%.1f GiB' % (props['total_global_mem'] / 2.0 ** 30)),
        ]
    return records


def show_config(*, _full=False):
    """Prints the current runtime configuration to standard output
    (reference: cupy/__init__.py:942-946, cupyx/_runtime.py:309-420)."""
    import builtins
    import sys
    records = _runtime_records()
    width = builtins.max(len(label) for label, _ in records) + 1
    sys.stdout.write(''.join('%s: %s\n' % (label.ljust(width), value)
                             for label, value in records))
    sys.stdout.flush()

from cupy_amd._core._reduction import (  # noqa
    ReductionKernel, create_reduction_func)
from cupy_amd._core.fusion import fuse  # noqa
from cupy_amd._core.raw import RawKernel, RawModule  # noqa
from cupy_amd._core._routines_math import (  # noqa
    sum, prod, nansum, nanprod, count_nonzero)
from cupy_amd._core._routines_statistics import (  # noqa
    amax, amin, argmax, argmin, mean, var, std, ptp, nanmin, nanmax, nanmean,
    nanvar, nanstd, nanargmax, nanargmin)
from cupy_amd._core._routines_logic import all, any  # noqa
from cupy_amd._core._scan import cumsum, cumprod, nancumsum, nancumprod  # noqa
from cupy_amd._creation import (  # noqa
    empty, empty_like, zeros, zeros_like, ones, ones_like, full, full_like, arange)

from cupy_amd._manipulation import (  # noqa
    shape, ndim, size, squeeze, swapaxes, moveaxis, rollaxis, expand_dims,
    atleast_1d, atleast_2d, atleast_3d, broadcast_arrays, flip, fliplr, flipud,
    astype, asanyarray, asfortranarray, isscalar, cumulative_sum, cumulative_prod,
    isneginf, isposinf, array_equal, array_equiv, average, linspace)
from cupy_amd._join import (  # noqa
    concatenate, stack, hstack, vstack, row_stack, dstack, column_stack,
    array_split, split, hsplit, vsplit, dsplit, tile, repeat, roll, rot90)

max = amax
min = amin


def transpose(a, axes=None):
    return a.transpose(axes)


def reshape(a, newshape, order='C'):
    return a.reshape(newshape, order=order)


def ravel(a, order='C'):
    return a.ravel(order)


def broadcast_to(array, shape):
    """Read-only zero-stride view of ``array`` with the given shape."""
    shape = tuple(shape) if isinstance(shape, (tuple, list)) else (shape,)
    if array.ndim > len(shape):
        raise ValueError('input operand has more dimensions than allowed by '
                         'the axis remapping')
    off = len(shape) - array.ndim
    strides = [0] * len(shape)
    for i, (ext, st) in enumerate(zip(array.shape, array.strides)):
        if ext == shape[off + i]:
            strides[off + i] = st
        elif ext != 1:
            raise ValueError(
                'operands could not be broadcast together with remapped shapes '
                '[original->remapped]: {} and requested shape {}'.format(
                    array.shape, shape))
    return array._view(shape, tuple(strides))


def copy(a, order='K'):
    from cupy_amd._core import _fusion_thread_local
    if _fusion_thread_local.is_fusing():
        return _ufuncs_module.elementwise_copy(a)
    return a.copy(order=order)


def copyto(dst, src, casting='same_kind', where=None):
    """Copies ``src`` into ``dst`` (broadcasting), optionally under a mask."""
    if where is None:
        _ufuncs_module.elementwise_copy(src, dst, casting=casting)
    else:
        _ufuncs_module.elementwise_copy(src, dst, casting=casting, _where=where)
