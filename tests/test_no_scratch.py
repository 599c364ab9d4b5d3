"""Generated kernels keep their per-lane state in registers.  Accumulators
that are structures (arg-reduction states, running summaries, complex numbers)
end up in scratch memory -- private memory behind the cache hierarchy -- as soon
as one loop indexes them by a run-time value; the code object records the
scratch size of every kernel, so the emitters can be checked without a GPU."""
import numpy as np
import pytest

import cupy_amd as cp
from cupy_amd import _dryrun
from cupy_amd.cuda import compiler

pytestmark = pytest.mark.skipif(not _dryrun.enabled(),
                                reason='drives the host path with fake allocations')


def scratch_users():
    bad = set()
    for mod in compiler._module_memo.values():
        for name, meta in mod.metadata.items():
            if meta['scratch']:
                bad.add((name, meta['scratch']))
    return bad


@pytest.mark.parametrize('dtype', ['float32', 'float64', 'complex64', 'complex128', 'int8',
                                   'float16', 'int16'])
def test_reductions_scans_and_elementwise_kernels_use_no_scratch(dtype):
    before = scratch_users()
    shapes = [(513, 1031), (1 << 14, 256), (3, 400001), (40000, 100)]
    for shape in shapes:
        arr = cp.empty(shape, dtype)
        for axis in (0, 1, None):
            arr.sum(axis=axis)
            arr.mean(axis=axis)
            cp.cumsum(arr, axis=axis)
            cp.cumsum(arr, axis=axis, dtype=arr.dtype)
            if arr.dtype.kind != 'c':
                arr.argmax(axis=axis)
                arr.max(axis=axis)
                arr.var(axis=axis)
            if arr.dtype.kind == 'f':
                cp.nanmean(arr, axis=axis)
                cp.nanargmin(arr, axis=axis)
    a = cp.empty((513, 1031), dtype)
    a + a
    a.T * 2
    abs(a)
    view = cp.empty((20, 30, 40), dtype)[::2, ::3, ::2]
    view + 1
    view.sum(axis=1)
    assert scratch_users() - before == set()
