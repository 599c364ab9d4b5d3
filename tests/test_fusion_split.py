"""Fused functions that need several kernels are cut at their reductions: one
map-reduce kernel per reduction (with everything elementwise that feeds it), one
elementwise kernel for what is left.  These tests look at the recorded launches
(compile-check mode); tests/test_gpu_fuse.py checks the values on the GPU."""
import numpy as np
import pytest

import cupy_amd as cp
from cupy_amd import _dryrun

pytestmark = pytest.mark.skipif(not _dryrun.enabled(),
                                reason='inspects recorded launches')


def kernels_of(f, *args):
    n0 = len(_dryrun.launches)
    out = f(*args)
    return out, [l[0] for l in _dryrun.launches[n0:]]


def arrays(*shapes, dtype=np.float32):
    return [cp.asarray(np.ones(s, dtype)) for s in shapes]


def test_softmax_is_three_kernels_with_no_full_size_temporary():
    @cp.fuse()
    def softmax(x):
        e = cp.exp(x - cp.amax(x, axis=1, keepdims=True))
        return e / cp.sum(e, axis=1, keepdims=True)

    x, = arrays((70, 33))
    pool = cp.get_default_memory_pool()
    out, names = kernels_of(softmax, x)
    assert names == ['softmax_part0', 'softmax_part1', 'softmax_part2']
    assert out.shape == (70, 33) and out.dtype == np.float32
    # the eager evaluation of the same function launches five kernels
    _, eager = kernels_of(softmax.func, x)
    assert len(eager) == 5
    # second call: the plan is remembered, same three launches
    _, again = kernels_of(softmax, x)
    assert again == names
    assert pool is not None


def test_elementwise_work_feeding_two_reductions_is_fused_into_each():
    @cp.fuse()
    def ratio(x, y, s):
        return cp.sum((x - y) ** 2, axis=1) / cp.sum(x * x * s, axis=1), x + y

    x, y = arrays((40, 50), (40, 50))
    (r, t), names = kernels_of(ratio, x, y, 2.0)
    assert r.shape == (40,) and t.shape == (40, 50)
    # two map-reduce kernels, then one elementwise kernel per result shape
    assert names == ['ratio_part0', 'ratio_part1', 'ratio_part2', 'ratio_part3']
    _, eager = kernels_of(ratio.func, x, y, 2.0)
    assert len(eager) > len(names)


def test_shapes_are_available_while_recording_and_key_the_plan():
    @cp.fuse()
    def var0(x):
        m = x.sum(axis=0) / x.shape[0]
        return ((x - m) ** 2).sum(axis=0) / x.shape[0]

    a, b = arrays((64, 8), (32, 8))
    ra, _ = kernels_of(var0, a)
    rb, _ = kernels_of(var0, b)
    assert ra.shape == rb.shape == (8,)
    assert len(var0._plans) == 2           # x.shape[0] is baked into each plan


def test_what_cannot_be_recorded_runs_as_written():
    @cp.fuse()
    def inplace(x, y):
        t = cp.sum(x, axis=0)
        y += t
        return y

    x, y = arrays((6, 5), (6, 5))
    out, names = kernels_of(inplace, x, y)
    assert out is y
    assert not any(n.startswith('inplace_part') for n in names)
    assert list(inplace._plans.values()) == [False]

    @cp.fuse()
    def looks_at_dtype(x):
        t = cp.sum(x, axis=0)
        return (x - t).astype(t.dtype)

    out, names = kernels_of(looks_at_dtype, x)
    assert out.dtype == np.float32 and list(looks_at_dtype._plans.values()) == [False]


def test_single_kernel_functions_do_not_take_this_route():
    @cp.fuse()
    def f(x, y):
        return cp.sqrt(cp.sum(x * y, axis=1))

    x, y = arrays((10, 20), (10, 20))
    _, names = kernels_of(f, x, y)
    assert names == ['f'] and not f._plans
