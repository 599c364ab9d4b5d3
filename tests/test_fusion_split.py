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


def _softmax(x):
    e = cp.exp(x - cp.amax(x, axis=1, keepdims=True))
    return e / cp.sum(e, axis=1, keepdims=True)


def test_softmax_over_long_rows_is_three_kernels_with_no_full_size_temporary():
    softmax = cp.fuse(kernel_name='softmax')(_softmax)
    x, = arrays((4, 100000))                  # a row does not fit the registers of a workgroup
    out, names = kernels_of(softmax, x)
    # (few long rows: each map-reduce kernel is followed by its combine kernel)
    assert [n for n in names if not n.endswith('_combine')] == [
        'softmax_part0', 'softmax_part1', 'softmax_part2']
    assert out.shape == (4, 100000) and out.dtype == np.float32
    # the eager evaluation of the same function launches five kernels (and two
    # full-size temporaries)
    _, eager = kernels_of(_softmax, x)
    assert len([n for n in eager if not n.endswith('_combine')]) == 5
    # second call: the plan is remembered, same three launches
    _, again = kernels_of(softmax, x)
    assert again == names


@pytest.mark.parametrize('shape', [(70, 33), (64, 4096), (3, 5, 1000), (1000,)])
def test_reductions_along_short_rows_become_one_kernel(shape):
    def standardise(x, eps):
        m = cp.sum(x, axis=-1, keepdims=True) / x.shape[-1]
        d = x - m
        v = cp.sum(d * d, axis=-1, keepdims=True) / x.shape[-1]
        return d / cp.sqrt(v + eps), m

    f = cp.fuse(kernel_name='standardise')(standardise)
    x, = arrays(shape)
    (out, mean), names = kernels_of(f, x, 1e-5)
    assert names == ['standardise']            # the matrix is read once
    assert out.shape == shape and mean.shape == shape[:-1] + (1,)
    assert out.dtype == mean.dtype == np.float32
    # a view that is not contiguous goes through the kernel sequence instead
    if len(shape) == 2:
        wide, = arrays((shape[0], 2 * shape[1]))
        (out2, _), names2 = kernels_of(f, wide[:, ::2], 1e-5)
        assert out2.shape == shape and all('_part' in n for n in names2)


def test_elementwise_work_feeding_two_reductions_is_fused_into_each():
    def ratio(x, y, s):
        return cp.sum((x - y) ** 2, axis=0) / cp.sum(x * x * s, axis=0), x + y

    f = cp.fuse(kernel_name='ratio')(ratio)
    x, y = arrays((40, 50), (40, 50))
    (r, t), names = kernels_of(f, x, y, 2.0)
    assert r.shape == (50,) and t.shape == (40, 50)
    # two map-reduce kernels, then one elementwise kernel per result shape
    assert names == ['ratio_part0', 'ratio_part1', 'ratio_part2', 'ratio_part3']
    _, eager = kernels_of(ratio, x, y, 2.0)
    assert len(eager) > len(names)
    # the same along the rows: everything in one kernel, both results written by it
    def ratio_rows(x, y, s):
        return cp.sum((x - y) ** 2, axis=1) / cp.sum(x * x * s, axis=1), x + y
    g = cp.fuse(kernel_name='ratio_rows')(ratio_rows)
    (r, t), names = kernels_of(g, x, y, 2.0)
    assert names == ['ratio_rows'] and r.shape == (40,) and t.shape == (40, 50)


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


CASES = {
    # name: (function of (xp, captured), number of arrays, extra args, kernels, result shapes)
    'tuple_axis': (lambda xp, c: lambda a: a - xp.sum(a, axis=(0, 2), keepdims=True) / 24,
                   1, (), 2, [(6, 5, 4)]),
    'negative_axis': (lambda xp, c: lambda a: xp.sum(a, axis=-1) * xp.amax(a, axis=-1),
                      1, (), 3, [(6, 5)]),
    'captured_array': (lambda xp, c: lambda a: (a + c) / xp.sum(a + c, axis=2, keepdims=True),
                       1, (), 2, [(6, 5, 4)]),
    'scalar_argument': (lambda xp, c: lambda a, s: a * s - xp.sum(a * s),
                        1, (2.5,), 2, [(6, 5, 4)]),
    'returns_an_argument': (lambda xp, c: lambda a: (a, a - xp.amin(a)),
                            1, (), 2, [(6, 5, 4), (6, 5, 4)]),
    'none_argument': (lambda xp, c: lambda a, b: a - xp.sum(a) if b is None else a + b,
                      1, (None,), 2, [(6, 5, 4)]),
    'zero_dimensional': (lambda xp, c: lambda a: xp.sum(a) / xp.amax(a),
                         1, (), 3, [()]),
    'astype': (lambda xp, c: lambda a: (a - xp.sum(a, axis=0)).astype(np.float64),
               1, (), 2, [(6, 5, 4)]),
    'methods': (lambda xp, c: lambda a: a.max(axis=1) - a.min(axis=1) + a.sum(axis=1),
                1, (), 4, [(6, 4)]),
    'logic': (lambda xp, c: lambda a: xp.where(xp.all(a > 0, axis=0), xp.sum(a, axis=0), 0),
              1, (), 3, [(5, 4)]),
    'two_arrays': (lambda xp, c: lambda a, b: (a - b) / xp.sum(a * b, axis=1, keepdims=True),
                   2, (), 2, [(6, 5, 4)]),
}


@pytest.fixture
def one_kernel_per_piece():
    from cupy_amd._core import _tuning
    _tuning.set(fused_rows=False)
    yield
    _tuning.set(fused_rows=True)


@pytest.mark.parametrize('name', sorted(CASES))
def test_recorded_shapes_and_kernel_counts(name, one_kernel_per_piece):
    make, n_arrays, extra, n_kernels, shapes = CASES[name]
    captured = cp.asarray(np.ones(4, np.float32))
    f = cp.fuse(make(cp, captured))
    args = arrays(*[(6, 5, 4)] * n_arrays) + list(extra)
    out, names = kernels_of(f, *args)
    outs = out if isinstance(out, tuple) else (out,)
    assert [o.shape for o in outs] == shapes
    assert len(names) == n_kernels and all('_part' in n for n in names)
    host = [np.ones((6, 5, 4), np.float32)] * n_arrays + list(extra)
    want = make(np, np.ones(4, np.float32))(*host)
    wants = want if isinstance(want, tuple) else (want,)
    assert [o.dtype for o in outs] == [np.asarray(w).dtype for w in wants]


def test_errors_of_the_function_surface():
    x, = arrays((6, 5, 4))
    with pytest.raises(ValueError):
        cp.fuse(lambda a: a - cp.sum(a, axis=(0, 0)))(x)
    with pytest.raises(cp.AxisError):
        cp.fuse(lambda a: a - cp.sum(a, axis=5))(x)


def test_nested_fused_functions_are_inlined_in_the_pieces():
    @cp.fuse()
    def inner(a, b):
        return a * b + 1

    @cp.fuse()
    def outer(a, b):
        return inner(a, b) - cp.sum(inner(a, b), axis=0)

    x, y = arrays((6, 5), (6, 5))
    out, names = kernels_of(outer, x, y)
    assert out.shape == (6, 5) and names[0] == 'outer_part0' and names[-1] == 'outer_part1'
