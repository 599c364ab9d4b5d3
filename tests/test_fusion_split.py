"""Fused functions that need several kernels are cut at their reductions: one
map-reduce kernel per reduction (with everything elementwise that feeds it), one
elementwise kernel for what is left.  These tests look at the recorded launches
(compile-check mode); tests/test_gpu_fuse.py checks the values on the GPU."""
import numpy as np
import pytest

import cupy_amd as cp
from cupy_amd import _dryrun
from cupy_amd._core import _tuning

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
    # (few long rows: the workgroups of a row hand their partial results over
    # in memory that the first such launch on a stream clears)
    names = [n for n in names if not n.startswith('cupy_copy')]
    assert names == ['softmax_part0', 'softmax_part1', 'softmax_part2']
    assert out.shape == (4, 100000) and out.dtype == np.float32
    # the eager evaluation of the same function launches five kernels (and two
    # full-size temporaries)
    _, eager = kernels_of(_softmax, x)
    assert len([n for n in eager if not n.endswith('_combine')]) == 5
    # second call: the plan is remembered, same three launches
    _, again = kernels_of(softmax, x)
    assert again == names
    # with the finishing in the launch switched off, each map-reduce kernel is
    # followed by its combine kernel
    _tuning.set(reduce_finish=False)
    try:
        _, two = kernels_of(cp.fuse(kernel_name='softmax')(_softmax), x)
    finally:
        _tuning.set(reduce_finish=True)
    assert two == ['softmax_part0', 'softmax_part0_combine', 'softmax_part1',
                   'softmax_part1_combine', 'softmax_part2']


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


def test_in_place_updates_and_dtype_queries_are_recorded():
    @cp.fuse()
    def inplace(x, y):
        t = cp.sum(x, axis=0)
        y += t
        return y

    x, y = arrays((6, 5), (6, 5))
    out, names = kernels_of(inplace, x, y)
    assert out is y
    # the reduction, then one elementwise kernel that writes y
    assert names == ['inplace_part0', 'inplace_part1']

    @cp.fuse()
    def looks_at_dtype(x):
        t = cp.sum(x, axis=0)
        return (x - t).astype(t.dtype)

    out, names = kernels_of(looks_at_dtype, x)
    assert out.dtype == np.float32
    assert names == ['looks_at_dtype_part0', 'looks_at_dtype_part1']


def test_what_cannot_be_recorded_runs_as_written():
    @cp.fuse()
    def indexes_an_intermediate(x):
        return (x + 1)[0] * 2

    x, = arrays((6, 5))
    out, names = kernels_of(indexes_an_intermediate, x)
    assert out.shape == (5,)
    assert names == ['cupy_add__float32_float_float32', 'cupy_multiply__float32_float_float32']
    assert indexes_an_intermediate._memo and \
        list(indexes_an_intermediate._memo.values()) == ['eager']

    @cp.fuse()
    def reduces_into_an_argument(x, y):
        cp.sum(x, axis=0, out=y)
        return y

    y, = arrays((5,))
    out, names = kernels_of(reduces_into_an_argument, x, y)
    assert out is y and names == ['cupy_sum']

    @cp.fuse()
    def writes_what_it_indexes(x):
        first = x[0]
        x += 1
        return first

    out, names = kernels_of(writes_what_it_indexes, x)
    assert out.shape == (5,) and not any('writes_what' in n for n in names)


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


# In-place operators, out= and indexing inside fused functions: the scenarios of
# the reference's tests/cupy_tests/core_tests/fusion_tests/test_misc.py:32-54,
# 126-141 and test_indexing.py:48-124.  Each must be ONE launch (or none, where
# nothing is computed); tests/test_gpu_fuse.py checks the values.

def _outarg_mixed(xp):
    def func(x, y, z, u, v):
        xp.add(x, y, out=z)
        xp.subtract(z, x, out=u)
        xp.multiply(z, x, out=v)
        return u
    return func


def _iadd_multiple_times(xp):
    def func(x, y):
        x += y
        x += y
        x += y
        return x
    return func


def _iadd_once(xp):
    def func(x):
        x += 2
    return func


def _iadd_twice(xp):
    def func(x):
        x += x
        x += x
    return func


def _swap(xp):
    def func(x, y, z):
        w = x * y + z
        (x, w) = (w, x)
        return z * w + y + x
    return func


ONE_LAUNCH = {
    'outarg_mixed': (_outarg_mixed, 5),
    'iadd_multiple_times': (_iadd_multiple_times, 2),
    'iadd_once': (_iadd_once, 1),
    'iadd_twice': (_iadd_twice, 1),
    'swap': (_swap, 3),
    'return_tuple': (lambda xp: lambda x, y, z: (x + y, y + z, z * x), 3),
    'astype_mix': (lambda xp: lambda x, y, z: (
        x.astype('int32') + x.astype('int32').astype('float32'),
        x.astype('int32').astype('float32') + z, z + x.astype('int32')), 3),
}


@pytest.mark.parametrize('name', sorted(ONE_LAUNCH))
@pytest.mark.parametrize('dtype', [np.float32, np.int16])
def test_in_place_and_out_arguments_are_one_launch(name, dtype):
    make, nargs = ONE_LAUNCH[name]
    f = cp.fuse(kernel_name='scenario')(make(cp))
    args = arrays(*[(3, 4)] * nargs, dtype=dtype)
    _, names = kernels_of(f, *args)
    assert names == ['scenario']
    _, again = kernels_of(f, *args)            # and the replay of the recorded call
    assert again == ['scenario']


def test_in_place_results_are_the_argument_arrays_themselves():
    x, y = arrays((3, 4), (3, 4))
    assert cp.fuse(_iadd_multiple_times(cp))(x, y) is x
    assert cp.fuse(_iadd_once(cp))(x) is None
    z, u, v = arrays((3, 4), (3, 4), (3, 4))
    assert cp.fuse(_outarg_mixed(cp))(x, y, z, u, v) is u
    assert cp.fuse(lambda a: ())(x) == ()
    (only,) = cp.fuse(lambda a: (a,))(x)
    assert only is x


INDICES = [
    1, -1, (1,), (1, 0), (1, 0, 2), (-1, 0, -2), slice(None), slice(None, None, 1),
    slice(None, None, -1), (slice(None), slice(None, None, -1)), Ellipsis, (Ellipsis,), None,
    (None,), (None, None, None), (slice(None), 0, slice(None, None, -1)),
    (1, None, slice(None, None, -1), None, 2), (Ellipsis, 2), (1, Ellipsis),
]


@pytest.mark.parametrize('indices', INDICES, ids=str)
def test_indexing_an_argument_is_a_view_and_launches_nothing(indices):
    x, = arrays((2, 3, 4))
    out, names = kernels_of(cp.fuse(lambda a: a[indices]), x)
    assert names == []
    assert out.shape == np.ones((2, 3, 4))[indices].shape
    assert out.data.ptr >= x.data.ptr and out.data.ptr < x.data.ptr + x.nbytes


@pytest.mark.parametrize('shape,indices', [((), 0), ((2, 3), (0, 0, 0)), ((2, 3, 4), -3),
                                           ((2, 3, 4), 3)])
def test_invalid_index_raises_as_numpy_does(shape, indices):
    x, = arrays(shape)
    with pytest.raises(IndexError):
        cp.fuse(lambda a: a[indices])(x)


INDEXED_SUMS = {
    'add_1': lambda x, y, z: x + y[1],
    'add_2': lambda x, y, z: x + z[0] + y,
    'add_3': lambda x, y, z: x + x[0] + x[1],
    'add_4': lambda x, y, z: x + x[0, 1] + x[1] + x + x[2, 1],
    'twice_2': lambda x, y, z: x[0][1] + x[1][0],
    'reversed': lambda x, y, z: x[::-1] + y,
}


@pytest.mark.parametrize('name', sorted(INDEXED_SUMS))
def test_indexed_operands_are_inputs_of_one_kernel(name):
    x, y, z = arrays((3, 4), (4,), (1,))
    f = cp.fuse(kernel_name='indexed')(INDEXED_SUMS[name])
    out, names = kernels_of(f, x, y, z)
    assert names == ['indexed']
    want = INDEXED_SUMS[name](np.ones((3, 4), np.float32), np.ones(4, np.float32),
                              np.ones(1, np.float32))
    assert out.shape == want.shape and out.dtype == want.dtype
    # other extents: recorded anew (integer indices were checked against the shape)
    x2, y2 = arrays((5, 4), (4,))
    out2, names2 = kernels_of(f, x2, y2, z)
    assert names2 == ['indexed'] and out2.shape[-1:] == (4,)[:out2.ndim]
