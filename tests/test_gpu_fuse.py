"""cupy.fuse on the GPU.  Each fused function is evaluated four ways -- NumPy,
eager on the device, the fused Python function on NumPy arrays, the fused
kernel -- and all must agree (the reference's protocol,
tests/cupy_tests/core_tests/fusion_tests/fusion_utils.py:14-148, with the
tolerance of this task instead of its 3e-3)."""
import numpy as np
import pytest

import cupy_amd as cp
from helpers import assert_exact, shaped_random
from oracle import numpy_oracle as o

pytestmark = pytest.mark.gpu


def four_way(func, host_args, exact=True, rtol=1e-5):
    dev_args = [cp.asarray(a) if isinstance(a, np.ndarray) else a for a in host_args]

    def run(xp, fused, args):
        f = cp.fuse(func(xp)) if fused else func(xp)
        return f(*args)

    r_np = run(np, False, host_args)
    r_eager = run(cp, False, dev_args)
    r_fused_np = run(np, True, host_args)
    r_fused = run(cp, True, dev_args)
    for r in (r_eager, r_fused):
        got = r.get()
        assert got.dtype == np.asarray(r_np).dtype, (got.dtype, np.asarray(r_np).dtype)
        if exact:
            assert_exact(got, np.asarray(r_np))
        else:
            assert np.allclose(got, r_np, rtol=rtol, atol=rtol)
    assert np.array_equal(np.asarray(r_fused_np), np.asarray(r_np), equal_nan=True)


def test_elementwise_chain():
    x = shaped_random((50, 30), 'float32', 1)
    y = shaped_random((50, 30), 'float32', 2)
    four_way(lambda xp: lambda a, b: (a - b) * (a - b) + a, [x, y])
    four_way(lambda xp: lambda a, b: xp.sqrt(xp.absolute(a)) + b * 2, [x, y])
    four_way(lambda xp: lambda a, b: xp.maximum(a, b) - xp.minimum(a, 0.5), [x, y])


def test_scalars_and_promotion():
    x = shaped_random((64,), 'int32', 3)
    four_way(lambda xp: lambda a: a * 2 + 1, [x])
    four_way(lambda xp: lambda a: a * 2.5, [x])
    four_way(lambda xp: lambda a, s: a + s, [x, 3])
    four_way(lambda xp: lambda a, s: a + s, [x, 2.5])
    h = shaped_random((64,), 'float16', 4)
    four_way(lambda xp: lambda a: a * 2 + 1, [h])
    four_way(lambda xp: lambda a, b: a + b, [h, x.astype(np.float32)])
    four_way(lambda xp: lambda a, s: a * s, [h, np.float32(1.5)])


BCAST = [((10,), (1,)), ((3, 1), (1, 4)), ((2, 1, 4), (3, 1)), ((256, 256), (256, 1)),
         ((5, 6), (6,)), ((0,), (1,))]


@pytest.mark.parametrize('sa,sb', BCAST)
def test_broadcast_shapes(sa, sb):
    a = shaped_random(sa, 'float32', 5)
    b = shaped_random(sb, 'float32', 6)
    four_way(lambda xp: lambda p, q: p * q + q, [a, b])


def test_invalid_broadcast():
    f = cp.fuse(lambda p, q: p + q)
    with pytest.raises(ValueError):
        f(cp.zeros((3,), np.float32), cp.zeros((4,), np.float32))


def test_power_shortcuts_match_numpy():
    h = shaped_random((500,), 'float16', 7, scale=3)
    four_way(lambda xp: lambda a: a ** 2, [h])
    f = shaped_random((500,), 'float32', 8, scale=3)
    four_way(lambda xp: lambda a: a ** 2 + a, [f])
    four_way(lambda xp: lambda a: xp.absolute(a) ** 0.5, [f])
    i = shaped_random((100,), 'int32', 9, scale=5)
    four_way(lambda xp: lambda a: a ** 2, [i])
    four_way(lambda xp: lambda a: a ** 3, [np.abs(i)])


def test_non_contiguous_inputs_and_multiple_outputs():
    x = shaped_random((40, 60), 'float32', 10)
    y = shaped_random((60, 40), 'float32', 11)
    d, e = cp.asarray(x), cp.asarray(y)
    f = cp.fuse(lambda a, b: (a + b, a - b))
    s, t = f(d, e.T)
    assert_exact(s.get(), x + y.T)
    assert_exact(t.get(), x - y.T)
    g = cp.fuse(lambda a, b: a[...] if False else a * b)
    assert_exact(g(d[::2, 1::2], e.T[::2, 1::2]).get(), x[::2, 1::2] * y.T[::2, 1::2])


def test_in_place_update_of_an_argument():
    x = shaped_random((100,), 'float32', 12)
    y = shaped_random((100,), 'float32', 13)

    @cp.fuse()
    def update(a, b):
        a += b * 2
        return a

    d = cp.asarray(x)
    r = update(d, cp.asarray(y))
    assert_exact(d.get(), x + y * 2)
    assert_exact(r.get(), x + y * 2)


def test_astype_and_comparison():
    x = shaped_random((80,), 'float32', 14)
    four_way(lambda xp: lambda a: (a > 0).astype(np.int32) * 3, [x])
    four_way(lambda xp: lambda a: a.astype(np.float16) + a.astype(np.float16), [x])


# -- reductions ------------------------------------------------------------------------------

def test_fused_sum_over_each_axis():
    x = shaped_random((37, 53), 'float32', 15, scale=1)
    y = shaped_random((37, 53), 'float32', 16, scale=1)
    for axis in (0, 1, -1, None):
        four_way(lambda xp: lambda a, b: xp.sum(a * b + a, axis=axis), [x, y], exact=False)
    four_way(lambda xp: lambda a: xp.sum(a), [x], exact=False)
    i = shaped_random((37, 53), 'int32', 17)
    four_way(lambda xp: lambda a: xp.sum(a * a, axis=0), [i])


def test_fused_config_small(small_configs):
    c = small_configs

    @cp.fuse()
    def f(x, y, w):
        return cp.sum((x - y) ** 2 * w, axis=-1)

    got = f(cp.asarray(c['c5_x']), cp.asarray(c['c5_y']), cp.asarray(c['c5_w']))
    assert got.dtype == np.float32 and got.shape == (70,)
    assert np.allclose(got.get(), c['c5_out'], rtol=1e-5)
    assert np.allclose(got.get(), o.fused_sqdiff_wsum(c['c5_x'], c['c5_y'], c['c5_w']), rtol=1e-5)
    # the float16 roundings of the pipeline are reproduced: an unrounded float32
    # evaluation is farther away than the tolerance on at least one row
    x32, y32 = c['c5_x'].astype(np.float32), c['c5_y'].astype(np.float32)
    unrounded = ((x32 - y32) ** 2 * c['c5_w']).sum(axis=-1)
    assert np.abs(got.get() - c['c5_out']).max() < np.abs(unrounded - c['c5_out']).max()
    # identical inputs: exactly zero
    z = f(cp.asarray(c['c5_x']), cp.asarray(c['c5_x']), cp.asarray(c['c5_w']))
    assert_exact(z.get(), np.zeros(70, np.float32))


def test_post_reduction_operations():
    x = shaped_random((30, 200), 'float32', 18, scale=1)
    four_way(lambda xp: lambda a: xp.sqrt(xp.sum(a * a, axis=1)), [x], exact=False)
    four_way(lambda xp: lambda a: xp.sum(a, axis=0) * 2 + 1, [x], exact=False)


def test_fused_min_max_prod():
    x = shaped_random((20, 30), 'float32', 19, scale=2)
    four_way(lambda xp: lambda a: xp.amax(a * 2, axis=1), [x])
    four_way(lambda xp: lambda a: xp.amin(a + 1, axis=0), [x])
    four_way(lambda xp: lambda a: xp.prod(a * 0.5 + 1, axis=1), [x], exact=False, rtol=1e-4)


def test_functions_the_single_kernel_cannot_express_still_compute():
    # two chained reductions, and a reduced value broadcast back over the
    # input: neither is one map-reduce kernel; both run as kernel sequences
    h = shaped_random((5, 7), 'float32', 19)

    @cp.fuse()
    def two(a):
        return cp.sum(cp.sum(a, axis=0))

    np.testing.assert_allclose(two(cp.asarray(h)).get(), h.sum(axis=0).sum(), rtol=1e-5)

    @cp.fuse()
    def mixed(a):
        return cp.sum(a, axis=0) + a

    np.testing.assert_allclose(mixed(cp.asarray(h)).get(), h.sum(axis=0) + h, rtol=1e-5)


def test_nested_fused_functions():
    @cp.fuse()
    def inner(a, b):
        return a * b

    @cp.fuse()
    def outer(a, b):
        return inner(a, b) + a

    x = shaped_random((64,), 'float32', 20)
    y = shaped_random((64,), 'float32', 21)
    assert_exact(outer(cp.asarray(x), cp.asarray(y)).get(), x * y + x)


def test_fused_where_and_clip_follow_numpy():
    rng = np.random.default_rng(41)
    a = rng.standard_normal((70, 33)).astype(np.float32)
    b = rng.standard_normal((70, 33)).astype(np.float32)

    @cp.fuse()
    def f(x, y):
        return cp.where(x > y, x, y) + cp.clip(x, 0, 1)
    got = f(cp.asarray(a), cp.asarray(b)).get()
    want = np.where(a > b, a, b) + np.clip(a, 0, 1)
    assert got.dtype == want.dtype
    assert np.array_equal(got, want)



def test_functions_beyond_one_kernel_run_as_a_kernel_sequence():
    rng = np.random.default_rng(42)
    a = rng.standard_normal((70, 33)).astype(np.float32)
    b = rng.standard_normal((70, 33)).astype(np.float32)

    @cp.fuse()
    def two_reductions(x):
        return cp.sum(x, axis=1) + cp.amax(x, axis=1)

    @cp.fuse()
    def normalise(x, y):
        return (x - cp.sum(x, axis=0)) * y          # a reduced value meets an array

    for _ in range(2):                                # second call: remembered as a sequence
        got = two_reductions(cp.asarray(a)).get()
        np.testing.assert_allclose(got, a.sum(axis=1) + a.max(axis=1), rtol=1e-5, atol=1e-5)
        got = normalise(cp.asarray(a), cp.asarray(b)).get()
        np.testing.assert_allclose(got, (a - a.sum(axis=0)) * b, rtol=1e-5, atol=1e-5)

    @cp.fuse()
    def broken(x):
        return x + undefined_name                     # noqa: F821
    with pytest.raises(NameError):
        broken(cp.asarray(a))


def test_kernel_sequences_match_numpy():
    rng = np.random.default_rng(43)
    a = rng.standard_normal((301, 77)).astype(np.float32)
    b = rng.standard_normal((301, 77)).astype(np.float32)

    def softmax(xp):
        def f(x):
            e = xp.exp(x - xp.amax(x, axis=1, keepdims=True))
            return e / xp.sum(e, axis=1, keepdims=True)
        return f

    def ratio(xp):
        def f(x, y, s):
            return xp.sum((x - y) ** 2, axis=1) / xp.sum(x * x * s, axis=1)
        return f

    def var0(xp):
        def f(x):
            m = x.sum(axis=0) / x.shape[0]
            return ((x - m) ** 2).sum(axis=0) / x.shape[0]
        return f

    def centred(xp):
        def f(x, y):
            return (x - xp.sum(x) / x.size) * y, xp.amin(y, axis=0)
        return f

    for make, args in ((softmax, (a,)), (ratio, (a, b, 2.0)), (var0, (a,)), (centred, (a, b))):
        want = make(np)(*args)
        fused = cp.fuse(make(cp))
        dev = [cp.asarray(v) if isinstance(v, np.ndarray) else v for v in args]
        for _ in range(2):                                   # plan, then remembered plan
            got = fused(*dev)
            assert fused._plans and all(fused._plans.values())
            if not isinstance(want, tuple):
                got, ref = (got,), (want,)
            else:
                ref = want
            for g, w in zip(got, ref):
                assert g.dtype == w.dtype and g.shape == w.shape
                np.testing.assert_allclose(g.get(), w, rtol=2e-5, atol=2e-5)

    # float16 intermediates round like the eager evaluation
    h = rng.standard_normal((64, 40)).astype(np.float16)

    @cp.fuse()
    def spread(x):
        return (x - cp.amax(x, axis=1, keepdims=True)) * (x - cp.amin(x, axis=1, keepdims=True))
    want = (h - h.max(axis=1, keepdims=True)) * (h - h.min(axis=1, keepdims=True))
    assert_exact(spread(cp.asarray(h)).get(), want)


def test_kernel_sequence_cases_match_numpy():
    from test_fusion_split import CASES
    rng = np.random.default_rng(44)
    captured = rng.uniform(0.5, 1.5, 4).astype(np.float32)
    for name in sorted(CASES):
        make, n_arrays, extra, _, shapes = CASES[name]
        host = [rng.uniform(0.5, 1.5, (6, 5, 4)).astype(np.float32) for _ in range(n_arrays)]
        want = make(np, captured)(*host, *extra)
        fused = cp.fuse(make(cp, cp.asarray(captured)))
        got = fused(*[cp.asarray(h) for h in host], *extra)
        assert all(fused._plans.values()), name
        gots = got if isinstance(got, tuple) else (got,)
        wants = want if isinstance(want, tuple) else (want,)
        for g, w in zip(gots, wants):
            assert g.shape == np.shape(w) and g.dtype == np.asarray(w).dtype, name
            np.testing.assert_allclose(g.get(), w, rtol=1e-5, atol=1e-5, err_msg=name)


@pytest.mark.parametrize('shape', [(301, 77), (70, 33), (64, 4096), (17, 5, 1000), (1000,),
                                   (129, 8192), (300, 1001), (64, 4099), (128, 777), (33, 18),
                                   (5000, 10), (777, 3), (100, 2), (4099, 7),
                                   (70001, 100), (140003, 33), (600001, 5), (66000, 64)])
def test_row_wise_functions_in_one_kernel_match_numpy(shape):
    """Functions whose reductions all run along short rows compile to a single
    kernel that holds the row in registers (wave-per-row and workgroup-per-row
    variants, vector widths 1 to 4, ragged row lengths; with rows in plenty,
    four or two short rows in flight per group of lanes and a last pass that
    has fewer)."""
    rng = np.random.default_rng(45)
    h = rng.standard_normal(shape).astype(np.float32)
    w = rng.uniform(0.5, 1.5, shape[-1]).astype(np.float32)

    def softmax(xp):
        def f(x):
            e = xp.exp(x - xp.amax(x, axis=-1, keepdims=True))
            return e / xp.sum(e, axis=-1, keepdims=True)
        return f

    def layernorm(xp):
        def f(x, g, eps):
            m = xp.sum(x, axis=-1, keepdims=True) / x.shape[-1]
            d = x - m
            v = xp.sum(d * d, axis=-1, keepdims=True) / x.shape[-1]
            return d / xp.sqrt(v + eps) * g, m, v
        return f

    def rownorm(xp):
        def f(x):
            return xp.sqrt(xp.sum(x * x, axis=-1)), xp.amin(x, axis=-1), x * 2
        return f

    from cupy_amd._core import _fusion_rows
    for make, args in ((softmax, (h,)), (layernorm, (h, w, 1e-5)), (rownorm, (h,))):
        want = make(np)(*args)
        fused = cp.fuse(make(cp))
        dev = [cp.asarray(v) if isinstance(v, np.ndarray) else v for v in args]
        for _ in range(2):
            got = fused(*dev)
            (plan,) = fused._plans.values()
            assert isinstance(plan, _fusion_rows.RowPlan), make.__name__
            gots = got if isinstance(got, tuple) else (got,)
            wants = want if isinstance(want, tuple) else (want,)
            for g, wv in zip(gots, wants):
                assert g.shape == np.shape(wv) and g.dtype == np.asarray(wv).dtype
                np.testing.assert_allclose(g.get(), wv, rtol=2e-5, atol=2e-5)
    # float16 rows with float32 weights; a misaligned view of the same shape
    # takes the general route and still agrees
    if len(shape) == 2:
        h16 = h.astype(np.float16)

        @cp.fuse()
        def centre(x, g):
            return (x - cp.amax(x, axis=1, keepdims=True)) * g
        want = (h16 - h16.max(axis=1, keepdims=True)) * w
        got = centre(cp.asarray(h16), cp.asarray(w))
        assert got.dtype == want.dtype
        np.testing.assert_allclose(got.get(), want, rtol=1e-3, atol=1e-3)
        flat = cp.asarray(np.concatenate([[0], h16.ravel()]).astype(np.float16))
        shifted = flat[1:].reshape(shape)           # same shape, data 2 bytes off alignment
        got = centre(shifted, cp.asarray(w))
        np.testing.assert_allclose(got.get(), want, rtol=1e-3, atol=1e-3)


def test_row_kernel_follows_scalars_types_and_captured_arrays():
    rng = np.random.default_rng(46)
    shift = cp.asarray(rng.standard_normal(96).astype(np.float32))      # captured by the function

    @cp.fuse()
    def f(x, y, eps, k):
        m = cp.sum(x * y, axis=1, keepdims=True) / k
        above = (x + shift) > m
        return cp.where(above, x, m) * eps, above, cp.sum(above, axis=1)

    hshift = shift.get()
    for trial, (eps, k) in enumerate(((0.5, 96), (2.0, 7), (np.float32(3), np.int64(5)))):
        hx = rng.integers(-5, 5, (50, 96)).astype(np.int32)
        hy = rng.standard_normal((50, 96)).astype(np.float16)
        got = f(cp.asarray(hx), cp.asarray(hy), eps, k)
        m = np.sum(hx * hy, axis=1, keepdims=True) / k
        above = (hx + hshift) > m
        want = (np.where(above, hx, m) * eps, above, np.sum(above, axis=1))
        for g, w in zip(got, want):
            assert g.dtype == w.dtype and g.shape == w.shape, (trial, g.dtype, w.dtype)
            if w.dtype.kind == 'f':
                np.testing.assert_allclose(g.get(), w, rtol=2e-3, atol=2e-3)
            else:
                # a comparison may flip where x + shift and the mean agree to rounding
                assert (g.get() != w).mean() < 0.01


# ---- in-place operators, out= and indexing inside fused functions --------------------------
# Scenarios of the reference's fusion_tests/test_misc.py:32-54,126-141 and
# test_indexing.py:48-124, evaluated on NumPy and by the fused kernel on the
# same seeded inputs; integer results bit-exact, float results too (every step is
# one IEEE operation in the same order).

ALL_DTYPES = ['int8', 'int16', 'int32', 'int64', 'uint8', 'uint16', 'uint32', 'uint64',
              'float16', 'float32', 'float64']


def _inputs(n, dtype, shape=(3, 4)):
    return [shaped_random(shape, dtype, seed) for seed in range(n)]


def _run_both(make, host_args):
    """Runs ``make(numpy)`` on copies of the host arrays and the fused
    ``make(cupy)`` on device copies; returns (numpy result, numpy args after,
    fused result, device args after)."""
    h = [a.copy() if isinstance(a, np.ndarray) else a for a in host_args]
    d = [cp.asarray(a) if isinstance(a, np.ndarray) else a for a in host_args]
    with np.errstate(all='ignore'):
        want = make(np)(*h)
    got = cp.fuse(make(cp))(*d)
    return want, h, got, d


def _same(got, want):
    if want is None:
        assert got is None
        return
    if isinstance(want, tuple):
        assert isinstance(got, tuple) and len(got) == len(want)
        for g, w in zip(got, want):
            _same(g, w)
        return
    g = got.get() if isinstance(got, cp.ndarray) else np.asarray(got)
    assert g.dtype == np.asarray(want).dtype, (g.dtype, np.asarray(want).dtype)
    assert g.shape == np.asarray(want).shape
    assert np.array_equal(g, want, equal_nan=True)


@pytest.mark.parametrize('dtype', ALL_DTYPES)
def test_out_arguments_mixed(dtype):
    def make(xp):
        def func(x, y, z, u, v):
            xp.add(x, y, out=z)
            xp.subtract(z, x, out=u)
            xp.multiply(z, x, out=v)
            return u
        return func
    want, h, got, d = _run_both(make, _inputs(5, dtype))
    _same(got, want)
    for a, b in zip(d, h):
        _same(a, b)                      # z, u and v were written, x and y were not
    assert got is d[3]


@pytest.mark.parametrize('dtype', ALL_DTYPES)
def test_in_place_add_several_times(dtype):
    def thrice(xp):
        def func(x, y):
            x += y
            x += y
            x += y
            return x
        return func

    def once(xp):
        def func(x):
            x += 2
        return func

    def twice(xp):
        def func(x):
            x += x
            x += x
        return func
    for make, n in ((thrice, 2), (once, 1), (twice, 1)):
        want, h, got, d = _run_both(make, _inputs(n, dtype))
        _same(got, want)
        for a, b in zip(d, h):
            _same(a, b)


@pytest.mark.parametrize('dtype', ['int32', 'uint8', 'float16', 'float32', 'float64', 'bool'])
def test_tuples_swaps_and_casts(dtype):
    def swap(xp):
        def func(x, y, z):
            w = x * y + z
            (x, w) = (w, x)
            return z * w + y + x
        return func

    def triple(xp):
        return lambda x, y, z: (x + y, y + z, z * x)

    def casts(xp):
        def func(x, y, z):
            x = x.astype('int32')
            y = x.astype('float32')
            return x + y, y + z, z + x
        return func
    for make in (swap, triple, casts):
        want, h, got, d = _run_both(make, _inputs(3, dtype))
        _same(got, want)
    x = cp.asarray(_inputs(1, dtype)[0])
    assert cp.fuse(lambda a: ())(x) == ()
    (only,) = cp.fuse(lambda a: (a,))(x)
    assert only is x
    assert cp.fuse(lambda: None)() is None


FUSE_INDICES = [
    1, -1, (1,), (1, 0), (1, 0, 2), (-1, 0, -2), slice(None), slice(None, None, -1),
    (slice(None), slice(None, None, -1)), Ellipsis, None, (None, None, None),
    (slice(None), 0, slice(None, None, -1)), (1, None, slice(None, None, -1), None, 2),
    (Ellipsis, 2), (1, Ellipsis),
]


@pytest.mark.parametrize('indices', FUSE_INDICES, ids=str)
def test_getitem_inside_a_fused_function(indices):
    for dtype in ('int16', 'float32', 'bool'):
        x = shaped_random((2, 3, 4), dtype, 0)
        want, _, got, _ = _run_both(lambda xp: lambda a: a[indices], [x])
        _same(got, want)
        # and as an operand of arithmetic
        want, _, got, _ = _run_both(lambda xp: lambda a: a[indices] + a[indices], [x])
        _same(got, want)
    x4 = shaped_random((2, 3, 4, 5), 'float32', 1)
    want, _, got, _ = _run_both(lambda xp: lambda a: a[1, ..., 3] * 2, [x4])
    _same(got, want)


@pytest.mark.parametrize('dtype1', ['int8', 'int32', 'uint16', 'float16', 'float32', 'float64'])
@pytest.mark.parametrize('dtype2', ['int16', 'uint32', 'float32', 'float64'])
def test_indexing_combined_with_arithmetic(dtype1, dtype2):
    x = shaped_random((3, 4), dtype1, 0)
    y = shaped_random((4,), dtype2, 1)
    z = shaped_random((1,), dtype1, 2)
    cases = [
        lambda xp: lambda x, y, z: x + y[1],
        lambda xp: lambda x, y, z: x + z[0] + y,
        lambda xp: lambda x, y, z: x + x[0] + x[1],
        lambda xp: lambda x, y, z: x + x[0, 1] + x[1] + x + x[2, 1],
        lambda xp: lambda x, y, z: x[0][1],
        lambda xp: lambda x, y, z: x[0][1] + x[1][0],
        lambda xp: lambda x, y, z: x[::-1] - y[::-1],
    ]
    for make in cases:
        want, _, got, _ = _run_both(make, [x, y, z])
        _same(got, want)


def test_in_place_with_reductions_and_overlapping_arguments():
    rng = np.random.default_rng(50)
    a = rng.standard_normal((40, 30)).astype(np.float32)
    b = rng.standard_normal((40, 30)).astype(np.float32)

    def various(xp):
        def func(x, y):
            s = x + y
            t = xp.sum(s, axis=0)
            x += t
            c = xp.sum(x, axis=0)
            y += c
            return c, t, x, y, s
        return func
    want, h, got, d = _run_both(various, [a, b])
    for g, w in zip(got, want):
        np.testing.assert_allclose(g.get(), w, rtol=1e-5, atol=1e-4)
    assert got[2] is d[0] and got[3] is d[1]
    np.testing.assert_allclose(d[0].get(), h[0], rtol=1e-5, atol=1e-4)
    np.testing.assert_allclose(d[1].get(), h[1], rtol=1e-5, atol=1e-4)

    # the written array overlaps another argument: what NumPy does, step by step
    @cp.fuse()
    def shift(x, y):
        x += y
        x += y
        return x
    base = cp.asarray(np.arange(20, dtype=np.float32))
    hbase = np.arange(20, dtype=np.float32)
    shift(base[1:], base[:-1])
    hx, hy = hbase[1:], hbase[:-1]
    hx += hy
    hx += hy
    _same(base, hbase)
    # the same array twice
    c = cp.asarray(a)
    shift(c, c)
    _same(c, a * 4)


def test_division_by_a_value_of_the_row_stays_within_one_ulp():
    """Fused row kernels divide by a value the row shares through its
    reciprocal and one correction step; where that is not safe (reciprocal or
    quotient zero, subnormal, infinite, NaN) they divide.  Against NumPy's
    division: at most one ulp apart, and identical wherever zeros, infinities
    or NaN are involved."""
    rng = np.random.default_rng(71)
    n_rows, n_cols = 4096, 100
    scale = np.float32(2.0) ** rng.integers(-60, 60, (n_rows, 1)).astype(np.float32)
    x = (rng.standard_normal((n_rows, n_cols)) * scale).astype(np.float32)
    # the divisor of row i is column 0 times the row length (all other columns
    # of the divisor operand are zero): every magnitude, and the special values
    d = np.zeros((n_rows, n_cols), np.float32)
    d[:, 0] = (rng.standard_normal(n_rows) * 2.0 ** rng.integers(-100, 100, n_rows)).astype(np.float32)
    specials = [0.0, -0.0, np.inf, -np.inf, np.nan, 1e-39, -1e-39, 1e-45, 3e38, -3e38, 1e-37, 2e37,
                1.0, 3.0, np.float32(1) - np.float32(2) ** -24, 1.9999999]
    d[:len(specials), 0] = specials
    x[::7, 3] = np.inf
    x[::11, 5] = -np.inf
    x[::13, 8] = np.nan
    x[::5, 9] = 0.0
    x[::9, 10] = -0.0
    x[::17, 11] = 1e-40
    x[::19, 12] = 3.3e38
    x[::23, 13] = -1e-45

    @cp.fuse()
    def scaled(x, d):
        return x / cp.sum(d, axis=1, keepdims=True)

    from cupy_amd._core import _fusion_rows
    with np.errstate(all='ignore'):
        want = x / d.sum(axis=1, keepdims=True)
    got = scaled(cp.asarray(x), cp.asarray(d)).get()
    (plan,) = scaled._plans.values()
    assert isinstance(plan, _fusion_rows.RowPlan)
    assert np.array_equal(np.isnan(got), np.isnan(want))
    ok = ~np.isnan(want)
    g, w = got[ok], want[ok]
    # infinities exactly; the sign of every result, zeros included
    assert np.array_equal(np.isinf(g), np.isinf(w))
    assert np.array_equal(np.signbit(g), np.signbit(w))

    def ordered(a):
        """Floats as integers in their own order (one apart = one ulp apart)."""
        bits = a.view(np.int32).astype(np.int64)
        return np.where(bits < 0, -(bits & 0x7fffffff), bits)
    apart = np.abs(ordered(g) - ordered(w))
    assert apart.max() <= 1, apart.max()
    # ... and all but a handful are the correctly rounded quotient itself
    assert (apart != 0).mean() < 1e-3
    # the cases that must take the exact route did get exact results
    exact = np.isinf(w) | (np.abs(w) > 1e30)
    assert np.array_equal(g[exact].view(np.uint32), w[exact].view(np.uint32))
