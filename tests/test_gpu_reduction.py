"""Reduction path on the GPU against NumPy: sums (all dtypes, axes, layouts,
sizes around powers of two), argmax/argmin (ties, NaN, first occurrence),
min/max/any/all/prod and user ReductionKernels.

Tolerances: integer and index results bit-exact; floating-point sums within
rtol 1e-5 (fp32) / 1e-12 (fp64) / 1e-3 (fp16) of NumPy, measured against the
sum of absolute addends (the order of additions differs from NumPy's)."""
import numpy as np
import pytest

import cupy_amd as cp
from helpers import assert_exact, assert_sum_close, shaped_random
from oracle import numpy_oracle as o

pytestmark = pytest.mark.gpu


def check_sum(a, axis=None, keepdims=False, dtype=None, view=None):
    d = cp.asarray(a)
    if view is not None:
        a, d = view(a), view(d)
    got = d.sum(axis=axis, keepdims=keepdims, dtype=dtype)
    expect = a.sum(axis=axis, keepdims=keepdims, dtype=dtype)
    if expect.dtype.kind == 'f':
        mag = np.abs(a.astype(np.float64)).sum(axis=axis, keepdims=keepdims)
        assert_sum_close(got.get(), np.asarray(expect), mag, expect.dtype, data=a, axis=axis)
    else:
        assert_exact(got.get(), np.asarray(expect))
    return got


@pytest.mark.parametrize('dtype', ['bool', 'int8', 'uint8', 'int16', 'uint16', 'int32',
                                   'uint32', 'int64', 'uint64', 'float16', 'float32', 'float64'])
def test_sum_all_dtypes(dtype):
    a = shaped_random((21, 37), dtype, 1, scale=100)
    for axis in (None, 0, 1, (0, 1), -1):
        check_sum(a, axis)
    check_sum(a, 1, keepdims=True)
    check_sum(a, None, keepdims=True)


def test_int8_sums_wrap_like_numpy(small_configs):
    i8 = small_configs['i8']
    d = cp.asarray(i8)
    assert_exact(d.sum(axis=0).get(), small_configs['i8_ax0'])
    assert_exact(d.sum(axis=1).get(), small_configs['i8_ax1'])
    assert_exact(d.sum(axis=0, dtype=np.int8).get(), i8.sum(axis=0, dtype=np.int8))
    assert_exact(d.sum(dtype=np.int8).get(), np.asarray(i8.sum(dtype=np.int8)))


@pytest.mark.parametrize('i', range(1, 14))
def test_sum_sizes_around_powers_of_two(i):
    for n in (2 ** i - 1, 2 ** i, 2 ** i + 1):
        a = shaped_random((n,), 'int8', n, scale=100)
        check_sum(a)
        f = shaped_random((n,), 'float32', n)
        check_sum(f)


@pytest.mark.parametrize('shape', [(2, 1000), (1000, 2), (65, 1000), (1000, 65), (512, 65536 // 64),
                                   (513, 1025), (1, 5000), (5000, 1), (3, 70000), (70000, 3)])
def test_sum_rectangular(shape):
    a = shaped_random(shape, 'float32', 3)
    check_sum(a, 0)
    check_sum(a, 1)
    check_sum(a)
    i = shaped_random(shape, 'int32', 4, scale=1000)
    check_sum(i, 0)
    check_sum(i, 1)


def test_sum_small_config(small_configs):
    c = small_configs
    for name, rtol in (('f32', 1e-5), ('f64', 1e-12)):
        a = c['c3_' + name]
        d = cp.asarray(a)
        for axis, key in ((0, 'ax0'), (1, 'ax1'), (None, 'all')):
            mag = np.abs(a.astype(np.float64)).sum(axis=axis)
            assert_sum_close(d.sum(axis=axis).get(), c['c3_%s_%s' % (name, key)], mag, a.dtype,
                             data=a, axis=axis)


TRANSPOSES = [
    ((2, 3, 4), (1, 0, 2), 0), ((2, 3, 4), (1, 0, 2), 1), ((2, 3, 4), (2, 0, 1), 2),
    ((2, 3, 4), (2, 1, 0), (0, 2)), ((2, 3, 4, 5), (3, 1, 0, 2), (1, 2)),
    ((2, 3, 4, 5), (0, 2, 1, 3), (0, 3)), ((2, 3, 4, 5), (1, 3, 0, 2), None),
    ((6, 0, 4), (1, 0, 2), 2), ((3, 5, 7), (2, 1, 0), (0, 1, 2)),
]


@pytest.mark.parametrize('shape,perm,axis', TRANSPOSES)
def test_sum_of_transposed_views(shape, perm, axis):
    a = shaped_random(shape, 'float64', 5)
    check_sum(a, axis, view=lambda x: x.transpose(perm))
    check_sum(a, axis, keepdims=True, view=lambda x: x.transpose(perm))


def test_sum_strided_and_broadcast_views():
    a = shaped_random((40, 30, 20), 'float32', 6)
    check_sum(a, 1, view=lambda x: x[::2, :, ::3])
    check_sum(a, (0, 2), view=lambda x: x[:, ::-1, 1:])
    check_sum(a, 0, view=lambda x: x[5:6])
    b = shaped_random((64, 1, 32), 'float32', 7)
    d = cp.broadcast_to(cp.asarray(b), (64, 16, 32))
    e = np.broadcast_to(b, (64, 16, 32))
    assert_sum_close(d.sum(axis=2).get(), e.sum(axis=2),
                     np.abs(e.astype(np.float64)).sum(axis=2), np.float32, data=e, axis=2)
    assert_sum_close(d.sum(axis=1).get(), e.sum(axis=1),
                     np.abs(e.astype(np.float64)).sum(axis=1), np.float32, data=e, axis=1)


def test_sum_many_dims_keepdims():
    a = shaped_random((2, 3, 2, 3, 2, 3, 2), 'float64', 8)
    check_sum(a, (1, 3, 4, 6), keepdims=True)
    check_sum(a, (0, 2, 5))


def test_sum_out_and_dtype_arguments():
    a = shaped_random((30, 50), 'float32', 9)
    d = cp.asarray(a)
    out = cp.empty((50,), np.float32)
    assert d.sum(axis=0, out=out) is out
    assert_sum_close(out.get(), a.sum(axis=0), np.abs(a).sum(axis=0, dtype=np.float64), np.float32,
                     data=a, axis=0)
    out64 = cp.empty((30,), np.float64)
    d.sum(axis=1, out=out64)
    assert np.allclose(out64.get(), a.sum(axis=1), rtol=1e-5)
    strided = cp.zeros((30, 2), np.float32)
    d.sum(axis=1, out=strided[:, 1])
    assert np.allclose(strided.get()[:, 1], a.sum(axis=1), rtol=1e-5)
    assert np.all(strided.get()[:, 0] == 0)
    i = shaped_random((30, 50), 'int32', 10)
    assert_exact(cp.asarray(i).sum(axis=0, dtype=np.float64).get(), i.sum(axis=0, dtype=np.float64))
    assert_exact(cp.sum(cp.asarray(i), axis=1).get(), i.sum(axis=1))
    assert_exact(cp.add.reduce(cp.asarray(i), axis=1).get(), np.add.reduce(i, axis=1))


def test_float16_sum_accumulates_in_float32():
    a = np.full((4096,), 0.1, np.float16)
    got = cp.asarray(a).sum().get()
    assert got.dtype == np.float16
    # accumulating in float16 would stall far below the true value
    assert abs(float(got) - float(np.float32(a).sum())) <= 1.0


def test_prod_min_max_any_all():
    a = shaped_random((12, 9), 'float32', 11, scale=2)
    d = cp.asarray(a)
    for axis in (None, 0, 1):
        assert np.allclose(d.prod(axis=axis).get(), a.prod(axis=axis), rtol=1e-4)
        assert_exact(d.max(axis=axis).get(), np.asarray(a.max(axis=axis)))
        assert_exact(d.min(axis=axis).get(), np.asarray(a.min(axis=axis)))
        assert_exact((d > 0).any(axis=axis).get(), np.asarray((a > 0).any(axis=axis)))
        assert_exact((d > -1.9).all(axis=axis).get(), np.asarray((a > -1.9).all(axis=axis)))
    n = a.copy()
    n[3, 4] = np.nan
    dn = cp.asarray(n)
    assert_exact(dn.max(axis=0).get(), n.max(axis=0))
    assert_exact(dn.min(axis=1).get(), n.min(axis=1))
    i = shaped_random((7, 300), 'int16', 12, scale=1000)
    assert_exact(cp.amax(cp.asarray(i), axis=1).get(), i.max(axis=1))
    assert_exact(cp.amin(cp.asarray(i)).get(), np.asarray(i.min()))
    assert np.allclose(d.mean(axis=0).get(), a.mean(axis=0), rtol=1e-5)


# -- argmax / argmin ------------------------------------------------------------------------

@pytest.mark.parametrize('dtype', ['bool', 'int8', 'uint8', 'int16', 'int32', 'uint32', 'int64',
                                   'uint64', 'float16', 'float32', 'float64'])
def test_arg_extreme_golden_cases(golden, dtype):
    dt = np.dtype(dtype)
    for case in golden['argmax_cases']:
        if case.get('float_only') and dt.kind != 'f':
            continue
        a = np.array([float(v) for v in case['values']]).astype(dt)
        got = cp.asarray(a).argmax()
        assert got.dtype == np.int64
        assert int(got.get()) == (case['argmax'] if dt.kind != 'b' else int(np.argmax(a)))
    for case in golden['argmin_cases']:
        if case.get('float_only') and dt.kind != 'f':
            continue
        a = np.array([float(v) for v in case['values']]).astype(dt)
        assert int(cp.asarray(a).argmin().get()) == (
            case['argmin'] if dt.kind != 'b' else int(np.argmin(a)))


@pytest.mark.parametrize('shape', [(2, 3), (3, 1000), (1000, 3), (2, 3, 4), (17, 128), (5, 129),
                                   (300, 2), (9, 4096), (4, 5000)])
def test_arg_extreme_heavy_ties(shape):
    a = shaped_random(shape, 'int32', 13, scale=3)
    d = cp.asarray(a)
    for axis in list(range(len(shape))) + [None, -1]:
        assert_exact(d.argmax(axis=axis).get(), np.asarray(a.argmax(axis=axis)))
        assert_exact(d.argmin(axis=axis).get(), np.asarray(a.argmin(axis=axis)))
    if len(shape) == 2:
        assert_exact(d.argmax(axis=1).get(), o.argmax_first(a, 1))
        assert_exact(d.argmin(axis=0).get(), o.argmin_first(a, 0))


def test_arg_extreme_small_config(small_configs):
    c = small_configs
    d = cp.asarray(c['c4_i32'])
    assert_exact(d.argmax(axis=-1).get(), c['c4_i32_argmax'])
    assert_exact(d.argmin(axis=-1).get(), c['c4_i32_argmin'])
    assert_exact(cp.asarray(c['c4_f32']).argmax(axis=1).get(), c['c4_f32_argmax'])


def test_arg_extreme_nan_positions():
    a = shaped_random((50, 260), 'float32', 14)
    a[3, 100] = np.nan
    a[3, 7] = np.nan          # two NaNs in a row: the first one wins
    a[9, 259] = np.nan
    a[20, 0] = np.nan
    a[:, 33] = np.nan         # a NaN in every row: competes with the others above
    a[3, 7] = np.nan
    d = cp.asarray(a)
    for axis in (0, 1, None):
        assert_exact(d.argmax(axis=axis).get(), np.asarray(a.argmax(axis=axis)))
        assert_exact(d.argmin(axis=axis).get(), np.asarray(a.argmin(axis=axis)))
    h = a.astype(np.float16)
    assert_exact(cp.asarray(h).argmax(axis=1).get(), h.argmax(axis=1))
    assert_exact(cp.asarray(a.astype(np.float64)).argmin(axis=0).get(), a.argmin(axis=0))
    inf = np.array([1.0, np.inf, -np.inf, np.inf, 2.0] * 30, np.float32)
    assert int(cp.asarray(inf).argmax().get()) == 1
    assert int(cp.asarray(inf).argmin().get()) == 2


def test_arg_extreme_layouts_and_options():
    a = shaped_random((6, 7, 8), 'float64', 15, scale=2).round()
    d = cp.asarray(a)
    for perm in ((1, 0, 2), (2, 1, 0), (0, 2, 1)):
        for axis in (0, 1, 2, None):
            assert_exact(d.transpose(perm).argmax(axis=axis).get(),
                         np.asarray(a.transpose(perm).argmax(axis=axis)))
    f = np.asfortranarray(a[0])
    assert_exact(cp.asarray(f).argmax().get(), np.asarray(f.argmax()))   # C-order flattening
    assert_exact(d[::2, :, ::-1].argmin(axis=2).get(), a[::2, :, ::-1].argmin(axis=2))
    assert_exact(d.argmax(axis=1, keepdims=True).get(), a.argmax(axis=1, keepdims=True))
    for dt in (np.int8, np.int16, np.int32, np.int64):
        assert_exact(d.argmax(axis=2, dtype=dt).get(), a.argmax(axis=2).astype(dt))
    out = cp.empty((6, 8), np.int64)
    assert d.argmin(axis=1, out=out) is out
    assert_exact(out.get(), a.argmin(axis=1))
    assert_exact(cp.argmax(d, axis=0).get(), a.argmax(axis=0))


# -- user reduction kernels --------------------------------------------------------------------

def test_l2norm_kernel():
    l2 = cp.ReductionKernel('T x', 'T y', 'x * x', 'a + b', 'y = sqrt(a)', '0', 'l2norm')
    a = np.arange(10, dtype=np.float32).reshape(2, 5)
    assert np.allclose(l2(cp.asarray(a), axis=1).get(), np.sqrt((a * a).sum(axis=1)), rtol=1e-6)
    b = shaped_random((33, 700), 'float64', 16)
    d = cp.asarray(b)
    for axis in (0, 1, None):
        assert np.allclose(l2(d, axis=axis).get(), np.sqrt((b * b).sum(axis=axis)), rtol=1e-12)
    assert np.allclose(l2(d, axis=1, keepdims=True).get(),
                       np.sqrt((b * b).sum(axis=1, keepdims=True)), rtol=1e-12)
    out = cp.empty((700,), np.float64)
    l2(d, out=out, axis=0)
    assert np.allclose(out.get(), np.sqrt((b * b).sum(axis=0)), rtol=1e-12)


def test_multi_input_broadcast_and_scalars():
    dot = cp.ReductionKernel('T x, T y, T scale', 'T z', 'x * y * scale', 'a + b', 'z = a', '0',
                             'scaled_dot')
    x = shaped_random((40, 300), 'float32', 17, scale=1)
    y = shaped_random((300,), 'float32', 18, scale=1)
    got = dot(cp.asarray(x), cp.asarray(y), 2.0, axis=1)
    expect = (x * y * np.float32(2)).sum(axis=1)
    assert np.allclose(got.get(), expect, rtol=1e-5, atol=1e-4)
    got0 = dot(cp.asarray(x), cp.asarray(y), 2.0, axis=0)
    assert np.allclose(got0.get(), (x * y * np.float32(2)).sum(axis=0), rtol=1e-5, atol=1e-4)
    col = shaped_random((40, 1), 'float32', 19, scale=1)
    got = dot(cp.asarray(x), cp.asarray(col), 1.0)
    assert np.allclose(got.get(), (x * col).sum(), rtol=1e-4)


def test_reduce_type_identity_and_post_map():
    # count of positives as int64 even for float input; post map adds a bias
    cnt = cp.ReductionKernel('T x, int64 bias', 'int64 y', 'x > 0 ? 1 : 0', 'a + b',
                             'y = a + bias', '0', 'count_pos', reduce_type='long long')
    a = shaped_random((77, 91), 'float32', 20)
    assert_exact(cnt(cp.asarray(a), 5, axis=0).get(), (a > 0).sum(axis=0) + 5)
    assert_exact(cnt(cp.asarray(a), 0).get(), np.asarray((a > 0).sum()))
    mx = cp.ReductionKernel('T x', 'T y', 'x', 'max(a, b)', 'y = a', '-1e30f', 'my_max')
    assert_exact(mx(cp.asarray(a), axis=1).get(), a.max(axis=1))


def test_raw_input_with_leading_reduce_axes():
    # raw arrays are legal when the reduced axes come first
    k = cp.ReductionKernel(
        'T x, raw T w', 'T y', 'x * w[_j / _out_ind.size()]', 'a + b', 'y = a', '0',
        'weighted_rows')
    x = shaped_random((6, 50), 'float64', 21)
    w = shaped_random((6,), 'float64', 22)
    got = k(cp.asarray(x), cp.asarray(w), axis=0)
    assert np.allclose(got.get(), (x * w[:, None]).sum(axis=0), rtol=1e-12)
    with pytest.raises(NotImplementedError):
        k(cp.asarray(x), cp.asarray(w), axis=1)


def test_large_full_reduction_is_split_and_deterministic():
    a = shaped_random((3_000_001,), 'float32', 23, scale=1)
    d = cp.asarray(a)
    r1 = d.sum().get()
    r2 = d.sum().get()
    assert r1 == r2
    assert abs(float(r1) - o.sum_exact(a)) <= 1e-5 * float(np.abs(a).sum(dtype=np.float64))
    i = shaped_random((3_000_001,), 'int32', 24, scale=2 ** 30)
    assert_exact(cp.asarray(i).sum().get(), np.asarray(i.sum()))
    assert int(cp.asarray(i).argmax().get()) == int(i.argmax())


MIDDLE = [((3, 5, 7), 'int32'), ((33, 65, 311), 'float32'), ((7, 3, 70001), 'int8'),
          ((300, 17, 9), 'float64'), ((2, 2000, 130), 'float16'), ((64, 8, 1031), 'float32'),
          ((5, 1, 1000), 'int16'), ((1, 40, 5000), 'float32'), ((9, 4000, 3), 'int64')]


@pytest.mark.parametrize('shape,dtype', MIDDLE)
def test_reduction_over_a_middle_axis(shape, dtype):
    x = shaped_random(shape, dtype, 21)
    dx = cp.asarray(x)
    if np.dtype(dtype).kind == 'f':
        got = dx.sum(axis=1).get()
        want = x.astype(np.float64).sum(axis=1)
        tol = {'float16': 2e-3, 'float32': 1e-5, 'float64': 1e-12}[dtype]
        scale = np.abs(x.astype(np.float64)).sum(axis=1)
        assert got.dtype == x.sum(axis=1).dtype
        assert np.all(np.abs(got - want) <= tol * np.maximum(scale, 1))
    else:
        assert_exact(dx.sum(axis=1).get(), x.sum(axis=1))
    assert_exact(dx.max(axis=1).get(), x.max(axis=1))
    assert_exact(dx.argmax(axis=1).get(), x.argmax(axis=1))
    assert_exact(dx.argmin(axis=1, keepdims=True).get(), x.argmin(axis=1, keepdims=True))
    assert_exact(dx.min(axis=1, keepdims=True).get(), x.min(axis=1, keepdims=True))
    # a window whose rows and batches are spaced wider than their length
    if shape[0] > 1 and shape[2] > 4:
        w, dw = x[1:, :, 1:-2], dx[1:, :, 1:-2]
        assert_exact(dw.max(axis=1).get(), w.max(axis=1))
        assert_exact(dw.argmax(axis=1).get(), w.argmax(axis=1))
        out = cp.zeros(w.max(axis=1).shape, dtype)
        r = dw.min(axis=1, out=out)
        assert r is out
        assert_exact(out.get(), w.min(axis=1))


def test_middle_axis_of_four_dimensions_and_broadcast_batches():
    x = shaped_random((4, 6, 50, 33), 'int32', 22)
    dx = cp.asarray(x)
    assert_exact(dx.sum(axis=2).get(), x.sum(axis=2))             # (4*6, 50, 33)
    assert_exact(dx.sum(axis=1).get(), x.sum(axis=1))             # (4, 6, 50*33)
    assert_exact(dx.sum(axis=(1, 2)).get(), x.sum(axis=(1, 2)))
    b = np.broadcast_to(x[:1], (5, 6, 50, 33))
    db = cp.broadcast_to(dx[:1], (5, 6, 50, 33))
    assert_exact(db.sum(axis=2).get(), b.sum(axis=2))
    assert_exact(db.argmax(axis=1).get(), b.argmax(axis=1))
    k = cp.ReductionKernel('T x, T y', 'T z', 'x * y', 'a + b', 'z = a', '0', 'dot_middle')
    y = shaped_random((4, 6, 50, 33), 'int32', 23)
    assert_exact(k(dx, cp.asarray(y), axis=2).get(), (x * y).sum(axis=2, dtype=np.int32))


@pytest.mark.parametrize('width', [3, 5, 7, 10, 17, 24, 33, 48, 67, 100, 129, 255])
@pytest.mark.parametrize('dtype', ['int8', 'float16', 'float32', 'float64'])
def test_short_rows_stored_back_to_back(width, dtype):
    for n_rows in (4096, 5000, 70001):
        x = shaped_random((n_rows, width), dtype, 41)
        dx = cp.asarray(x)
        if np.dtype(dtype).kind == 'f':
            got = dx.sum(axis=1).get()
            want = x.astype(np.float64).sum(axis=1)
            tol = {'float16': 2e-3, 'float32': 1e-5, 'float64': 1e-12}[dtype]
            scale = np.abs(x.astype(np.float64)).sum(axis=1)
            assert got.dtype == np.dtype(dtype)
            assert np.all(np.abs(got - want) <= tol * np.maximum(scale, 1))
        else:
            assert_exact(dx.sum(axis=1).get(), x.sum(axis=1))
        assert_exact(dx.max(axis=1).get(), x.max(axis=1))
        assert_exact(dx.argmin(axis=1).get(), x.argmin(axis=1))
        assert_exact(dx.argmax(axis=1).get(), x.argmax(axis=1))
    # rows that start anywhere, and a strided output
    lo, hi = width + 1, width + 1 + (n_rows - 2) * width
    v, dv = x.reshape(-1)[lo:hi].reshape(-1, width), dx.reshape(-1)[lo:hi].reshape(-1, width)
    assert_exact(dv.min(axis=1).get(), v.min(axis=1))
    out = cp.zeros((v.shape[0], 2), dx.dtype)
    dv.max(axis=1, out=out[:, 1])
    assert_exact(out.get()[:, 1], v.max(axis=1))
    assert not out.get()[:, 0].any()


def test_short_rows_with_two_inputs_and_mixed_types():
    k = cp.ReductionKernel('T x, S y', 'float32 z', '(float)x * (float)y', 'a + b', 'z = a', '0',
                           'dot_short_rows')
    x = shaped_random((9000, 11), 'float32', 42)
    y = shaped_random((9000, 11), 'int8', 43)
    got = k(cp.asarray(x), cp.asarray(y), axis=1).get()
    want = (x.astype(np.float64) * y).sum(axis=1)
    np.testing.assert_allclose(got, want, rtol=1e-5, atol=1e-3)
    nan = x.copy()
    nan[::7, 3] = np.nan
    assert_exact(cp.asarray(nan).argmax(axis=1).get(), nan.argmax(axis=1))
    assert_exact(cp.asarray(nan).max(axis=1).get(), nan.max(axis=1))
    np.testing.assert_allclose(cp.nansum(cp.asarray(nan), axis=1).get(), np.nansum(nan, axis=1),
                               rtol=1e-5, atol=1e-4)


@pytest.mark.parametrize('shape,dtype', [((16, 5, 300), 'float32'), ((3, 64, 4099), 'int8'),
                                         ((8, 3, 100000), 'float32'), ((100, 7, 33), 'float64'),
                                         ((2, 2, 2), 'int32'), ((40, 31, 1000), 'float16')])
def test_reduction_over_the_outer_and_the_innermost_axis(shape, dtype):
    x = shaped_random(shape, dtype, 51)
    dx = cp.asarray(x)
    if np.dtype(dtype).kind == 'f':
        tol = {'float16': 2e-3, 'float32': 1e-5, 'float64': 1e-12}[dtype]
        want = x.astype(np.float64).sum(axis=(0, 2))
        scale = np.abs(x.astype(np.float64)).sum(axis=(0, 2))
        got = dx.sum(axis=(0, 2)).get()
        assert got.dtype == np.dtype(dtype)
        assert np.all(np.abs(got - want) <= tol * np.maximum(scale, 1))
        np.testing.assert_allclose(dx.mean(axis=(0, 2)).get().astype(np.float64),
                                   x.astype(np.float64).mean(axis=(0, 2)),
                                   rtol=max(tol, 1e-6), atol=tol * 10)
    else:
        assert_exact(dx.sum(axis=(0, 2)).get(), x.sum(axis=(0, 2)))
        assert_exact(dx.mean(axis=(0, 2)).get(), x.mean(axis=(0, 2)))
    assert_exact(dx.max(axis=(0, 2)).get(), x.max(axis=(0, 2)))
    assert_exact(dx.min(axis=(0, 2), keepdims=True).get(), x.min(axis=(0, 2), keepdims=True))
    assert_exact((dx > 0).any(axis=(0, 2)).get(), (x > 0).any(axis=(0, 2)))
    # windows do not qualify for the two-stage path and must still be right
    if shape[2] > 4:
        w, dw = x[:, :, 1:-1], dx[:, :, 1:-1]
        assert_exact(dw.max(axis=(0, 2)).get(), w.max(axis=(0, 2)))
        # a post-map that asks for the number of reduced elements, after a split
        np.testing.assert_allclose(dw.mean(axis=(0, 2)).get().astype(np.float64),
                                   w.astype(np.float64).mean(axis=(0, 2)), rtol=2e-3, atol=2e-2)
    out = cp.zeros((2 * shape[1],), dx.max().dtype)
    dx.max(axis=(0, 2), out=out[::2])
    assert_exact(out.get()[::2], x.max(axis=(0, 2)))


@pytest.mark.parametrize('width', [3, 7, 10, 33, 100])
def test_short_rows_with_a_row_of_weights_shared_by_all_rows(width):
    rng = np.random.default_rng(44)
    x = rng.standard_normal((50001, width)).astype(np.float32)
    y = rng.standard_normal((50001, width)).astype(np.float32)
    w = rng.uniform(0, 1, width).astype(np.float32)
    k = cp.ReductionKernel('T x, T y, T w', 'T z', '(x - y) * (x - y) * w', 'a + b', 'z = a', '0',
                           'weighted_sqdiff_rows')
    got = k(cp.asarray(x), cp.asarray(y), cp.asarray(w), axis=1).get()
    want = (((x.astype(np.float64) - y) ** 2) * w).sum(axis=1)
    np.testing.assert_allclose(got, want, rtol=2e-5, atol=1e-5)
    fused = cp.fuse(lambda a, b, c: cp.sum((a - b) ** 2 * c, axis=-1))
    np.testing.assert_allclose(fused(cp.asarray(x), cp.asarray(y), cp.asarray(w)).get(), want,
                               rtol=2e-5, atol=1e-5)
    # a value per row beside the row itself: the variance's pivot
    np.testing.assert_allclose(cp.asarray(x).var(axis=1).get(), x.astype(np.float64).var(axis=1),
                               rtol=1e-4, atol=1e-6)
    np.testing.assert_allclose(cp.asarray(x + 1000).std(axis=1, ddof=1).get(),
                               (x + 1000).astype(np.float64).std(axis=1, ddof=1), rtol=2e-3)
    am = cp.ReductionKernel('T x, T w', 'int64 z', 'cupy_pair(x * w, _J)', 'a.v >= b.v ? a : b',
                            'z = a.i', 'cupy_pair(-1e30f, 0)', 'weighted_argmax_rows',
                            reduce_type='cupy_pair',
                            preamble='struct cupy_pair { float v; long long i; '
                                     '__device__ cupy_pair() : v(0), i(0) {} '
                                     '__device__ cupy_pair(float a, long long b) : v(a), i(b) {} };')
    got = am(cp.asarray(x), cp.asarray(w), axis=1).get()
    prod = x * w
    assert np.array_equal(prod[np.arange(len(got)), got], prod.max(axis=1))


@pytest.mark.parametrize('shape', [(40000, 4, 4), (30001, 16, 2), (5000, 2, 32), (20011, 5, 3),
                                   (7001, 9, 7), (1500, 33, 8), (100000, 3, 2), (2049, 100, 5),
                                   (1025, 7, 100), (3, 700, 4, 5), (4096, 2, 128)])
def test_middle_axis_reductions_of_short_slices_with_few_columns(shape):
    """(slices, lines, columns) reduced over the lines: workgroups stage runs
    of whole slices in the LDS."""
    rng = np.random.default_rng(sum(shape))
    axis = len(shape) - 2
    h = rng.integers(-9, 10, shape).astype(np.int32)
    d = cp.asarray(h)
    assert_exact(d.sum(axis=axis).get(), h.sum(axis=axis))
    assert_exact(d.max(axis=axis).get(), h.max(axis=axis))
    assert_exact(d.argmax(axis=axis).get(), h.argmax(axis=axis))          # first of the ties
    assert_exact(d.argmin(axis=axis).get(), h.argmin(axis=axis))
    assert_exact((d > 7).any(axis=axis).get(), (h > 7).any(axis=axis))
    assert_exact(cp.count_nonzero(d, axis=axis).get(), np.count_nonzero(h, axis=axis))
    h8 = h.astype(np.int8)
    assert_exact(cp.asarray(h8).sum(axis=axis).get(), h8.sum(axis=axis))
    assert_exact(cp.asarray(h8).min(axis=axis).get(), h8.min(axis=axis))
    hp = np.where(rng.uniform(size=shape) < 0.3, -1, 1).astype(np.int64)
    assert_exact(cp.asarray(hp).prod(axis=axis).get(), hp.prod(axis=axis))
    out = cp.empty(h.sum(axis=axis, keepdims=True).shape, np.int64)
    d.sum(axis=axis, keepdims=True, out=out)
    assert_exact(out.get(), h.sum(axis=axis, keepdims=True))
    hf = rng.standard_normal(shape)
    df = cp.asarray(hf)
    np.testing.assert_allclose(df.sum(axis=axis).get(), hf.sum(axis=axis), rtol=1e-12, atol=1e-12)
    np.testing.assert_allclose(df.mean(axis=axis).get(), hf.mean(axis=axis), rtol=1e-12, atol=1e-12)
    np.testing.assert_allclose(df.var(axis=axis).get(), hf.var(axis=axis), rtol=1e-10, atol=1e-12)
    hn = hf.astype(np.float32)
    hn[..., ::3, 1] = np.nan
    dn = cp.asarray(hn)
    assert_exact(dn.argmax(axis=axis).get(), hn.argmax(axis=axis))        # the first NaN wins
    np.testing.assert_allclose(cp.nansum(dn, axis=axis).get(),
                               np.nansum(hn.astype(np.float64), axis=axis), rtol=1e-5, atol=1e-5)
    hc = (hf + 1j * rng.standard_normal(shape)).astype(np.complex64)
    np.testing.assert_allclose(cp.asarray(hc).sum(axis=axis).get(),
                               hc.astype(np.complex128).sum(axis=axis), rtol=1e-4, atol=1e-4)
    h16 = rng.uniform(0, 1, shape).astype(np.float16)
    np.testing.assert_allclose(cp.asarray(h16).sum(axis=axis).get().astype(np.float64),
                               h16.astype(np.float64).sum(axis=axis), rtol=2e-3, atol=1e-2)
    # a view that does not start on a 16-byte boundary
    flat = rng.integers(-9, 10, h.size + 1).astype(np.int32)
    assert_exact(cp.asarray(flat)[1:].reshape(shape).sum(axis=axis).get(),
                 flat[1:].reshape(shape).sum(axis=axis))


@pytest.mark.parametrize('width', [2, 3, 5, 7, 10, 12, 17, 33, 67, 100, 129, 255])
@pytest.mark.parametrize('dtype', ['int8', 'float16', 'float32', 'float64', 'complex64'])
def test_columns_of_narrow_matrices(width, dtype):
    """Reductions down the columns of narrow dense matrices walk the matrix as
    one piece of memory (``emit_cols_flat``): every row count modulo the
    kernel's trip, a last vector that is a partial one, every reduction
    family, against NumPy."""
    from cupy_amd._core import _tuning
    from cupy_amd import _dryrun  # noqa: F401
    _tuning.set(cols_flat_min_bytes=0, cols_flat='always')
    try:
        for n_rows in (4096, 5001, 70001):
            x = shaped_random((n_rows, width), dtype, 43)
            dx = cp.asarray(x)
            kind = np.dtype(dtype).kind
            if kind in 'fc':
                got = dx.sum(axis=0).get()
                wide = np.complex128 if kind == 'c' else np.float64
                want = x.astype(wide).sum(axis=0)
                tol = {'float16': 2e-3, 'float32': 1e-5, 'float64': 1e-12, 'complex64': 1e-5}[dtype]
                scale = np.abs(x.astype(wide)).sum(axis=0)
                assert got.dtype == np.dtype(dtype)
                assert np.all(np.abs(got - want) <= tol * np.maximum(scale, 1))
            else:
                assert_exact(dx.sum(axis=0).get(), x.sum(axis=0))
            assert_exact(dx.max(axis=0).get(), x.max(axis=0))
            assert_exact(dx.argmin(axis=0).get(), x.argmin(axis=0))
            assert_exact(dx.argmax(axis=0).get(), x.argmax(axis=0))
            if kind == 'f' and dtype != 'float16':
                v = dx.var(axis=0).get()
                assert np.allclose(v, x.astype(np.float64).var(axis=0), rtol=1e-4)
                m = dx.mean(axis=0).get()
                assert np.allclose(m, x.astype(np.float64).mean(axis=0), rtol=1e-4, atol=1e-5)
            if kind == 'i':
                # (states of four doubles per element: too wide for this
                # kernel's LDS, the column kernel takes them)
                assert np.allclose(dx.var(axis=0).get(), x.var(axis=0), rtol=1e-10)
                assert np.allclose(dx.mean(axis=0).get(), x.mean(axis=0), rtol=1e-12)
        # NaN in one column, keepdims, an output given
        if np.dtype(dtype).kind == 'f':
            x[7, width // 2] = np.nan
            dx = cp.asarray(x)
            assert_exact(dx.max(axis=0, keepdims=True).get(), x.max(axis=0, keepdims=True))
            assert_exact(dx.argmax(axis=0).get(), x.argmax(axis=0))
            out = cp.zeros((width,), dx.dtype)
            cp.nanmax(dx, axis=0, out=out)
            assert_exact(out.get(), np.nanmax(x, axis=0))
    finally:
        _tuning.set(cols_flat_min_bytes=1 << 20, cols_flat=True)


def test_columns_of_a_narrow_matrix_use_the_flat_kernel_and_replay():
    rng = np.random.default_rng(44)
    h = rng.integers(-100, 100, (150007, 131)).astype(np.int32)
    d = cp.asarray(h)
    from cupy_amd.cuda import function
    seen = []
    orig = function.Function.launch_packed
    function.Function.launch_packed = lambda self, grid, *a, **k: (
        seen.append((self.name, grid)), orig(self, grid, *a, **k))[1]
    try:
        got = d.sum(axis=0)
    finally:
        function.Function.launch_packed = orig
    assert [s[0] for s in seen] == ['cupy_sum', 'cupy_sum_combine']
    assert seen[0][1][1] == 1            # one grid dimension: workgroups walk trips, not column blocks
    assert_exact(got.get(), h.sum(axis=0))
    for _ in range(3):                   # replays
        assert_exact(d.sum(axis=0).get(), h.sum(axis=0))
    # a view that starts elsewhere takes the same route when aligned, the
    # column kernel otherwise; both agree with NumPy
    assert_exact(d[4:].sum(axis=0).get(), h[4:].sum(axis=0))
    assert_exact(d[1:].sum(axis=0).get(), h[1:].sum(axis=0))


@pytest.mark.parametrize('mode', ['auto', True, False])
@pytest.mark.parametrize('shape,axis', [((1031, 4099), 0), ((7, 33, 1001), 1), ((300, 70001), 0),
                                        ((4099, 16363), 0), ((64, 2048), 0), ((9, 65, 31277), 1),
                                        ((5000, 129 * 8 + 4), 0)])
def test_column_blocks_numbered_die_by_die(shape, axis, mode):
    """Column reductions whose workgroups are renumbered so that neighbouring
    column blocks run on one compute die (grids that are and are not a multiple
    of eight workgroups, split and unsplit reduce axes, batches): every
    workgroup still takes exactly one (column block, slice) pair."""
    from cupy_amd._core import _tuning
    _tuning.set(cols_xcd=mode)
    try:
        rng = np.random.default_rng(51)
        h = rng.integers(-1000, 1000, shape).astype(np.int32)
        d = cp.asarray(h)
        assert_exact(d.sum(axis=axis).get(), h.sum(axis=axis))
        assert_exact(d.argmax(axis=axis).get(), h.argmax(axis=axis))
        assert_exact(d.min(axis=axis).get(), h.min(axis=axis))
        hf = rng.standard_normal(shape).astype(np.float32)
        got = cp.asarray(hf).sum(axis=axis).get()
        want = hf.astype(np.float64).sum(axis=axis)
        scale = np.abs(hf).astype(np.float64).sum(axis=axis)
        assert np.all(np.abs(got - want) <= 1e-5 * np.maximum(scale, 1))
    finally:
        _tuning.set(cols_xcd='auto')


@pytest.mark.parametrize('via_copy', [True, False])
def test_interleaved_kept_and_reduced_axes_with_a_tiny_innermost_axis(via_copy):
    # kept and reduced axes alternate and the last axis holds a few elements: the
    # input is copied with the reduced axes last and reduced row by row
    from cupy_amd._core import _tuning
    _tuning.set(reduce_via_copy=via_copy)
    try:
        rng = np.random.default_rng(17)
        for shape, dtype in [((83, 126, 40, 4), 'int32'), ((100, 64, 50, 3), 'float32'),
                             ((3000, 50, 3, 2), 'float64'), ((257, 33, 65, 5), 'float16'),
                             ((70000, 8, 5), 'float32')]:
            h = rng.integers(-3, 4, size=shape).astype(dtype)
            d = cp.asarray(h)
            nd = len(shape)
            axes = [(1, 3), (0, 2), (0, 1, 3), (0, 3), (1, 2)] if nd == 4 else [(0, 2)]
            for axis in axes:
                for keepdims in (False, True):
                    got = d.sum(axis=axis, keepdims=keepdims)
                    want = h.sum(axis=axis, keepdims=keepdims, dtype=np.float64 if h.dtype.kind == 'f' else None)
                    assert got.shape == want.shape
                    np.testing.assert_allclose(got.get().astype(np.float64), want, rtol=2e-3)
                np.testing.assert_array_equal(d.max(axis=axis).get(), h.max(axis=axis))
                np.testing.assert_array_equal(d.any(axis=axis).get(), h.any(axis=axis))
                if h.dtype.kind == 'f' and h.dtype.itemsize >= 4:
                    np.testing.assert_allclose(d.var(axis=axis).get(), h.var(axis=axis, dtype=np.float64),
                                               rtol=1e-4)
                    np.testing.assert_allclose(d.mean(axis=axis).get(), h.mean(axis=axis, dtype=np.float64),
                                               rtol=1e-5, atol=1e-6)
            # into a given output, on another stream, from a view
            axis = axes[0]
            out = cp.zeros(h.sum(axis=axis).shape, d.sum(axis=axis).dtype)
            with cp.cuda.Stream() as s:
                v = d[1:]
                v.sum(axis=axis, out=out[1:] if 0 not in axis else out)
                s.synchronize()
            want = h[1:].sum(axis=axis)
            np.testing.assert_allclose((out[1:] if 0 not in axis else out).get().astype(np.float64),
                                       want.astype(np.float64), rtol=2e-3)
            # the same call again (nothing of the copy may be replayed from a record)
            h2 = h + 1
            d2 = cp.asarray(h2)
            for _ in range(2):
                np.testing.assert_array_equal(d2.max(axis=axes[0]).get(), h2.max(axis=axes[0]))
    finally:
        _tuning.set(reduce_via_copy=True)
