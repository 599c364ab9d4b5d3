"""Elementwise path on the GPU against NumPy on the same inputs: user kernels,
ufunc dispatch, broadcasting, memory layouts, scalars.  Tolerance: bit-exact
for +,-,* and every integer/bool result (<= 1 ulp is the stated bar for fp32 /
fp16 elementwise; these operations are expected to hit 0)."""
import numpy as np
import pytest

import cupy_amd as cp
from helpers import assert_exact, assert_ulp, shaped_random

pytestmark = pytest.mark.gpu

ALL = ['bool', 'int8', 'uint8', 'int16', 'uint16', 'int32', 'uint32', 'int64', 'uint64',
       'float16', 'float32', 'float64']
NUMERIC = ALL[1:]


def both(fn, *host_args):
    """fn evaluated with NumPy on host arrays and with cupy on device copies."""
    dev_args = [cp.asarray(a) if isinstance(a, np.ndarray) else a for a in host_args]
    return fn(np, *host_args), fn(cp, *dev_args)


# -- user kernels ---------------------------------------------------------------------

def test_saxpy_small_config(small_configs):
    c = small_configs
    k = cp.ElementwiseKernel('float32 x, float32 y, float32 a', 'float32 z',
                             'z = a * x + y', 'saxpy')
    z = k(cp.asarray(c['c1_x']), cp.asarray(c['c1_y']), 2.5)
    assert_exact(z.get(), c['c1_z'])


@pytest.mark.parametrize('n', [1, 2, 3, 63, 64, 65, 255, 256, 257, 1023, 1025, 4099, 70001])
def test_flat_kernel_all_sizes_and_tails(n):
    x = shaped_random((n,), 'float32', 1)
    y = shaped_random((n,), 'float32', 2)
    k = cp.ElementwiseKernel('T x, T y', 'T z', 'z = x * y - x', 'muladd_sizes')
    assert_exact(k(cp.asarray(x), cp.asarray(y)).get(), x * y - x)


@pytest.mark.parametrize('offset', [0, 1, 2, 3, 5])
def test_unaligned_views(offset):
    n = 5000
    x = shaped_random((n + 8,), 'float32', 3)
    y = shaped_random((n + 8,), 'float16', 4)
    dx, dy = cp.asarray(x), cp.asarray(y)
    got = cp.multiply(dx[offset:offset + n], dy[offset + 1:offset + 1 + n])
    assert_exact(got.get(), x[offset:offset + n] * y[offset + 1:offset + 1 + n])


def test_denormals_and_specials_survive():
    x = np.array([1e-45, -1e-45, 1e-40, 0.0, -0.0, np.inf, -np.inf, np.nan, 3e38] * 40, np.float32)
    y = np.array([-1e-45, 1e-45, 1e-41, -0.0, 0.0, -np.inf, 1.0, 1.0, 3e38] * 40, np.float32)
    k = cp.ElementwiseKernel('float32 x, float32 y, float32 a', 'float32 z',
                             'z = a * x + y', 'saxpy')
    with np.errstate(all='ignore'):
        expect = np.float32(2.5) * x + y
    got = k(cp.asarray(x), cp.asarray(y), 2.5).get()
    assert_exact(got, expect)
    assert np.array_equal(np.signbit(got), np.signbit(expect))


def test_no_fma_contraction():
    rng = np.random.default_rng(12)
    x = rng.uniform(-1, 1, 100000).astype(np.float32)
    y = rng.uniform(-1, 1, 100000).astype(np.float32)
    k = cp.ElementwiseKernel('float32 x, float32 y', 'float32 z', 'z = x * x + y', 'sq_add')
    got = k(cp.asarray(x), cp.asarray(y)).get()
    assert_exact(got, x * x + y)
    fused = (x.astype(np.float64) * x.astype(np.float64) + y.astype(np.float64)).astype(np.float32)
    assert not np.array_equal(fused, got)      # the inputs do distinguish the two


def test_raw_arrays_and_manual_indexing():
    x = shaped_random((6, 7), 'float32', 5)
    dx = cp.asarray(x)
    rev = cp.ElementwiseKernel('raw T x', 'T y', 'y = x[_ind.size() - i - 1]', 'reverse')
    assert_exact(rev(dx, cp.empty((6, 7), np.float32)).get(), x.reshape(-1)[::-1].reshape(6, 7))
    # multi-dimensional index into a transposed (non-contiguous) raw array
    xt = dx.T                       # shape (7, 6)
    k2 = cp.ElementwiseKernel(
        'raw T x, int32 ncol', 'T y',
        'ptrdiff_t idx[] = {i / ncol, i % ncol}; y = x[idx]', 'gather_t2')
    out = k2(xt, 6, size=42)
    assert_exact(out.get(), x.T.reshape(-1))
    # size(), shape(), strides() of a raw array
    meta = cp.ElementwiseKernel(
        'raw T x', 'int64 y',
        'y = i == 0 ? x.size() : i == 1 ? x.shape()[0] : i == 2 ? x.shape()[1] : '
        'i == 3 ? x.strides()[0] : x.strides()[1]', 'carray_meta')
    got = meta(xt, size=5).get()
    assert got.tolist() == [42, 7, 6, 4, 28]
    # linear indexing of a non-contiguous raw array follows C order of the view
    lin = cp.ElementwiseKernel('raw T x', 'T y', 'y = x[i]', 'linear_raw')
    assert_exact(lin(xt, size=42).get(), x.T.reshape(-1))


def test_python_and_numpy_scalars_take_parameter_dtype():
    x = shaped_random((100,), 'int32', 6)
    k = cp.ElementwiseKernel('T x, T y', 'T z', 'z = x + y', 'add_scalar')
    assert_exact(k(cp.asarray(x), 2).get(), x + np.int32(2))
    assert_exact(k(cp.asarray(x), np.int32(7)).get(), x + np.int32(7))
    xf = shaped_random((100,), 'float16', 7)
    assert_exact(k(cp.asarray(xf), 1.5).get(), xf + np.float16(1.5))
    for v in (-1, 2 ** 31 - 1, -2 ** 31):
        assert_exact(k(cp.asarray(x), np.int64(v)).get(), x + np.int64(v).astype(np.int32))
    with pytest.raises(TypeError, match='Type is mismatched'):
        k(cp.asarray(x), cp.asarray(xf))


def test_in_place_and_partial_writes():
    x = shaped_random((1000,), 'float32', 8)
    y = shaped_random((1000,), 'float32', 9)
    acc = cp.ElementwiseKernel('T x', 'T y', 'y += x', 'accumulate')
    dy = cp.asarray(y)
    r = acc(cp.asarray(x), dy)
    assert r is dy
    assert_exact(dy.get(), y + x)
    cond = cp.ElementwiseKernel('T x', 'T y', 'if (x > 0) y = x', 'cond_write')
    dy = cp.asarray(y)
    cond(cp.asarray(x), dy)
    assert_exact(dy.get(), np.where(x > 0, x, y))
    skip = cp.ElementwiseKernel('T x', 'T y', 'if (x <= 0) continue; y = x', 'skip_write')
    dy = cp.asarray(y)
    skip(cp.asarray(x), dy)
    assert_exact(dy.get(), np.where(x > 0, x, y))


def test_multiple_outputs_and_return_forms():
    x = shaped_random((300,), 'float32', 10)
    k = cp.ElementwiseKernel('T x', 'T a, T b', 'a = x + 1; b = x * 2', 'two_out')
    a, b = k(cp.asarray(x))
    assert_exact(a.get(), x + 1)
    assert_exact(b.get(), x * 2)
    k1 = cp.ElementwiseKernel('T x', 'T a', 'a = x', 'ret_tuple', return_tuple=True)
    assert isinstance(k1(cp.asarray(x)), tuple)
    k0 = cp.ElementwiseKernel('T x', 'T a', 'a = x', 'no_ret', no_return=True)
    assert k0(cp.asarray(x)) is None


@pytest.mark.parametrize('block_size', [1, 32, 128, 1024])
def test_block_size_argument(block_size):
    x = shaped_random((5, 7), 'float32', 11)
    k = cp.ElementwiseKernel('raw T x', 'T y', 'y = x[i] * 2', 'dbl_raw')
    assert_exact(k(cp.asarray(x), size=35, block_size=block_size).get(), (x * 2).reshape(-1))


def test_preamble_loop_prep_and_options():
    x = shaped_random((500,), 'float32', 12)
    k = cp.ElementwiseKernel(
        'T x', 'T y', 'y = helper(x) + offset',
        'with_preamble',
        preamble='__device__ float helper(float v) { return v * SCALE; }',
        options=('-DSCALE=3.0f',), loop_prep='const float offset = 0.5f')
    assert_exact(k(cp.asarray(x)).get(), x * np.float32(3) + np.float32(0.5))


# -- ufuncs ------------------------------------------------------------------------------

@pytest.mark.parametrize('name', ['add', 'subtract', 'multiply'])
@pytest.mark.parametrize('dtype', NUMERIC)
def test_arithmetic_same_dtype(name, dtype):
    a = shaped_random((37, 5), dtype, 1)
    b = shaped_random((37, 5), dtype, 2)
    e, g = both(lambda xp, p, q: getattr(xp, name)(p, q), a, b)
    assert_exact(g.get(), e)


@pytest.mark.parametrize('da', ['bool', 'int8', 'uint8', 'int32', 'uint64', 'float16', 'float32',
                                'float64'])
@pytest.mark.parametrize('db', ['bool', 'int8', 'uint16', 'int64', 'float16', 'float32',
                                'float64'])
def test_mixed_dtype_promotion(da, db):
    a = shaped_random((64,), da, 3)
    b = shaped_random((64,), db, 4)
    e, g = both(lambda xp, p, q: xp.add(p, q), a, b)
    assert_exact(g.get(), e)
    e, g = both(lambda xp, p, q: xp.multiply(p, q), a, b)
    assert_exact(g.get(), e)


def test_nep50_examples(golden):
    def run(xp, ex):
        scope = {'array': xp.array, 'uint8': np.uint8, 'int64': np.int64,
                 'float32': np.float32, 'float64': np.float64, 'int16': np.int16,
                 'bool_': np.bool_, 'int32': np.int32, 'int8': np.int8}
        return eval(ex, scope)

    for ex in golden['nep50_examples']:
        if 'array' not in ex:
            continue                     # scalar-only expressions never reach the package
        try:
            with np.errstate(all='ignore'):
                expect = run(np, ex)
        except OverflowError:
            with pytest.raises(OverflowError):
                run(cp, ex)
            continue
        got = run(cp, ex)
        assert_exact(got.get(), np.asarray(expect))


SHAPES = [((10,), (1,)), ((3, 1), (1, 4)), ((2, 1, 4), (3, 1)), ((256, 256), (256, 1)),
          ((5, 6), (6,)), ((1, 1), (7, 3)), ((), (4, 2)), ((2, 3, 4, 5), (4, 1)),
          ((0,), (1,)), ((3, 0, 2), (1, 2))]


@pytest.mark.parametrize('sa,sb', SHAPES)
def test_broadcasting(sa, sb):
    a = shaped_random(sa, 'float32', 5)
    b = shaped_random(sb, 'float64', 6)
    e, g = both(lambda xp, p, q: xp.subtract(p, q), a, b)
    assert_exact(g.get(), e)
    e, g = both(lambda xp, p, q: q * p + p, a, b)
    assert_exact(g.get(), e)


def test_broadcast_mixed_small_config(small_configs):
    c = small_configs
    x = cp.asarray(c['c2_base']).T
    y = cp.asarray(c['c2_y'])
    out = x * y + 1
    assert out.flags.c_contiguous
    assert_exact(out.get(), c['c2_out'])


LAYOUTS = [
    lambda a: a.T,
    lambda a: a[::2],
    lambda a: a[:, ::3],
    lambda a: a[::-1],
    lambda a: a[:, ::-1],
    lambda a: a[1:-1, 2:-2],
    lambda a: a.T[::2, 1::2],
    lambda a: a.reshape(2, -1, a.shape[1]).transpose(1, 0, 2),
    lambda a: a.reshape(2, -1, a.shape[1]).transpose(2, 1, 0),
]


@pytest.mark.parametrize('layout', range(len(LAYOUTS)))
@pytest.mark.parametrize('shape', [(8, 12), (70, 66), (130, 260)])
def test_non_contiguous_operands(layout, shape):
    f = LAYOUTS[layout]
    a = shaped_random(shape, 'float32', 7)
    b = shaped_random(shape, 'float16', 8)
    da, db = cp.asarray(a), cp.asarray(b)
    assert_exact(cp.add(f(da), f(db)).get(), f(a) + f(b))
    assert_exact(cp.multiply(f(da), 3).get(), f(a) * 3)
    # strided destination
    out = cp.zeros(shape, np.float32)
    cp.subtract(f(da), f(db), out=f(out))
    expect = np.zeros(shape, np.float32)
    np.subtract(f(a), f(b), out=f(expect))
    assert_exact(out.get(), expect)


@pytest.mark.parametrize('rows,cols', [(1, 64), (64, 1), (63, 65), (64, 64), (65, 63), (200, 7),
                                       (7, 200), (129, 513)])
def test_transposed_times_row_broadcast(rows, cols):
    base = shaped_random((cols, rows), 'float32', 9)
    y = shaped_random((1, cols), 'float16', 10)
    col = shaped_random((rows, 1), 'float32', 11)
    d = cp.asarray(base)
    assert_exact((d.T * cp.asarray(y)).get(), base.T * y)
    assert_exact((d.T + cp.asarray(col)).get(), base.T + col)
    assert_exact((d.T - d.T).get(), base.T - base.T)
    # transposed destination too
    out = cp.zeros((cols, rows), np.float32)
    cp.multiply(d.T, 2, out=out.T)
    assert_exact(out.get(), (base.T * 2).T.copy())


def test_out_argument_forms_and_overlap():
    a = shaped_random((50,), 'float32', 12)
    da = cp.asarray(a)
    out = cp.empty((50,), np.float32)
    assert cp.add(da, 1, out) is out
    assert cp.add(da, 1, out=out) is out
    assert_exact(out.get(), a + 1)
    # in place
    db = cp.asarray(a)
    db += 2
    db *= db
    assert_exact(db.get(), (a + 2) * (a + 2))
    # input overlapping the output with a shift is read before it is written
    dc = cp.asarray(a)
    cp.add(dc[:-1], 0, out=dc[1:])
    assert_exact(dc.get(), np.concatenate([a[:1], a[:-1]]))


def test_where_mask():
    a = shaped_random((40, 3), 'float32', 13)
    m = shaped_random((40, 3), 'bool', 14)
    out0 = shaped_random((40, 3), 'float32', 15)
    d = cp.asarray(out0)
    cp.add(cp.asarray(a), 5, out=d, _where=cp.asarray(m))
    expect = out0.copy()
    np.add(a, 5, out=expect, where=m)
    assert_exact(d.get(), expect)


@pytest.mark.parametrize('name', ['negative', 'absolute', 'square', 'sign', 'floor', 'ceil',
                                  'trunc', 'rint', 'sqrt', 'reciprocal', 'isnan', 'isinf',
                                  'isfinite', 'logical_not'])
def test_exact_unary_ufuncs(name):
    for dtype in ('float16', 'float32', 'float64'):
        a = shaped_random((333,), dtype, 16, scale=4)
        a[::17] = np.nan
        a[5::29] = np.inf
        a[7::31] = 0
        with np.errstate(all='ignore'):
            e, g = both(lambda xp, p: getattr(xp, name)(p), a)
        assert_ulp(g.get(), e, 0 if name != 'reciprocal' else 1)
    if name in ('negative', 'absolute', 'square', 'sign', 'logical_not'):
        for dtype in ('int8', 'int32', 'int64', 'uint16'):
            if name == 'negative' and dtype.startswith('u'):
                continue
            a = shaped_random((100,), dtype, 17)
            e, g = both(lambda xp, p: getattr(xp, name)(p), a)
            assert_exact(g.get(), e)


@pytest.mark.parametrize('name', ['exp', 'log', 'sin', 'cos', 'tanh', 'log1p', 'expm1', 'arctan'])
def test_transcendental_ufuncs_are_close(name):
    # device libm vs host libm: not bit-identical by contract (parity unpinned),
    # checked to a few ulp
    a = np.abs(shaped_random((1000,), 'float32', 18, scale=3)) + np.float32(0.01)
    e, g = both(lambda xp, p: getattr(xp, name)(p), a)
    assert g.dtype == e.dtype
    assert np.allclose(g.get(), e, rtol=2e-6, atol=1e-7)
    a64 = a.astype(np.float64)
    e, g = both(lambda xp, p: getattr(xp, name)(p), a64)
    assert np.allclose(g.get(), e, rtol=1e-14, atol=1e-15)


@pytest.mark.parametrize('name', ['less', 'less_equal', 'greater', 'greater_equal', 'equal',
                                  'not_equal', 'maximum', 'minimum', 'logical_and', 'logical_or',
                                  'logical_xor'])
def test_comparison_and_minmax(name):
    for dtype in ('int32', 'uint8', 'float32', 'float16'):
        a = shaped_random((200,), dtype, 19, scale=3)
        b = shaped_random((200,), dtype, 20, scale=3)
        if np.dtype(dtype).kind == 'f':
            a[::11] = np.nan
            b[::13] = np.nan
        e, g = both(lambda xp, p, q: getattr(xp, name)(p, q), a, b)
        assert_exact(g.get(), e)


@pytest.mark.parametrize('name', ['bitwise_and', 'bitwise_or', 'bitwise_xor', 'left_shift',
                                  'right_shift'])
def test_bitwise(name):
    for dtype in ('int8', 'uint8', 'int32', 'uint64'):
        a = shaped_random((200,), dtype, 21, scale=100)
        b = shaped_random((200,), dtype, 22, scale=5)
        if name.endswith('shift'):
            b = np.abs(b).astype(dtype)
        e, g = both(lambda xp, p, q: getattr(xp, name)(p, q), a, b)
        assert_exact(g.get(), e)
    a = shaped_random((50,), 'bool', 23)
    e, g = both(lambda xp, p: xp.invert(p), a)
    assert_exact(g.get(), e)


def test_division_family():
    for dtype in ('int32', 'int8', 'uint16', 'float32', 'float64'):
        a = shaped_random((300,), dtype, 24, scale=50)
        b = shaped_random((300,), dtype, 25, scale=7)
        b[b == 0] = 3
        e, g = both(lambda xp, p, q: xp.true_divide(p, q), a, b)
        assert_ulp(g.get(), e, 0)
        e, g = both(lambda xp, p, q: xp.floor_divide(p, q), a, b)
        assert_ulp(g.get(), e, 0)
        e, g = both(lambda xp, p, q: xp.remainder(p, q), a, b)
        assert_ulp(g.get(), e, 1 if np.dtype(dtype).kind == 'f' else 0)


def test_power():
    a = shaped_random((200,), 'int32', 26, scale=6)
    b = np.abs(shaped_random((200,), 'int32', 27, scale=5))
    e, g = both(lambda xp, p, q: xp.power(p, q), a, b)
    assert_exact(g.get(), e)
    x = np.abs(shaped_random((200,), 'float32', 28, scale=3))
    d = cp.asarray(x)
    assert_exact((d ** 2).get(), x ** 2)
    assert_exact((d ** 0.5).get(), x ** 0.5)
    xh = shaped_random((200,), 'float16', 29, scale=3)
    assert_exact((cp.asarray(xh) ** 2).get(), xh ** 2)
    e = x ** np.float32(1.7)
    assert np.allclose((d ** 1.7).get(), e, rtol=1e-5)


@pytest.mark.parametrize('src', ALL)
@pytest.mark.parametrize('dst', ALL)
def test_astype_all_pairs(src, dst):
    a = shaped_random((120,), src, 30, scale=100)
    if np.dtype(src).kind == 'f' and np.dtype(dst).kind in 'iub':
        a = np.abs(a) if np.dtype(dst).kind == 'u' else a
        a = np.trunc(a).astype(src)          # conversions of in-range integers only
        if np.dtype(dst).itemsize == 1:
            a = (a % 100).astype(src)
    if np.dtype(src).kind == 'i' and np.dtype(dst).kind == 'u':
        a = np.abs(a)
    with np.errstate(all='ignore'):
        expect = a.astype(dst)
    got = cp.asarray(a).astype(dst)
    assert_exact(got.get(), expect)


def test_float64_to_float16_rounds_once():
    # values that round differently when passing through float32 first
    vals = np.array([1.0 + 2.0 ** -11 + 2.0 ** -30, 1.0 + 2.0 ** -11 - 2.0 ** -30,
                     2049.0 + 1e-9, 65519.999, 6.0e-8 + 1e-12], np.float64)
    vals = np.tile(vals, 30)
    assert_exact(cp.asarray(vals).astype(np.float16).get(), vals.astype(np.float16))


def test_copy_fill_and_views():
    a = shaped_random((6, 5, 4), 'float32', 31)
    d = cp.asarray(a)
    assert_exact(d.copy().get(), a)
    assert_exact(d.T.copy().get(), a.T.copy())
    assert d.T.copy().flags.c_contiguous
    assert_exact(d.transpose(1, 2, 0)[::2, 1:].get(), a.transpose(1, 2, 0)[::2, 1:])
    assert_exact(d.reshape(30, 4).get(), a.reshape(30, 4))
    assert_exact(d.T.reshape(-1).get(), a.T.reshape(-1))
    f = cp.empty((5, 3), np.int16)
    f.fill(-7)
    assert_exact(f.get(), np.full((5, 3), -7, np.int16))
    z = cp.zeros((4, 4), np.float64)
    z[1:3, ::2] = 2.5
    e = np.zeros((4, 4))
    e[1:3, ::2] = 2.5
    assert_exact(z.get(), e)
    z[...] = cp.asarray(e.T.copy()).T
    assert_exact(z.get(), e)
    assert_exact(cp.arange(10).get(), np.arange(10))
    assert_exact(cp.arange(2, 11, 3, dtype=np.float32).get(), np.arange(2, 11, 3, dtype=np.float32))
    assert_exact(cp.ones((3,), np.int8).get(), np.ones(3, np.int8))
    assert_exact(cp.full((2, 2), 3.5).get(), np.full((2, 2), 3.5))
    fo = cp.asarray(np.asfortranarray(a[0]))
    assert fo.flags.f_contiguous
    assert_exact(fo.get(), a[0])
    assert_exact((fo + fo).get(), a[0] + a[0])


def test_numpy_ufunc_dispatch_and_reflected_operators():
    a = shaped_random((30,), 'float32', 32)
    d = cp.asarray(a)
    assert_exact(np.add(d, 1).get(), a + 1)
    assert_exact((1 + d).get(), 1 + a)
    assert_exact((2 - d).get(), 2 - a)
    assert_exact((np.float32(3) * d).get(), np.float32(3) * a)
    assert_exact(np.multiply(d, d).get(), a * a)
    assert_exact((-d).get(), -a)
    assert_exact(abs(d).get(), abs(a))


def test_cuda_array_interface_round_trip():
    a = shaped_random((4, 6), 'float32', 33)
    d = cp.asarray(a)

    class Foreign:
        def __init__(self, arr):
            self.arr = arr
            self.__cuda_array_interface__ = arr.__cuda_array_interface__

    f = Foreign(d[:, ::2])
    assert_exact(cp.add(f, 1).get(), a[:, ::2] + 1)
    assert np.allclose(cp.asarray(f).sum(axis=0).get(), a[:, ::2].sum(axis=0), rtol=1e-5)
    assert d.__cuda_array_interface__['strides'] is None
    assert d.T.__cuda_array_interface__['strides'] == d.T.strides


# -- permuted operands of three and four dimensions -------------------------------------

import itertools


@pytest.mark.parametrize('shape', [(5, 70, 130), (33, 65, 31), (2, 129, 257), (64, 3, 200)])
@pytest.mark.parametrize('dtype', ['float32', 'int8', 'float64'])
def test_every_permutation_of_three_axes(shape, dtype):
    x = shaped_random(shape, dtype, 31)
    dx = cp.asarray(x)
    for perm in itertools.permutations(range(3)):
        t, dt = x.transpose(perm), dx.transpose(perm)
        assert_exact(cp.ascontiguousarray(dt).get(), np.ascontiguousarray(t))
        y = shaped_random(t.shape, dtype, 32)
        assert_exact((dt + cp.asarray(y)).get(), t + y)
        # both operands permuted, differently
        u = shaped_random(shape[::-1], dtype, 33)
        du = cp.asarray(u)
        if u.T.shape == t.shape:
            assert_exact((dt * du.T).get(), t * u.T)


@pytest.mark.parametrize('perm', [(0, 2, 1, 3), (0, 1, 3, 2), (2, 0, 1, 3), (3, 1, 2, 0),
                                  (1, 0, 3, 2), (0, 3, 1, 2), (3, 2, 1, 0)])
def test_permutations_of_four_axes(perm):
    shape = (3, 17, 66, 35)
    x = shaped_random(shape, 'float32', 34)
    dx = cp.asarray(x)
    t, dt = x.transpose(perm), dx.transpose(perm)
    assert_exact(cp.ascontiguousarray(dt).get(), np.ascontiguousarray(t))
    row = shaped_random((t.shape[-1],), 'float32', 35)
    assert_exact((dt * cp.asarray(row)).get(), t * row)
    col = shaped_random(t.shape[:2] + (1, 1), 'float32', 36)
    assert_exact((dt - cp.asarray(col)).get(), t - col)
    out = cp.zeros(t.shape, 'float32')
    cp.negative(dt, out=out)
    assert_exact(out.get(), -t)


def test_permuted_windows_and_mixed_types():
    x = shaped_random((20, 70, 90), 'float16', 37)
    y = shaped_random((90, 20, 70), 'float32', 38)
    dx, dy = cp.asarray(x), cp.asarray(y)
    a, da = x[1:, 2:-3, 5:], dx[1:, 2:-3, 5:]
    b, db = y.transpose(1, 2, 0)[1:, 2:-3, 5:], dy.transpose(1, 2, 0)[1:, 2:-3, 5:]
    assert_exact((da + db).get(), a + b)
    assert_exact((da.transpose(1, 0, 2) > db.transpose(1, 0, 2)).get(),
                 a.transpose(1, 0, 2) > b.transpose(1, 0, 2))


def test_reduce_dims_false_keeps_the_axes_for_the_kernel():
    """``reduce_dims=False`` (cupy/_core/_kernel.pyx:802-868): the kernel sees the
    broadcast arguments with all their axes, so ``_ind.get()[k]`` is the index
    along axis k and raw arrays can be addressed with it."""
    k = cp.ElementwiseKernel(
        'T x', 'int64 y',
        'y = _ind.get()[0] * 10000 + _ind.get()[1] * 100 + _ind.get()[2] + (x > 1e30f ? 1 : 0)',
        'multi_index', reduce_dims=False)
    x = cp.asarray(np.zeros((7, 11, 13), np.float32))
    i0, i1, i2 = np.meshgrid(np.arange(7), np.arange(11), np.arange(13), indexing='ij')
    assert_exact(k(x).get(), (i0 * 10000 + i1 * 100 + i2).astype(np.int64))
    # a transposed view keeps its axes too
    got = k(x.transpose(2, 0, 1)).get()
    j0, j1, j2 = np.meshgrid(np.arange(13), np.arange(7), np.arange(11), indexing='ij')
    assert_exact(got, (j0 * 10000 + j1 * 100 + j2).astype(np.int64))
    # gather along the last two axes of a raw array with the loop's own indices
    g = cp.ElementwiseKernel(
        'raw T src, int32 row', 'T out',
        'ptrdiff_t idx[2] = {row, _ind.get()[1]}; out = src[idx]', 'gather_rows',
        reduce_dims=False)
    src = np.arange(5 * 6, dtype=np.float32).reshape(5, 6)
    rows = np.array([[4], [0], [2]], np.int32)
    out = g(cp.asarray(src), cp.broadcast_to(cp.asarray(rows), (3, 6)))
    assert_exact(out.get(), src[rows[:, 0]])


@pytest.mark.parametrize('shape', [(100003, 3), (3, 100003), (65536, 15), (31, 40001), (50000, 32),
                                   (2, 70001), (4099, 1), (7, 5, 20001, 3), (6, 3, 20001),
                                   # widths that are no power of two: longer tiles
                                   (30011, 12), (24, 30011), (20001, 26), (28, 9001), (70001, 20),
                                   (18, 33333),
                                   # odd widths: the staged tile is read as one piece
                                   (40001, 31), (50001, 17), (70001, 7), (4, 30001, 5), (1, 3),
                                   (300, 13)])
def test_transposes_of_narrow_arrays(shape):
    """Points as rows of a few coordinates to or from a few long rows: tiles as
    narrow as the array."""
    rng = np.random.default_rng(sum(shape))
    perm = tuple(range(len(shape) - 2)) + (len(shape) - 1, len(shape) - 2)
    for dtype in (np.float32, np.float64, np.int8, np.complex64, np.float16):
        h = (rng.uniform(-100, 100, shape)).astype(dtype)
        d = cp.asarray(h)
        ht = np.swapaxes(h, -1, -2)
        dt = d.transpose(perm)
        assert_exact(cp.ascontiguousarray(dt).get(), np.ascontiguousarray(ht))
        if np.dtype(dtype).kind == 'f':
            other = rng.uniform(1, 2, ht.shape).astype(dtype)
            assert_exact((dt * cp.asarray(other)).get(), ht * other)
            assert_exact((dt + dt).get(), ht + ht)
    # a view that does not start on a 16-byte boundary
    n = int(np.prod(shape))
    flat = rng.integers(-9, 10, n + 1).astype(np.int32)
    got = cp.ascontiguousarray(cp.asarray(flat)[1:].reshape(shape).transpose(perm)).get()
    assert_exact(got, np.ascontiguousarray(np.swapaxes(flat[1:].reshape(shape), -1, -2)))


@pytest.mark.parametrize('perm', [(0, 1, 2), (2, 1, 0), (1, 2, 0)])
def test_orders_of_reshape_ravel_flatten_and_get(perm):
    """(reference: cupy/_core/_routines_manipulation.pyx:135-208, core.pyx:2098-2160)"""
    rng = np.random.default_rng(17)
    h = rng.standard_normal((6, 10, 14)).astype(np.float32).transpose(perm)
    d = cp.asarray(np.ascontiguousarray(h.transpose(np.argsort(perm)))).transpose(perm)
    assert d.strides == h.strides
    for order in ('C', 'F', 'A', 'K'):
        assert np.array_equal(d.ravel(order=order).get(), h.ravel(order=order)), order
        assert np.array_equal(d.flatten(order=order).get(), h.flatten(order=order)), order
    for order in ('C', 'F', 'A'):
        want = h.reshape((20, 42), order=order)
        assert np.array_equal(d.reshape((20, 42), order=order).get(), want), order
        got = d.get(order=order)
        assert np.array_equal(got, h)
        assert got.flags.f_contiguous == np.asarray(h, order=order).flags.f_contiguous
    out = np.empty(h.shape, np.float32, order='F')
    assert d.get(out=out) is out and np.array_equal(out, h)
    part = d[1:, ::2]
    assert np.array_equal(part.get(order='F'), h[1:, ::2])
    assert part.get(order='F').flags.f_contiguous


@pytest.mark.parametrize('mode,strip', [('auto', 16), (True, 16), (True, 3), (True, 64), (False, 16)])
@pytest.mark.parametrize('shape', [(1031, 2053), (2049, 515), (127, 4099), (3001, 129), (1024, 1040)])
def test_tiles_numbered_die_by_die(shape, mode, strip):
    """Transposed operands whose rows do not start on cache lines: the tiles are
    renumbered so that a compute die works on neighbouring ones (strips of
    tiles, a last strip that is narrower, tile counts that are no multiple of
    eight).  Every tile must still be visited exactly once."""
    from cupy_amd._core import _tuning
    _tuning.set(tiled_xcd=mode, tiled_xcd_strip=strip)
    try:
        rng = np.random.default_rng(61)
        a = rng.integers(-1000, 1000, shape).astype(np.int32)
        b = rng.integers(-1000, 1000, shape[::-1]).astype(np.int32)
        da, db = cp.asarray(a), cp.asarray(b)
        assert_exact(cp.ascontiguousarray(da.T).get(), np.ascontiguousarray(a.T))
        assert_exact((da.T + db).get(), a.T + b)
        out = cp.full(shape, -7, np.int32)
        cp.add(db.T, da, out=out)
        assert_exact(out.get(), b.T + a)
        # a batch of such matrices
        c = rng.integers(-1000, 1000, (5,) + shape[::-1]).astype(np.int32)[:, :301, :257]
        dc = cp.asarray(c)
        assert_exact(cp.ascontiguousarray(dc.transpose(0, 2, 1)).get(),
                     np.ascontiguousarray(c.transpose(0, 2, 1)))
        assert_exact(cp.ascontiguousarray(dc.transpose(2, 1, 0)).get(),
                     np.ascontiguousarray(c.transpose(2, 1, 0)))
    finally:
        _tuning.set(tiled_xcd='auto', tiled_xcd_strip=16)
