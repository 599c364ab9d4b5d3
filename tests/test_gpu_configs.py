"""The five benchmark configurations at their full shapes, compared with NumPy
evaluating the same expression on the same seeded inputs, plus size-independent
properties of each operation.  Stated bars: bit-exact integers and indices,
<= 1 ulp elementwise, rtol 1e-5 (fp32) / 1e-12 (fp64) for sums."""
import numpy as np
import pytest

import cupy_amd as cp
from helpers import assert_exact, assert_sum_close, assert_ulp, check_sum_forward
from oracle import numpy_oracle as o

pytestmark = pytest.mark.gpu


def test_c1_saxpy_full():
    n = 1 << 26
    rng = np.random.default_rng(1)
    x = rng.uniform(-1, 1, n).astype(np.float32)
    y = rng.uniform(-1, 1, n).astype(np.float32)
    k = cp.ElementwiseKernel('float32 x, float32 y, float32 a', 'float32 z',
                             'z = a * x + y', 'saxpy')
    dx, dy = cp.asarray(x), cp.asarray(y)
    z = k(dx, dy, 2.5)
    assert_ulp(z.get(), o.saxpy(2.5, x, y), 1)
    assert_exact(z.get(), o.saxpy(2.5, x, y))
    # properties: a = 0 returns y exactly; a = 1, y = -x cancels to zero
    assert_exact(k(dx, dy, 0.0).get(), y)
    neg = cp.negative(dx)
    assert not k(dx, neg, 1.0).any()


def test_c2_broadcast_mixed_full():
    m = 8192
    rng = np.random.default_rng(2)
    base = rng.standard_normal((m, m), dtype=np.float32)
    y = rng.uniform(0, 2, (1, m)).astype(np.float16)
    db = cp.asarray(base)
    dx = db.T
    dy = cp.asarray(y)
    assert not dx.flags.c_contiguous
    out = dx * dy + 1
    assert out.dtype == np.float32 and out.shape == (m, m) and out.flags.c_contiguous
    expect = o.broadcast_mul_add(base.T, y, 1)
    assert_ulp(out.get(), expect, 1)
    assert_exact(out.get(), expect)
    # property: transposing back reproduces multiplication by a column vector
    back = (dx * dy).T
    assert_exact(back.get(), base * y.T)


@pytest.mark.parametrize('dtype,n,seed', [('float32', 16384, 3), ('float64', 8192, 4)])
def test_c3_sums_full(dtype, n, seed):
    rng = np.random.default_rng(seed)
    a = rng.standard_normal((n, n), dtype=np.float32) if dtype == 'float32' \
        else rng.standard_normal((n, n))
    d = cp.asarray(a)
    mag = np.abs(a)
    s1 = d.sum(axis=1)
    s0 = d.sum(axis=0)
    sa = d.sum()
    # backward bound (rtol * sum|a|) AND forward bound on the result itself:
    # |got - float64 sum| <= rtol * max(|float64 sum|, sigma * sqrt(N reduced))
    r1 = assert_sum_close(s1.get(), o.sum_fp(a, 1), mag.sum(axis=1, dtype=np.float64), dtype,
                          data=a, axis=1)
    r0 = assert_sum_close(s0.get(), o.sum_fp(a, 0), mag.sum(axis=0, dtype=np.float64), dtype,
                          data=a, axis=0)
    ra = assert_sum_close(sa.get(), np.asarray(o.sum_fp(a)), mag.sum(dtype=np.float64), dtype,
                          data=a, axis=None)
    print('forward bound, largest err/bound: axis=1 %.3g, axis=0 %.3g, all %.3g' % (r1, r0, ra))
    # the gate bites: had the kernel dropped one partial result's worth of input
    # (131072 consecutive elements = 1/2048 of the f32 matrix), the value it
    # would have produced -- the sum of everything else -- is rejected
    chunk = 131072
    cut = a.reshape(-1)[5 * chunk:6 * chunk]
    missing = np.asarray(float(sa.get()) - cut.sum(dtype=np.float64)).astype(a.dtype)
    assert check_sum_forward(missing, a, None, dtype) > 1.0
    rows = chunk // n
    short1 = s1.get().copy()
    short1[:rows] = 0
    assert check_sum_forward(short1, a, 1, dtype) > 1.0
    # a sum of sums is the same total, whichever axis goes first
    t1 = float(s1.astype(np.float64).sum().get())
    t0 = float(s0.astype(np.float64).sum().get())
    total = float(mag.sum(dtype=np.float64))
    rtol = 1e-5 if dtype == 'float32' else 1e-12
    assert abs(t1 - t0) <= rtol * total
    assert abs(t1 - float(sa.get())) <= rtol * total
    # linearity: sum(2a) == 2 sum(a) exactly (scaling by two is exact)
    assert_exact((d * 2).sum(axis=1).get(), (s1 * 2).get())


def test_c4_argmax_argmin_int32_full():
    rng = np.random.default_rng(5)
    a = rng.integers(0, 16, (1 << 20, 128), dtype=np.int32)
    d = cp.asarray(a)
    imax = d.argmax(axis=-1)
    imin = d.argmin(axis=-1)
    assert imax.dtype == np.int64 and imax.shape == (1 << 20,)
    assert_exact(imax.get(), o.argmax_fast(a, -1))
    assert_exact(imin.get(), o.argmin_fast(a, -1))
    assert_exact(imax.get(), a.argmax(axis=-1))
    # first occurrence: nothing before the reported index attains the maximum
    rows = np.arange(a.shape[0])
    got = imax.get()
    best = a[rows, got]
    assert np.array_equal(best, a.max(axis=1))
    before = np.arange(128)[None, :] < got[:, None]
    assert not np.any((a == best[:, None]) & before)
    # negating the data swaps argmax and argmin
    assert_exact((-d).argmin(axis=-1).get(), got)


def test_c4_argmax_float32_full():
    rng = np.random.default_rng(6)
    a = rng.standard_normal((1 << 16, 4096), dtype=np.float32)
    d = cp.asarray(a)
    got = d.argmax(axis=1)
    assert_exact(got.get(), a.argmax(axis=1))
    # planted NaNs win, first one per row
    a[5, 4000] = np.nan
    a[5, 17] = np.nan
    a[70, 4095] = np.nan
    assert_exact(cp.asarray(a).argmax(axis=1).get(), a.argmax(axis=1))


def test_c5_fused_full():
    rows = 1 << 18
    rng = np.random.default_rng(7)
    x = rng.standard_normal((rows, 256)).astype(np.float16)
    y = rng.standard_normal((rows, 256)).astype(np.float16)
    w = rng.uniform(0, 1, 256).astype(np.float32)

    @cp.fuse()
    def f(x, y, w):
        return cp.sum((x - y) ** 2 * w, axis=-1)

    dx, dy, dw = cp.asarray(x), cp.asarray(y), cp.asarray(w)
    got = f(dx, dy, dw)
    assert got.dtype == np.float32 and got.shape == (rows,)
    expect = o.fused_sqdiff_wsum(x, y, w)
    assert np.allclose(got.get(), expect, rtol=1e-5, atol=0)
    # symmetric in x and y; zero for identical inputs; one launch only
    assert_exact(f(dy, dx, dw).get(), got.get())
    assert not f(dx, dx, dw).any()
    # eager evaluation (four kernels and temporaries) agrees with the fused one
    eager = cp.sum((dx - dy) ** 2 * dw, axis=-1)
    assert np.allclose(eager.get(), got.get(), rtol=1e-5, atol=0)
