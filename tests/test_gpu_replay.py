"""Repeated calls with the same argument signature replay the recorded launch:
results must follow the new data, the new scalar values and the new outputs."""
import numpy as np
import pytest

import cupy_amd as cp
from helpers import assert_exact, assert_sum_close
from oracle import numpy_oracle as oracle

pytestmark = pytest.mark.gpu


def test_elementwise_kernel_repeated_calls_follow_data_and_scalars():
    saxpy = cp.ElementwiseKernel('float32 x, float32 y, float32 a', 'float32 z',
                                 'z = a * x + y', 'saxpy_repeat')
    rng = np.random.default_rng(11)
    n = 100003
    for k, a in enumerate((2.5, -0.75, 1e-3, 3.0, float('inf'))):
        x = rng.uniform(-1, 1, n).astype(np.float32)
        y = rng.uniform(-1, 1, n).astype(np.float32)
        z = saxpy(cp.asarray(x), cp.asarray(y), a)
        assert_exact(z.get(), oracle.saxpy(a, x, y))
    assert len(saxpy._fast_calls) >= 1


def test_ufunc_repeated_calls_transposed_broadcast_mixed():
    rng = np.random.default_rng(12)
    for k in range(4):
        base = rng.standard_normal((384, 640), dtype=np.float32)
        y = rng.uniform(0, 2, (1, 384)).astype(np.float16)
        dx = cp.asarray(base).T
        dy = cp.asarray(y)
        out = dx * dy + (k + 1)
        assert_exact(out.get(), oracle.broadcast_mul_add(base.T, y, k + 1))
        o2 = cp.empty((640, 384), np.float32)
        assert cp.multiply(dx, dy, out=o2) is o2
        assert_exact(o2.get(), base.T * y)


def test_ufunc_repeated_in_place_and_overlapping():
    rng = np.random.default_rng(13)
    for k in range(3):
        h = rng.integers(-100, 100, 4097).astype(np.int32)
        d = cp.asarray(h)
        a, b = d[:-1], d[1:]
        cp.add(a, 7, a)                       # in place: same array in and out
        h[:-1] += 7
        assert_exact(d.get(), h)
        cp.add(a, 1, b)                       # shifted overlap: input copied first
        h[1:] = h[:-1] + 1
        assert_exact(d.get(), h)


@pytest.mark.parametrize('dtype', [np.float32, np.float64, np.int32])
def test_reductions_repeated(dtype):
    rng = np.random.default_rng(14)
    for k in range(3):
        if np.dtype(dtype).kind == 'f':
            h = rng.standard_normal((700, 1300)).astype(dtype)
        else:
            h = rng.integers(-50, 50, (700, 1300)).astype(dtype)
        d = cp.asarray(h)
        for axis in (0, 1, None):
            got = d.sum(axis=axis).get()
            want = h.sum(axis=axis)
            if np.dtype(dtype).kind == 'f':
                assert_sum_close(got, want, np.abs(h).sum(axis=axis, dtype=np.float64), dtype,
                                 data=h, axis=axis)
            else:
                assert_exact(got, want)
        h[rng.integers(0, 700), :] = h.max()          # ties
        d = cp.asarray(h)
        assert_exact(d.argmax(axis=1).get(), oracle.argmax_first(h, 1))
        assert_exact(d.argmin(axis=0).get(), oracle.argmin_first(h, 0))
        out = cp.empty((1300,), dtype if np.dtype(dtype).kind == 'f' else np.int64)
        assert d.sum(axis=0, out=out) is out
        if np.dtype(dtype).kind == 'i':
            assert_exact(out.get(), h.sum(axis=0))


def test_large_split_reduction_repeated_uses_fresh_partials():
    rng = np.random.default_rng(15)
    for k in range(3):
        h = rng.standard_normal(1 << 22, dtype=np.float32)
        d = cp.asarray(h)
        got = d.sum().get()
        assert_sum_close(got, h.sum(dtype=np.float32), np.abs(h).sum(dtype=np.float64),
                         np.float32, data=h, axis=None)


def test_fused_and_reduction_kernel_repeated():
    f = cp.fuse(lambda x, y, w: cp.sum((x - y) ** 2 * w, axis=-1))
    l2 = cp.ReductionKernel('T x, T y', 'T z', '(x - y) * (x - y)', 'a + b', 'z = sqrt(a)',
                            '0', 'l2_repeat')
    rng = np.random.default_rng(16)
    for k in range(3):
        x = rng.standard_normal((2048, 256)).astype(np.float16)
        y = rng.standard_normal((2048, 256)).astype(np.float16)
        w = rng.uniform(0, 1, 256).astype(np.float32)
        got = f(cp.asarray(x), cp.asarray(y), cp.asarray(w)).get()
        want = oracle.fused_sqdiff_wsum(x, y, w)
        bound = np.abs(((x - y) ** 2).astype(np.float32) * w).sum(axis=-1, dtype=np.float64)
        terms = ((x - y) ** 2).astype(np.float32) * w
        assert_sum_close(got, want, bound, np.float32, data=terms, axis=-1)
        xf, yf = x.astype(np.float32), y.astype(np.float32)
        got = l2(cp.asarray(xf), cp.asarray(yf), axis=1).get()
        want = np.sqrt(((xf - yf) ** 2).sum(axis=1))
        np.testing.assert_allclose(got, want, rtol=1e-5)
