"""Operands that start at, or whose rows are spaced by, an address that is not
a multiple of the kernels' vector width: views at an element offset, odd row
lengths, outputs given as such views.  The kernels keep their wide accesses
there, so every family is checked against NumPy on the same data, bit-exact
where the operation is."""
import numpy as np
import pytest

import cupy_amd as cp
from helpers import assert_exact, shaped_random

pytestmark = pytest.mark.gpu

DTYPES = ['int8', 'float16', 'int32', 'float32', 'float64', 'complex64']


@pytest.mark.parametrize('dtype', DTYPES)
def test_flat_kernel_at_every_offset_of_inputs_and_output(dtype):
    n = 70001
    x = shaped_random((n + 24,), dtype, 1)
    y = shaped_random((n + 24,), dtype, 2)
    dx, dy = cp.asarray(x), cp.asarray(y)
    for ox, oy, oo in [(0, 0, 0), (1, 0, 0), (0, 3, 0), (1, 2, 0), (0, 0, 1), (3, 5, 7),
                       (7, 7, 7), (2, 9, 13), (15, 1, 6)]:
        out = cp.zeros(n + 24, dtype)
        r = cp.add(dx[ox:ox + n], dy[oy:oy + n], out=out[oo:oo + n])
        assert r.data.ptr == out.data.ptr + oo * out.itemsize
        host = out.get()
        assert_exact(host[oo:oo + n], x[ox:ox + n] + y[oy:oy + n])
        # nothing written outside the view
        assert not host[:oo].any() and not host[oo + n:].any()


def test_flat_kernel_mixed_widths_at_odd_offsets():
    n = 123457
    a = shaped_random((n + 8,), 'int8', 3)
    b = shaped_random((n + 8,), 'float16', 4)
    c = shaped_random((n + 8,), 'float64', 5)
    da, db, dc = cp.asarray(a), cp.asarray(b), cp.asarray(c)
    k = cp.ElementwiseKernel('int8 a, float16 b, float64 c', 'float32 z',
                             'z = (float)a + (float)b * 2.0f + (float)c', 'mixed_offsets')
    for oa, ob, oc in [(1, 1, 1), (3, 2, 0), (5, 0, 3), (0, 7, 1)]:
        got = k(da[oa:oa + n], db[ob:ob + n], dc[oc:oc + n]).get()
        want = (a[oa:oa + n].astype(np.float32) + b[ob:ob + n].astype(np.float32) * np.float32(2)
                + c[oc:oc + n].astype(np.float32))
        assert_exact(got, want)


@pytest.mark.parametrize('dtype', ['int8', 'float16', 'float32', 'float64'])
@pytest.mark.parametrize('shape', [(257, 1023), (1000, 67), (67, 1001), (130, 129), (513, 515)])
def test_rows_of_odd_length(dtype, shape):
    x = shaped_random(shape, dtype, 6)
    y = shaped_random(shape, dtype, 7)
    row = shaped_random((1, shape[1]), dtype, 8)
    col = shaped_random((shape[0], 1), dtype, 9)
    dx, dy, drow, dcol = map(cp.asarray, (x, y, row, col))
    assert_exact((dx * dy).get(), x * y)
    assert_exact((dx + drow).get(), x + row)
    assert_exact((dx - dcol).get(), x - col)
    # transposed operand against a row-major one: rows of both start anywhere
    t = shaped_random(shape[::-1], dtype, 10)
    dt = cp.asarray(t)
    assert_exact((dt.T + dx).get(), t.T + x)
    # a window into a wider array
    assert_exact((dx[1:, 1:] + dy[:-1, :-1]).get(), x[1:, 1:] + y[:-1, :-1])
    out = cp.zeros(shape, dtype)
    cp.add(dx[1:, 1:], dy[:-1, :-1], out=out[1:, :-1])
    want = np.zeros(shape, dtype)
    np.add(x[1:, 1:], y[:-1, :-1], out=want[1:, :-1])
    assert_exact(out.get(), want)


@pytest.mark.parametrize('dtype', ['int8', 'float16', 'float32', 'float64'])
@pytest.mark.parametrize('shape', [(1000, 67), (67, 1001), (4099, 129), (3, 70001), (70001, 3),
                                   (300, 4097), (33, 65, 31)])
def test_reductions_over_odd_shapes(dtype, shape):
    x = shaped_random(shape, dtype, 11)
    dx = cp.asarray(x)
    for axis in list(range(len(shape))) + [None]:
        got = dx.sum(axis=axis).get()
        if dtype.startswith('float'):
            want = x.astype(np.float64).sum(axis=axis)
            tol = {'float16': 2e-3, 'float32': 1e-5, 'float64': 1e-12}[dtype]
            scale = np.abs(x.astype(np.float64)).sum(axis=axis)
            assert np.all(np.abs(got.astype(np.float64) - want) <= tol * np.maximum(scale, 1)), axis
        else:
            assert_exact(got, x.sum(axis=axis))
        assert_exact(dx.max(axis=axis).get(), x.max(axis=axis))
        assert_exact(dx.argmin(axis=axis).get(), x.argmin(axis=axis))


@pytest.mark.parametrize('dtype', ['int8', 'float32'])
def test_reductions_of_offset_windows(dtype):
    base = shaped_random((515, 1031), dtype, 12)
    db = cp.asarray(base)
    for r0, c0 in [(0, 1), (1, 3), (2, 5), (3, 2)]:
        w, dw = base[r0:r0 + 500, c0:c0 + 1000], db[r0:r0 + 500, c0:c0 + 1000]
        for axis in (0, 1, None):
            if dtype == 'int8':
                assert_exact(dw.sum(axis=axis).get(), w.sum(axis=axis))
            else:
                np.testing.assert_allclose(dw.sum(axis=axis).get(), w.sum(axis=axis, dtype=np.float64),
                                           rtol=1e-5, atol=1e-3)
            assert_exact(dw.argmax(axis=axis).get(), w.argmax(axis=axis))
    flat = db.reshape(-1)
    hflat = base.reshape(-1)
    for off in (1, 2, 3, 7):
        if dtype == 'int8':
            assert_exact(flat[off:].sum().get(), hflat[off:].sum())
        assert_exact(flat[off:].argmax().get(), hflat[off:].argmax())
        assert_exact(flat[off:].min().get(), hflat[off:].min())


def _check_cumsum(dev, host, axis=None):
    got = cp.cumsum(dev, axis=axis).get()
    if host.dtype.kind == 'f':
        np.testing.assert_allclose(got, np.cumsum(host, axis=axis), rtol=1e-12, atol=1e-9)
    else:
        assert_exact(got, np.cumsum(host, axis=axis))


@pytest.mark.parametrize('dtype', ['int8', 'int32', 'float64'])
def test_scans_of_offset_views_and_odd_rows(dtype):
    n = 100003
    x = shaped_random((n + 8,), dtype, 13)
    dx = cp.asarray(x)
    for off in (1, 3, 5):
        _check_cumsum(dx[off:off + n], x[off:off + n])
    m = shaped_random((301, 67), dtype, 14)
    dm = cp.asarray(m)
    for axis in (0, 1):
        _check_cumsum(dm, m, axis)
        _check_cumsum(dm[1:, 3:], m[1:, 3:], axis)
    m = shaped_random((1001, 16), dtype, 15)
    dm = cp.asarray(m).reshape(-1)[3:3 + 1000 * 16].reshape(1000, 16)
    _check_cumsum(dm, m.reshape(-1)[3:3 + 1000 * 16].reshape(1000, 16), 0)


@cp.fuse()
def _centred(x):
    return x - cp.sum(x, axis=1, keepdims=True) / x.shape[1]


def test_fused_rows_with_offset_operands():
    base = shaped_random((64 * 1031 + 8,), 'float32', 15)
    db = cp.asarray(base)
    for off in (0, 1, 2, 3):
        for cols in (1031, 1024):
            x = base[off:off + 64 * cols].reshape(64, cols)
            dx = db[off:off + 64 * cols].reshape(64, cols)
            want = x - (x.sum(axis=1, keepdims=True, dtype=np.float64) / cols).astype(np.float32)
            np.testing.assert_allclose(_centred(dx).get(), want, rtol=1e-5, atol=1e-5)


def test_array_that_ends_with_its_allocation():
    # the last vector of a view must not reach past the end of the memory
    for n in (4096 + 1, 4096 + 3, 65536 + 5):
        x = shaped_random((n,), 'float32', 16)
        dx = cp.asarray(x)
        for off in (1, 2, 3):
            v, hv = dx[off:], x[off:]
            assert_exact((v + v).get(), hv + hv)
            np.testing.assert_allclose(v.sum().get(), hv.sum(dtype=np.float64), rtol=1e-5, atol=1e-3)
            assert_exact(v.argmax().get(), hv.argmax())


@pytest.mark.parametrize('shape', [(70001, 3), (5000, 1000), (3, 70001), (4099, 67), (2, 2), (1000, 1),
                                   (129, 4099), (100000, 2)])
def test_matrix_with_a_value_per_row_or_per_column(shape):
    nr, nc = shape
    x = shaped_random(shape, 'float32', 61)
    row = shaped_random((1, nc), 'float32', 62)
    col = shaped_random((nr, 1), 'float16', 63)
    one = shaped_random((1, 1), 'float64', 64)
    dx, drow, dcol, done = map(cp.asarray, (x, row, col, one))
    assert_exact((dx + drow).get(), x + row)
    assert_exact((dx * dcol).get(), x * col)
    assert_exact(((dx - drow) * dcol).get(), (x - row) * col)
    assert_exact((drow - dx).get(), row - x)
    assert_exact((dx + done).get(), x + one)
    out = cp.zeros(shape, 'float32')
    cp.add(drow, dcol, out)
    assert_exact(out.get(), (row + col).astype(np.float32))
    assert_exact(cp.where(dx > drow, dx, dcol).get(), np.where(x > row, x, col))
    # 1-d row vector (broadcast from the left), strided column vector
    assert_exact((dx + drow[0]).get(), x + row[0])
    wide = shaped_random((nr, 3), 'float32', 65)
    assert_exact((dx * cp.asarray(wide)[:, 1:2]).get(), x * wide[:, 1:2])
    assert_exact((dx * cp.asarray(wide.T.copy())[1][:, None]).get(), x * wide[:, 1:2])
    long_row = shaped_random((1, 2 * nc), 'float32', 66)
    assert_exact((dx - cp.asarray(long_row)[:, ::2]).get(), x - long_row[:, ::2])
    # the element index of a user kernel runs over the matrix row after row
    k = cp.ElementwiseKernel('T x, T r', 'T y, int64 at', 'y = x + r; at = i', 'row_add_with_index')
    y, at = k(dx, drow)
    assert_exact(y.get(), x + row)
    assert_exact(at.get(), np.arange(nr * nc, dtype=np.int64).reshape(shape))


@pytest.mark.parametrize('dtype', ['int8', 'float16', 'float32', 'float64'])
@pytest.mark.parametrize('shape', [(300, 1001), (1000, 3), (70, 4099), (5, 5), (2000, 130)])
def test_rows_spaced_apart_and_strided_columns(dtype, shape):
    nr, nc = shape
    x = shaped_random((nr + 3, 2 * nc + 6), dtype, 71)
    y = shaped_random((nr + 3, 2 * nc + 6), dtype, 72)
    dx, dy = cp.asarray(x), cp.asarray(y)
    views = [
        lambda a: a[1:nr + 1, 2:nc + 2],            # window
        lambda a: a[:nr, 1:2 * nc + 1:2],           # every second column
        lambda a: a[:nr, nc - 1::-1],               # columns backwards
        lambda a: a[:2 * (nr // 2):2, :nc],         # every second row
        lambda a: a[nr - 1::-1, 3:nc + 3],          # rows backwards
    ]
    for va in views:
        for vb in views:
            p, q = va(x), vb(y)
            if p.shape != q.shape:
                continue
            assert_exact((va(dx) + vb(dy)).get(), p + q)
    # into a window, in place, with a value per row and a user kernel's index
    out = cp.zeros_like(dx)
    w = out[1:nr + 1, 2:nc + 2]
    cp.multiply(dx[:nr, :nc], dy[2:nr + 2, 3:4], out=w)
    want = np.zeros_like(x)
    np.multiply(x[:nr, :nc], y[2:nr + 2, 3:4], out=want[1:nr + 1, 2:nc + 2])
    assert_exact(out.get(), want)
    w += dx[:nr, 1:2 * nc + 1:2]
    want[1:nr + 1, 2:nc + 2] += x[:nr, 1:2 * nc + 1:2]
    assert_exact(out.get(), want)
    k = cp.ElementwiseKernel('T a', 'int64 at', 'at = i + (a == a ? 0 : 1)', 'index_of_window')
    assert_exact(k(dx[1:nr + 1, 2:nc + 2]).get(), np.arange(nr * nc, dtype=np.int64).reshape(shape))
    # matrices stored column after column
    xf, yf = np.asfortranarray(x[:nr, :nc]), np.asfortranarray(y[:nr, :nc])
    dxf, dyf = cp.asarray(x[:nr, :nc].T.copy()).T, cp.asarray(y[:nr, :nc].T.copy()).T
    of = cp.zeros((nc, nr), dtype).T
    cp.add(dxf, dyf, out=of)
    assert_exact(of.get(), xf + yf)
    assert_exact((dxf[1:, :] - dyf[:-1, :]).get(), xf[1:, :] - yf[:-1, :])
    # one strided axis
    flat, dflat = x.reshape(-1), dx.reshape(-1)
    assert_exact((dflat[::2] * dflat[1::2]).get(), flat[::2] * flat[1::2])
    assert_exact((dflat[::-1] + dflat).get(), flat[::-1] + flat)
    o1 = cp.zeros(flat.size + 3, dtype)
    cp.negative(dflat[::3], out=o1[1::3][:dflat[::3].size])
    w1 = np.zeros(flat.size + 3, dtype)
    np.negative(flat[::3], out=w1[1::3][:flat[::3].size])
    assert_exact(o1.get(), w1)
