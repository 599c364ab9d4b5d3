"""Seeded random shapes, views, dtypes and axes against NumPy: every dispatch
route of the elementwise, reduction and scan families is reached by some case
(dense, offset, strided, reversed, transposed, broadcast operands; one to four
axes; extents from 1 to a few hundred thousand elements)."""
import numpy as np
import pytest

import cupy_amd as cp
from helpers import assert_exact

pytestmark = pytest.mark.gpu

DTYPES = ['int8', 'uint8', 'int32', 'int64', 'float16', 'float32', 'float64', 'bool']


def random_shape(rng, max_elems):
    ndim = int(rng.integers(1, 5))
    while True:
        kind = rng.integers(0, 4)
        if kind == 0:
            dims = rng.integers(1, 7, ndim)
        elif kind == 1:
            dims = rng.integers(1, 40, ndim)
        else:
            dims = rng.integers(1, 9, ndim)
            dims[int(rng.integers(0, ndim))] = int(rng.integers(1, max_elems))
        if int(np.prod(dims)) <= max_elems:
            return tuple(int(d) for d in dims)


def random_view(rng, shape, dtype, seed):
    """(host view, device view) of the given shape over a larger base array:
    a combination of offsets, steps, reversed axes, a permutation of the axes
    and broadcast axes."""
    r = np.random.default_rng(seed)
    ndim = len(shape)
    perm = list(rng.permutation(ndim)) if rng.random() < 0.4 else list(range(ndim))
    base_shape = [0] * ndim
    slices = [None] * ndim
    bcast = []
    for ax in range(ndim):
        n = shape[ax]
        if n > 1 and rng.random() < 0.15:
            bcast.append(ax)
            base_shape[ax] = 1
            slices[ax] = slice(None)
            continue
        step = int(rng.choice([1, 1, 1, 2, 3, -1, -2]))
        lo = int(rng.integers(0, 3))
        hi_pad = int(rng.integers(0, 3))
        extent = lo + (n - 1) * abs(step) + 1 + hi_pad
        base_shape[ax] = extent
        if step > 0:
            slices[ax] = slice(lo, lo + (n - 1) * step + 1, step)
        else:
            start = lo + (n - 1) * (-step)
            stop = lo - 1
            slices[ax] = slice(start, stop if stop >= 0 else None, step)
    # the base is laid out with its axes in the order `perm`
    stored = [base_shape[p] for p in perm]
    dt = np.dtype(dtype)
    if dt.kind == 'b':
        host = r.integers(0, 2, stored).astype(dt)
    elif dt.kind in 'iu':
        host = r.integers(0 if dt.kind == 'u' else -20, 20, stored).astype(dt)
    else:
        host = (r.random(stored) * 16 - 8).astype(dt)
    dev = cp.asarray(host)
    inv = np.argsort(perm)
    host_v = host.transpose(inv)[tuple(slices)]
    dev_v = dev.transpose(tuple(int(i) for i in inv))[tuple(slices)]
    if bcast:
        host_v = np.broadcast_to(host_v, shape)
        dev_v = cp.broadcast_to(dev_v, shape)
    assert host_v.shape == tuple(shape) and dev_v.shape == tuple(shape)
    return host_v, dev_v


def assert_close(got, want, rtol, scale=None):
    got = np.asarray(got).astype(np.float64)
    want = np.asarray(want).astype(np.float64)
    assert got.shape == want.shape
    bound = rtol * (np.abs(want) if scale is None else scale) + 1e-30
    with np.errstate(invalid='ignore'):
        bad = ~(np.abs(got - want) <= bound) & ~(np.isnan(got) & np.isnan(want)) & ~(got == want)
    assert not bad.any(), (got[bad][:3], want[bad][:3])


@pytest.mark.parametrize('block', range(16))
def test_elementwise_random_views(block):
    rng = np.random.default_rng(1000 + block)
    for case in range(60):
        shape = random_shape(rng, 200000 if case % 8 == 0 else 4000)
        da, db = (str(rng.choice(DTYPES)) for _ in range(2))
        a, xa = random_view(rng, shape, da, int(rng.integers(1 << 30)))
        b, xb = random_view(rng, shape, db, int(rng.integers(1 << 30)))
        tag = (block, case, shape, da, db, xa.strides, xb.strides)
        op = int(rng.integers(0, 5))
        if op == 0:
            assert_exact((xa + xb).get(), a + b), tag
        elif op == 1:
            got, want = cp.multiply(xa, xb), np.multiply(a, b)
            assert got.dtype == want.dtype, tag
            if want.dtype.kind == 'f':
                assert_close(got.get(), want, 1e-3 if want.dtype == np.float16 else 1e-6)
            else:
                assert_exact(got.get(), want)
        elif op == 2:
            assert_exact(cp.where(xa > xb, xa, xb).get(), np.where(a > b, a, b)), tag
        elif op == 3:
            # into a view given as output
            out_h, out_d = random_view(rng, shape, 'float64', 7)
            if out_d.size and not any(s == 0 for s, n in zip(out_d.strides, shape) if n > 1):
                res = cp.subtract(xa.astype('float64'), xb.astype('float64'), out=out_d)
                assert res is out_d
                assert_exact(out_d.get(), a.astype('float64') - b.astype('float64')), tag
        else:
            assert_exact(cp.ascontiguousarray(xa).get(), np.ascontiguousarray(a)), tag
            assert_exact(xa.astype('float32').get(), a.astype('float32')), tag


@pytest.mark.parametrize('block', range(16))
def test_reductions_random_views(block):
    rng = np.random.default_rng(2000 + block)
    for case in range(50):
        shape = random_shape(rng, 300000 if case % 5 == 0 else 5000)
        dt = str(rng.choice(['int8', 'int32', 'float32', 'float64', 'float16', 'bool']))
        a, xa = random_view(rng, shape, dt, int(rng.integers(1 << 30)))
        ndim = len(shape)
        n_ax = int(rng.integers(1, ndim + 1))
        axes = tuple(sorted(int(i) for i in rng.choice(ndim, n_ax, replace=False)))
        axis = axes if len(axes) > 1 else axes[0]
        if rng.random() < 0.15:
            axis = None
        keep = bool(rng.random() < 0.3)
        tag = (block, case, shape, dt, xa.strides, axis, keep)
        kind = np.dtype(dt).kind
        want = a.sum(axis=axis, keepdims=keep)
        got = xa.sum(axis=axis, keepdims=keep)
        assert got.dtype == want.dtype and got.shape == want.shape, tag
        if kind == 'f':
            scale = np.abs(a.astype(np.float64)).sum(axis=axis, keepdims=keep)
            tol = {'float16': 4e-3, 'float32': 2e-5, 'float64': 1e-12}[dt]
            exact = a.astype(np.float64).sum(axis=axis, keepdims=keep)
            if dt == 'float16':
                with np.errstate(over='ignore'):
                    exact = exact.astype(np.float16).astype(np.float64)   # overflows like the result
            assert_close(got.get(), exact, tol, np.maximum(scale, 1))
        else:
            assert_exact(got.get(), want), tag
        assert_exact(xa.max(axis=axis, keepdims=keep).get(), a.max(axis=axis, keepdims=keep)), tag
        if kind != 'b':
            m_got = xa.mean(axis=axis, keepdims=keep)
            m_want = a.mean(axis=axis, keepdims=keep)
            assert m_got.dtype == m_want.dtype, tag
            assert_close(m_got.get(), a.astype(np.float64).mean(axis=axis, keepdims=keep),
                         4e-3 if dt == 'float16' else 2e-5,
                  np.maximum(np.abs(a.astype(np.float64)).mean(axis=axis, keepdims=keep), 1))
        one = axis if (axis is None or isinstance(axis, int)) else axis[0]
        assert_exact(xa.argmax(axis=one).get(), a.argmax(axis=one)), tag
        assert_exact(xa.argmin(axis=one, keepdims=keep).get(), a.argmin(axis=one, keepdims=keep)), tag
        if kind == 'f' and dt != 'float16':
            v_want = a.astype(np.float64).var(axis=axis, keepdims=keep)
            assert_close(xa.var(axis=axis, keepdims=keep).get(), v_want, 1e-4 if dt == 'float32' else 1e-10,
                  np.maximum(v_want, 1e-3))


@pytest.mark.parametrize('block', range(8))
def test_scans_random_views(block):
    rng = np.random.default_rng(3000 + block)
    for case in range(40):
        shape = random_shape(rng, 100000 if case % 5 == 0 else 3000)
        dt = str(rng.choice(['int8', 'int32', 'int64', 'float64']))
        a, xa = random_view(rng, shape, dt, int(rng.integers(1 << 30)))
        axis = int(rng.integers(0, len(shape))) if rng.random() < 0.85 else None
        tag = (block, case, shape, dt, xa.strides, axis)
        want = np.cumsum(a, axis=axis)
        got = cp.cumsum(xa, axis=axis)
        assert got.dtype == want.dtype and got.shape == want.shape, tag
        if dt == 'float64':
            assert_close(got.get(), want, 1e-12, np.maximum(np.cumsum(np.abs(a), axis=axis), 1))
        else:
            assert_exact(got.get(), want), tag


def _fused_templates(xp):
    def chain(x, y):
        return xp.sqrt(xp.abs(x)) + y * 2 - xp.minimum(x, y)

    def dot_last(x, y):
        return xp.sum(x * y, axis=-1)

    def dot_first(x, y):
        return xp.sum(x * y, axis=0)

    def centre(x, y):
        return x - xp.sum(x, axis=-1, keepdims=True) / x.shape[-1] + y

    def softmax(x, y):
        e = xp.exp(x - xp.amax(x, axis=-1, keepdims=True))
        return e / xp.sum(e, axis=-1, keepdims=True)

    def two_results(x, y):
        return xp.sum(x, axis=0), xp.amax(x * y, axis=0)

    def normalise(x, y):
        m = xp.sum(x, axis=-1, keepdims=True) / x.shape[-1]
        d = x - m
        v = xp.sum(d * d, axis=-1, keepdims=True) / x.shape[-1]
        return d / xp.sqrt(v + 1e-3) * y

    def total(x, y):
        return xp.sum(xp.where(x > y, x, y))

    return [chain, dot_last, dot_first, centre, softmax, two_results, normalise, total]


@pytest.mark.parametrize('template', range(8))
def test_fused_functions_random_views(template):
    rng = np.random.default_rng(4000 + template)
    host_f = _fused_templates(np)[template]
    dev_f = cp.fuse(_fused_templates(cp)[template])
    for case in range(40):
        ndim = int(rng.integers(1, 4))
        if case % 4 == 0:
            shape = tuple(int(d) for d in rng.integers(2, 9, ndim - 1)) + (
                int(rng.choice([64, 100, 256, 1000, 4096, 5000])),)
        else:
            shape = tuple(int(d) for d in rng.integers(1, 30, ndim))
        dt = str(rng.choice(['float32', 'float64', 'float32', 'float16']))
        plain = rng.random() < 0.5
        if plain:
            r = np.random.default_rng(case)
            a = (r.random(shape) * 4 - 2).astype(dt)
            b = (r.random(shape) * 4 - 2).astype(dt)
            xa, xb = cp.asarray(a), cp.asarray(b)
        else:
            a, xa = random_view(rng, shape, dt, int(rng.integers(1 << 30)))
            b, xb = random_view(rng, shape, dt, int(rng.integers(1 << 30)))
            a, b = a / 4, b / 4
            xa, xb = xa / 4, xb / 4
            if rng.random() < 0.5:
                # the division above made them dense; take views of those again
                a, b, xa, xb = a[..., ::-1], b[..., 1:], xa[..., ::-1], xb[..., 1:]
                a, xa = a[..., 1:], xa[..., 1:]
        if a.shape[-1] == 0:
            continue
        with np.errstate(all='ignore'):
            want = host_f(a.astype(np.float64), b.astype(np.float64))
            like = host_f(a, b)
        got = dev_f(xa, xb)
        wants = want if isinstance(want, tuple) else (want,)
        likes = like if isinstance(like, tuple) else (like,)
        gots = got if isinstance(got, tuple) else (got,)
        tol = {'float16': 2e-2, 'float32': 2e-4, 'float64': 1e-9}[dt]
        for g, w, l in zip(gots, wants, likes):
            tag = (template, case, shape, dt, plain, xa.strides, xb.strides)
            assert g.shape == np.shape(w) and g.dtype == np.asarray(l).dtype, tag
            if dt == 'float16':
                w = np.where(np.abs(w) > 65504, np.sign(w) * np.inf, w)     # overflows like the result
            assert_close(g.get(), w, tol, np.maximum(np.abs(w), 1) * (a.shape[-1] ** 0.5))
