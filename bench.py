"""Benchmark of the generated-kernel hot path on one MI355X.

A "step" is one pass over the five benchmark configurations at their full
shapes (13 operations, inputs resident in HBM, outputs preallocated):

  C1  saxpy via ElementwiseKernel, float32, N = 2**26
  C2  x.T * y (+ 1): float32 (8192, 8192) transposed view times float16 (1, 8192)
      row, then add of a Python scalar (two ufunc calls)
  C3  sum over axis=1, axis=0 and all elements: float32 (16384, 16384) and
      float64 (8192, 8192)
  C4  argmax and argmin of int32 (2**20, 128) along the last axis, argmax of
      float32 (2**16, 4096) along axis 1
  C5  fused sum((x - y)**2 * w, axis=-1): float16 (2**18, 256) x 2, float32 (256,)

``value`` is the algorithmic bytes of one step divided by the wall time of a
step (all launches enqueued through the public API, one synchronisation at the
end of the timed region).  ``per_config`` gives each operation's own figure:
fifteen more steps after the timed region in which every kernel carries a pair
of HIP events that receive the start and the end of its execution on the
launch stream, so that an operation is timed where it stands in the step (no
operation finds its own operands in the memory-side cache) and nothing is added
to the stream between the kernels; ``roofline`` repeats the entry of the
operation that takes the largest share of a step.  ``cpu_baseline`` is NumPy
evaluating the same operations on the same host arrays, single-threaded.

Prints exactly one JSON line on stdout.
"""
import argparse
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBPS = 8000.0

# HBM bytes per launch (read + written) from the rocprofv3 FETCH_SIZE and
# WRITE_SIZE counters, scaled by what the same counters read for the plain copy
# kernel that --calibrate adds.  `python bench_profiles.py pmc` digests the
# counter runs into this file (operation name -> bytes; two-pass reductions
# count both of their kernels); an operation it does not list reports null.
TRAFFIC_FILE = os.path.join(ROOT, 'bench_traffic.json')


def measured_traffic():
    try:
        with open(TRAFFIC_FILE) as f:
            return json.load(f).get('hbm_bytes_per_launch', {})
    except (OSError, ValueError):
        return {}


def log(*a):
    print(*a, file=sys.stderr, flush=True)


def build_cases(cp, scale=1):
    """Returns a list of dicts: name, algorithmic bytes, gpu callable, numpy
    callable, parity check."""
    from oracle import numpy_oracle as oracle
    cases = []

    def add(name, config, nbytes, gpu, cpu, check, kernel):
        cases.append(dict(name=name, config=config, bytes=int(nbytes), gpu=gpu, cpu=cpu,
                          check=check, kernel=kernel))

    # ---- C1 ---------------------------------------------------------------------------
    n1 = (1 << 26) // scale
    rng = np.random.default_rng(1)
    x1 = rng.uniform(-1, 1, n1).astype(np.float32)
    y1 = rng.uniform(-1, 1, n1).astype(np.float32)
    dx1, dy1 = cp.asarray(x1), cp.asarray(y1)
    z1 = cp.empty((n1,), np.float32)
    hz1 = np.empty(n1, np.float32)
    saxpy = cp.ElementwiseKernel('float32 x, float32 y, float32 a', 'float32 z',
                                 'z = a * x + y', 'saxpy')

    def cpu_saxpy():
        np.multiply(np.float32(2.5), x1, out=hz1)
        np.add(hz1, y1, out=hz1)
        return hz1

    add('C1 saxpy f32 2^26', 'C1', 12 * n1, lambda: saxpy(dx1, dy1, 2.5, z1), cpu_saxpy,
        lambda: np.array_equal(z1.get(), oracle.saxpy(2.5, x1, y1)), 'saxpy')

    # ---- C2 ---------------------------------------------------------------------------
    m = 8192 // (4 if scale > 1 else 1)
    rng = np.random.default_rng(2)
    base = rng.standard_normal((m, m), dtype=np.float32)
    y2 = rng.uniform(0, 2, (1, m)).astype(np.float16)
    dbase = cp.asarray(base)
    dx2 = dbase.T
    dy2 = cp.asarray(y2)
    tmp2 = cp.empty((m, m), np.float32)
    out2 = cp.empty((m, m), np.float32)
    htmp2 = np.empty((m, m), np.float32)
    hout2 = np.empty((m, m), np.float32)
    add('C2a x.T*y f32(T)xf16 8192^2', 'C2', 8 * m * m + 2 * m,
        lambda: cp.multiply(dx2, dy2, tmp2), lambda: np.multiply(base.T, y2, out=htmp2),
        lambda: np.array_equal(tmp2.get(), base.T * y2),
        'cupy_multiply__float32_float16_float32')
    add('C2b tmp+1 f32 8192^2', 'C2', 8 * m * m,
        lambda: cp.add(tmp2, 1, out2), lambda: np.add(htmp2, 1, out=hout2),
        lambda: np.array_equal(out2.get(), oracle.broadcast_mul_add(base.T, y2, 1)),
        'cupy_add__float32_float_float32')

    # ---- C3 ---------------------------------------------------------------------------
    for dt, n, seed, rtol in ((np.float32, 16384, 3, 1e-5), (np.float64, 8192, 4, 1e-12)):
        n = n // (4 if scale > 1 else 1)
        rng = np.random.default_rng(seed)
        a = rng.standard_normal((n, n), dtype=np.float32) if dt == np.float32 \
            else rng.standard_normal((n, n))
        da = cp.asarray(a)
        item = a.dtype.itemsize
        for axis in (1, 0, None):
            oshape = () if axis is None else (n,)
            out = cp.empty(oshape, dt)
            hout = np.empty(oshape, dt)

            def gpu(da=da, axis=axis, out=out):
                return da.sum(axis=axis, out=out)

            def cpu(a=a, axis=axis, hout=hout):
                return np.sum(a, axis=axis, out=hout)

            def check(a=a, axis=axis, out=out, rtol=rtol, dt=dt):
                # backward bound against NumPy's own sum, and the bound on the
                # result itself: |got - float64 sum| <= rtol * max(|float64
                # sum|, sigma * sqrt(N reduced)), which a missing partial breaks
                got = out.get()
                mag = np.abs(a).sum(axis=axis, dtype=np.float64)
                err = np.abs(got.astype(np.float64) - np.sum(a, axis=axis))
                ratio = oracle.check_sum_forward(got, a, axis, dt)
                log('  forward bound %s axis=%s: largest err/bound %.3g' % (
                    np.dtype(dt).name, axis, ratio))
                return bool(np.all(err <= rtol * mag)) and ratio <= 1.0

            add('C3 sum %s axis=%s %d^2' % (np.dtype(dt).name, axis, n), 'C3',
                a.nbytes + (item if axis is None else n * item), gpu, cpu, check, 'cupy_sum')

    # ---- C4 ---------------------------------------------------------------------------
    r4 = (1 << 20) // scale
    rng = np.random.default_rng(5)
    a4 = rng.integers(0, 16, (r4, 128), dtype=np.int32)
    d4 = cp.asarray(a4)
    o4a = cp.empty((r4,), np.int64)
    o4b = cp.empty((r4,), np.int64)
    add('C4 argmax i32 (2^20,128)', 'C4', a4.nbytes + r4 * 8,
        lambda: d4.argmax(axis=-1, out=o4a), lambda: a4.argmax(axis=-1),
        lambda: np.array_equal(o4a.get(), oracle.argmax_fast(a4, -1)), 'cupy_argmax')
    add('C4 argmin i32 (2^20,128)', 'C4', a4.nbytes + r4 * 8,
        lambda: d4.argmin(axis=-1, out=o4b), lambda: a4.argmin(axis=-1),
        lambda: np.array_equal(o4b.get(), oracle.argmin_fast(a4, -1)), 'cupy_argmin')
    r4f = (1 << 16) // scale
    rng = np.random.default_rng(6)
    a4f = rng.standard_normal((r4f, 4096), dtype=np.float32)
    d4f = cp.asarray(a4f)
    o4f = cp.empty((r4f,), np.int64)
    add('C4 argmax f32 (2^16,4096)', 'C4', a4f.nbytes + r4f * 8,
        lambda: d4f.argmax(axis=1, out=o4f), lambda: a4f.argmax(axis=1),
        lambda: np.array_equal(o4f.get(), a4f.argmax(axis=1)), 'cupy_argmax')

    # ---- C5 ---------------------------------------------------------------------------
    r5 = (1 << 18) // scale
    rng = np.random.default_rng(7)
    x5 = rng.standard_normal((r5, 256)).astype(np.float16)
    y5 = rng.standard_normal((r5, 256)).astype(np.float16)
    w5 = rng.uniform(0, 1, 256).astype(np.float32)
    dx5, dy5, dw5 = cp.asarray(x5), cp.asarray(y5), cp.asarray(w5)

    @cp.fuse(kernel_name='fused_sqdiff_wsum')
    def fused(x, y, w):
        return cp.sum((x - y) ** 2 * w, axis=-1)

    res5 = [None]

    def gpu5():
        res5[0] = fused(dx5, dy5, dw5)
        return res5[0]

    add('C5 fused sum((x-y)^2*w) f16 (2^18,256)', 'C5',
        2 * x5.nbytes + w5.nbytes + r5 * 4, gpu5,
        lambda: np.sum((x5 - y5) ** 2 * w5, axis=-1),
        lambda: bool(np.allclose(res5[0].get(), oracle.fused_sqdiff_wsum(x5, y5, w5),
                                 rtol=1e-5, atol=0)), 'fused_sqdiff_wsum')
    return cases


def build_next_cases(cp):
    """Operations of the components built after the five configurations (scans,
    statistics, complex types, multi-kernel fused functions), at shapes of the
    same size class.  ``bytes`` is the algorithmic traffic: every input element
    read once, every output element written once -- also where the operation as
    defined takes several passes (variance, softmax), so that the fraction of
    peak shows the cost of those passes."""
    cases = []

    def add(name, nbytes, gpu, cpu, check, kernel):
        cases.append(dict(name=name, config='next', bytes=int(nbytes), gpu=gpu, cpu=cpu,
                          check=check, kernel=kernel))

    def close(got, want, rtol, scale=None):
        got = got.get().astype(np.float64 if got.dtype.kind != 'c' else np.complex128)
        err = np.abs(got - want)
        bound = rtol * (np.abs(want) if scale is None else scale) + 1e-30
        return bool(np.all(err <= bound))

    rng = np.random.default_rng(11)
    # ---- scans ------------------------------------------------------------------------
    for shape, axis in (((1 << 20, 64), 1), ((8192, 8192), 1), ((8192, 8192), 0),
                        ((64, 1 << 20), 0), ((1 << 26,), 0)):
        a = rng.standard_normal(shape, dtype=np.float32)
        da = cp.asarray(a)
        out = cp.empty(shape, np.float32)
        label = 'cumsum f32 %s axis=%d' % ('x'.join(str(s) for s in shape), axis)

        def check(a=a, out=out, axis=axis):
            return close(out, np.cumsum(a, axis=axis, dtype=np.float64), 1e-5,
                         np.cumsum(np.abs(a), axis=axis, dtype=np.float64))
        add(label, 2 * a.nbytes, lambda da=da, axis=axis, out=out: cp.cumsum(da, axis=axis, out=out),
            lambda a=a, axis=axis: np.cumsum(a, axis=axis), check, 'cupy_scan')
    # ---- statistics -------------------------------------------------------------------
    m = rng.standard_normal((16384, 8192), dtype=np.float32)
    dm = cp.asarray(m)
    o_mean = cp.empty((16384,), np.float32)
    add('mean f32 16384x8192 axis=1', m.nbytes + 16384 * 4,
        lambda: dm.mean(axis=1, out=o_mean), lambda: m.mean(axis=1),
        lambda: close(o_mean, m.mean(axis=1, dtype=np.float64), 1e-5,
                      np.abs(m).mean(axis=1, dtype=np.float64)), 'cupy_mean')
    res_var = [None]

    def gpu_var():
        res_var[0] = dm.var(axis=0)
    add('var f32 16384x8192 axis=0 (one pass; combine kernel included)', m.nbytes + 8192 * 4,
        gpu_var, lambda: m.var(axis=0),
        lambda: close(res_var[0], m.var(axis=0, dtype=np.float64), 1e-4), 'cupy_var_float32')
    mn = m.copy()
    mn[::7, ::5] = np.nan
    dmn = cp.asarray(mn)
    o_nanmax = cp.empty((16384,), np.float32)
    add('nanmax f32 16384x8192 axis=1', m.nbytes + 16384 * 4,
        lambda: cp.nanmax(dmn, axis=1, out=o_nanmax), lambda: np.nanmax(mn, axis=1),
        lambda: bool(np.array_equal(o_nanmax.get(), np.nanmax(mn, axis=1))), 'cupy_nanmax')
    # ---- complex ----------------------------------------------------------------------
    n = 1 << 25
    z1 = (rng.standard_normal(n) + 1j * rng.standard_normal(n)).astype(np.complex64)
    z2 = (rng.standard_normal(n) + 1j * rng.standard_normal(n)).astype(np.complex64)
    dz1, dz2 = cp.asarray(z1), cp.asarray(z2)
    oz = cp.empty((n,), np.complex64)
    add('multiply complex64 2^25', 3 * z1.nbytes, lambda: cp.multiply(dz1, dz2, oz),
        lambda: np.multiply(z1, z2),
        lambda: close(oz, z1.astype(np.complex128) * z2.astype(np.complex128), 5e-7), 'cupy_multiply')
    oa = cp.empty((n,), np.float32)
    add('absolute complex64 2^25', z1.nbytes + n * 4, lambda: cp.absolute(dz1, oa),
        lambda: np.absolute(z1),
        lambda: close(oa, np.abs(z1.astype(np.complex128)), 3e-7), 'cupy_absolute')
    w1 = (rng.standard_normal(n // 2) + 1j * rng.standard_normal(n // 2))
    dw1 = cp.asarray(w1)
    osum = cp.empty((), np.complex128)
    add('sum complex128 2^24', w1.nbytes + 16, lambda: dw1.sum(out=osum), lambda: w1.sum(),
        lambda: close(osum, np.asarray(w1.sum()), 1e-12, np.abs(w1).sum()), 'cupy_sum')
    # ---- multi-kernel fused function ----------------------------------------------------
    s = rng.standard_normal((16384, 4096), dtype=np.float32)
    ds = cp.asarray(s)

    @cp.fuse(kernel_name='softmax_rows')
    def softmax(x):
        e = cp.exp(x - cp.amax(x, axis=1, keepdims=True))
        return e / cp.sum(e, axis=1, keepdims=True)
    res_sm = [None]

    def gpu_softmax():
        res_sm[0] = softmax(ds)

    def cpu_softmax():
        e = np.exp(s - s.max(axis=1, keepdims=True))
        return e / e.sum(axis=1, keepdims=True)
    add('fused softmax f32 16384x4096 (one kernel, rows in registers)', 2 * s.nbytes, gpu_softmax,
        cpu_softmax, lambda: close(res_sm[0], cpu_softmax().astype(np.float64), 1e-5), 'softmax_rows')
    ex = cp.empty((16384, 4096), np.float32)
    add('exp f32 2^26', 2 * s.nbytes, lambda: cp.exp(ds, ex), lambda: np.exp(s),
        lambda: close(ex, np.exp(s.astype(np.float64)), 3e-7), 'cupy_exp')
    return cases


def build_layout_cases(cp):
    """Operand layouts beyond the five configurations, at the same size class
    (2^26 float32 elements unless stated): views at an element offset, rows of
    odd length, tall narrow matrices with a value per row or column, windows,
    permuted axes, operands of different widths, reductions over a middle axis
    or over the outer and the innermost axis.  ``bytes`` as in the other
    suites: every input element read once, every output element written once."""
    cases = []

    def add(name, nbytes, gpu, cpu, check, kernel):
        cases.append(dict(name=name, config='layouts', bytes=int(nbytes), gpu=gpu, cpu=cpu,
                          check=check, kernel=kernel))

    def same(out, want):
        return bool(np.array_equal(out.get(), want))

    def close(got, want, rtol, scale):
        err = np.abs(got.get().astype(np.float64) - want)
        return bool(np.all(err <= rtol * scale + 1e-30))

    rng = np.random.default_rng(12)
    n = 1 << 26
    flat = rng.standard_normal(n, dtype=np.float32)
    dflat = cp.asarray(flat)
    res = {}

    def run(key, fn):
        def call():
            res[key] = fn()
        return call

    # ---- elementwise ------------------------------------------------------------------
    add('x[1:] + x[:-1] f32 2^26 (x counted once)', 2 * 4 * (n - 1), run('off', lambda: dflat[1:] + dflat[:-1]),
        lambda: flat[1:] + flat[:-1], lambda: same(res['off'], flat[1:] + flat[:-1]), 'cupy_add')
    rows3 = n // 3
    a3, d3 = flat[:rows3 * 3].reshape(rows3, 3), dflat[:rows3 * 3].reshape(rows3, 3)
    row3 = rng.standard_normal((1, 3), dtype=np.float32)
    drow3 = cp.asarray(row3)
    add('(N,3) - row f32', 2 * a3.nbytes, run('n3', lambda: d3 - drow3), lambda: a3 - row3,
        lambda: same(res['n3'], a3 - row3), 'cupy_subtract')
    sq, dsq = flat.reshape(8192, 8192), dflat.reshape(8192, 8192)
    col = rng.standard_normal((8192, 1), dtype=np.float32)
    row = rng.standard_normal((1, 8192), dtype=np.float32)
    dcol, drow = cp.asarray(col), cp.asarray(row)
    add('a * col(n,1) f32 8192x8192', 2 * sq.nbytes, run('col', lambda: dsq * dcol), lambda: sq * col,
        lambda: same(res['col'], sq * col), 'cupy_multiply')
    add('col + row -> 8192x8192 f32', sq.nbytes, run('outer', lambda: dcol + drow), lambda: col + row,
        lambda: same(res['outer'], col + row), 'cupy_add')
    add('a[1:-1,1:-1] + a[:-2,2:] f32 8192x8192 (a counted once)', 2 * 4 * 8190 * 8190,
        run('win', lambda: dsq[1:-1, 1:-1] + dsq[:-2, 2:]), lambda: sq[1:-1, 1:-1] + sq[:-2, 2:],
        lambda: same(res['win'], sq[1:-1, 1:-1] + sq[:-2, 2:]), 'cupy_add')
    cube, dcube = flat.reshape(256, 512, 512), dflat.reshape(256, 512, 512)
    for perm in ((0, 2, 1), (2, 1, 0), (1, 0, 2)):
        key = 'perm%d%d%d' % perm
        add('transpose%r copy f32 256x512x512' % (perm,), 2 * cube.nbytes,
            run(key, lambda perm=perm: cp.ascontiguousarray(dcube.transpose(perm))),
            lambda perm=perm: np.ascontiguousarray(cube.transpose(perm)),
            lambda perm=perm, key=key: same(res[key], cube.transpose(perm)), 'cupy_copy')
    q, dq = flat.reshape(16, 512, 64, 128), dflat.reshape(16, 512, 64, 128)
    add('(B,S,H,D) -> (B,H,S,D) copy f32 16x512x64x128', 2 * q.nbytes,
        run('bshd', lambda: cp.ascontiguousarray(dq.transpose(0, 2, 1, 3))),
        lambda: np.ascontiguousarray(q.transpose(0, 2, 1, 3)),
        lambda: same(res['bshd'], q.transpose(0, 2, 1, 3)), 'cupy_copy')
    add('f32 > 0 -> bool 2^26', 5 * n, run('gt', lambda: dflat > 0), lambda: flat > 0,
        lambda: same(res['gt'], flat > 0), 'cupy_greater')
    mask = flat > 0
    dmask = cp.asarray(mask)
    other = rng.standard_normal(n, dtype=np.float32)
    dother = cp.asarray(other)
    add('where(mask, f32, f32) 2^26', 13 * n, run('where', lambda: cp.where(dmask, dflat, dother)),
        lambda: np.where(mask, flat, other), lambda: same(res['where'], np.where(mask, flat, other)),
        'cupy_where')
    add('astype f32 -> f16 2^26', 6 * n, run('half', lambda: dflat.astype(np.float16)),
        lambda: flat.astype(np.float16), lambda: same(res['half'], flat.astype(np.float16)),
        'cupy_copy')
    i8 = rng.integers(-100, 100, n).astype(np.int8)
    di8 = cp.asarray(i8)
    add('astype int8 -> int64 2^26', 9 * n, run('wide', lambda: di8.astype(np.int64)),
        lambda: i8.astype(np.int64), lambda: same(res['wide'], i8.astype(np.int64)), 'cupy_copy')
    # ---- reductions -------------------------------------------------------------------
    def red(name, arr, darr, axis, kernel='cupy_sum'):
        want = arr.sum(axis=axis, dtype=np.float64)
        scale = np.abs(arr).sum(axis=axis, dtype=np.float64)
        key = name
        add(name, arr.nbytes + want.size * 4, run(key, lambda: darr.sum(axis=axis)),
            lambda: arr.sum(axis=axis), lambda: close(res[key], want, 1e-5, scale), kernel)
    r67 = 1000003
    a67, d67 = flat[:r67 * 67].reshape(r67, 67), dflat[:r67 * 67].reshape(r67, 67)
    red('sum f32 1000003x67 axis=0', a67, d67, 0)
    red('sum f32 1000003x67 axis=1', a67, d67, 1)
    r7 = n // 7
    a7, d7 = flat[:r7 * 7].reshape(r7, 7), dflat[:r7 * 7].reshape(r7, 7)
    red('sum f32 (2^26/7)x7 axis=1', a7, d7, 1)
    add('argmax f32 (2^26/7)x7 axis=1', a7.nbytes + r7 * 8, run('am7', lambda: d7.argmax(axis=1)),
        lambda: a7.argmax(axis=1), lambda: same(res['am7'], a7.argmax(axis=1)), 'cupy_argmax')
    am, dm3 = flat[:33 * 65 * 31277].reshape(33, 65, 31277), dflat[:33 * 65 * 31277].reshape(33, 65, 31277)
    red('sum f32 33x65x31277 axis=1', am, dm3, 1)
    ac, dc = flat.reshape(512, 256, 512), dflat.reshape(512, 256, 512)
    red('sum f32 512x256x512 axis=(0,2)', ac, dc, (0, 2))
    a2, d2 = flat.reshape(2, n // 2), dflat.reshape(2, n // 2)
    red('sum f32 2x2^25 axis=0', a2, d2, 0)
    # ---- scan along an axis with an odd tail, fused rows of 100 ---------------------------
    want_scan = np.cumsum(a3, axis=0, dtype=np.float64)
    scale_scan = np.cumsum(np.abs(a3), axis=0, dtype=np.float64)
    add('cumsum f32 (2^26/3)x3 axis=0', 2 * a3.nbytes, run('scan3', lambda: cp.cumsum(d3, axis=0)),
        lambda: np.cumsum(a3, axis=0), lambda: close(res['scan3'], want_scan, 1e-5, scale_scan),
        'cupy_scan_lanes')
    # ---- narrow arrays and short slices (points, channels-last data) -------------------
    add('(N,3) -> (3,N) copy f32', 2 * a3.nbytes, run('t3', lambda: cp.ascontiguousarray(d3.T)),
        lambda: np.ascontiguousarray(a3.T), lambda: same(res['t3'], a3.T), 'cupy_copy')
    ach, dch = flat.reshape(n // 32, 16, 2), dflat.reshape(n // 32, 16, 2)
    add('sum f32 (2^21,16,2) axis=1', ach.nbytes + (n // 16) * 4, run('ch', lambda: dch.sum(axis=1)),
        lambda: ach.sum(axis=1),
        lambda: close(res['ch'], ach.sum(axis=1, dtype=np.float64), 1e-5,
                      np.abs(ach).sum(axis=1, dtype=np.float64)), 'cupy_sum')
    a44, d44 = flat.reshape(n // 16, 4, 4), dflat.reshape(n // 16, 4, 4)
    add('cumsum f32 (2^22,4,4) axis=1', 2 * a44.nbytes, run('s44', lambda: cp.cumsum(d44, axis=1)),
        lambda: np.cumsum(a44, axis=1),
        lambda: close(res['s44'], np.cumsum(a44, axis=1, dtype=np.float64), 1e-5,
                      np.cumsum(np.abs(a44), axis=1, dtype=np.float64)), 'cupy_scan_tile_packed')
    r33 = n // 33
    a33, d33 = flat[:r33 * 33].reshape(r33, 33), dflat[:r33 * 33].reshape(r33, 33)
    add('cumsum f32 (2^26/33)x33 axis=1', 2 * a33.nbytes, run('s33', lambda: cp.cumsum(d33, axis=1)),
        lambda: np.cumsum(a33, axis=1),
        lambda: close(res['s33'], np.cumsum(a33, axis=1, dtype=np.float64), 1e-5,
                      np.cumsum(np.abs(a33), axis=1, dtype=np.float64)), 'cupy_scan_tile_packed')
    rw = n // (16 * 257)
    aw = flat[:rw * 16 * 257].reshape(rw, 16, 257)
    dw = dflat[:rw * 16 * 257].reshape(rw, 16, 257)
    add('cumsum f32 (2^26/4112)x16x257 axis=1', 2 * aw.nbytes, run('sw', lambda: cp.cumsum(dw, axis=1)),
        lambda: np.cumsum(aw, axis=1),
        lambda: close(res['sw'], np.cumsum(aw, axis=1, dtype=np.float64), 1e-5,
                      np.cumsum(np.abs(aw), axis=1, dtype=np.float64)), 'cupy_scan_slab')
    r100 = n // 100
    a100, d100 = flat[:r100 * 100].reshape(r100, 100), dflat[:r100 * 100].reshape(r100, 100)

    @cp.fuse(kernel_name='softmax_rows_of_100')
    def softmax(x):
        e = cp.exp(x - cp.amax(x, axis=1, keepdims=True))
        return e / cp.sum(e, axis=1, keepdims=True)

    def cpu_softmax():
        e = np.exp(a100 - a100.max(axis=1, keepdims=True))
        return e / e.sum(axis=1, keepdims=True)
    add('fused softmax f32 (2^26/100)x100', 2 * a100.nbytes, run('sm100', lambda: softmax(d100)),
        cpu_softmax, lambda: close(res['sm100'], cpu_softmax().astype(np.float64), 1e-5, 1.0),
        'softmax_rows_of_100')
    # ---- rows that do not start on cache lines: neighbouring workgroups share lines -----------
    odd = flat[:8191 * 8193].reshape(8191, 8193)
    dodd = dflat[:8191 * 8193].reshape(8191, 8193)
    add('transposed copy f32 8191x8193', 2 * odd.nbytes, run('oddT', lambda: cp.ascontiguousarray(dodd.T)),
        lambda: np.ascontiguousarray(odd.T), lambda: same(res['oddT'], np.ascontiguousarray(odd.T)),
        'cupy_copy')
    add('sum f32 8191x8193 axis=0', odd.nbytes + 4 * 8193, run('oddS', lambda: dodd.sum(axis=0)),
        lambda: odd.sum(axis=0),
        lambda: close(res['oddS'], odd.sum(axis=0, dtype=np.float64), 1e-5,
                      np.abs(odd).sum(axis=0, dtype=np.float64)), 'cupy_sum')
    add('cumsum f32 8191x8193 axis=0', 2 * odd.nbytes, run('oddC', lambda: cp.cumsum(dodd, axis=0)),
        lambda: np.cumsum(odd, axis=0),
        lambda: close(res['oddC'], np.cumsum(odd, axis=0, dtype=np.float64), 1e-5,
                      np.cumsum(np.abs(odd), axis=0, dtype=np.float64)), 'cupy_scan_chain_cols')
    add('cumsum f32 2^26 - 1 axis=0 (no whole number of vectors)', 2 * 4 * (n - 1),
        run('odd1', lambda: cp.cumsum(dflat[:n - 1])), lambda: np.cumsum(flat[:n - 1]),
        lambda: close(res['odd1'], np.cumsum(flat[:n - 1], dtype=np.float64), 1e-5,
                      np.cumsum(np.abs(flat[:n - 1]), dtype=np.float64)), 'cupy_scan_chain')
    # ---- small trailing axes under a permutation: tiles that span several axes ------------------
    m88, dm88 = flat.reshape(n // 64, 8, 8), dflat.reshape(n // 64, 8, 8)
    add('(2^20,8,8) -> matrices transposed, copy f32', 2 * m88.nbytes,
        run('m88', lambda: cp.ascontiguousarray(dm88.transpose(0, 2, 1))),
        lambda: np.ascontiguousarray(m88.transpose(0, 2, 1)),
        lambda: same(res['m88'], np.ascontiguousarray(m88.transpose(0, 2, 1))), 'cupy_copy')
    nb43 = n // 12
    h43 = flat[:nb43 * 12].astype(np.float16).reshape(nb43, 4, 3)
    d43 = cp.asarray(h43)
    add('(N,4,3) -> (N,3,4) copy f16', 2 * h43.nbytes,
        run('m43', lambda: cp.ascontiguousarray(d43.transpose(0, 2, 1))),
        lambda: np.ascontiguousarray(h43.transpose(0, 2, 1)),
        lambda: same(res['m43'], np.ascontiguousarray(h43.transpose(0, 2, 1))), 'cupy_copy')
    q4, dq4 = flat.reshape(4, n // 16, 4), dflat.reshape(4, n // 16, 4)
    add('(4,2^22,4) -> axes reversed, copy f32', 2 * q4.nbytes,
        run('q4', lambda: cp.ascontiguousarray(dq4.transpose(2, 1, 0))),
        lambda: np.ascontiguousarray(q4.transpose(2, 1, 0)),
        lambda: same(res['q4'], np.ascontiguousarray(q4.transpose(2, 1, 0))), 'cupy_copy')
    r164 = flat.reshape(n // 64, 16, 4)
    dr164 = dflat.reshape(n // 64, 16, 4)
    mid = rng.standard_normal((n // 64, 1, 4), dtype=np.float32)
    dmid = cp.asarray(mid)
    add('(2^20,16,4) + (2^20,1,4) f32', 2 * r164.nbytes + mid.nbytes, run('mid', lambda: dr164 + dmid),
        lambda: r164 + mid, lambda: same(res['mid'], r164 + mid), 'cupy_add')
    # ---- joining, tiling, rolling: copies into windows of the result ---------------------------------
    h2, dh2 = flat.reshape(8192, 8192)[:, :4096], dsq[:, :4096]
    g2, dg2 = flat.reshape(8192, 8192)[:, 4096:], dsq[:, 4096:]
    add('concatenate two (8192,4096) f32 windows along axis 0', 2 * (h2.nbytes + g2.nbytes),
        run('cat0', lambda: cp.concatenate([dh2, dg2])), lambda: np.concatenate([h2, g2]),
        lambda: same(res['cat0'], np.concatenate([h2, g2])), 'cupy_copy')
    t1, dt1 = flat[:1 << 25].reshape(4096, 8192), dflat[:1 << 25].reshape(4096, 8192)
    t2, dt2 = flat[1 << 25:].reshape(4096, 8192), dflat[1 << 25:].reshape(4096, 8192)
    add('concatenate two (4096,8192) f32 along axis 1', 2 * flat.nbytes,
        run('cat1', lambda: cp.concatenate([dt1, dt2], axis=1)), lambda: np.concatenate([t1, t2], axis=1),
        lambda: same(res['cat1'], np.concatenate([t1, t2], axis=1)), 'cupy_copy')
    tl, dtl = flat[:1 << 24].reshape(4096, 4096), dflat[:1 << 24].reshape(4096, 4096)
    add('tile (4096,4096) f32 by (2,2)', 5 * tl.nbytes, run('tile', lambda: cp.tile(dtl, (2, 2))),
        lambda: np.tile(tl, (2, 2)), lambda: same(res['tile'], np.tile(tl, (2, 2))), 'cupy_copy')
    add('roll f32 8192x8192 by (1,1)', 2 * sq.nbytes, run('roll', lambda: cp.roll(dsq, (1, 1), (0, 1))),
        lambda: np.roll(sq, (1, 1), (0, 1)), lambda: same(res['roll'], np.roll(sq, (1, 1), (0, 1))), 'cupy_copy')
    return cases


CEILING_SOURCE = r'''
#include <cupy/carray.cuh>
typedef float T;
typedef cupy::Vec<T, 4> V4;
// Plain streaming kernels written by hand: 16 bytes per lane and access, KUN
// accesses per operand in flight per lane before the first is used, grid-stride
// over whole blocks of work, streaming (non-temporal) hints on loads and stores.
// KBLOCK (workgroup size) and KUN come from the command line: the suite runs a
// grid of variants and the best one per stream kind is the yardstick.  n is a
// multiple of 4*KBLOCK*KUN.
extern "C" __global__ void __launch_bounds__(KBLOCK)
ceil_read(const T* __restrict__ x, T* __restrict__ sink, long nvec) {
  const long per_iter = (long)KBLOCK * KUN;
  float s = 0;
  for (long base = (long)blockIdx.x * per_iter; base + per_iter <= nvec;
       base += (long)gridDim.x * per_iter) {
    V4 a[KUN];
#pragma unroll
    for (int u = 0; u < KUN; ++u)
      a[u] = cupy::load_vec<T, 4, true>(x + (base + u * KBLOCK + threadIdx.x) * 4);
#pragma unroll
    for (int u = 0; u < KUN; ++u) s += a[u].v[0] + a[u].v[1] + a[u].v[2] + a[u].v[3];
  }
  if (s == 12345.678f) sink[0] = s;   // keeps the loads alive, never true for the zeros read
}
extern "C" __global__ void __launch_bounds__(KBLOCK)
ceil_fill(T* __restrict__ z, long nvec) {
  const long per_iter = (long)KBLOCK * KUN;
  V4 a;
  a.v[0] = a.v[1] = a.v[2] = a.v[3] = 1.0f;
  for (long base = (long)blockIdx.x * per_iter; base + per_iter <= nvec;
       base += (long)gridDim.x * per_iter) {
#pragma unroll
    for (int u = 0; u < KUN; ++u)
      cupy::store_vec<T, 4, true>(z + (base + u * KBLOCK + threadIdx.x) * 4, a);
  }
}
extern "C" __global__ void __launch_bounds__(KBLOCK)
ceil_copy(const T* __restrict__ x, T* __restrict__ z, long nvec) {
  const long per_iter = (long)KBLOCK * KUN;
  for (long base = (long)blockIdx.x * per_iter; base + per_iter <= nvec;
       base += (long)gridDim.x * per_iter) {
    V4 a[KUN];
#pragma unroll
    for (int u = 0; u < KUN; ++u)
      a[u] = cupy::load_vec<T, 4, true>(x + (base + u * KBLOCK + threadIdx.x) * 4);
#pragma unroll
    for (int u = 0; u < KUN; ++u)
      cupy::store_vec<T, 4, true>(z + (base + u * KBLOCK + threadIdx.x) * 4, a[u]);
  }
}
extern "C" __global__ void __launch_bounds__(KBLOCK)
ceil_saxpy(const T* __restrict__ x, const T* __restrict__ y, T* __restrict__ z, long nvec) {
  const long per_iter = (long)KBLOCK * KUN;
  for (long base = (long)blockIdx.x * per_iter; base + per_iter <= nvec;
       base += (long)gridDim.x * per_iter) {
    V4 a[KUN], b[KUN];
#pragma unroll
    for (int u = 0; u < KUN; ++u) {
      a[u] = cupy::load_vec<T, 4, true>(x + (base + u * KBLOCK + threadIdx.x) * 4);
      b[u] = cupy::load_vec<T, 4, true>(y + (base + u * KBLOCK + threadIdx.x) * 4);
    }
#pragma unroll
    for (int u = 0; u < KUN; ++u) {
#pragma unroll
      for (int k = 0; k < 4; ++k) a[u].v[k] = 2.5f * a[u].v[k] + b[u].v[k];
      cupy::store_vec<T, 4, true>(z + (base + u * KBLOCK + threadIdx.x) * 4, a[u]);
    }
  }
}
'''


def build_ceiling_cases(cp):
    """The streaming ceiling of the device: what plain read-only, write-only,
    copy and two-in-one-out kernels reach, (a) written by hand (RawKernel) over
    a grid of workgroup sizes, accesses in flight per lane and grid sizes, (b)
    through ElementwiseKernel / ``sum`` / ``fill`` of this package, (c) as a
    device-to-device ``rt_memcpy_async``.  Arrays of 256 MiB and 1 GiB; every
    call works on the next of several buffer sets, so that nothing of a call's
    operands is left in the 256 MB memory-side cache from the call before."""
    cases = []

    def add(name, nbytes, gpu, kernel):
        cases.append(dict(name=name, config='ceiling', bytes=int(nbytes), gpu=gpu,
                          cpu=lambda: None, check=lambda: True, kernel=kernel))

    mods = {}
    for block in (256, 512, 1024):
        for un in (1, 2, 4):
            mods[block, un] = cp.RawModule(
                code=CEILING_SOURCE, options=('-DKBLOCK=%d' % block, '-DKUN=%d' % un))
    e_copy = cp.ElementwiseKernel('T x', 'T y', 'y = x', 'ew_copy')
    e_saxpy = cp.ElementwiseKernel('float32 x, float32 y, float32 a', 'float32 z',
                                   'z = a * x + y', 'ew_saxpy')
    sink = cp.zeros((4,), np.float32)
    cus = 256
    for mib in (256, 1024):
        n = mib * (1 << 20) // 4
        nvec = n // 4
        sets = 6 if mib == 256 else 3
        xs = [cp.zeros((n,), np.float32) for _ in range(sets)]
        ys = [cp.zeros((n,), np.float32) for _ in range(sets)]
        zs = [cp.empty((n,), np.float32) for _ in range(sets)]
        souts = [cp.empty((), np.float32) for _ in range(sets)]
        turn = [0]

        def rot(fn, sets=sets, turn=turn):
            def call():
                turn[0] = (turn[0] + 1) % sets
                fn(turn[0])
            return call
        tag = '%d MiB' % mib
        for (block, un), mod in mods.items():
            k_read, k_fill = mod.get_function('ceil_read'), mod.get_function('ceil_fill')
            k_copy, k_saxpy = mod.get_function('ceil_copy'), mod.get_function('ceil_saxpy')
            full = nvec // (block * un)
            for per_cu in (1, 4, 0):         # resident workgroups' worth of grid; 0 = no loop
                grid = (full if per_cu == 0 else min(full, cus * (2048 // block) * per_cu),)
                var = ' [block %d, %d in flight, grid %d]' % (block, un, grid[0])
                add('read   hand-written %s%s' % (tag, var), 4 * n,
                    rot(lambda i, k=k_read, g=grid, b=block, xs=xs, nvec=nvec:
                        k(g, (b,), (xs[i], sink, nvec))), 'ceil_read')
                add('fill   hand-written %s%s' % (tag, var), 4 * n,
                    rot(lambda i, k=k_fill, g=grid, b=block, zs=zs, nvec=nvec:
                        k(g, (b,), (zs[i], nvec))), 'ceil_fill')
                add('copy   hand-written %s%s' % (tag, var), 8 * n,
                    rot(lambda i, k=k_copy, g=grid, b=block, xs=xs, zs=zs, nvec=nvec:
                        k(g, (b,), (xs[i], zs[i], nvec))), 'ceil_copy')
                add('saxpy  hand-written %s%s' % (tag, var), 12 * n,
                    rot(lambda i, k=k_saxpy, g=grid, b=block, xs=xs, ys=ys, zs=zs, nvec=nvec:
                        k(g, (b,), (xs[i], ys[i], zs[i], nvec))), 'ceil_saxpy')
        add('read   sum() of this package %s' % tag, 4 * n,
            rot(lambda i, xs=xs, souts=souts: xs[i].sum(out=souts[i])), 'cupy_sum')
        add('fill   ndarray.fill of this package %s' % tag, 4 * n,
            rot(lambda i, zs=zs: zs[i].fill(1.0)), 'cupy_fill')
        add('copy   ElementwiseKernel of this package %s' % tag, 8 * n,
            rot(lambda i, xs=xs, zs=zs: e_copy(xs[i], zs[i])), 'ew_copy')
        add('copy   rt_memcpy_async device to device %s' % tag, 8 * n,
            rot(lambda i, xs=xs, zs=zs, n=n: zs[i].data.copy_from_device_async(xs[i].data, 4 * n)),
            'hipMemcpyAsync')
        add('saxpy  ElementwiseKernel of this package %s' % tag, 12 * n,
            rot(lambda i, xs=xs, ys=ys, zs=zs: e_saxpy(xs[i], ys[i], 2.5, zs[i])), 'ew_saxpy')
    return cases


def time_case_events(cp, fn, repeats, inner):
    """Median over ``repeats`` of the time per call, each sample being
    ``inner`` back-to-back calls bracketed by two events on the launch stream."""
    e0 = cp.cuda.Event()
    e1 = cp.cuda.Event()
    samples = []
    for _ in range(repeats):
        e0.record()
        for _ in range(inner):
            fn()
        e1.record()
        e1.synchronize()
        samples.append(cp.cuda.get_elapsed_time(e0, e1) * 1e-3 / inner)
    return float(np.median(samples)), float(np.min(samples))


def time_cases_in_step(cp, cases, steps):
    """Median and minimum over ``steps`` steps of every operation's time INSIDE
    the step: every kernel of the step is launched with a pair of events that
    receive the start and the end of its own execution (``KernelTimer``), an
    operation's time is the sum over its kernels.  Every operation starts on
    whatever its predecessor left in the caches, exactly as in the timed
    region, and the figures are what a profiler's kernel trace of the same
    step shows.  (Ten calls in a row on the same arrays, as
    ``time_case_events`` makes them, let operands of up to 512 MiB survive in
    part in the 256 MB memory-side cache and read a few percent too fast;
    events recorded BETWEEN the operations put a marker into the stream that
    costs 1 to 5 us per operation.)  Also returns the kernels of each operation."""
    from cupy_amd.profiler import KernelTimer
    n = len(cases)
    samples = [[] for _ in range(n)]
    kernels = [None] * n
    with KernelTimer() as timer:
        for c in cases:             # (the launch-by-launch path, once, untimed)
            c['gpu']()
        timer.durations()
        for _ in range(steps):
            marks = [0]
            for c in cases:
                c['gpu']()
                marks.append(timer.mark())
            spans = timer.durations()
            for i in range(n):
                mine = spans[marks[i]:marks[i + 1]]
                samples[i].append(sum(t for _, t in mine))
                kernels[i] = [name for name, _ in mine]
    return [(float(np.median(ts)), float(np.min(ts))) for ts in samples], kernels


def launch_latency(cp):
    """Host enqueue cost (us per call, 2000 asynchronous calls on tiny arrays)
    and event-bracketed single-call latency on an idle stream."""
    out = {}
    x = cp.zeros((1,), np.float32)
    y = cp.zeros((1,), np.float32)
    y0 = y.reshape(())
    k = cp.ElementwiseKernel('T x', 'T y', 'y = x + 1', 'tiny_add')

    @cp.fuse(kernel_name='tiny_fused')
    def fz(a):
        return a * 2 + 1

    pool = cp.get_default_memory_pool()

    def pool_cycle():
        pool.malloc(4096)

    ops = {'ElementwiseKernel': lambda: k(x, y), 'ufunc_add': lambda: cp.add(x, x, y),
           'sum': lambda: x.sum(out=y0), 'fuse': lambda: fz(x),
           'pool_malloc_free': pool_cycle}
    for name, fn in ops.items():
        for _ in range(20):
            fn()
        cp.cuda.Device().synchronize()
        n = 2000
        t0 = time.perf_counter()
        for _ in range(n):
            fn()
        t1 = time.perf_counter()
        cp.cuda.Device().synchronize()
        entry = {'host_enqueue_us': round((t1 - t0) / n * 1e6, 2)}
        if name != 'pool_malloc_free':
            e0, e1 = cp.cuda.Event(), cp.cuda.Event()
            lat = []
            for _ in range(50):
                cp.cuda.Device().synchronize()
                e0.record()
                fn()
                e1.record()
                e1.synchronize()
                lat.append(cp.cuda.get_elapsed_time(e0, e1) * 1e3)
            entry['single_call_us'] = round(float(np.median(lat)), 2)
        out[name] = entry
    return out


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument('--gpus', type=int, default=1)
    ap.add_argument('--steps', type=int, default=20)
    ap.add_argument('--warmup', type=int, default=3)
    ap.add_argument('--scale', type=int, default=1,
                    help='divide the problem sizes (for quick checks only; the '
                         'reported figure is then not the benchmark figure)')
    ap.add_argument('--no-cpu', action='store_true', help='skip the NumPy baseline')
    ap.add_argument('--no-detail', action='store_true',
                    help='skip per-operation event timing and launch latency')
    ap.add_argument('--only', default='', help='run only cases whose name contains this')
    ap.add_argument('--suite', default='configs', choices=('configs', 'next', 'layouts', 'ceiling'),
                    help="'configs': the five benchmark configurations (the headline figure); "
                         "'next': scans, statistics, complex types and multi-kernel fused "
                         "functions at shapes of the same size class; 'layouts': offset views, "
                         "odd and narrow rows, windows, permuted axes, mixed widths; 'ceiling': plain "
                         "read / fill / copy / saxpy streams over rotating buffers, the "
                         "yardstick the other suites are read against")
    ap.add_argument('--plan', default='',
                    help='write the names of the kernels every operation launches, in step '
                         'order, to this JSON file (bench_profiles.py maps profiler rows to '
                         'operations with it)')
    ap.add_argument('--calibrate', action='store_true',
                    help='add a plain copy kernel of known size (256 MiB in, 256 MiB out) to '
                         'every step, as the yardstick for hardware traffic counters')
    args = ap.parse_args()
    if args.gpus != 1:
        print('bench.py measures one GPU: every operation of this path runs on a '
              'single device; --gpus %d is not supported.' % args.gpus, file=sys.stderr)
        sys.exit(2)

    import cupy_amd as cp
    dev = cp.cuda.Device(0)
    dev.use()
    props = cp.cuda.device.get_device_properties(0)
    log('device:', props['arch'], props['compute_units'], 'CUs')
    t0 = time.perf_counter()
    cases = (build_cases(cp, args.scale) if args.suite == 'configs' else
             build_next_cases(cp) if args.suite == 'next' else
             build_ceiling_cases(cp) if args.suite == 'ceiling' else build_layout_cases(cp))
    if args.suite == 'ceiling':
        args.no_cpu = True
    if args.only:
        cases = [c for c in cases if args.only in c['name']]
    log('inputs ready in %.1f s' % (time.perf_counter() - t0))

    calib = None
    if args.calibrate:
        n_cal = 1 << 26
        cal_src = cp.zeros((n_cal,), np.float32)
        cal_dst = cp.empty((n_cal,), np.float32)
        cal_kernel = cp.ElementwiseKernel('T x', 'T y', 'y = x', 'calib_copy_256MiB')

        def calib():
            cal_kernel(cal_src, cal_dst)

    def step():
        for c in cases:
            c['gpu']()
        if calib is not None:
            calib()

    # warm-up (compiles / loads kernels, grows the pool)
    for _ in range(max(args.warmup, 1)):
        step()
    dev.synchronize()
    if args.plan:
        from cupy_amd.cuda import function as _function
        from cupy_amd._core import _launch_plan
        _launch_plan.use_quick = False      # every launch through Function.launch_packed
        seen = []
        real_launch = _function.Function.launch_packed

        def spy(self, *a, **k):
            seen.append(self.name)
            return real_launch(self, *a, **k)
        _function.Function.launch_packed = spy
        plan = []
        try:
            for c in cases + ([dict(name='calibration copy 256 MiB', bytes=2 << 28,
                                    gpu=calib)] if calib is not None else []):
                del seen[:]
                c['gpu']()
                plan.append({'name': c['name'], 'bytes': c['bytes'], 'kernels': list(seen)})
        finally:
            _function.Function.launch_packed = real_launch
            _launch_plan.use_quick = True
        dev.synchronize()
        os.makedirs(os.path.dirname(os.path.abspath(args.plan)), exist_ok=True)
        with open(args.plan, 'w') as f:
            json.dump({'suite': args.suite, 'scale': args.scale, 'steps': args.steps,
                       'warmup': max(args.warmup, 1), 'operations': plan}, f, indent=1)
    parity = {}
    for c in cases:
        parity[c['name']] = bool(c['check']())
        if not parity[c['name']]:
            log('PARITY FAILURE:', c['name'])

    # ---- timed region: exactly `steps` steps ------------------------------------------
    dev.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step()
    dev.synchronize()
    t1 = time.perf_counter()
    step_s = (t1 - t0) / args.steps
    total_bytes = sum(c['bytes'] for c in cases)
    value = total_bytes / step_s / 1e9

    per_config = []
    roof = None
    if not args.no_detail:
        in_step = kernels = None
        if args.suite != 'ceiling':
            in_step, kernels = time_cases_in_step(cp, cases, 15)
        for k, c in enumerate(cases):
            rep, rep_min = time_case_events(cp, c['gpu'], repeats=7 if in_step is None else 9,
                                            inner=10)
            med, mn = (rep, rep_min) if in_step is None else in_step[k]
            gbps = c['bytes'] / med / 1e9
            per_config.append({
                'name': c['name'], 'config': c['config'], 'kernel': c['kernel'],
                'bytes': c['bytes'], 'us': round(med * 1e6, 2), 'min_us': round(mn * 1e6, 2),
                'gbps': round(gbps, 1), 'frac': round(gbps / HBM_PEAK_GBPS, 4),
                'timing': 'ten calls in a row over rotating buffers' if in_step is None
                else 'inside the step, kernel by kernel',
                'kernels': None if kernels is None else kernels[k],
                'us_repeated_calls': round(rep * 1e6, 2),
                'parity': parity[c['name']]})
            log('%-42s %9.1f us  %8.1f GB/s  %5.1f%%   (ten calls in a row: %.1f us)' % (
                c['name'], med * 1e6, gbps, gbps / HBM_PEAK_GBPS * 100, rep * 1e6))
        dom = max(per_config, key=lambda e: e['us'])
        roof = {'bound': 'hbm', 'kernel': dom['kernel'], 'operation': dom['name'],
                'achieved': dom['gbps'], 'peak': HBM_PEAK_GBPS, 'unit': 'GB/s',
                'frac': dom['frac'],
                'traffic': measured_traffic().get(dom['name'])
                if args.scale == 1 and args.suite == 'configs' else None,
                'launch_us': dom['us'], 'algorithmic_bytes': dom['bytes']}
    else:
        roof = {'bound': 'hbm', 'achieved': round(value, 1), 'peak': HBM_PEAK_GBPS,
                'unit': 'GB/s', 'frac': round(value / HBM_PEAK_GBPS, 4), 'traffic': None}

    cpu = None
    if not args.no_cpu:
        # NumPy, single-threaded, one warm pass then the best of five passes
        # over the whole suite (about 15-25 s of CPU work)
        best = None
        for _ in range(6):
            c0 = time.perf_counter()
            for c in cases:
                c['cpu']()
            dt = time.perf_counter() - c0
            best = dt if best is None else min(best, dt)
        try:
            model = [l.split(':', 1)[1].strip() for l in open('/proc/cpuinfo')
                     if l.startswith('model name')][0]
        except Exception:
            model = 'unknown'
        cpu = {'value': round(total_bytes / best / 1e9, 2), 'unit': 'GB/s', 'cores': 1,
               'kind': 'port',
               'sample': 'one full pass of the same %d operations with NumPy %s on the host '
                         '(best of 5 after a warm pass, outputs preallocated where NumPy allows); '
                         '%d host cores visible, CPU: %s' % (
                             len(cases), np.__version__, os.cpu_count(), model),
               'seconds_per_pass': round(best, 3)}

    result = {
        'metric': 'achieved HBM GB/s (elementwise + reduction suite, algorithmic bytes / time)',
        'value': round(value, 1),
        'unit': 'GB/s',
        'n_gpus': 1,
        'steps': args.steps,
        'warmup': args.warmup,
        'ms_per_step': round(step_s * 1e3, 4),
        'higher_is_better': True,
        'scaling': 'weak',
        'vs_baseline': None,
        'dtype': 'f32/f64/f16/i32 (the element types of the five configurations)',
        'data': 'synthetic (seeded NumPy RNG, uploaded once)',
        'config': {'workload': 'C1-C5 of BASELINE.json at full shapes, 13 operations per step'
                   if args.scale == 1 and not args.only and args.suite == 'configs' else
                   'NOT the benchmark figure: scans, statistics, complex types and multi-kernel '
                   'fused functions, %d operations per step' % len(cases)
                   if args.suite == 'next' and not args.only else
                   'NOT the benchmark figure: offset views, odd and narrow rows, windows, permuted '
                   'axes, mixed widths, %d operations per step' % len(cases)
                   if args.suite == 'layouts' and not args.only else
                   'NOT the benchmark figure: plain streaming kernels over rotating buffers, '
                   '%d operations per step' % len(cases)
                   if args.suite == 'ceiling' and not args.only else
                   'REDUCED run (scale=%d only=%r): not the benchmark figure' % (args.scale, args.only),
                   'bytes_per_step': total_bytes, 'operations': len(cases)},
        'frac_of_hbm_peak': round(value / HBM_PEAK_GBPS, 4),
        'parity_ok': all(parity.values()),
        'roofline': roof,
        'cpu_baseline': cpu,
        'per_config': per_config,
    }
    if not args.no_detail:
        result['launch_us'] = launch_latency(cp)
    print(json.dumps(result))


if __name__ == '__main__':
    main()
