"""CPU oracle for the generated-kernel hot path -- TEST INFRASTRUCTURE, never
imported by the product (``cupy_amd``).

The parity target of this path is NumPy itself: the reference's own test suite
is a differential test against NumPy on identical inputs
(cupy/testing/_loops.py:270-375 ``numpy_cupy_allclose`` and friends), and every
result of ElementwiseKernel / ufunc / ReductionKernel / fuse calls in the five
benchmark configurations is defined as "what NumPy computes".  Each function
below states one of those operations with explicit rounding steps, and cites
the reference code whose device-side behaviour it stands for.

How each function is pinned (see tests/test_oracle.py):

* ``saxpy``, ``broadcast_mul_add``  exact arithmetic identities: every step is a
  single IEEE operation, checked against float64 evaluation rounded once per
  step, and against NumPy's own ufuncs.
* ``promote``       NumPy's ``result_type`` and the NEP-50 examples the reference
  holds in tests/cupy_tests/core_tests/test_nep50_examples.py:10-38.
* ``argmax_first`` / ``argmin_first``  brute-force definition; fixtures from
  tests/cupy_tests/sorting_tests/test_search.py:26-30,62-66,100-104,142-146 and
  ``numpy.argmax``.
* ``sum_fp``        ``math.fsum`` (exactly rounded) within the tolerance the task
  states; integer sums are exact (wrap-around in int64).
* ``fused_sqdiff_wsum``  per-step float16 rounding checked against float32
  evaluation followed by one rounding, and the closed form for x == y.
* ``ref_block_reduce_order`` (C, oracle/ref_kernels.c)  the summation ORDER of
  the reference's generic reduction kernel; pinned only through invariants
  (permutation of the same addends: equals fsum within rtol; exact for
  integers).  parity unpinned beyond that: the reference cannot run here.

Operations beyond the five configurations (the rest of the ufunc catalogue,
complex numbers, scans, statistics) have no restatement here: their tests call
NumPy directly on the same seeded inputs.  For the complex elementary functions
NumPy's value comes from the host C library, so agreement is to a stated
tolerance (32 eps * (1 + |result|) on the device, 4 eps for a host build of the
same formulas); parity unpinned below that tolerance.
"""
import math

import numpy as np


# --------------------------------------------------------------------------------
# elementwise
# --------------------------------------------------------------------------------

def saxpy(a, x, y):
    """z = a*x + y in float32 with two roundings (no fused multiply-add).

    Stands for ElementwiseKernel('float32 x, float32 y, float32 a',
    'float32 z', 'z = a * x + y') -- reference kernel template
    cupy/_core/_kernel.pyx:86-97; the Python scalar takes the parameter's
    dtype (cupy/_core/_kernel.pyx:920-922)."""
    a = np.float32(a)
    x = np.asarray(x, dtype=np.float32)
    y = np.asarray(y, dtype=np.float32)
    prod = np.multiply(a, x, dtype=np.float32)
    return np.add(prod, y, dtype=np.float32)


def promote(*operands):
    """Result dtype of a binary arithmetic ufunc under NEP 50: Python scalars
    are weak.  Stands for the first-matching-loop search with weak scalars,
    cupy/_core/_kernel.pyx:1656-1741."""
    return np.result_type(*operands)


def broadcast_mul_add(x, y, c=1):
    """out = x * y + c with NumPy broadcasting and promotion (two ufunc calls,
    the second with a weak Python scalar).  Stands for config 2: ufunc dispatch
    cupy/_core/_kernel.pyx:1241-1401, multiply/add loops
    cupy/_core/_routines_math.pyx:878-905,989-996."""
    t = np.multiply(x, y)
    return np.add(t, c)


# --------------------------------------------------------------------------------
# reductions
# --------------------------------------------------------------------------------

def sum_fp(a, axis=None, dtype=None):
    """NumPy's sum (pairwise summation along contiguous runs).  Stands for
    cupy_sum, cupy/_core/_routines_math.pyx:795-797; results are compared with a
    relative tolerance because the order of additions differs."""
    return np.sum(a, axis=axis, dtype=dtype)


def sum_tolerances(dtype):
    """rtol for floating-point reductions whose order differs from NumPy's."""
    return {'float16': 1e-3, 'float32': 1e-5, 'float64': 1e-12}[np.dtype(dtype).name]


def _square_sum64(a, axis):
    """Sum of squares in float64, without a float64 copy of a large array."""
    a = np.asarray(a)
    if a.size <= 1 << 24 or a.ndim == 0:
        return np.sum(np.square(a, dtype=np.float64), axis=axis)
    # large arrays in the tests are matrices: go through them in row blocks
    step = max(1, (1 << 24) // max(1, a.size // a.shape[0]))
    axes = tuple(range(a.ndim)) if axis is None else \
        tuple(ax % a.ndim for ax in (axis if isinstance(axis, tuple) else (axis,)))
    if 0 in axes:
        total = None
        for i in range(0, a.shape[0], step):
            part = np.sum(np.square(a[i:i + step], dtype=np.float64), axis=axes)
            total = part if total is None else total + part
        return total
    parts = [np.sum(np.square(a[i:i + step], dtype=np.float64), axis=axes)
             for i in range(0, a.shape[0], step)]
    return np.concatenate(parts, axis=0)


def forward_sum_bound(data, axis, dtype):
    """``(ref64, bound)`` of the forward check on a floating-point sum:
    ``|got - ref64| <= rtol * max(|ref64|, sigma * sqrt(N))`` with ``ref64``
    NumPy's float64 sum of the same data and ``sigma * sqrt(N)`` the root of the
    addends' square sum -- the size a sum of N values of spread sigma has when
    its mean is zero, so heavy cancellation does not turn rtol into nothing,
    while a dropped or doubled block of addends (which moves the result by
    about sigma * sqrt(block)) is far outside."""
    ref64 = np.sum(data, axis=axis, dtype=np.float64)
    floor = np.sqrt(_square_sum64(data, axis))
    return ref64, sum_tolerances(dtype) * np.maximum(np.abs(ref64), floor)


def check_sum_forward(got, data, axis, dtype):
    """Largest ``err / bound`` of the forward check (<= 1 passes)."""
    ref64, bound = forward_sum_bound(data, axis, dtype)
    err = np.abs(np.asarray(got).astype(np.float64).reshape(np.shape(ref64)) - ref64)
    return float(np.max(err / (bound + 1e-300))) if err.size else 0.0


def sum_exact(values):
    """Correctly rounded float64 sum of a 1-d sequence (``math.fsum``)."""
    return math.fsum(float(v) for v in np.asarray(values).ravel())


def sum_int(a, axis=None):
    """Integer sums: bool/signed -> int64, unsigned -> uint64, wrapping."""
    a = np.asarray(a)
    if a.dtype.kind in 'bi':
        return np.sum(a, axis=axis, dtype=np.int64)
    return np.sum(a, axis=axis, dtype=np.uint64)


def _arg_extreme_1d(v, want_max):
    """Index of the first extreme element of a 1-d array; NaN counts as more
    extreme than any number and the first NaN wins."""
    best = 0
    best_val = v[0]
    best_nan = best_val != best_val
    for j in range(1, len(v)):
        if best_nan:
            break
        x = v[j]
        if x != x:
            best, best_val, best_nan = j, x, True
        elif (x > best_val) if want_max else (x < best_val):
            best, best_val = j, x
    return best


def _arg_extreme(a, axis, want_max):
    a = np.asarray(a)
    if axis is None:
        flat = a.reshape(-1)           # C order, also for F-ordered input
        if flat.size == 0:
            raise ValueError('attempt to get argmax of an empty sequence')
        return np.int64(_arg_extreme_1d(flat, want_max))
    moved = np.moveaxis(a, axis, -1)
    if moved.shape[-1] == 0:
        raise ValueError('attempt to get argmax of an empty sequence')
    out = np.empty(moved.shape[:-1], dtype=np.int64)
    for idx in np.ndindex(*moved.shape[:-1]):
        out[idx] = _arg_extreme_1d(moved[idx], want_max)
    return out


def argmax_first(a, axis=None):
    """First index of the maximum (brute force).  Stands for cupy_argmax,
    cupy/_core/_routines_statistics.pyx:234-274,342-353."""
    return _arg_extreme(a, axis, True)


def argmin_first(a, axis=None):
    """First index of the minimum (brute force).  Stands for cupy_argmin,
    cupy/_core/_routines_statistics.pyx:234-274,328-340."""
    return _arg_extreme(a, axis, False)


def argmax_fast(a, axis=None):
    """Vectorised statement of the same rule for large inputs: where the
    maximum is attained, take the smallest index.  Only valid without NaNs."""
    a = np.asarray(a)
    if axis is None:
        a = a.reshape(-1)
        axis = 0
    m = a.max(axis=axis, keepdims=True)
    n = a.shape[axis]
    idx_shape = [1] * a.ndim
    idx_shape[axis] = n
    idx = np.arange(n, dtype=np.int64).reshape(idx_shape)
    return np.where(a == m, idx, n).min(axis=axis)


def argmin_fast(a, axis=None):
    a = np.asarray(a)
    if axis is None:
        a = a.reshape(-1)
        axis = 0
    m = a.min(axis=axis, keepdims=True)
    n = a.shape[axis]
    idx_shape = [1] * a.ndim
    idx_shape[axis] = n
    idx = np.arange(n, dtype=np.int64).reshape(idx_shape)
    return np.where(a == m, idx, n).min(axis=axis)


# --------------------------------------------------------------------------------
# fuse
# --------------------------------------------------------------------------------

def fused_sqdiff_wsum(x, y, w, axis=-1):
    """sum((x - y)**2 * w, axis) for float16 x, y and float32 w, with every
    intermediate rounded the way NumPy's loops round it: the difference and the
    square in float16 (computed in float32, rounded once), the product and the
    sum in float32.  Stands for the fused map-reduce of config 5
    (cupy/_core/fusion.pyx:744-785; loops 'ee->e' subtract/square, 'ff->f'
    multiply, 'f->f' sum)."""
    x = np.asarray(x, dtype=np.float16)
    y = np.asarray(y, dtype=np.float16)
    w = np.asarray(w, dtype=np.float32)
    d = (x.astype(np.float32) - y.astype(np.float32)).astype(np.float16)
    sq = (d.astype(np.float32) * d.astype(np.float32)).astype(np.float16)
    prod = sq.astype(np.float32) * w
    return np.sum(prod, axis=axis, dtype=np.float32)


# --------------------------------------------------------------------------------
# host helpers restated in closed form
# --------------------------------------------------------------------------------

def element_offsets(shape, strides):
    """Byte offset of every element of a strided view in C order
    (offset = sum(index[d] * strides[d])); the set of addresses a kernel may
    touch.  Used to check stride canonicalisation: a reduced view must visit
    the same offsets in the same order."""
    offs = np.zeros(shape, dtype=np.int64)
    for d, (n, st) in enumerate(zip(shape, strides)):
        idx_shape = [1] * len(shape)
        idx_shape[d] = n
        offs = offs + (np.arange(n, dtype=np.int64) * st).reshape(idx_shape)
    return offs.reshape(-1)
