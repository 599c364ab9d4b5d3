"""Prefix scans: cumsum / cumprod and their NaN-skipping variants.

Counterpart of the reference's ``scan_core`` (cupy/_core/_routines_math.pyx:
160-751; dtype rules :693-706).  The reference copies the input into the result
and scans it in place with a work-efficient LDS tree per 512-element block, a
recursive scan of the block sums and a fix-up pass.  Here the input is read
directly (converted on load) and there are two kernels for the two memory
orders of the scanned axis of a C-contiguous (outer, n, inner) problem:

``rows``  inner == 1, the scanned axis is contiguous.  A wave owns a chunk of
          the row: every lane loads TRIPS 128-bit vectors (all requested
          before the first is used), scans its elements in registers, the wave
          scans the lane totals with six shuffle steps per trip, and a running
          carry links the trips.  No LDS, no barrier.
``cols``  inner > 1, the scanned axis is strided.  A thread owns adjacent inner
          positions and walks down the scanned axis with a running value,
          several rows requested at a time.

A problem with too few rows (or columns) to fill the device is cut into chunks
along the scanned axis: pass 1 reduces every chunk to its total, the totals
are scanned by the same code, pass 3 scans the chunks seeded with the total of
everything before them.  Nothing spins on another workgroup's progress.
"""
import struct
import threading

import numpy

from cupy_amd._core import _tuning
from cupy_amd._core import internal
from cupy_amd._core._scalar import get_typename as _get_typename
from cupy_amd._core.core import ndarray
from cupy_amd.cuda import compiler
from cupy_amd.cuda import device as _device
from cupy_amd.cuda import stream as _stream

_SUM, _PROD = 0, 1
_BLOCK = 256
_WAVE = 64

_memo = {}
_lock = threading.Lock()


def _acc_type(t):
    return 'float' if t == 'float16' else t


def _emit(in_t, out_t, op, skip_nan, vec, trips, idx64, group=64):
    acc_t = _acc_type(out_t)
    idx_t = 'ptrdiff_t' if idx64 else 'int'
    op_c = '+' if op == _SUM else '*'
    ident = '0' if op == _SUM else '1'
    if skip_nan:
        conv = ('(_x != _x) ? _acc_t(%s) : static_cast<_acc_t>(_x)' % ident)
    else:
        conv = 'static_cast<_acc_t>(_x)'
    return '''#include <cupy/carray.cuh>
typedef %(in_t)s _in_t;
typedef %(out_t)s _out_t;
typedef %(acc_t)s _acc_t;
typedef %(idx_t)s _idx_t;
#define SCAN_OP(a, b) ((a) %(op_c)s (b))
#define SCAN_IDENTITY (_acc_t(%(ident)s))
#define VEC %(vec)d
#define TRIPS %(trips)d
#define GROUP %(group)d
__device__ __forceinline__ _acc_t _load_value(_in_t _x) { return %(conv)s; }

// mode 0: scan, no carry-in.  mode 1: write only the chunk totals.
// mode 2: scan seeded with carry[chunk - 1] (the inclusive scan of the totals).
template <int kMode>
__device__ __forceinline__ void scan_rows_impl(
    const _in_t* __restrict__ in, _out_t* __restrict__ out, _acc_t* __restrict__ totals,
    const _idx_t n_rows, const _idx_t n, const _idx_t n_chunks, const _idx_t chunk_len) {
  const int lane = threadIdx.x %% GROUP;
  const _idx_t n_work = n_rows * n_chunks;
  const _idx_t group_step = (_idx_t)gridDim.x * (%(block)d / GROUP);
  for (_idx_t w = (_idx_t)blockIdx.x * (%(block)d / GROUP) + threadIdx.x / GROUP; w < n_work;
       w += group_step) {
    const _idx_t row = w / n_chunks;
    const _idx_t chunk = w - row * n_chunks;
    const _idx_t j0 = chunk * chunk_len;
    const _idx_t j1 = (j0 + chunk_len < n) ? (j0 + chunk_len) : n;
    const _in_t* src = in + (ptrdiff_t)row * n;
    _acc_t carry = SCAN_IDENTITY;
    if (kMode == 2 && chunk > 0) carry = totals[(ptrdiff_t)row * n_chunks + chunk - 1];
    for (_idx_t base = j0; base < j1; base += GROUP * VEC * TRIPS) {
      // every load of this lane first ...
      cupy::Vec<_in_t, VEC> raw[TRIPS];
#pragma unroll
      for (int t = 0; t < TRIPS; ++t) {
        const _idx_t j = base + (t * GROUP + lane) * VEC;
        const _idx_t jc = (j + VEC <= j1) ? j : 0;       // the row start always holds a vector
        if (VEC > 1) raw[t] = cupy::load_vec<_in_t, VEC, true>(src + jc);
        else raw[t].v[0] = src[(j < j1) ? j : j0];
      }
#pragma unroll
      for (int t = 0; t < TRIPS; ++t) {
        const _idx_t j = base + (t * GROUP + lane) * VEC;
        _acc_t v[VEC];
        if (VEC > 1 && j + VEC > j1) {
          // ragged end of the chunk: element-wise, past-the-end = identity
#pragma unroll
          for (int k = 0; k < VEC; ++k) v[k] = (j + k < j1) ? _load_value(src[j + k]) : SCAN_IDENTITY;
        } else {
#pragma unroll
          for (int k = 0; k < VEC; ++k) v[k] = (j + k < j1) ? _load_value(raw[t].v[k]) : SCAN_IDENTITY;
        }
#pragma unroll
        for (int k = 1; k < VEC; ++k) v[k] = SCAN_OP(v[k - 1], v[k]);
        // inclusive scan of the lane totals across the wave
        _acc_t incl = v[VEC - 1];
#pragma unroll
        for (int d = 1; d < GROUP; d <<= 1) {
          const _acc_t o = cupy::shfl_up<GROUP>(incl, d);
          if (lane >= d) incl = SCAN_OP(o, incl);
        }
        const _acc_t trip_total = cupy::shfl_idx<GROUP>(incl, GROUP - 1);
        if (kMode != 1) {
          _acc_t before = cupy::shfl_up<GROUP>(incl, 1);
          before = (lane == 0) ? carry : SCAN_OP(carry, before);
          _out_t* dst = out + (ptrdiff_t)row * n + j;
          if (VEC > 1 && j + VEC <= j1) {
            cupy::Vec<_out_t, VEC> r;
#pragma unroll
            for (int k = 0; k < VEC; ++k) r.v[k] = static_cast<_out_t>(SCAN_OP(before, v[k]));
            cupy::store_vec<_out_t, VEC, false>(dst, r);
          } else {
#pragma unroll
            for (int k = 0; k < VEC; ++k)
              if (j + k < j1) dst[k] = static_cast<_out_t>(SCAN_OP(before, v[k]));
          }
        }
        carry = SCAN_OP(carry, trip_total);
      }
    }
    if (kMode == 1 && lane == 0) totals[(ptrdiff_t)row * n_chunks + chunk] = carry;
  }
}

template <int kMode>
__device__ __forceinline__ void scan_cols_impl(
    const _in_t* __restrict__ in, _out_t* __restrict__ out, _acc_t* __restrict__ totals,
    const _idx_t n_outer, const _idx_t n, const _idx_t inner, const _idx_t n_chunks,
    const _idx_t chunk_len) {
  const _idx_t inner_v = inner / VEC;            // the host guarantees inner %% VEC == 0
  const _idx_t n_work = n_outer * n_chunks * inner_v;
  for (_idx_t w = (_idx_t)blockIdx.x * %(block)d + threadIdx.x; w < n_work;
       w += (_idx_t)gridDim.x * %(block)d) {
    const _idx_t iv = w %% inner_v;
    const _idx_t oc = w / inner_v;
    const _idx_t chunk = oc %% n_chunks;
    const _idx_t o = oc / n_chunks;
    const _idx_t j0 = chunk * chunk_len;
    const _idx_t j1 = (j0 + chunk_len < n) ? (j0 + chunk_len) : n;
    const ptrdiff_t col = (ptrdiff_t)o * n * inner + (ptrdiff_t)iv * VEC;
    _acc_t run[VEC];
#pragma unroll
    for (int k = 0; k < VEC; ++k) run[k] = SCAN_IDENTITY;
    if (kMode == 2 && chunk > 0) {
#pragma unroll
      for (int k = 0; k < VEC; ++k)
        run[k] = totals[((ptrdiff_t)o * n_chunks + chunk - 1) * inner + (ptrdiff_t)iv * VEC + k];
    }
    _idx_t j = j0;
    for (; j + TRIPS <= j1; j += TRIPS) {
      cupy::Vec<_in_t, VEC> raw[TRIPS];
#pragma unroll
      for (int t = 0; t < TRIPS; ++t)
        raw[t] = cupy::load_vec<_in_t, VEC, true>(in + col + (ptrdiff_t)(j + t) * inner);
#pragma unroll
      for (int t = 0; t < TRIPS; ++t) {
        cupy::Vec<_out_t, VEC> r;
#pragma unroll
        for (int k = 0; k < VEC; ++k) {
          run[k] = SCAN_OP(run[k], _load_value(raw[t].v[k]));
          r.v[k] = static_cast<_out_t>(run[k]);
        }
        if (kMode != 1) cupy::store_vec<_out_t, VEC, false>(out + col + (ptrdiff_t)(j + t) * inner, r);
      }
    }
    for (; j < j1; ++j) {
      const cupy::Vec<_in_t, VEC> raw = cupy::load_vec<_in_t, VEC, true>(in + col + (ptrdiff_t)j * inner);
      cupy::Vec<_out_t, VEC> r;
#pragma unroll
      for (int k = 0; k < VEC; ++k) {
        run[k] = SCAN_OP(run[k], _load_value(raw.v[k]));
        r.v[k] = static_cast<_out_t>(run[k]);
      }
      if (kMode != 1) cupy::store_vec<_out_t, VEC, false>(out + col + (ptrdiff_t)j * inner, r);
    }
    if (kMode == 1) {
#pragma unroll
      for (int k = 0; k < VEC; ++k)
        totals[((ptrdiff_t)o * n_chunks + chunk) * inner + (ptrdiff_t)iv * VEC + k] = run[k];
    }
  }
}

#define ROWS_KERNEL(NAME, MODE) \\
extern "C" __global__ void __launch_bounds__(%(block)d) NAME( \\
    const _in_t* in, _out_t* out, _acc_t* totals, const _idx_t n_rows, const _idx_t n, \\
    const _idx_t n_chunks, const _idx_t chunk_len) { \\
  scan_rows_impl<MODE>(in, out, totals, n_rows, n, n_chunks, chunk_len); }
#define COLS_KERNEL(NAME, MODE) \\
extern "C" __global__ void __launch_bounds__(%(block)d) NAME( \\
    const _in_t* in, _out_t* out, _acc_t* totals, const _idx_t n_outer, const _idx_t n, \\
    const _idx_t inner, const _idx_t n_chunks, const _idx_t chunk_len) { \\
  scan_cols_impl<MODE>(in, out, totals, n_outer, n, inner, n_chunks, chunk_len); }
ROWS_KERNEL(cupy_scan_rows, 0)
ROWS_KERNEL(cupy_scan_rows_totals, 1)
ROWS_KERNEL(cupy_scan_rows_seeded, 2)
COLS_KERNEL(cupy_scan_cols, 0)
COLS_KERNEL(cupy_scan_cols_totals, 1)
COLS_KERNEL(cupy_scan_cols_seeded, 2)
''' % dict(in_t=in_t, out_t=out_t, acc_t=acc_t, idx_t=idx_t, op_c=op_c, ident=ident,
           vec=vec, trips=trips, conv=conv, block=_BLOCK, group=group)


def _module(in_dtype, out_dtype, op, skip_nan, vec, trips, idx64, group=64):
    key = (_device.get_device_id(), in_dtype.char, out_dtype.char, op, skip_nan, vec,
           trips, idx64, group)
    mod = _memo.get(key)
    if mod is None:
        src = _emit(_get_typename(in_dtype), _get_typename(out_dtype), op, skip_nan,
                    vec, trips, idx64, group)
        mod = compiler.compile_with_cache(src)
        with _lock:
            mod = _memo.setdefault(key, mod)
    return mod


def _acc_dtype(out_dtype):
    return numpy.dtype('float32') if out_dtype == numpy.float16 else out_dtype


def _scan_contiguous(src, dst, outer, n, inner, op, skip_nan, stream_ptr, may_chunk=True):
    """Scans the middle axis of C-contiguous (outer, n, inner) ``src`` into
    ``dst`` (same layout; may be the same memory if the dtypes agree)."""
    if outer * n * inner == 0:
        return
    in_dtype, out_dtype = src.dtype, dst.dtype
    cus = _device.get_compute_units(_device.get_device_id())
    idx64 = outer * n * inner > 0x7fffffff - (1 << 24)
    ic = 'q' if idx64 else 'i'
    item = max(in_dtype.itemsize, out_dtype.itemsize)
    if inner == 1:
        vec = max(1, 16 // item)
        while vec > 1 and (src.data.ptr % (vec * in_dtype.itemsize)
                           or dst.data.ptr % (vec * out_dtype.itemsize)
                           or (outer > 1 and n % vec) or n < vec):
            vec //= 2
        # short rows: a group of lanes smaller than a wave per row, each lane
        # with up to four vectors; long rows: whole waves
        trips = 4
        group = _WAVE
        while group > 1 and (group // 2) * vec * trips >= n:
            group //= 2
        while trips > 1 and group * vec * (trips // 2) >= n:
            trips //= 2
        per_group = group * vec * trips
        # enough waves to fill the device: cut rows into chunks if there are few
        want = cus * 16
        n_chunks = 1
        if may_chunk and group == _WAVE and outer < want and n > 2 * per_group:
            n_chunks = min((want + outer - 1) // outer, (n + per_group - 1) // per_group)
        chunk_len = (n + n_chunks - 1) // n_chunks
        chunk_len = (chunk_len + per_group - 1) // per_group * per_group
        n_chunks = (n + chunk_len - 1) // chunk_len
        mod = _module(in_dtype, out_dtype, op, skip_nan, vec, trips, idx64, group)
        groups = outer * n_chunks
        per_block = _BLOCK // group
        grid = max(1, min((groups + per_block - 1) // per_block, cus * 32))
        fmt = '@PPP' + ic * 4

        def launch(name, totals_ptr):
            blob = struct.pack(fmt, src.data.ptr, dst.data.ptr, totals_ptr, outer, n,
                               n_chunks, chunk_len)
            mod.get_function(name).launch_packed(
                (grid, 1, 1), (_BLOCK, 1, 1), blob, 0, stream_ptr)
        prefix = 'cupy_scan_rows'
        totals_shape = (outer, n_chunks, 1)
    else:
        vec = max(1, 16 // item)
        while vec > 1 and (src.data.ptr % (vec * in_dtype.itemsize)
                           or dst.data.ptr % (vec * out_dtype.itemsize)
                           or inner % vec):
            vec //= 2
        trips = 4
        threads = outer * (inner // vec)
        want = cus * 1024
        n_chunks = 1
        if may_chunk and threads < want and n >= 128:
            n_chunks = min((want + threads - 1) // threads, n // 64)
        chunk_len = (n + n_chunks - 1) // n_chunks
        n_chunks = (n + chunk_len - 1) // chunk_len
        mod = _module(in_dtype, out_dtype, op, skip_nan, vec, trips, idx64)
        work = threads * n_chunks
        grid = max(1, min((work + _BLOCK - 1) // _BLOCK, cus * 64))
        fmt = '@PPP' + ic * 5

        def launch(name, totals_ptr):
            blob = struct.pack(fmt, src.data.ptr, dst.data.ptr, totals_ptr, outer, n,
                               inner, n_chunks, chunk_len)
            mod.get_function(name).launch_packed(
                (grid, 1, 1), (_BLOCK, 1, 1), blob, 0, stream_ptr)
        prefix = 'cupy_scan_cols'
        totals_shape = (outer, n_chunks, inner)
    if n_chunks == 1:
        launch(prefix, 0)
        return
    totals = ndarray._new_contiguous(totals_shape, _acc_dtype(out_dtype))
    launch(prefix + '_totals', totals.data.ptr)
    # the totals are few: one more level of chunks would cost more launches
    # than it saves
    _scan_contiguous(totals, totals, totals_shape[0], n_chunks, totals_shape[2], op, False,
                     stream_ptr, may_chunk=totals.size > (1 << 20))
    launch(prefix + '_seeded', totals.data.ptr)


def scan_core(a, axis, op, dtype=None, out=None, skip_nan=False):
    """Inclusive scan of ``a`` along ``axis`` (``None``: of the flattened
    array) -- the body of cumsum / cumprod (dtype rules of
    cupy/_core/_routines_math.pyx:693-706)."""
    from cupy_amd._core import _ufuncs
    if out is None:
        if dtype is None:
            kind = a.dtype.kind
            if kind in 'bi':
                dtype = numpy.dtype('int64')
            elif kind == 'u':
                dtype = numpy.dtype('uint64')
            else:
                dtype = a.dtype
        dtype = numpy.dtype(dtype)
    else:
        dtype = out.dtype
    if dtype.kind not in 'biuf':
        raise TypeError('scan does not support dtype %s' % dtype)
    src = a
    if not src._c_contiguous or src.dtype.kind not in 'biuf':
        src = src.astype(dtype, order='C')
    if axis is None:
        shape = (a.size,)
        outer, n, inner = 1, a.size, 1
    else:
        axis = internal._normalize_axis_index(axis, a.ndim)
        shape = a.shape
        outer = internal.prod(shape[:axis])
        n = shape[axis]
        inner = internal.prod(shape[axis + 1:])
    if out is not None and out.shape != shape:
        raise ValueError('invalid shape of the output array')
    direct = out is not None and out._c_contiguous
    result = out if direct else ndarray._new_contiguous(shape, dtype)
    if direct and src is a and out.data.ptr != a.data.ptr:
        from cupy_amd._core._carray import may_share_bounds
        if may_share_bounds(a, out):
            src = a.copy()
    stream_ptr = _stream.get_current_stream_ptr()
    _scan_contiguous(src, result, outer, n, inner, op, skip_nan and src.dtype.kind == 'f',
                     stream_ptr)
    if out is not None and not direct:
        _ufuncs.elementwise_copy(result, out)
        return out
    return result


def cumsum(a, axis=None, dtype=None, out=None):
    """Cumulative sum along an axis (of the flattened array by default).

    .. seealso:: :func:`numpy.cumsum`
    """
    return scan_core(a, axis, _SUM, dtype, out)


def cumprod(a, axis=None, dtype=None, out=None):
    """Cumulative product along an axis (of the flattened array by default).

    .. seealso:: :func:`numpy.cumprod`
    """
    return scan_core(a, axis, _PROD, dtype, out)


def nancumsum(a, axis=None, dtype=None, out=None):
    """Cumulative sum with NaNs counted as zero.

    .. seealso:: :func:`numpy.nancumsum`
    """
    return scan_core(a, axis, _SUM, dtype, out, skip_nan=True)


def nancumprod(a, axis=None, dtype=None, out=None):
    """Cumulative product with NaNs counted as one.

    .. seealso:: :func:`numpy.nancumprod`
    """
    return scan_core(a, axis, _PROD, dtype, out, skip_nan=True)
