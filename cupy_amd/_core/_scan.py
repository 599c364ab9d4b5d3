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
from cupy_amd._core._kernel import _aligned
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


def _emit(in_t, out_t, op, skip_nan, vec, trips, idx64, group=64, stream=(True, False),
          ragged=True, reuse=False):
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
#define NT_LOAD %(ntl)s
#define NT_STORE %(nts)s
// CHUNK_REUSE: the totals pass and the seeded pass of a chunked scan read the
// input with plain loads, the seeded pass works through the chunks from the
// last to the first and stores past the cache: what the totals pass read last
// is still in the memory-side cache when the seeded pass asks for it first.
#define CHUNK_REUSE %(reuse)d
#define NT_LOAD_OF(MODE) ((MODE) == 0 || !CHUNK_REUSE ? NT_LOAD : false)
#define NT_STORE_OF(MODE) ((MODE) == 2 && CHUNK_REUSE ? true : NT_STORE)
#define GROUP %(group)d
// RAGGED: a row may end inside a vector (its length is no multiple of VEC)
#define RAGGED %(ragged)d
__device__ __forceinline__ _acc_t _load_value(_in_t _x) { return %(conv)s; }

// One round of loads of a group: TRIPS vectors per lane, all unconditional (a
// vector that would start past the end of the chunk is read from the row start
// instead, which always holds one; its values are not used).
template <bool kStream>
__device__ __forceinline__ void _rows_load(
    cupy::Vec<_in_t, VEC> (&raw)[TRIPS], const _in_t* __restrict__ src, const _idx_t base,
    const _idx_t j0, const _idx_t j1, const int lane) {
#pragma unroll
  for (int t = 0; t < TRIPS; ++t) {
    const _idx_t j = base + (t * GROUP + lane) * VEC;
    const _idx_t jc = (j + VEC <= j1) ? j : 0;
    if (VEC > 1) raw[t] = cupy::load_vec<_in_t, VEC, kStream>(src + jc);
    else raw[t].v[0] = src[(j < j1) ? j : j0];
  }
}

// mode 0: scan, no carry-in.  mode 1: write only the chunk totals.
// mode 2: scan seeded with carry[chunk - 1] (the inclusive scan of the totals).
template <int kMode>
__device__ __forceinline__ void scan_rows_impl(
    const _in_t* __restrict__ in, _out_t* __restrict__ out, _acc_t* __restrict__ totals,
    const _idx_t n_rows, const _idx_t n, const _idx_t n_chunks, const _idx_t chunk_len) {
  const int lane = threadIdx.x %% GROUP;
  const _idx_t n_work = n_rows * n_chunks;
  const _idx_t group_step = (_idx_t)gridDim.x * (%(block)d / GROUP);
  for (_idx_t w0 = (_idx_t)blockIdx.x * (%(block)d / GROUP) + threadIdx.x / GROUP; w0 < n_work;
       w0 += group_step) {
    const _idx_t w = (kMode == 2 && CHUNK_REUSE) ? n_work - 1 - w0 : w0;
    const _idx_t row = w / n_chunks;
    const _idx_t chunk = w - row * n_chunks;
    const _idx_t j0 = chunk * chunk_len;
    const _idx_t j1 = (j0 + chunk_len < n) ? (j0 + chunk_len) : n;
    const _in_t* src = in + (ptrdiff_t)row * n;
    _acc_t carry = SCAN_IDENTITY;
    if (kMode == 2 && chunk > 0) carry = totals[(ptrdiff_t)row * n_chunks + chunk - 1];
    // the vectors of the first round; later rounds are requested one round
    // ahead, before the current one is scanned
    cupy::Vec<_in_t, VEC> raw[TRIPS];
    _rows_load<NT_LOAD_OF(kMode)>(raw, src, j0, j0, j1, lane);
    for (_idx_t base = j0; base < j1; base += GROUP * VEC * TRIPS) {
      cupy::Vec<_in_t, VEC> next[TRIPS];
      const _idx_t nbase = base + GROUP * VEC * TRIPS;
      if (nbase < j1) _rows_load<NT_LOAD_OF(kMode)>(next, src, nbase, j0, j1, lane);
      _acc_t v[TRIPS][VEC];
#pragma unroll
      for (int t = 0; t < TRIPS; ++t) {
        const _idx_t j = base + (t * GROUP + lane) * VEC;
        if (RAGGED && VEC > 1 && j + VEC > j1) {
          // a row that ends inside this vector: element-wise, past-the-end = identity
#pragma unroll
          for (int k = 0; k < VEC; ++k)
            v[t][k] = (j + k < j1) ? _load_value(src[j + k]) : SCAN_IDENTITY;
        } else {
#pragma unroll
          for (int k = 0; k < VEC; ++k)
            v[t][k] = ((RAGGED ? j + k : j) < j1) ? _load_value(raw[t].v[k]) : SCAN_IDENTITY;
        }
#pragma unroll
        for (int k = 1; k < VEC; ++k) v[t][k] = SCAN_OP(v[t][k - 1], v[t][k]);
      }
      if (kMode == 1) {
        // only the chunk total is wanted: a per-lane running value, combined
        // across the lanes once, after the last round
#pragma unroll
        for (int t = 0; t < TRIPS; ++t) carry = SCAN_OP(carry, v[t][VEC - 1]);
      } else {
        // inclusive scans of the lane totals across the group, the TRIPS
        // independent scans step by step side by side
        _acc_t incl[TRIPS];
#pragma unroll
        for (int t = 0; t < TRIPS; ++t) incl[t] = v[t][VEC - 1];
#pragma unroll
        for (int d = 1; d < GROUP; d <<= 1) {
#pragma unroll
          for (int t = 0; t < TRIPS; ++t) {
            const _acc_t o = cupy::shfl_up<GROUP>(incl[t], d);
            incl[t] = (lane >= d) ? SCAN_OP(o, incl[t]) : incl[t];
          }
        }
#pragma unroll
        for (int t = 0; t < TRIPS; ++t) {
          const _idx_t j = base + (t * GROUP + lane) * VEC;
          const _acc_t trip_total = cupy::shfl_idx<GROUP>(incl[t], GROUP - 1);
          _acc_t before = cupy::shfl_up<GROUP>(incl[t], 1);
          before = (lane == 0) ? carry : SCAN_OP(carry, before);
          _out_t* dst = out + (ptrdiff_t)row * n + j;
          if (VEC > 1 && (RAGGED ? j + VEC <= j1 : j < j1)) {
            cupy::Vec<_out_t, VEC> r;
#pragma unroll
            for (int k = 0; k < VEC; ++k) r.v[k] = static_cast<_out_t>(SCAN_OP(before, v[t][k]));
            cupy::store_vec<_out_t, VEC, NT_STORE_OF(kMode)>(dst, r);
          } else if (RAGGED || VEC == 1) {
#pragma unroll
            for (int k = 0; k < VEC; ++k)
              if (j + k < j1) dst[k] = static_cast<_out_t>(SCAN_OP(before, v[t][k]));
          }
          carry = SCAN_OP(carry, trip_total);
        }
      }
#pragma unroll
      for (int t = 0; t < TRIPS; ++t) raw[t] = next[t];
    }
    if (kMode == 1) {
#pragma unroll
      for (int m = GROUP / 2; m > 0; m >>= 1) carry = SCAN_OP(carry, cupy::shfl_xor(carry, m));
      if (lane == 0) totals[(ptrdiff_t)row * n_chunks + chunk] = carry;
    }
  }
}

template <int kMode>
__device__ __forceinline__ void scan_cols_impl(
    const _in_t* __restrict__ in, _out_t* __restrict__ out, _acc_t* __restrict__ totals,
    const _idx_t n_outer, const _idx_t n, const _idx_t inner, const _idx_t n_chunks,
    const _idx_t chunk_len) {
  const _idx_t inner_v = inner / VEC;            // the host guarantees inner %% VEC == 0
  const _idx_t n_work = n_outer * n_chunks * inner_v;
  for (_idx_t w0 = (_idx_t)blockIdx.x * %(block)d + threadIdx.x; w0 < n_work;
       w0 += (_idx_t)gridDim.x * %(block)d) {
    const _idx_t w = (kMode == 2 && CHUNK_REUSE) ? n_work - 1 - w0 : w0;
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
        raw[t] = cupy::load_vec<_in_t, VEC, NT_LOAD_OF(kMode)>(in + col + (ptrdiff_t)(j + t) * inner);
#pragma unroll
      for (int t = 0; t < TRIPS; ++t) {
        cupy::Vec<_out_t, VEC> r;
#pragma unroll
        for (int k = 0; k < VEC; ++k) {
          run[k] = SCAN_OP(run[k], _load_value(raw[t].v[k]));
          r.v[k] = static_cast<_out_t>(run[k]);
        }
        if (kMode != 1) cupy::store_vec<_out_t, VEC, NT_STORE_OF(kMode)>(out + col + (ptrdiff_t)(j + t) * inner, r);
      }
    }
    for (; j < j1; ++j) {
      const cupy::Vec<_in_t, VEC> raw = cupy::load_vec<_in_t, VEC, NT_LOAD_OF(kMode)>(in + col + (ptrdiff_t)j * inner);
      cupy::Vec<_out_t, VEC> r;
#pragma unroll
      for (int k = 0; k < VEC; ++k) {
        run[k] = SCAN_OP(run[k], _load_value(raw.v[k]));
        r.v[k] = static_cast<_out_t>(run[k]);
      }
      if (kMode != 1) cupy::store_vec<_out_t, VEC, NT_STORE_OF(kMode)>(out + col + (ptrdiff_t)j * inner, r);
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
           vec=vec, trips=trips, conv=conv, block=_BLOCK, group=group,
           ntl='true' if stream[0] else 'false', nts='true' if stream[1] else 'false',
           ragged=1 if ragged else 0, reuse=1 if reuse else 0)


def _emit_lanes(in_t, out_t, op, skip_nan, vec, trips, idx64, lstride, stream):
    """Scan along the middle axis of (outer, n, inner) when ``inner`` is a few
    vectors wide: a row of ``inner = lstride * vec`` elements sits in
    ``lstride`` adjacent lanes, a wave holds ``64 / lstride`` consecutive rows
    per load -- contiguous in memory, so accesses stay coalesced however narrow
    the array is -- and the scan runs across the lanes in steps of ``lstride``
    (Kogge-Stone over rows; the ``vec`` columns of a lane never mix).
    ``lstride`` need not be a power of two: the lanes past the last whole row
    of a wave stay idle."""
    acc_t = _acc_type(out_t)
    op_c = '+' if op == _SUM else '*'
    ident = '0' if op == _SUM else '1'
    if skip_nan:
        conv = ('(_x != _x) ? _acc_t(%s) : static_cast<_acc_t>(_x)' % ident)
    else:
        conv = 'static_cast<_acc_t>(_x)'
    return """#include <cupy/carray.cuh>
typedef %(in_t)s _in_t;
typedef %(out_t)s _out_t;
typedef %(acc_t)s _acc_t;
typedef %(idx_t)s _idx_t;
#define SCAN_OP(a, b) ((a) %(op_c)s (b))
#define SCAN_IDENTITY (_acc_t(%(ident)s))
#define VEC %(vec)d
#define TRIPS %(trips)d
#define NT_LOAD %(ntl)s
#define NT_STORE %(nts)s
#define LSTRIDE %(lstride)d
#define INNER (LSTRIDE * VEC)
#define TRIP_ROWS (64 / LSTRIDE)
__device__ __forceinline__ _acc_t _load_value(_in_t _x) { return %(conv)s; }

// mode 0: scan, no carry-in.  mode 1: write only the chunk totals (one per
// column).  mode 2: scan seeded with the inclusive scan of the totals.
template <int kMode>
__device__ __forceinline__ void scan_lanes_impl(
    const _in_t* __restrict__ in, _out_t* __restrict__ out, _acc_t* __restrict__ totals,
    const _idx_t n_outer, const _idx_t n, const _idx_t n_chunks, const _idx_t chunk_rows) {
  const int lane = threadIdx.x %% 64;
  const int lrow = lane / LSTRIDE;
  const int lcol = (lane %% LSTRIDE) * VEC;
  const _idx_t n_work = n_outer * n_chunks;
  const _idx_t wave_step = (_idx_t)gridDim.x * (%(block)d / 64);
  for (_idx_t w = (_idx_t)blockIdx.x * (%(block)d / 64) + threadIdx.x / 64; w < n_work;
       w += wave_step) {
    const _idx_t o = w / n_chunks;
    const _idx_t chunk = w - o * n_chunks;
    const _idx_t r0 = chunk * chunk_rows;
    const _idx_t r1 = (r0 + chunk_rows < n) ? (r0 + chunk_rows) : n;
    const _in_t* src = in + (ptrdiff_t)o * n * INNER + lcol;
    _out_t* dst = out + (ptrdiff_t)o * n * INNER + lcol;
    _acc_t carry[VEC];
#pragma unroll
    for (int k = 0; k < VEC; ++k) carry[k] = SCAN_IDENTITY;
    if (kMode == 2 && chunk > 0) {
#pragma unroll
      for (int k = 0; k < VEC; ++k)
        carry[k] = totals[((ptrdiff_t)o * n_chunks + chunk - 1) * INNER + lcol + k];
    }
    for (_idx_t rb = r0; rb < r1; rb += TRIP_ROWS * TRIPS) {
      // every load of the round is requested before the first value is used; a
      // row past the end of the chunk is read from the chunk's first row instead
      cupy::Vec<_in_t, VEC> raw[TRIPS];
#pragma unroll
      for (int t = 0; t < TRIPS; ++t) {
        const _idx_t r = rb + t * TRIP_ROWS + lrow;
        raw[t] = cupy::load_vec<_in_t, VEC, NT_LOAD>(
            src + (ptrdiff_t)((r < r1 && lrow < TRIP_ROWS) ? r : r0) * INNER);
      }
      _acc_t v[TRIPS][VEC];
#pragma unroll
      for (int t = 0; t < TRIPS; ++t) {
        const _idx_t r = rb + t * TRIP_ROWS + lrow;
#pragma unroll
        for (int k = 0; k < VEC; ++k)
          v[t][k] = (r < r1 && lrow < TRIP_ROWS) ? _load_value(raw[t].v[k]) : SCAN_IDENTITY;
      }
      if (kMode == 1) {
        // only the column totals of the chunk are wanted: every lane adds up
        // its own rows; the lanes are combined once, after the last round
#pragma unroll
        for (int t = 0; t < TRIPS; ++t) {
#pragma unroll
          for (int k = 0; k < VEC; ++k) carry[k] = SCAN_OP(carry[k], v[t][k]);
        }
        continue;
      }
      // inclusive scan over the rows of each trip: lanes LSTRIDE apart hold the
      // same columns of neighbouring rows
#pragma unroll
      for (int d = LSTRIDE; d < 64; d <<= 1) {
#pragma unroll
        for (int t = 0; t < TRIPS; ++t) {
#pragma unroll
          for (int k = 0; k < VEC; ++k) {
            const _acc_t up = cupy::shfl_up<64>(v[t][k], d);
            v[t][k] = (lane >= d) ? SCAN_OP(up, v[t][k]) : v[t][k];
          }
        }
      }
#pragma unroll
      for (int t = 0; t < TRIPS; ++t) {
        const _idx_t r = rb + t * TRIP_ROWS + lrow;
        cupy::Vec<_out_t, VEC> res;
#pragma unroll
        for (int k = 0; k < VEC; ++k) {
          // the trip's total of this column sits in the last row of the wave
          const _acc_t total = cupy::shfl_idx<64>(
              v[t][k], (TRIP_ROWS - 1) * LSTRIDE + lane %% LSTRIDE);
          res.v[k] = static_cast<_out_t>(SCAN_OP(carry[k], v[t][k]));
          carry[k] = SCAN_OP(carry[k], total);
        }
        if (kMode != 1 && r < r1 && lrow < TRIP_ROWS)
          cupy::store_vec<_out_t, VEC, NT_STORE>(dst + (ptrdiff_t)r * INNER, res);
      }
    }
    if (kMode == 1) {
      // the rows of the wave are combined like a scan; its last row then holds
      // the totals
#pragma unroll
      for (int d = LSTRIDE; d < 64; d <<= 1) {
#pragma unroll
        for (int k = 0; k < VEC; ++k) {
          const _acc_t up = cupy::shfl_up<64>(carry[k], d);
          carry[k] = (lane >= d) ? SCAN_OP(up, carry[k]) : carry[k];
        }
      }
      if (lrow == TRIP_ROWS - 1) {
#pragma unroll
        for (int k = 0; k < VEC; ++k)
          totals[((ptrdiff_t)o * n_chunks + chunk) * INNER + lcol + k] = carry[k];
      }
    }
  }
}

#define LANES_KERNEL(NAME, MODE) \\
extern "C" __global__ void __launch_bounds__(%(block)d) NAME( \\
    const _in_t* in, _out_t* out, _acc_t* totals, const _idx_t n_outer, const _idx_t n, \\
    const _idx_t n_chunks, const _idx_t chunk_rows) { \\
  scan_lanes_impl<MODE>(in, out, totals, n_outer, n, n_chunks, chunk_rows); }
LANES_KERNEL(cupy_scan_lanes, 0)
LANES_KERNEL(cupy_scan_lanes_totals, 1)
LANES_KERNEL(cupy_scan_lanes_seeded, 2)
""" % dict(in_t=in_t, out_t=out_t, acc_t=acc_t, idx_t='ptrdiff_t' if idx64 else 'int',
           op_c=op_c, ident=ident, vec=vec, trips=trips, conv=conv, block=_BLOCK,
           lstride=lstride, ntl='true' if stream[0] else 'false',
           nts='true' if stream[1] else 'false')


def _tile_geometry(inner, vec, trips):
    """(rows per round, segments, rows per segment, words between segments in
    the LDS) of the staged kernel for ``inner`` columns."""
    tile = _WAVE * vec * trips
    seg = _WAVE // inner
    lrows = (tile // inner) // seg
    # segments start `inner` banks apart, so the lanes of one access touch
    # distinct banks
    pad = (inner - (lrows * inner) % 32) % 32
    return seg * lrows, seg, lrows, lrows * inner + pad


def _emit_tile(in_t, out_t, op, skip_nan, vec, trips, idx64, inner, stream, reuse):
    """Scan along the middle axis of (outer, n, inner) for 2 <= inner <= 32.

    A wave takes ``ROWS_T`` consecutive rows per round -- one contiguous piece
    of memory, read with full 128-bit vectors on consecutive lanes whatever the
    width of the array -- and lays them out in the LDS.  Lane (s, c) then owns
    ``LROWS`` consecutive rows of column c (segment s of the tile): it scans them
    in registers, the totals of the segments of a column are scanned across the
    lanes (shuffles in steps of ``INNER`` lanes), every lane adds what came
    before its segment, and the tile goes back through the LDS into one
    contiguous store.  No barrier: a wave only ever reads what it wrote itself."""
    acc_t = _acc_type(out_t)
    op_c = '+' if op == _SUM else '*'
    ident = '0' if op == _SUM else '1'
    if skip_nan:
        conv = ('(_x != _x) ? _acc_t(%s) : static_cast<_acc_t>(_x)' % ident)
    else:
        conv = 'static_cast<_acc_t>(_x)'
    rows_t, seg, lrows, stride = _tile_geometry(inner, vec, trips)
    return """#include <cupy/carray.cuh>
typedef %(in_t)s _in_t;
typedef %(out_t)s _out_t;
typedef %(acc_t)s _acc_t;
typedef %(idx_t)s _idx_t;
#define SCAN_OP(a, b) ((a) %(op_c)s (b))
#define SCAN_IDENTITY (_acc_t(%(ident)s))
#define VEC %(vec)d
#define TRIPS %(trips)d
#define NT_LOAD %(ntl)s
#define NT_STORE %(nts)s
#define CHUNK_REUSE %(reuse)d
#define NT_LOAD_OF(MODE) ((MODE) == 0 || !CHUNK_REUSE ? NT_LOAD : false)
#define NT_STORE_OF(MODE) ((MODE) == 2 && CHUNK_REUSE ? true : NT_STORE)
#define INNER %(inner)d
#define ROWS_T %(rows_t)d
#define SEG %(seg)d
#define LROWS %(lrows)d
#define SEG_STRIDE %(stride)d
#define LDS_WORDS (SEG * SEG_STRIDE)
__device__ __forceinline__ _acc_t _load_value(_in_t _x) { return %(conv)s; }
// position in the LDS of element p of the tile (p = row * INNER + column)
__device__ __forceinline__ int _lds_at(int p) { return p + (p / (LROWS * INNER)) * (SEG_STRIDE - LROWS * INNER); }

template <int kMode>
__device__ __forceinline__ void scan_tile_impl(
    const _in_t* __restrict__ in, _out_t* __restrict__ out, _acc_t* __restrict__ totals,
    const _idx_t n_outer, const _idx_t n, const _idx_t n_chunks, const _idx_t chunk_rows) {
  __shared__ _acc_t _lds_all[%(block)d / 64][LDS_WORDS];
  _acc_t* lds = _lds_all[threadIdx.x / 64];
  const int lane = threadIdx.x %% 64;
  const int seg = lane / INNER;
  const int col = lane - seg * INNER;
  const bool active = lane < SEG * INNER;
  const _idx_t n_work = n_outer * n_chunks;
  const _idx_t wave_step = (_idx_t)gridDim.x * (%(block)d / 64);
  for (_idx_t w0 = (_idx_t)blockIdx.x * (%(block)d / 64) + threadIdx.x / 64; w0 < n_work;
       w0 += wave_step) {
    const _idx_t w = (kMode == 2 && CHUNK_REUSE) ? n_work - 1 - w0 : w0;
    const _idx_t o = w / n_chunks;
    const _idx_t chunk = w - o * n_chunks;
    const _idx_t r0 = chunk * chunk_rows;
    const _idx_t r1 = (r0 + chunk_rows < n) ? (r0 + chunk_rows) : n;
    _acc_t carry = SCAN_IDENTITY;
    if (kMode == 2 && chunk > 0 && active)
      carry = totals[((ptrdiff_t)o * n_chunks + chunk - 1) * INNER + col];
    for (_idx_t rb = r0; rb < r1; rb += ROWS_T) {
      const int rows_here = (r1 - rb < ROWS_T) ? (int)(r1 - rb) : ROWS_T;
      const int valid = rows_here * INNER;
      const _in_t* src = in + ((ptrdiff_t)o * n + rb) * INNER;
      _out_t* dst = out + ((ptrdiff_t)o * n + rb) * INNER;
      // every load of the round is requested before the first value is used
      cupy::Vec<_in_t, VEC> raw[TRIPS];
#pragma unroll
      for (int t = 0; t < TRIPS; ++t) {
        const int p = (t * 64 + lane) * VEC;
        if (p + VEC <= valid) {
          raw[t] = cupy::load_vec<_in_t, VEC, NT_LOAD_OF(kMode)>(src + p);
        } else {
#pragma unroll
          for (int k = 0; k < VEC; ++k) raw[t].v[k] = (p + k < valid) ? src[p + k] : _in_t();
        }
      }
#pragma unroll
      for (int t = 0; t < TRIPS; ++t) {
        const int p = (t * 64 + lane) * VEC;
#pragma unroll
        for (int k = 0; k < VEC; ++k)
          if (p + k < ROWS_T * INNER)
            lds[_lds_at(p + k)] = (p + k < valid) ? _load_value(raw[t].v[k]) : SCAN_IDENTITY;
      }
      __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
      __builtin_amdgcn_wave_barrier();
      // the lane's own rows of its column, scanned in registers
      _acc_t v[LROWS];
      if (active) {
#pragma unroll
        for (int i = 0; i < LROWS; ++i) v[i] = lds[seg * SEG_STRIDE + i * INNER + col];
#pragma unroll
        for (int i = 1; i < LROWS; ++i) v[i] = SCAN_OP(v[i - 1], v[i]);
      } else {
#pragma unroll
        for (int i = 0; i < LROWS; ++i) v[i] = SCAN_IDENTITY;
      }
      // totals of the segments of one column sit INNER lanes apart
      _acc_t incl = v[LROWS - 1];
#pragma unroll
      for (int d = 1; d < SEG; d <<= 1) {
        const _acc_t other = cupy::shfl_up<64>(incl, d * INNER);
        incl = (lane >= d * INNER) ? SCAN_OP(other, incl) : incl;
      }
      const _acc_t column_total = cupy::shfl_idx<64>(incl, (SEG - 1) * INNER + col);
      if (kMode != 1) {
        _acc_t before = cupy::shfl_up<64>(incl, INNER);
        before = (seg == 0) ? carry : SCAN_OP(carry, before);
        if (active) {
#pragma unroll
          for (int i = 0; i < LROWS; ++i)
            lds[seg * SEG_STRIDE + i * INNER + col] = SCAN_OP(before, v[i]);
        }
        __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
        __builtin_amdgcn_wave_barrier();
#pragma unroll
        for (int t = 0; t < TRIPS; ++t) {
          const int p = (t * 64 + lane) * VEC;
          if (p + VEC <= valid) {
            cupy::Vec<_out_t, VEC> r;
#pragma unroll
            for (int k = 0; k < VEC; ++k) r.v[k] = static_cast<_out_t>(lds[_lds_at(p + k)]);
            cupy::store_vec<_out_t, VEC, NT_STORE_OF(kMode)>(dst + p, r);
          } else {
#pragma unroll
            for (int k = 0; k < VEC; ++k)
              if (p + k < valid) dst[p + k] = static_cast<_out_t>(lds[_lds_at(p + k)]);
          }
        }
        __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
        __builtin_amdgcn_wave_barrier();
      }
      carry = SCAN_OP(carry, column_total);
    }
    if (kMode == 1 && lane < INNER)
      totals[((ptrdiff_t)o * n_chunks + chunk) * INNER + col] = carry;
  }
}

#define TILE_KERNEL(NAME, MODE) \\
extern "C" __global__ void __launch_bounds__(%(block)d) NAME( \\
    const _in_t* in, _out_t* out, _acc_t* totals, const _idx_t n_outer, const _idx_t n, \\
    const _idx_t n_chunks, const _idx_t chunk_rows) { \\
  scan_tile_impl<MODE>(in, out, totals, n_outer, n, n_chunks, chunk_rows); }
TILE_KERNEL(cupy_scan_tile, 0)
TILE_KERNEL(cupy_scan_tile_totals, 1)
TILE_KERNEL(cupy_scan_tile_seeded, 2)
""" % dict(in_t=in_t, out_t=out_t, acc_t=acc_t, idx_t='ptrdiff_t' if idx64 else 'int',
           op_c=op_c, ident=ident, vec=vec, trips=trips, conv=conv, block=_BLOCK,
           inner=inner, rows_t=rows_t, seg=seg, lrows=lrows, stride=stride,
           ntl='true' if stream[0] else 'false', nts='true' if stream[1] else 'false',
           reuse=1 if reuse else 0)


def _module_tile(in_dtype, out_dtype, op, skip_nan, vec, trips, idx64, inner, stream, reuse):
    key = ('tile', _device.get_device_id(), in_dtype.char, out_dtype.char, op, skip_nan, vec,
           trips, idx64, inner, stream, reuse)
    mod = _memo.get(key)
    if mod is None:
        src = _emit_tile(_get_typename(in_dtype), _get_typename(out_dtype), op, skip_nan,
                         vec, trips, idx64, inner, stream, reuse)
        mod = compiler.compile_with_cache(src)
        with _lock:
            mod = _memo.setdefault(key, mod)
    return mod


def _module_lanes(in_dtype, out_dtype, op, skip_nan, vec, trips, idx64, lstride, stream):
    key = ('lanes', _device.get_device_id(), in_dtype.char, out_dtype.char, op, skip_nan, vec,
           trips, idx64, lstride, stream)
    mod = _memo.get(key)
    if mod is None:
        src = _emit_lanes(_get_typename(in_dtype), _get_typename(out_dtype), op, skip_nan,
                          vec, trips, idx64, lstride, stream)
        mod = compiler.compile_with_cache(src)
        with _lock:
            mod = _memo.setdefault(key, mod)
    return mod


def _module(in_dtype, out_dtype, op, skip_nan, vec, trips, idx64, group=64,
            stream=(True, False), ragged=True, reuse=False):
    key = (_device.get_device_id(), in_dtype.char, out_dtype.char, op, skip_nan, vec,
           trips, idx64, group, stream, ragged, reuse)
    mod = _memo.get(key)
    if mod is None:
        src = _emit(_get_typename(in_dtype), _get_typename(out_dtype), op, skip_nan,
                    vec, trips, idx64, group, stream, ragged, reuse)
        mod = compiler.compile_with_cache(src)
        with _lock:
            mod = _memo.setdefault(key, mod)
    return mod


def _acc_dtype(out_dtype):
    return numpy.dtype('float32') if out_dtype == numpy.float16 else out_dtype


def _lanes_geometry(src, dst, inner, item):
    """(vec, lanes per row) for the lane-interleaved kernel, or None when a row
    of the inner extent does not fit half a wave."""
    if inner < 2:
        return None
    vec = max(1, 16 // item)
    while vec >= 1:
        if (inner % vec == 0 and _aligned(src.data.ptr, vec * src.dtype.itemsize)
                and _aligned(dst.data.ptr, vec * dst.dtype.itemsize)):
            lstride = inner // vec
            if lstride <= 32:
                return vec, lstride
            return None
        vec //= 2
    return None


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
    total = outer * n * inner
    setting = _tuning.get('scan_stream')
    if setting == 'auto':
        # Inputs stream.  Many rows (or column strips) are written at once, far
        # apart in memory: such writes gain from being collected in the
        # memory-side cache as long as the output fits it.
        stream = (True, total * out_dtype.itemsize > _tuning.get('cache_bytes'))
    else:
        stream = _tuning.stream_policy(setting, total * in_dtype.itemsize,
                                       total * out_dtype.itemsize)
    # A chunked scan reads its input twice.  While the input is not much larger
    # than the memory-side cache, the second reading starts where the first
    # ended and finds (part of) it there.
    reuse_ok = (_tuning.get('scan_chunk_reuse')
                and total * in_dtype.itemsize <= 2 * _tuning.get('cache_bytes'))
    if inner == 1:
        vec = max(1, 16 // item)
        while vec > 1 and (not _aligned(src.data.ptr, vec * in_dtype.itemsize)
                           or not _aligned(dst.data.ptr, vec * out_dtype.itemsize)
                           or (outer > 1 and n % vec) or n < vec):
            vec //= 2
        # short rows: a group of lanes smaller than a wave per row, each lane
        # with up to four vectors; long rows: whole waves
        trips = 4
        group = _WAVE
        while trips > 1 and group * vec * (trips // 2) >= n:
            trips //= 2
        while group > 1 and (group // 2) * vec * trips >= n:
            group //= 2
        per_group = group * vec * trips
        # enough waves to fill the device: cut rows into chunks if there are few
        want = cus * _tuning.get('scan_waves_per_cu')
        n_chunks = 1
        # (three launches cost about 30 us: a wave on its own is quicker for
        # up to a dozen rounds)
        if may_chunk and group == _WAVE and outer < want and n > 12 * per_group:
            n_chunks = min((want + outer - 1) // outer, (n + per_group - 1) // per_group)
        chunk_len = (n + n_chunks - 1) // n_chunks
        chunk_len = (chunk_len + per_group - 1) // per_group * per_group
        n_chunks = (n + chunk_len - 1) // chunk_len
        mod = _module(in_dtype, out_dtype, op, skip_nan, vec, trips, idx64, group, stream,
                      ragged=n % vec != 0, reuse=n_chunks > 1 and reuse_ok)
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
        middle_round = _WAVE * 4 * 4          # elements one wave takes per round
    elif 2 <= inner <= 32 and _tuning.get('scan_tile'):
        vec = max(1, 16 // item)
        trips = 4
        rows_t, _, _, _ = _tile_geometry(inner, vec, trips)
        want = cus * _tuning.get('scan_waves_per_cu')
        n_chunks = 1
        if may_chunk and outer < want and n > 2 * rows_t:
            n_chunks = min((want + outer - 1) // outer, (n + rows_t - 1) // rows_t)
        chunk_len = (n + n_chunks - 1) // n_chunks
        chunk_len = (chunk_len + rows_t - 1) // rows_t * rows_t
        n_chunks = (n + chunk_len - 1) // chunk_len
        mod = _module_tile(in_dtype, out_dtype, op, skip_nan, vec, trips, idx64, inner, stream,
                           n_chunks > 1 and reuse_ok)
        waves = outer * n_chunks
        per_block = _BLOCK // _WAVE
        grid = max(1, min((waves + per_block - 1) // per_block, cus * 32))
        fmt = '@PPP' + ic * 4

        def launch(name, totals_ptr):
            blob = struct.pack(fmt, src.data.ptr, dst.data.ptr, totals_ptr, outer, n,
                               n_chunks, chunk_len)
            mod.get_function(name).launch_packed(
                (grid, 1, 1), (_BLOCK, 1, 1), blob, 0, stream_ptr)
        prefix = 'cupy_scan_tile'
        totals_shape = (outer, n_chunks, inner)
        middle_round = rows_t
    elif _lanes_geometry(src, dst, inner, item) is not None:
        vec, lstride = _lanes_geometry(src, dst, inner, item)
        trips = 4
        trip_rows = _WAVE // lstride
        per_wave = trip_rows * trips
        want = cus * _tuning.get('scan_waves_per_cu')
        n_chunks = 1
        if may_chunk and outer < want and n > 2 * per_wave:
            n_chunks = min((want + outer - 1) // outer, (n + per_wave - 1) // per_wave)
        chunk_len = (n + n_chunks - 1) // n_chunks
        chunk_len = (chunk_len + per_wave - 1) // per_wave * per_wave
        n_chunks = (n + chunk_len - 1) // chunk_len
        mod = _module_lanes(in_dtype, out_dtype, op, skip_nan, vec, trips, idx64, lstride,
                            stream)
        waves = outer * n_chunks
        per_block = _BLOCK // _WAVE
        grid = max(1, min((waves + per_block - 1) // per_block, cus * 32))
        fmt = '@PPP' + ic * 4

        def launch(name, totals_ptr):
            blob = struct.pack(fmt, src.data.ptr, dst.data.ptr, totals_ptr, outer, n,
                               n_chunks, chunk_len)
            mod.get_function(name).launch_packed(
                (grid, 1, 1), (_BLOCK, 1, 1), blob, 0, stream_ptr)
        prefix = 'cupy_scan_lanes'
        totals_shape = (outer, n_chunks, inner)
        middle_round = per_wave
    else:
        vec = max(1, 16 // item)
        while vec > 1 and (not _aligned(src.data.ptr, vec * in_dtype.itemsize)
                           or not _aligned(dst.data.ptr, vec * out_dtype.itemsize)
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
        mod = _module(in_dtype, out_dtype, op, skip_nan, vec, trips, idx64, 64, stream,
                      reuse=n_chunks > 1 and reuse_ok)
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
        middle_round = 16                     # rows a lane takes per round
    if n_chunks == 1:
        launch(prefix, 0)
        return
    totals = ndarray._new_contiguous(totals_shape, _acc_dtype(out_dtype))
    launch(prefix + '_totals', totals.data.ptr)
    # The scan of the totals is one dependent chain per row (or column): when
    # it would take many rounds it is cut into chunks in its turn.
    _scan_contiguous(totals, totals, totals_shape[0], n_chunks, totals_shape[2], op, False,
                     stream_ptr, may_chunk=n_chunks > 8 * middle_round)
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
    if dtype.kind not in 'biufc':
        raise TypeError('scan does not support dtype %s' % dtype)
    src = a
    if not src._c_contiguous or src.dtype.kind not in 'biufc':
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
    _scan_contiguous(src, result, outer, n, inner, op, skip_nan and src.dtype.kind in 'fc',
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
