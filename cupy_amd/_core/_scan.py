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
from cupy_amd.cuda import _giveup
from cupy_amd.cuda import compiler
from cupy_amd.cuda import device as _device
from cupy_amd.cuda import stream as _stream

_SUM, _PROD = 0, 1
_BLOCK = 256
_WAVE = 64

_memo = {}
_lock = threading.Lock()


def _start_text(op, acc_t):
    """Arguments of the accumulator's constructor for the value a scan starts
    from.  For sums of floating-point values that is the NEGATIVE zero, the
    one value that leaves every other unchanged when added to it
    (0.0 + -0.0 is 0.0: a scan that starts from 0.0 turns a leading -0.0 into
    0.0, which neither NumPy nor the reference's in-place scan does;
    cupy/_core/_routines_math.pyx:160-751).  A NaN that ``nancumsum`` skips
    still counts as 0.0."""
    if op != _SUM:
        return '1'
    if acc_t.startswith('complex'):
        return '-0.0, -0.0'
    if acc_t in ('float', 'double'):
        return '-0.0'
    return '0'


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
#define SCAN_IDENTITY (_acc_t(%(start)s))
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
    // the whole vectors of the chunk end here (a row that is no whole number
    // of vectors ends up to VEC - 1 elements later: see the end of the loop)
    const _idx_t jv = RAGGED ? j0 + (j1 - j0) / VEC * VEC : j1;
    const _in_t* src = in + (ptrdiff_t)row * n;
    _acc_t carry = SCAN_IDENTITY;
    if (kMode == 2 && chunk > 0) carry = totals[(ptrdiff_t)row * n_chunks + chunk - 1];
    // the vectors of the first round; later rounds are requested one round
    // ahead, before the current one is scanned
    cupy::Vec<_in_t, VEC> raw[TRIPS];
    _rows_load<NT_LOAD_OF(kMode)>(raw, src, j0, j0, jv, lane);
    for (_idx_t base = j0; base < jv; base += GROUP * VEC * TRIPS) {
      cupy::Vec<_in_t, VEC> next[TRIPS];
      const _idx_t nbase = base + GROUP * VEC * TRIPS;
      if (nbase < jv) _rows_load<NT_LOAD_OF(kMode)>(next, src, nbase, j0, jv, lane);
      _acc_t v[TRIPS][VEC];
#pragma unroll
      for (int t = 0; t < TRIPS; ++t) {
        const _idx_t j = base + (t * GROUP + lane) * VEC;
#pragma unroll
        for (int k = 0; k < VEC; ++k)
          v[t][k] = (j < jv) ? _load_value(raw[t].v[k]) : SCAN_IDENTITY;
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
          if (j < jv) {
            cupy::Vec<_out_t, VEC> r;
#pragma unroll
            for (int k = 0; k < VEC; ++k) r.v[k] = static_cast<_out_t>(SCAN_OP(before, v[t][k]));
            if (VEC > 1) cupy::store_vec<_out_t, VEC, NT_STORE_OF(kMode)>(dst, r);
            else dst[0] = r.v[0];
          }
          carry = SCAN_OP(carry, trip_total);
        }
      }
#pragma unroll
      for (int t = 0; t < TRIPS; ++t) raw[t] = next[t];
    }
    // The elements after the last whole vector of a row: one lane goes through
    // them, from the running value, which every lane holds (in mode 1 it adds
    // them to its share of the total).  Kept out of the loop above: element by
    // element loads inside it were asked for late and by few lanes (2^26
    // float32 in rows of 4099: 110 us against 83 for rows of 4096).
    if (RAGGED && jv < j1 && lane == 0) {
      _acc_t a = carry;
      for (_idx_t i = jv; i < j1; ++i) {
        a = SCAN_OP(a, _load_value(src[i]));
        if (kMode != 1) out[(ptrdiff_t)row * n + i] = static_cast<_out_t>(a);
      }
      if (kMode == 1) carry = a;
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
  // vectors per row; where the row is no whole number of them, the last one
  // starts VEC columns before the end of the row and overlaps its neighbour
  // (both then compute and store the same values for the shared columns)
  const _idx_t inner_v = (inner + VEC - 1) / VEC;            // the host guarantees inner >= VEC
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
    const _idx_t c0 = (iv * VEC + VEC <= inner) ? iv * VEC : inner - VEC;
    const ptrdiff_t col = (ptrdiff_t)o * n * inner + c0;
    _acc_t run[VEC];
#pragma unroll
    for (int k = 0; k < VEC; ++k) run[k] = SCAN_IDENTITY;
    if (kMode == 2 && chunk > 0) {
#pragma unroll
      for (int k = 0; k < VEC; ++k)
        run[k] = totals[((ptrdiff_t)o * n_chunks + chunk - 1) * inner + c0 + k];
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
        totals[((ptrdiff_t)o * n_chunks + chunk) * inner + c0 + k] = run[k];
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
''' % dict(in_t=in_t, out_t=out_t, acc_t=acc_t, idx_t=idx_t, op_c=op_c, ident=ident, start=_start_text(op, acc_t),
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
#define SCAN_IDENTITY (_acc_t(%(start)s))
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
           op_c=op_c, ident=ident, start=_start_text(op, acc_t), vec=vec, trips=trips, conv=conv, block=_BLOCK,
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
    """Scan along the middle axis of (outer, n, inner) for 2 <= inner <= 64.

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
#define SCAN_IDENTITY (_acc_t(%(start)s))
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
           op_c=op_c, ident=ident, start=_start_text(op, acc_t), vec=vec, trips=trips, conv=conv, block=_BLOCK,
           inner=inner, rows_t=rows_t, seg=seg, lrows=lrows, stride=stride,
           ntl='true' if stream[0] else 'false', nts='true' if stream[1] else 'false',
           reuse=1 if reuse else 0)


def _emit_tile_packed(in_t, out_t, op, skip_nan, vec, trips, idx64, inner, stream):
    """Scan along the middle axis of (outer, n, inner) for 2 <= inner <= 64 and
    slices so short that many fit the rows a wave stages per round: the
    staging of ``_emit_tile``, with the (outer x n) rows taken as one long run
    cut into rounds of whole slices.  The scan starts over wherever a slice
    starts: inside a lane's own rows, and -- through a flag that travels with
    the running values -- in the combination across the lanes.  Rounds are
    independent of one another: nothing is carried from round to round."""
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
#define SCAN_IDENTITY (_acc_t(%(start)s))
#define VEC %(vec)d
#define TRIPS %(trips)d
#define NT_LOAD %(ntl)s
#define NT_STORE %(nts)s
#define INNER %(inner)d
#define ROWS_T %(rows_t)d
#define SEG %(seg)d
#define LROWS %(lrows)d
#define SEG_STRIDE %(stride)d
#define LDS_WORDS (SEG * SEG_STRIDE)
__device__ __forceinline__ _acc_t _load_value(_in_t _x) { return %(conv)s; }
// position in the LDS of element p of the round (p = row * INNER + column)
__device__ __forceinline__ int _lds_at(int p) { return p + (p / (LROWS * INNER)) * (SEG_STRIDE - LROWS * INNER); }

// total_rows = outer * n rows of INNER elements; a round is round_rows of them,
// a multiple of n not above ROWS_T (so that every round starts a slice).
extern "C" __global__ void __launch_bounds__(%(block)d) cupy_scan_tile_packed(
    const _in_t* __restrict__ in, _out_t* __restrict__ out, const _idx_t total_rows,
    const int n, const int round_rows) {
  __shared__ _acc_t _lds_all[%(block)d / 64][LDS_WORDS];
  _acc_t* lds = _lds_all[threadIdx.x / 64];
  const int lane = threadIdx.x %% 64;
  const int seg = lane / INNER;
  const int col = lane - seg * INNER;
  const bool active = lane < SEG * INNER;
  // where the lane's rows start over (the same in every round): bit i is set
  // if its row i is the first of a slice
  unsigned long long starts = 0ull;      // (LROWS <= 64)
  {
    int j = (seg * LROWS) %% n;
#pragma unroll
    for (int i = 0; i < LROWS; ++i) {
      if (j == 0) starts |= 1ull << i;
      j = (j + 1 == n) ? 0 : j + 1;
    }
  }
  const _idx_t n_rounds = (total_rows + round_rows - 1) / round_rows;
  const _idx_t wave_step = (_idx_t)gridDim.x * (%(block)d / 64);
  for (_idx_t w = (_idx_t)blockIdx.x * (%(block)d / 64) + threadIdx.x / 64; w < n_rounds;
       w += wave_step) {
    const _idx_t rb = w * round_rows;
    const int rows_here = (total_rows - rb < round_rows) ? (int)(total_rows - rb) : round_rows;
    const int valid = rows_here * INNER;
    const _in_t* src = in + (ptrdiff_t)rb * INNER;
    _out_t* dst = out + (ptrdiff_t)rb * INNER;
    // every load of the round is requested before the first value is used
    cupy::Vec<_in_t, VEC> raw[TRIPS];
#pragma unroll
    for (int t = 0; t < TRIPS; ++t) {
      const int p = (t * 64 + lane) * VEC;
      if (p + VEC <= valid) {
        raw[t] = cupy::load_vec<_in_t, VEC, NT_LOAD>(src + p);
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
      for (int i = 1; i < LROWS; ++i) v[i] = ((starts >> i) & 1ull) ? v[i] : SCAN_OP(v[i - 1], v[i]);
    } else {
#pragma unroll
      for (int i = 0; i < LROWS; ++i) v[i] = SCAN_IDENTITY;
    }
    // what runs into the next segment of the column: the lane's last value,
    // and whether a slice started inside the lane (then nothing from the
    // segments before passes through it)
    _acc_t run = v[LROWS - 1];
    bool cut = starts != 0ull;
#pragma unroll
    for (int d = 1; d < SEG; d <<= 1) {
      const _acc_t other = cupy::shfl_up<64>(run, d * INNER);
      const int other_cut = cupy::shfl_up<64>((int)cut, d * INNER);
      if (lane >= d * INNER) {
        run = cut ? run : SCAN_OP(other, run);
        cut = cut || other_cut != 0;
      }
    }
    const _acc_t before = cupy::shfl_up<64>(run, INNER);
    if (active) {
      // rows before the lane's first start continue the segments before it
      bool open = seg > 0;
#pragma unroll
      for (int i = 0; i < LROWS; ++i) {
        open = open && !((starts >> i) & 1ull);
        lds[seg * SEG_STRIDE + i * INNER + col] = open ? SCAN_OP(before, v[i]) : v[i];
      }
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
        cupy::store_vec<_out_t, VEC, NT_STORE>(dst + p, r);
      } else {
#pragma unroll
        for (int k = 0; k < VEC; ++k)
          if (p + k < valid) dst[p + k] = static_cast<_out_t>(lds[_lds_at(p + k)]);
      }
    }
    __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
    __builtin_amdgcn_wave_barrier();
  }
}
""" % dict(in_t=in_t, out_t=out_t, acc_t=acc_t, idx_t='ptrdiff_t' if idx64 else 'int',
           op_c=op_c, ident=ident, start=_start_text(op, acc_t), vec=vec, trips=trips, conv=conv, block=_BLOCK,
           inner=inner, rows_t=rows_t, seg=seg, lrows=lrows, stride=stride,
           ntl='true' if stream[0] else 'false', nts='true' if stream[1] else 'false')


def _module_tile_packed(in_dtype, out_dtype, op, skip_nan, vec, trips, idx64, inner, stream):
    key = ('tile packed', _device.get_device_id(), in_dtype.char, out_dtype.char, op, skip_nan,
           vec, trips, idx64, inner, stream)
    mod = _memo.get(key)
    if mod is None:
        src = _emit_tile_packed(_get_typename(in_dtype), _get_typename(out_dtype), op, skip_nan,
                                vec, trips, idx64, inner, stream)
        mod = compiler.compile_with_cache(src)
        with _lock:
            mod = _memo.setdefault(key, mod)
    return mod


_SLAB_TRIPS = 8


def _emit_slab(in_t, out_t, op, skip_nan, vec, idx64, stream):
    """Scan along the middle axis of (outer, n, inner) where a whole slice of
    n x inner elements fits the LDS of a workgroup, however wide and however
    aligned its rows: a workgroup takes a slab of consecutive whole slices --
    one contiguous piece of memory, read with full vectors on consecutive
    lanes --, lays it out in the LDS, a thread per column walks down the rows
    there, and the slab goes back in one contiguous store."""
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
#define VEC %(vec)d
#define TRIPS %(trips)d
#define BLOCK %(block)d
#define NT_LOAD %(ntl)s
#define NT_STORE %(nts)s
#define SLAB_ELEMS (BLOCK * VEC * TRIPS)
__device__ __forceinline__ _acc_t _load_value(_in_t _x) { return %(conv)s; }

// total = outer * n * inner elements; a slab is slab_elems of them, a whole
// number of slices and SLAB_ELEMS at most.
extern "C" __global__ void __launch_bounds__(BLOCK) cupy_scan_slab(
    const _in_t* __restrict__ in, _out_t* __restrict__ out, const _idx_t total,
    const int n, const int inner, const int slab_elems) {
  __shared__ _acc_t lds[SLAB_ELEMS];
  const int slice_elems = n * inner;
  const _idx_t n_slabs = (total + slab_elems - 1) / slab_elems;
  for (_idx_t slab = blockIdx.x; slab < n_slabs; slab += gridDim.x) {
    const _idx_t base = slab * slab_elems;
    const int valid = (total - base < slab_elems) ? (int)(total - base) : slab_elems;
    const _in_t* src = in + (ptrdiff_t)base;
    _out_t* dst = out + (ptrdiff_t)base;
    // every load of the slab is requested before the first value is used
    cupy::Vec<_in_t, VEC> raw[TRIPS];
#pragma unroll
    for (int t = 0; t < TRIPS; ++t) {
      const int p = (t * BLOCK + (int)threadIdx.x) * VEC;
      if (p + VEC <= valid) {
        raw[t] = cupy::load_vec<_in_t, VEC, NT_LOAD>(src + p);
      } else {
#pragma unroll
        for (int k = 0; k < VEC; ++k) raw[t].v[k] = (p + k < valid) ? src[p + k] : _in_t();
      }
    }
#pragma unroll
    for (int t = 0; t < TRIPS; ++t) {
      const int p = (t * BLOCK + (int)threadIdx.x) * VEC;
      if (p < valid) {
#pragma unroll
        for (int k = 0; k < VEC; ++k) lds[p + k] = _load_value(raw[t].v[k]);
      }
    }
    __syncthreads();
    // a thread per column of a slice
    const int columns = (valid / slice_elems) * inner;
    for (int q = threadIdx.x; q < columns; q += BLOCK) {
      const int s = q / inner;
      _acc_t* at = lds + s * slice_elems + (q - s * inner);
      _acc_t acc = at[0];
      int r = 1;
      // (eight rows requested before the first is used: the compiler keeps
      // every read behind the write before it, which would cost the latency
      // of the LDS per row)
      for (; r + 8 <= n; r += 8) {
        _acc_t x[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) x[u] = at[(r + u) * inner];
#pragma unroll
        for (int u = 0; u < 8; ++u) { acc = SCAN_OP(acc, x[u]); x[u] = acc; }
#pragma unroll
        for (int u = 0; u < 8; ++u) at[(r + u) * inner] = x[u];
      }
      for (; r < n; ++r) {
        acc = SCAN_OP(acc, at[r * inner]);
        at[r * inner] = acc;
      }
    }
    __syncthreads();
#pragma unroll
    for (int t = 0; t < TRIPS; ++t) {
      const int p = (t * BLOCK + (int)threadIdx.x) * VEC;
      if (p + VEC <= valid) {
        cupy::Vec<_out_t, VEC> r;
#pragma unroll
        for (int k = 0; k < VEC; ++k) r.v[k] = static_cast<_out_t>(lds[p + k]);
        cupy::store_vec<_out_t, VEC, NT_STORE>(dst + p, r);
      } else {
#pragma unroll
        for (int k = 0; k < VEC; ++k)
          if (p + k < valid) dst[p + k] = static_cast<_out_t>(lds[p + k]);
      }
    }
    // (the next slab overwrites what the stores above read)
    __syncthreads();
  }
}
""" % dict(in_t=in_t, out_t=out_t, acc_t=acc_t, idx_t='ptrdiff_t' if idx64 else 'int',
           op_c=op_c, ident=ident, start=_start_text(op, acc_t), vec=vec, trips=_SLAB_TRIPS, conv=conv, block=_BLOCK,
           ntl='true' if stream[0] else 'false', nts='true' if stream[1] else 'false')


def _module_slab(in_dtype, out_dtype, op, skip_nan, vec, idx64, stream):
    key = ('slab', _device.get_device_id(), in_dtype.char, out_dtype.char, op, skip_nan,
           vec, idx64, stream)
    mod = _memo.get(key)
    if mod is None:
        src = _emit_slab(_get_typename(in_dtype), _get_typename(out_dtype), op, skip_nan,
                         vec, idx64, stream)
        mod = compiler.compile_with_cache(src)
        with _lock:
            mod = _memo.setdefault(key, mod)
    return mod


def _slab_pays(src, dst, n, inner, item):
    """Whether slices that fit the LDS of a workgroup go through
    ``_emit_slab``, which runs at 65-70 % of peak whatever the shape, rather
    than through the kernels for narrow, medium and wide rows.  Measured on
    2^26 floats (us, slab against the others): rows that are no whole vectors
    -- 2 x 65 103 / 165, 64 x 65 109 / 178, 16 x 257 111 / 168, 33 x 33
    101 / 131, 33 x 17 102 / 130 -- and rows that leave lanes of the
    lane-interleaved kernel idle -- 2 x 100 98 / 138, 33 x 100 99 / 126 -- gain;
    rows of whole vectors that fill the lanes do not: 2 x 128 97 / 89, 2 x 4096
    97 / 88, 7 x 64 96 / 90, but 7 x 1000 98 / 107."""
    setting = _tuning.get('scan_slab_min_inner')
    if setting is not None:
        return inner > setting
    vec = max(1, 16 // item)
    # (a thread walks down a column: long columns want a wave's worth of them
    # to a slab; 400 x 3: 180 us against 98, 126 x 65: 113 against 205)
    if n > 64 and (_BLOCK * min(vec, 4) * _SLAB_TRIPS) // (n * inner) * inner < _WAVE:
        return False
    whole = (inner % vec == 0 and _aligned(src.data.ptr, 16) and _aligned(dst.data.ptr, 16))
    if inner > 64:
        if not whole:
            return True
        lstride = inner // vec
        if lstride <= 32:
            return 64 % lstride != 0
        return n >= 5
    if whole:
        return False
    # narrow rows: where the staged kernels leave much of a round empty
    rows_t = _tile_geometry(inner, vec, 4)[0]
    if 2 * n <= rows_t:
        used = rows_t // n * n          # whole slices to a round
        rounds = 1
    else:
        used = n
        rounds = (n + rows_t - 1) // rows_t
    return used < 0.7 * rounds * rows_t


def _scan_slab(src, dst, outer, n, inner, op, skip_nan, idx64, stream, stream_ptr, cus):
    """Launches ``_emit_slab`` where a slice fits the LDS; returns False
    otherwise."""
    if not _tuning.get('scan_slab'):
        return False
    item = max(src.dtype.itemsize, dst.dtype.itemsize, _acc_dtype(dst.dtype).itemsize)
    vec = max(1, min(4, 16 // item))
    capacity = _BLOCK * vec * _SLAB_TRIPS
    slice_elems = n * inner
    if slice_elems > capacity:
        return False
    # whole slices to a slab, and slabs enough for every CU
    per_slab = max(1, min(capacity // slice_elems, outer // (cus * 8)))
    slab_elems = per_slab * slice_elems
    n_slabs = (outer + per_slab - 1) // per_slab
    mod = _module_slab(src.dtype, dst.dtype, op, skip_nan, vec, idx64, stream)
    grid = max(1, min(n_slabs, cus * _tuning.get('scan_blocks_per_cu')))
    blob = struct.pack('@PP' + ('q' if idx64 else 'i') + 'iii', src.data.ptr, dst.data.ptr,
                       outer * n * inner, n, inner, slab_elems)
    mod.get_function('cupy_scan_slab').launch_packed(
        (grid, 1, 1), (_BLOCK, 1, 1), blob, 0, stream_ptr)
    return True



_SLAB_LONG_COLUMNS = 2       # columns a thread may own in the kernel below


def _emit_slab_long(in_t, out_t, op, skip_nan, vec, idx64, stream):
    """``_emit_slab`` for slices that do not fit the LDS: a workgroup takes a
    slice, ``round_rows`` rows at a time -- again one contiguous piece of
    memory per round --, and every thread carries the running values of its
    columns (two at most) from round to round."""
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
#define SCAN_IDENTITY (_acc_t(%(start)s))
#define VEC %(vec)d
#define TRIPS %(trips)d
#define BLOCK %(block)d
#define COLUMNS %(columns)d
#define NT_LOAD %(ntl)s
#define NT_STORE %(nts)s
#define SLAB_ELEMS (BLOCK * VEC * TRIPS)
__device__ __forceinline__ _acc_t _load_value(_in_t _x) { return %(conv)s; }

// inner <= COLUMNS * BLOCK; round_rows * inner <= SLAB_ELEMS
extern "C" __global__ void __launch_bounds__(BLOCK) cupy_scan_slab_long(
    const _in_t* __restrict__ in, _out_t* __restrict__ out, const _idx_t outer,
    const int n, const int inner, const int round_rows) {
  __shared__ _acc_t lds[SLAB_ELEMS];
  for (_idx_t slice = blockIdx.x; slice < outer; slice += gridDim.x) {
    _acc_t carry[COLUMNS];
#pragma unroll
    for (int j = 0; j < COLUMNS; ++j) carry[j] = SCAN_IDENTITY;
    for (int r0 = 0; r0 < n; r0 += round_rows) {
      const int rows = (n - r0 < round_rows) ? n - r0 : round_rows;
      const int valid = rows * inner;
      const ptrdiff_t base = ((ptrdiff_t)slice * n + r0) * inner;
      const _in_t* src = in + base;
      _out_t* dst = out + base;
      cupy::Vec<_in_t, VEC> raw[TRIPS];
#pragma unroll
      for (int t = 0; t < TRIPS; ++t) {
        const int p = (t * BLOCK + (int)threadIdx.x) * VEC;
        if (p + VEC <= valid) {
          raw[t] = cupy::load_vec<_in_t, VEC, NT_LOAD>(src + p);
        } else {
#pragma unroll
          for (int k = 0; k < VEC; ++k) raw[t].v[k] = (p + k < valid) ? src[p + k] : _in_t();
        }
      }
#pragma unroll
      for (int t = 0; t < TRIPS; ++t) {
        const int p = (t * BLOCK + (int)threadIdx.x) * VEC;
        if (p < valid) {
#pragma unroll
          for (int k = 0; k < VEC; ++k) lds[p + k] = _load_value(raw[t].v[k]);
        }
      }
      __syncthreads();
#pragma unroll
      for (int j = 0; j < COLUMNS; ++j) {
        const int c = j * BLOCK + (int)threadIdx.x;
        if (c < inner) {
          // (the first row of a slice as it is: adding it to a zero would
          // lose the sign of a negative zero)
          _acc_t acc = (r0 == 0) ? lds[c] : carry[j];
          int r = (r0 == 0) ? 1 : 0;
          // (eight rows requested before the first is used: the compiler
          // keeps every read behind the write before it, which would cost
          // the latency of the LDS per row)
          for (; r + 8 <= rows; r += 8) {
            _acc_t x[8];
#pragma unroll
            for (int u = 0; u < 8; ++u) x[u] = lds[(r + u) * inner + c];
#pragma unroll
            for (int u = 0; u < 8; ++u) { acc = SCAN_OP(acc, x[u]); x[u] = acc; }
#pragma unroll
            for (int u = 0; u < 8; ++u) lds[(r + u) * inner + c] = x[u];
          }
          for (; r < rows; ++r) {
            acc = SCAN_OP(acc, lds[r * inner + c]);
            lds[r * inner + c] = acc;
          }
          carry[j] = acc;
        }
      }
      __syncthreads();
#pragma unroll
      for (int t = 0; t < TRIPS; ++t) {
        const int p = (t * BLOCK + (int)threadIdx.x) * VEC;
        if (p + VEC <= valid) {
          cupy::Vec<_out_t, VEC> r;
#pragma unroll
          for (int k = 0; k < VEC; ++k) r.v[k] = static_cast<_out_t>(lds[p + k]);
          cupy::store_vec<_out_t, VEC, NT_STORE>(dst + p, r);
        } else {
#pragma unroll
          for (int k = 0; k < VEC; ++k)
            if (p + k < valid) dst[p + k] = static_cast<_out_t>(lds[p + k]);
        }
      }
      // (the next round overwrites what the stores above read)
      __syncthreads();
    }
  }
}
""" % dict(in_t=in_t, out_t=out_t, acc_t=acc_t, idx_t='ptrdiff_t' if idx64 else 'int',
           op_c=op_c, ident=ident, start=_start_text(op, acc_t), vec=vec, trips=_SLAB_TRIPS, conv=conv, block=_BLOCK,
           columns=_SLAB_LONG_COLUMNS,
           ntl='true' if stream[0] else 'false', nts='true' if stream[1] else 'false')


def _module_slab_long(in_dtype, out_dtype, op, skip_nan, vec, idx64, stream):
    key = ('slab long', _device.get_device_id(), in_dtype.char, out_dtype.char, op, skip_nan,
           vec, idx64, stream)
    mod = _memo.get(key)
    if mod is None:
        src = _emit_slab_long(_get_typename(in_dtype), _get_typename(out_dtype), op, skip_nan,
                              vec, idx64, stream)
        mod = compiler.compile_with_cache(src)
        with _lock:
            mod = _memo.setdefault(key, mod)
    return mod


def _scan_slab_long(src, dst, outer, n, inner, op, skip_nan, idx64, stream, stream_ptr, cus):
    """Launches ``_emit_slab_long`` for many slices of rows that are no whole
    vectors, or that leave lanes of the lane-interleaved kernel idle; returns
    False where it does not apply."""
    if not _tuning.get('scan_slab_long'):
        return False
    item = max(src.dtype.itemsize, dst.dtype.itemsize, _acc_dtype(dst.dtype).itemsize)
    vec = max(1, min(4, 16 // item))
    capacity = _BLOCK * vec * _SLAB_TRIPS
    round_rows = capacity // inner
    if (inner <= 64 or inner > _SLAB_LONG_COLUMNS * _BLOCK or round_rows < 8
            or outer < cus * _tuning.get('scan_slab_long_slices_per_cu')):
        return False
    full = max(1, 16 // max(src.dtype.itemsize, dst.dtype.itemsize))
    whole = (inner % full == 0 and _aligned(src.data.ptr, 16) and _aligned(dst.data.ptr, 16))
    if whole and (inner // full > 32 or 64 % (inner // full) == 0):
        return False
    mod = _module_slab_long(src.dtype, dst.dtype, op, skip_nan, vec, idx64, stream)
    grid = max(1, min(outer, cus * _tuning.get('scan_blocks_per_cu')))
    blob = struct.pack('@PP' + ('q' if idx64 else 'i') + 'iii', src.data.ptr, dst.data.ptr,
                       outer, n, inner, round_rows)
    mod.get_function('cupy_scan_slab_long').launch_packed(
        (grid, 1, 1), (_BLOCK, 1, 1), blob, 0, stream_ptr)
    return True



_CHAIN_WAVES = _BLOCK // _WAVE
_CHAIN_HEADER_WORDS = 64            # the ticket counter, padded to 256 bytes


def _emit_chain(in_t, out_t, op, skip_nan, vec, trips, idx64, stream, ragged, parts=2, waves=_CHAIN_WAVES,
                bands=False):
    """One-pass scan of long rows: a workgroup per tile of 256 x VEC x TRIPS
    elements scans its tile in registers, publishes the tile's total and adds
    up the totals published by the tiles before it: the input is read once and
    the result written once.

    A tile waits only for tiles with smaller numbers (``blockIdx.x``), and
    workgroups start in the order of their numbers on every compute die, so
    the unfinished tile with the smallest number is always running and waits
    for nobody.  Every wait is bounded by ``spin_limit`` polls all the same:
    a tile that runs out of patience flags the failure in ``fault`` and still
    runs to its end, so the grid always drains.

    The totals before a tile are combined in an order that depends only on the
    tile's number: tiles form groups of ``group_tiles``; the last tile of a
    group publishes the group's total; a tile adds the totals of the groups
    before its own and the totals of the tiles before it in its group, each
    set folded lane by lane and then across the lanes.  Results therefore do
    not vary from run to run (a look-back that stops at whatever prefix happens
    to be published would make floating-point results depend on timing)."""
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
#define SCAN_IDENTITY (_acc_t(%(start)s))
#define VEC %(vec)d
#define TRIPS %(trips)d
#define NT_LOAD %(ntl)s
#define NT_STORE %(nts)s
#define RAGGED %(ragged)d
#define BANDS %(bands)d
#define WAVE 64
#define WAVES %(waves)d
#define PARTS %(parts)d
#define SPIN_SLEEP %(sleep)d      // pause between two polls, in units of 64 clocks
#define PART_ELEMS (WAVE * VEC * TRIPS)
#define WAVE_ELEMS (PARTS * PART_ELEMS)
#define TILE (WAVES * WAVE_ELEMS)
#define HEADER_WORDS %(header)d
__device__ __forceinline__ _acc_t _load_value(_in_t _x) { return %(conv)s; }

// A published value travels as 32-bit words, each in the low half of a 64-bit
// slot whose high half holds the number of this launch (`epoch`, never zero):
// one atomic store publishes a word together with its mark and one atomic load
// fetches both, so that no fence (and no write-back of a die's cache) is
// needed on either side, and nothing has to be cleared between launches: what
// an earlier launch left in a slot carries an older number.  The accesses have
// device scope: they pass the caches of the compute dies.
constexpr int kWords = (sizeof(_acc_t) + 3) / 4;
typedef unsigned long long _slot_t;

__device__ __forceinline__ void _publish(_slot_t* slots, const ptrdiff_t i, const _acc_t& v,
                                         const unsigned epoch) {
  unsigned w[kWords];
#pragma unroll
  for (int k = 0; k < kWords; ++k) w[k] = 0u;
  __builtin_memcpy(w, &v, sizeof(_acc_t));
#pragma unroll
  for (int k = 0; k < kWords; ++k)
    __hip_atomic_store(slots + i * kWords + k, ((_slot_t)epoch << 32) | w[k], __ATOMIC_RELAXED,
                       __HIP_MEMORY_SCOPE_AGENT);
}

// `count` published values from `first`, waited for and combined in an order
// that depends on `count` alone: every lane takes the values lane, lane + 64,
// ... as they appear, then the lanes are combined (every lane ends with the
// same value).  One wave, all lanes call.  `ok` turns false if the wave gave
// up after `spin_limit` rounds of polling (the value is then meaningless).
__device__ __forceinline__ _acc_t _await_fold(_slot_t* slots, const ptrdiff_t first,
                                              const int count, const int lane,
                                              const unsigned epoch, const unsigned spin_limit,
                                              bool& ok) {
  _acc_t s = SCAN_IDENTITY;
  int i = lane;
  unsigned spins = 0;
  // Tiles publish roughly in the order of their numbers: wait for the newest
  // value alone first (one address for the whole wave, so that thousands of
  // waiting workgroups do not hammer the few memory channels that hold the
  // slots), then collect all of them.
  for (;;) {
    const _slot_t x = __hip_atomic_load(slots + (first + count) * kWords - 1, __ATOMIC_RELAXED,
                                        __HIP_MEMORY_SCOPE_AGENT);
    if ((unsigned)(x >> 32) == epoch) break;
    if (spins >= spin_limit) { ok = false; break; }
    ++spins;
    __builtin_amdgcn_s_sleep(SPIN_SLEEP);
  }
  for (;;) {
    while (i < count) {
      _slot_t x[kWords];
#pragma unroll
      for (int k = 0; k < kWords; ++k)
        x[k] = __hip_atomic_load(slots + (first + i) * kWords + k, __ATOMIC_RELAXED,
                                 __HIP_MEMORY_SCOPE_AGENT);
      bool written = true;
      unsigned w[kWords];
#pragma unroll
      for (int k = 0; k < kWords; ++k) {
        written = written && (unsigned)(x[k] >> 32) == epoch;
        w[k] = (unsigned)x[k];
      }
      if (!written) break;
      _acc_t v;
      __builtin_memcpy(&v, w, sizeof(_acc_t));
      s = SCAN_OP(s, v);
      i += WAVE;
    }
    if (__ballot(i < count) == 0) break;
    if (spins >= spin_limit) { ok = false; break; }
    ++spins;
    __builtin_amdgcn_s_sleep(SPIN_SLEEP);
  }
#pragma unroll
  for (int m = WAVE / 2; m > 0; m >>= 1) s = SCAN_OP(s, cupy::shfl_xor(s, m));
  return s;
}

extern "C" __global__ void cupy_scan_chain_clear(unsigned* desc, const unsigned words) {
  for (unsigned i = blockIdx.x * blockDim.x + threadIdx.x; i < words; i += gridDim.x * blockDim.x)
    desc[i] = 0u;
}

// The TRIPS vectors of a lane for the part of tile `t_row` of a row that wave
// `wv` scans, all requested at once (a vector that would start past the end of
// the row is read from the row's start instead; its values are not used).
__device__ __forceinline__ void _tile_load(
    cupy::Vec<_in_t, VEC> (&raw)[TRIPS], const _in_t* __restrict__ src, const _idx_t j0,
    const _idx_t j1, const int lane) {
#pragma unroll
  for (int t = 0; t < TRIPS; ++t) {
    const _idx_t j = j0 + (t * WAVE + lane) * VEC;
    const _idx_t jc = (j + VEC <= j1) ? j : 0;
    if (VEC > 1) raw[t] = cupy::load_vec<_in_t, VEC, NT_LOAD>(src + jc);
    else raw[t].v[0] = src[(j < j1) ? j : 0];
  }
}

// One part of a wave's share of the tile (TRIPS vectors per lane, from `j0`):
// the values of every lane scanned in place (`v`), what precedes each of the
// lane's vectors inside the part (`pre`), and -- returned -- the part's total.
__device__ __forceinline__ _acc_t _part_scan(
    const cupy::Vec<_in_t, VEC> (&raw)[TRIPS], const _in_t* __restrict__ src, const _idx_t j0,
    const _idx_t j1, const int lane, _acc_t (&v)[TRIPS][VEC], _acc_t (&pre)[TRIPS]) {
#pragma unroll
  for (int t = 0; t < TRIPS; ++t) {
    const _idx_t j = j0 + (t * WAVE + lane) * VEC;
#pragma unroll
    for (int k = 0; k < VEC; ++k)
      v[t][k] = (j < j1) ? _load_value(raw[t].v[k]) : SCAN_IDENTITY;
#pragma unroll
    for (int k = 1; k < VEC; ++k) v[t][k] = SCAN_OP(v[t][k - 1], v[t][k]);
  }
  // inclusive scans of the lane totals across the wave, the trips side by side
  _acc_t incl[TRIPS];
#pragma unroll
  for (int t = 0; t < TRIPS; ++t) incl[t] = v[t][VEC - 1];
#pragma unroll
  for (int d = 1; d < WAVE; d <<= 1) {
#pragma unroll
    for (int t = 0; t < TRIPS; ++t) {
      const _acc_t o = cupy::shfl_up<WAVE>(incl[t], d);
      incl[t] = (lane >= d) ? SCAN_OP(o, incl[t]) : incl[t];
    }
  }
  _acc_t carry = SCAN_IDENTITY;
#pragma unroll
  for (int t = 0; t < TRIPS; ++t) {
    const _acc_t trip_total = cupy::shfl_idx<WAVE>(incl[t], WAVE - 1);
    const _acc_t before = cupy::shfl_up<WAVE>(incl[t], 1);
    pre[t] = (lane == 0) ? carry : SCAN_OP(carry, before);
    carry = (t == 0) ? trip_total : SCAN_OP(carry, trip_total);
  }
  return carry;
}

// The results of one part: `base` (if `has_base`) before everything.
__device__ __forceinline__ void _part_store(
    _out_t* __restrict__ row_out, const _idx_t j0, const _idx_t j1, const int lane,
    const _acc_t (&v)[TRIPS][VEC], const _acc_t (&pre)[TRIPS], const _acc_t base,
    const bool has_base) {
#pragma unroll
  for (int t = 0; t < TRIPS; ++t) {
    const _idx_t j = j0 + (t * WAVE + lane) * VEC;
    const bool has_pre = (t > 0) || (lane > 0);
    const _acc_t before = has_base ? (has_pre ? SCAN_OP(base, pre[t]) : base) : pre[t];
    const bool any = has_base || has_pre;
    _out_t* dst = row_out + j;
    if (j < j1) {
      cupy::Vec<_out_t, VEC> r;
#pragma unroll
      for (int k = 0; k < VEC; ++k)
        r.v[k] = static_cast<_out_t>(any ? SCAN_OP(before, v[t][k]) : v[t][k]);
      if (VEC > 1) cupy::store_vec<_out_t, VEC, NT_STORE>(dst, r);
      else dst[0] = r.v[0];
    }
  }
}

// desc: [HEADER_WORDS unused 32-bit words][slots of the tile totals][slots of
//       the group totals]; zero before its first use, then only ever written
//       by launches of this kernel, each with a number of its own.
// One workgroup per tile, tiles numbered by blockIdx.x: a tile waits only for
// tiles with smaller numbers.  Workgroups are handed to each compute die in the
// order of their numbers, so the unfinished tile with the smallest number is
// always running and owes nothing to anyone: every wait ends.  (Should that
// order ever not hold, the waits are bounded: see `spin_limit`.)
//
// A wave's share of the tile comes in PARTS parts of TRIPS vectors per lane,
// all requested at the start.  While the workgroup waits for its neighbours it
// has nothing in flight, so what it holds in registers meanwhile is what
// keeps the memory system busy: the first part is held scanned, the others as
// loaded (they are scanned twice: once for their total, once for the result).
extern "C" __global__ void __launch_bounds__(%(block)d) %(occupancy)s cupy_scan_chain(
    const _in_t* __restrict__ in, _out_t* __restrict__ out, unsigned* desc,
    const _idx_t n_rows, const _idx_t n, const _idx_t tiles_per_row, const _idx_t group_tiles,
    const _idx_t groups_per_row, const unsigned epoch, const unsigned spin_limit,
    unsigned* fault) {
  __shared__ __attribute__((aligned(16))) char sm_raw[(WAVES + 2) * sizeof(_acc_t)];
  _acc_t* sm_wave = reinterpret_cast<_acc_t*>(sm_raw);
  const ptrdiff_t n_tiles = (ptrdiff_t)n_rows * tiles_per_row;
  _slot_t* tile_totals = reinterpret_cast<_slot_t*>(desc + HEADER_WORDS);
  _slot_t* group_totals = tile_totals + n_tiles * kWords;
  const int lane = threadIdx.x %% WAVE;
  const int wv = threadIdx.x / WAVE;
  const _idx_t jn = n;
  const _idx_t j1 = RAGGED ? n - n %% VEC : n;           // the whole vectors of a row end here
#if BANDS
  // Workgroups are handed to the eight compute dies in turn (workgroup w goes
  // to die w %% 8, each die with a cache of its own), and neighbouring tiles of
  // a row share the cache lines at their borders when the rows do not start on
  // line boundaries.  Workgroup w takes tile number w / 8 of the rows r with
  // r %% 8 == w %% 8, counted row by row: a die works its way along whole rows,
  // and a tile still only waits for workgroups with smaller numbers (the
  // tiles before it in its row).
  const _idx_t band = (_idx_t)(blockIdx.x & 7u);
  const ptrdiff_t seq = (ptrdiff_t)(blockIdx.x >> 3);
  const _idx_t row = (_idx_t)(seq / tiles_per_row) * 8 + band;
  if (row >= n_rows) return;
  const _idx_t t_row = (_idx_t)(seq %% tiles_per_row);
  const ptrdiff_t tile = (ptrdiff_t)row * tiles_per_row + t_row;
#else
  const ptrdiff_t tile = blockIdx.x;
  if (tile >= n_tiles) return;
  const _idx_t row = (_idx_t)(tile / tiles_per_row);
  const _idx_t t_row = (_idx_t)(tile - (ptrdiff_t)row * tiles_per_row);
#endif
  const _in_t* src = in + (ptrdiff_t)row * n;
  _out_t* row_out = out + (ptrdiff_t)row * n;
  const _idx_t j0 = t_row * TILE + wv * WAVE_ELEMS;        // this wave's share of the tile
  cupy::Vec<_in_t, VEC> raw[PARTS][TRIPS];
#pragma unroll
  for (int p = 0; p < PARTS; ++p) _tile_load(raw[p], src, j0 + p * PART_ELEMS, j1, lane);
  _acc_t v[TRIPS][VEC];
  _acc_t pre[TRIPS];
  _acc_t part_total[PARTS];
  part_total[0] = _part_scan(raw[0], src, j0, j1, lane, v, pre);
  _acc_t carry = part_total[0];
#pragma unroll
  for (int p = 1; p < PARTS; ++p) {
    _acc_t v2[TRIPS][VEC];
    _acc_t pre2[TRIPS];
    part_total[p] = _part_scan(raw[p], src, j0 + p * PART_ELEMS, j1, lane, v2, pre2);
    carry = SCAN_OP(carry, part_total[p]);
  }
  if (lane == 0) sm_wave[wv] = carry;
  __syncthreads();
  _acc_t wave_before = SCAN_IDENTITY;
  _acc_t tile_total = sm_wave[0];
#pragma unroll
  for (int w = 1; w < WAVES; ++w) {
    if (w == wv) wave_before = tile_total;
    tile_total = SCAN_OP(tile_total, sm_wave[w]);
  }
  // ---- what precedes the tile in its row: the first wave collects the totals
  // of the tiles before it in its group, the second those of the groups before
  // its own
  const _idx_t g = t_row / group_tiles;
  const int t_group = (int)(t_row - g * group_tiles);
  const bool closes_group = (t_group == group_tiles - 1) || (t_row == tiles_per_row - 1);
  const ptrdiff_t row_groups = (ptrdiff_t)row * groups_per_row;
  if (wv == 0) {
    if (lane == 0) _publish(tile_totals, tile, tile_total, epoch);
    bool ok = true;
    _acc_t in_group = SCAN_IDENTITY;
    if (t_group > 0)
      in_group = _await_fold(tile_totals, tile - t_group, t_group, lane, epoch, spin_limit, ok);
    if (lane == 0) {
      if (closes_group)
        _publish(group_totals, row_groups + g,
                 (t_group > 0) ? SCAN_OP(in_group, tile_total) : tile_total, epoch);
      sm_wave[WAVES] = in_group;
      if (!ok && fault) *reinterpret_cast<volatile unsigned*>(fault) = 1u;
    }
  } else if (wv == 1 && g > 0) {
    bool ok = true;
    const _acc_t groups_before =
        _await_fold(group_totals, row_groups, (int)g, lane, epoch, spin_limit, ok);
    if (lane == 0) {
      sm_wave[WAVES + 1] = groups_before;
      if (!ok && fault) *reinterpret_cast<volatile unsigned*>(fault) = 1u;
    }
  }
  __syncthreads();
  const bool seeded = t_row > 0;
  _acc_t base = (g > 0) ? ((t_group > 0) ? SCAN_OP(sm_wave[WAVES + 1], sm_wave[WAVES])
                                         : sm_wave[WAVES + 1])
                        : sm_wave[WAVES];
  if (wv > 0) base = seeded ? SCAN_OP(base, wave_before) : wave_before;
  bool has_base = seeded || wv > 0;
  // ---- results
  _part_store(row_out, j0, j1, lane, v, pre, base, has_base);
#pragma unroll
  for (int p = 1; p < PARTS; ++p) {
    base = has_base ? SCAN_OP(base, part_total[p - 1]) : part_total[p - 1];
    has_base = true;
    (void)_part_scan(raw[p], src, j0 + p * PART_ELEMS, j1, lane, v, pre);
    _part_store(row_out, j0 + p * PART_ELEMS, j1, lane, v, pre, base, has_base);
  }
  // A row whose length is no whole number of vectors ends up to VEC - 1
  // elements after its last whole vector: the lane that has just stored that
  // vector goes on through them, one element after the other, from the result
  // it stored last.  (No tile's total needs them: nothing of the row follows.
  // Nothing is carried through the loops above for this: a register more
  // than 128 per lane would halve the workgroups a CU holds.)
  if (RAGGED) {
    const _idx_t rel = j1 - VEC - j0;                 // the last whole vector, within this wave's share
    if (rel >= 0 && rel < WAVE_ELEMS && (int)((rel / VEC) %% WAVE) == lane) {
      _acc_t a = static_cast<_acc_t>(row_out[j1 - 1]);
      for (_idx_t i = j1; i < jn; ++i) {
        a = SCAN_OP(a, _load_value(src[i]));
        row_out[i] = static_cast<_out_t>(a);
      }
    }
  }
}
''' % dict(in_t=in_t, out_t=out_t, acc_t=acc_t, idx_t=idx_t, op_c=op_c, ident=ident, start=_start_text(op, acc_t),
           vec=vec, trips=trips, conv=conv, block=waves * _WAVE, waves=waves,
           header=_CHAIN_HEADER_WORDS, parts=parts, sleep=_tuning.get('scan_chain_sleep'),
           occupancy='', bands=1 if bands else 0,
           ntl='true' if stream[0] else 'false', nts='true' if stream[1] else 'false',
           ragged=1 if ragged else 0)


def _module_chain(in_dtype, out_dtype, op, skip_nan, vec, trips, idx64, stream, ragged, parts,
                  waves=_CHAIN_WAVES, bands=False):
    key = ('chain', _device.get_device_id(), in_dtype.char, out_dtype.char, op, skip_nan, vec,
           trips, idx64, stream, ragged, parts, waves, _tuning.get('scan_chain_sleep'), bands)
    mod = _memo.get(key)
    if mod is None:
        src = _emit_chain(_get_typename(in_dtype), _get_typename(out_dtype), op, skip_nan,
                          vec, trips, idx64, stream, ragged, parts, waves, bands)
        mod = compiler.compile_with_cache(src)
        with _lock:
            mod = _memo.setdefault(key, mod)
    return mod


def _emit_chain_tile(in_t, out_t, op, skip_nan, vec, trips, idx64, inner, stream, parts, sleep):
    """One-pass scan along the middle axis of (outer, n, inner) for
    2 <= inner <= 32 and few, long (outer) slices: the staging of
    ``_emit_tile`` (a wave lays a run of whole rows out in the LDS and scans its
    columns) inside the tile protocol of ``_emit_chain`` (a workgroup per tile
    publishes the tile's totals -- one per column -- and folds those published
    before it, in an order fixed by the tile's number).  A wave holds PARTS
    rounds of rows as loaded; they go through the LDS twice, once for the
    totals and once, after the totals before the tile are known, for the
    results."""
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
#define SCAN_IDENTITY (_acc_t(%(start)s))
#define VEC %(vec)d
#define TRIPS %(trips)d
#define NT_LOAD %(ntl)s
#define NT_STORE %(nts)s
#define INNER %(inner)d
#define ROWS_T %(rows_t)d
#define SEG %(seg)d
#define LROWS %(lrows)d
#define SEG_STRIDE %(stride)d
#define LDS_WORDS (SEG * SEG_STRIDE)
#define WAVES %(waves)d
#define PARTS %(parts)d
#define WAVE_ROWS (PARTS * ROWS_T)
#define TILE_ROWS (WAVES * WAVE_ROWS)
#define HEADER_WORDS %(header)d
#define SPIN_SLEEP %(sleep)d
// tiles whose totals one round of a wave's polling covers, one per group of INNER lanes
#define FOLD_TILES (64 / INNER)
__device__ __forceinline__ _acc_t _load_value(_in_t _x) { return %(conv)s; }
// position in the LDS of element p of the round (p = row * INNER + column)
__device__ __forceinline__ int _lds_at(int p) { return p + (p / (LROWS * INNER)) * (SEG_STRIDE - LROWS * INNER); }

// Published values: see the one-pass kernel for contiguous rows.  Value
// `i * INNER + column` belongs to column `column` of tile (or group) `i`.
constexpr int kWords = (sizeof(_acc_t) + 3) / 4;
typedef unsigned long long _slot_t;

__device__ __forceinline__ void _publish(_slot_t* slots, const ptrdiff_t i, const _acc_t& v,
                                         const unsigned epoch) {
  unsigned w[kWords];
#pragma unroll
  for (int k = 0; k < kWords; ++k) w[k] = 0u;
  __builtin_memcpy(w, &v, sizeof(_acc_t));
#pragma unroll
  for (int k = 0; k < kWords; ++k)
    __hip_atomic_store(slots + i * kWords + k, ((_slot_t)epoch << 32) | w[k], __ATOMIC_RELAXED,
                       __HIP_MEMORY_SCOPE_AGENT);
}

// Totals of `count` tiles (or groups) from `first`, per column: lane (s, c)
// takes column c of the tiles s, s + FOLD_TILES, ...; the partial results of a
// column are then combined across the lane groups in order.  Every lane ends
// with the value of its column (lanes past the last whole group: undefined).
// A lane asks for FOLD_AHEAD of its values at a time (with wide rows a wave
// covers few tiles per round, and every round is a trip to memory).
#define FOLD_AHEAD 4
__device__ __forceinline__ _acc_t _await_fold(_slot_t* slots, const ptrdiff_t first,
                                              const int count, const int lane,
                                              const unsigned epoch, const unsigned spin_limit,
                                              bool& ok) {
  const int sub = lane / INNER;
  const int col = lane - sub * INNER;
  const bool active = sub < FOLD_TILES;
  _acc_t s = SCAN_IDENTITY;
  int i = active ? sub : count;
  unsigned spins = 0;
  // the newest totals first, alone (see the kernel for contiguous rows)
  for (;;) {
    const _slot_t x = __hip_atomic_load(slots + ((first + count) * INNER) * kWords - 1,
                                        __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    if ((unsigned)(x >> 32) == epoch) break;
    if (spins >= spin_limit) { ok = false; break; }
    ++spins;
    __builtin_amdgcn_s_sleep(SPIN_SLEEP);
  }
  for (;;) {
    while (i < count) {
      _slot_t x[FOLD_AHEAD][kWords];
#pragma unroll
      for (int a = 0; a < FOLD_AHEAD; ++a) {
        // (past the last value: the last one again, not used)
        const int ia = (i + a * FOLD_TILES < count) ? i + a * FOLD_TILES : i;
#pragma unroll
        for (int k = 0; k < kWords; ++k)
          x[a][k] = __hip_atomic_load(slots + ((first + ia) * INNER + col) * kWords + k,
                                      __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      }
      bool stalled = false;
#pragma unroll
      for (int a = 0; a < FOLD_AHEAD; ++a) {
        if (stalled || i >= count) break;
        bool written = true;
        unsigned w[kWords];
#pragma unroll
        for (int k = 0; k < kWords; ++k) {
          written = written && (unsigned)(x[a][k] >> 32) == epoch;
          w[k] = (unsigned)x[a][k];
        }
        if (!written) { stalled = true; break; }
        _acc_t v;
        __builtin_memcpy(&v, w, sizeof(_acc_t));
        s = SCAN_OP(s, v);
        i += FOLD_TILES;
      }
      if (stalled) break;
    }
    if (__ballot(i < count) == 0) break;
    if (spins >= spin_limit) { ok = false; break; }
    ++spins;
    __builtin_amdgcn_s_sleep(SPIN_SLEEP);
  }
  // running combination down the lane groups of a column; the last group holds all
#pragma unroll
  for (int d = 1; d < FOLD_TILES; d <<= 1) {
    const _acc_t other = cupy::shfl_up<64>(s, d * INNER);
    s = (lane >= d * INNER && active) ? SCAN_OP(other, s) : s;
  }
  return cupy::shfl_idx<64>(s, (FOLD_TILES - 1) * INNER + col);
}

// One round of a wave: its rows as loaded -> the LDS -> every lane's own rows
// of its column scanned in registers (`v`), the running combination of the
// segments of a column across the lanes (`incl`).  Returns the column's total.
__device__ __forceinline__ _acc_t _round_scan(
    const cupy::Vec<_in_t, VEC> (&raw)[TRIPS], _acc_t* lds, const int valid, const int lane,
    const int seg, const int col, const bool active, _acc_t (&v)[LROWS], _acc_t& incl) {
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
  if (active) {
#pragma unroll
    for (int i = 0; i < LROWS; ++i) v[i] = lds[seg * SEG_STRIDE + i * INNER + col];
#pragma unroll
    for (int i = 1; i < LROWS; ++i) v[i] = SCAN_OP(v[i - 1], v[i]);
  } else {
#pragma unroll
    for (int i = 0; i < LROWS; ++i) v[i] = SCAN_IDENTITY;
  }
  incl = v[LROWS - 1];
#pragma unroll
  for (int d = 1; d < SEG; d <<= 1) {
    const _acc_t other = cupy::shfl_up<64>(incl, d * INNER);
    incl = (lane >= d * INNER) ? SCAN_OP(other, incl) : incl;
  }
  __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
  __builtin_amdgcn_wave_barrier();
  return cupy::shfl_idx<64>(incl, (SEG - 1) * INNER + col);
}

extern "C" __global__ void cupy_scan_chain_clear(unsigned* desc, const unsigned words) {
  for (unsigned i = blockIdx.x * blockDim.x + threadIdx.x; i < words; i += gridDim.x * blockDim.x)
    desc[i] = 0u;
}

// One workgroup per tile of TILE_ROWS rows of one (outer) slice, tiles numbered
// by blockIdx.x; waits, slots and the order of combination as in the kernel for
// contiguous rows, with INNER values per tile instead of one.
extern "C" __global__ void __launch_bounds__(%(block)d) cupy_scan_chain_tile(
    const _in_t* __restrict__ in, _out_t* __restrict__ out, unsigned* desc,
    const _idx_t n_outer, const _idx_t n, const _idx_t tiles_per_row, const _idx_t group_tiles,
    const _idx_t groups_per_row, const unsigned epoch, const unsigned spin_limit,
    unsigned* fault) {
  __shared__ _acc_t _lds_all[WAVES][LDS_WORDS];
  __shared__ _acc_t sm_wave[WAVES + 2][INNER];
  const ptrdiff_t n_tiles = (ptrdiff_t)n_outer * tiles_per_row;
  _slot_t* tile_totals = reinterpret_cast<_slot_t*>(desc + HEADER_WORDS);
  _slot_t* group_totals = tile_totals + n_tiles * INNER * kWords;
  const int lane = threadIdx.x %% 64;
  const int wv = threadIdx.x / 64;
  _acc_t* lds = _lds_all[wv];
  const int seg = lane / INNER;
  const int col = lane - seg * INNER;
  const bool active = lane < SEG * INNER;
  const ptrdiff_t tile = blockIdx.x;
  if (tile >= n_tiles) return;
  const _idx_t o = (_idx_t)(tile / tiles_per_row);
  const _idx_t t_row = (_idx_t)(tile - (ptrdiff_t)o * tiles_per_row);
  const _idx_t r0 = t_row * TILE_ROWS + wv * WAVE_ROWS;      // this wave's first row
  // ---- the wave's rows as loaded, all requested at once
  cupy::Vec<_in_t, VEC> raw[PARTS][TRIPS];
  int valid[PARTS];
#pragma unroll
  for (int q = 0; q < PARTS; ++q) {
    const _idx_t rb = r0 + q * ROWS_T;
    const _idx_t left = n - rb;
    const int rows_here = left <= 0 ? 0 : (left < ROWS_T ? (int)left : ROWS_T);
    valid[q] = rows_here * INNER;
    const _in_t* src = in + ((ptrdiff_t)o * n + rb) * INNER;
#pragma unroll
    for (int t = 0; t < TRIPS; ++t) {
      const int p = (t * 64 + lane) * VEC;
      if (p + VEC <= valid[q]) {
        raw[q][t] = cupy::load_vec<_in_t, VEC, NT_LOAD>(src + p);
      } else {
#pragma unroll
        for (int k = 0; k < VEC; ++k) raw[q][t].v[k] = (p + k < valid[q]) ? src[p + k] : _in_t();
      }
    }
  }
  // ---- totals: of every round, of the wave, of the tile (per column)
  _acc_t round_total[PARTS];
  _acc_t carry = SCAN_IDENTITY;
#pragma unroll
  for (int q = 0; q < PARTS; ++q) {
    _acc_t v[LROWS];
    _acc_t incl;
    round_total[q] = _round_scan(raw[q], lds, valid[q], lane, seg, col, active, v, incl);
    carry = (q == 0) ? round_total[q] : SCAN_OP(carry, round_total[q]);
  }
  if (lane < INNER) sm_wave[wv][lane] = carry;
  __syncthreads();
  _acc_t wave_before = SCAN_IDENTITY;
  _acc_t tile_total = sm_wave[0][col];
#pragma unroll
  for (int w = 1; w < WAVES; ++w) {
    if (w == wv) wave_before = tile_total;
    tile_total = SCAN_OP(tile_total, sm_wave[w][col]);
  }
  // ---- what precedes the tile in its slice
  const _idx_t g = t_row / group_tiles;
  const int t_group = (int)(t_row - g * group_tiles);
  const bool closes_group = (t_group == group_tiles - 1) || (t_row == tiles_per_row - 1);
  const ptrdiff_t row_groups = (ptrdiff_t)o * groups_per_row;
  if (wv == 0) {
    if (lane < INNER) _publish(tile_totals, tile * INNER + lane, tile_total, epoch);
    bool ok = true;
    _acc_t in_group = SCAN_IDENTITY;
    if (t_group > 0)
      in_group = _await_fold(tile_totals, tile - t_group, t_group, lane, epoch, spin_limit, ok);
    if (lane < INNER) {
      if (closes_group)
        _publish(group_totals, (row_groups + g) * INNER + lane,
                 (t_group > 0) ? SCAN_OP(in_group, tile_total) : tile_total, epoch);
      sm_wave[WAVES][lane] = in_group;
    }
    if (!ok && lane == 0 && fault) *reinterpret_cast<volatile unsigned*>(fault) = 1u;
  } else if (wv == 1 && g > 0) {
    bool ok = true;
    const _acc_t groups_before =
        _await_fold(group_totals, row_groups, (int)g, lane, epoch, spin_limit, ok);
    if (lane < INNER) sm_wave[WAVES + 1][lane] = groups_before;
    if (!ok && lane == 0 && fault) *reinterpret_cast<volatile unsigned*>(fault) = 1u;
  }
  __syncthreads();
  _acc_t base = SCAN_IDENTITY;
  if (g > 0) base = sm_wave[WAVES + 1][col];
  if (t_group > 0) base = (g > 0) ? SCAN_OP(base, sm_wave[WAVES][col]) : sm_wave[WAVES][col];
  if (wv > 0) base = (t_row > 0) ? SCAN_OP(base, wave_before) : wave_before;
  // ---- results, round by round
  carry = base;
  bool seeded = t_row > 0 || wv > 0;
#pragma unroll
  for (int q = 0; q < PARTS; ++q) {
    _acc_t v[LROWS];
    _acc_t incl;
    (void)_round_scan(raw[q], lds, valid[q], lane, seg, col, active, v, incl);
    _acc_t before = cupy::shfl_up<64>(incl, INNER);
    const bool has_before = seg > 0;
    before = seeded ? (has_before ? SCAN_OP(carry, before) : carry) : before;
    const bool any = seeded || has_before;
    if (active) {
#pragma unroll
      for (int i = 0; i < LROWS; ++i)
        lds[seg * SEG_STRIDE + i * INNER + col] = any ? SCAN_OP(before, v[i]) : v[i];
    }
    __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
    __builtin_amdgcn_wave_barrier();
    _out_t* dst = out + ((ptrdiff_t)o * n + r0 + q * ROWS_T) * INNER;
#pragma unroll
    for (int t = 0; t < TRIPS; ++t) {
      const int p = (t * 64 + lane) * VEC;
      if (p + VEC <= valid[q]) {
        cupy::Vec<_out_t, VEC> r;
#pragma unroll
        for (int k = 0; k < VEC; ++k) r.v[k] = static_cast<_out_t>(lds[_lds_at(p + k)]);
        cupy::store_vec<_out_t, VEC, NT_STORE>(dst + p, r);
      } else {
#pragma unroll
        for (int k = 0; k < VEC; ++k)
          if (p + k < valid[q]) dst[p + k] = static_cast<_out_t>(lds[_lds_at(p + k)]);
      }
    }
    __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
    __builtin_amdgcn_wave_barrier();
    carry = seeded ? SCAN_OP(carry, round_total[q]) : round_total[q];
    seeded = true;
  }
}
""" % dict(in_t=in_t, out_t=out_t, acc_t=acc_t, idx_t='ptrdiff_t' if idx64 else 'int',
           op_c=op_c, ident=ident, start=_start_text(op, acc_t), vec=vec, trips=trips, conv=conv, block=_BLOCK,
           inner=inner, rows_t=rows_t, seg=seg, lrows=lrows, stride=stride,
           waves=_CHAIN_WAVES, parts=parts, header=_CHAIN_HEADER_WORDS, sleep=sleep,
           ntl='true' if stream[0] else 'false', nts='true' if stream[1] else 'false')


def _module_chain_tile(in_dtype, out_dtype, op, skip_nan, vec, trips, idx64, inner, stream,
                       parts):
    sleep = _tuning.get('scan_chain_sleep')
    key = ('chain tile', _device.get_device_id(), in_dtype.char, out_dtype.char, op, skip_nan,
           vec, trips, idx64, inner, stream, parts, sleep)
    mod = _memo.get(key)
    if mod is None:
        src = _emit_chain_tile(_get_typename(in_dtype), _get_typename(out_dtype), op, skip_nan,
                               vec, trips, idx64, inner, stream, parts, sleep)
        mod = compiler.compile_with_cache(src)
        with _lock:
            mod = _memo.setdefault(key, mod)
    return mod


def _emit_chain_cols(in_t, out_t, op, skip_nan, vec, trips, idx64, waves, stream, sleep,
                     ahead=2, bands=False):
    """One-pass scan along the middle axis of (outer, n, inner) where the
    columns are many and long but too few to give every thread a column of its
    own: a workgroup per tile of WAVES x TRIPS rows by 64 x VEC columns.  A
    lane owns VEC adjacent columns and TRIPS consecutive rows of them, which it
    keeps as loaded: it adds them up for the totals, and once more, from what
    precedes it, for the results.  Tiles publish their totals per column and
    fold those of the tiles above them as in ``_emit_chain`` (slots, waits and
    an order of combination fixed by the tile's number); tiles are numbered
    row of tiles by row of tiles, so that a tile only ever waits for smaller
    numbers.

    ``bands``: workgroups are handed to the eight compute dies in turn
    (workgroup w goes to die w % 8, each die with a cache of its own), and
    neighbouring tiles of a row of tiles share the cache lines at their borders
    whenever the rows of the array do not start on line boundaries.  Workgroup
    w then takes tile number w / 8 of band w % 8 of the columns (the column
    blocks cut into eight runs), the band's tiles counted row of tiles by row
    of tiles: a die works on neighbouring tiles, and a tile still only waits
    for workgroups with smaller numbers (the tiles above it lie in its own
    band, earlier in the band's count)."""
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
#define SCAN_IDENTITY (_acc_t(%(start)s))
#define VEC %(vec)d
#define TRIPS %(trips)d
#define NT_LOAD %(ntl)s
#define NT_STORE %(nts)s
#define WAVES %(waves)d
#define HALF (WAVES / 2)
#define COLS_T (64 * VEC)
#define TILE_ROWS (WAVES * TRIPS)
#define HEADER_WORDS %(header)d
#define SPIN_SLEEP %(sleep)d
#define FOLD_AHEAD %(ahead)d
#define BANDS %(bands)d
__device__ __forceinline__ _acc_t _load_value(_in_t _x) { return %(conv)s; }

// Published values: see the one-pass kernel for contiguous rows.  Value
// `i * COLS_T + c` belongs to column c of tile (or group) i.
constexpr int kWords = (sizeof(_acc_t) + 3) / 4;
typedef unsigned long long _slot_t;

__device__ __forceinline__ void _publish(_slot_t* slots, const ptrdiff_t i, const _acc_t& v,
                                         const unsigned epoch) {
  unsigned w[kWords];
#pragma unroll
  for (int k = 0; k < kWords; ++k) w[k] = 0u;
  __builtin_memcpy(w, &v, sizeof(_acc_t));
#pragma unroll
  for (int k = 0; k < kWords; ++k)
    __hip_atomic_store(slots + i * kWords + k, ((_slot_t)epoch << 32) | w[k], __ATOMIC_RELAXED,
                       __HIP_MEMORY_SCOPE_AGENT);
}

// The values `first + j * stride + k` (j < count, k < VEC) of a lane's own
// columns, waited for and combined over j in order.  A lane asks for
// FOLD_AHEAD values of j at a time.  One wave, all lanes call (`count` is 0
// for a lane without columns); `ok` turns false if the wave gave up after
// `spin_limit` rounds of polling.
__device__ __forceinline__ void _await_fold_cols(
    _slot_t* slots, const ptrdiff_t first, const ptrdiff_t stride, const int count,
    const unsigned epoch, const unsigned spin_limit, bool& ok, _acc_t (&s)[VEC]) {
#pragma unroll
  for (int k = 0; k < VEC; ++k) s[k] = SCAN_IDENTITY;
  int i = 0;
  unsigned spins = 0;
  for (;;) {
    while (i < count) {
      _slot_t x[FOLD_AHEAD][VEC * kWords];
#pragma unroll
      for (int a = 0; a < FOLD_AHEAD; ++a) {
        // (past the last value: the last one again, not used)
        const int ia = (i + a < count) ? i + a : count - 1;
        const _slot_t* at = slots + (first + (ptrdiff_t)ia * stride) * kWords;
#pragma unroll
        for (int m = 0; m < VEC * kWords; ++m)
          x[a][m] = __hip_atomic_load(at + m, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      }
      bool stalled = false;
#pragma unroll
      for (int a = 0; a < FOLD_AHEAD; ++a) {
        if (stalled || i >= count) break;
        bool written = true;
#pragma unroll
        for (int m = 0; m < VEC * kWords; ++m)
          written = written && (unsigned)(x[a][m] >> 32) == epoch;
        if (!written) { stalled = true; break; }
#pragma unroll
        for (int k = 0; k < VEC; ++k) {
          unsigned w[kWords];
#pragma unroll
          for (int m = 0; m < kWords; ++m) w[m] = (unsigned)x[a][k * kWords + m];
          _acc_t v;
          __builtin_memcpy(&v, w, sizeof(_acc_t));
          s[k] = (i == 0) ? v : SCAN_OP(s[k], v);
        }
        ++i;
      }
      if (stalled) break;
    }
    if (__ballot(i < count) == 0) break;
    if (spins >= spin_limit) { ok = false; break; }
    ++spins;
    __builtin_amdgcn_s_sleep(SPIN_SLEEP);
  }
}

// (launched with workgroups of any size up to the bound)
extern "C" __global__ void __launch_bounds__(%(block)d) cupy_scan_chain_clear(
    unsigned* desc, const unsigned words) {
  for (unsigned i = blockIdx.x * blockDim.x + threadIdx.x; i < words; i += gridDim.x * blockDim.x)
    desc[i] = 0u;
}

extern "C" __global__ void __launch_bounds__(%(block)d) cupy_scan_chain_cols(
    const _in_t* __restrict__ in, _out_t* __restrict__ out, unsigned* desc,
    const _idx_t n_outer, const _idx_t n, const _idx_t inner, const _idx_t col_blocks,
    const _idx_t row_tiles, const _idx_t group_tiles, const _idx_t groups_per_col,
    const unsigned epoch, const unsigned spin_limit, unsigned* fault) {
  __shared__ _acc_t sm_wave[WAVES][COLS_T];
  __shared__ _acc_t sm_part[WAVES][COLS_T];
  const ptrdiff_t n_tiles = (ptrdiff_t)n_outer * row_tiles * col_blocks;
  _slot_t* tile_totals = reinterpret_cast<_slot_t*>(desc + HEADER_WORDS);
  _slot_t* group_totals = tile_totals + n_tiles * COLS_T * kWords;
  const int lane = threadIdx.x %% 64;
  const int wv = __builtin_amdgcn_readfirstlane(threadIdx.x / 64);
#if BANDS
  const _idx_t band = (_idx_t)(blockIdx.x & 7u);
  const ptrdiff_t seq = (ptrdiff_t)(blockIdx.x >> 3);
  const _idx_t band_base = col_blocks / 8, band_rest = col_blocks %% 8;
  const _idx_t band_width = band_base + (band < band_rest ? 1 : 0);
  if (band_width == 0) return;
  const _idx_t cb = band * band_base + (band < band_rest ? band : band_rest)
                    + (_idx_t)(seq %% band_width);
  const ptrdiff_t slab = seq / band_width;                   // (o, t_row)
  if (slab >= (ptrdiff_t)n_outer * row_tiles) return;
  const ptrdiff_t tile = slab * col_blocks + cb;
#else
  const ptrdiff_t tile = blockIdx.x;
  if (tile >= n_tiles) return;
  const _idx_t cb = (_idx_t)(tile %% col_blocks);
  const ptrdiff_t slab = tile / col_blocks;                  // (o, t_row)
#endif
  const _idx_t t_row = (_idx_t)(slab %% row_tiles);
  const _idx_t o = (_idx_t)(slab / row_tiles);
  const int lc = lane * VEC;                     // the lane's first column within the block
  const bool has_cols = cb * COLS_T + lc < inner;
  // A vector that would pass the end of the rows (their length is no multiple
  // of VEC) starts VEC columns before the end instead and overlaps its
  // neighbour's: both lanes compute and store the same values for the shared
  // column (never in place: the host sees to that).  In the LDS and in the
  // slots the lane keeps its own places.
  const int lm = (VEC > 1 && cb * COLS_T + lc + VEC > inner) ? (int)(inner - VEC - cb * COLS_T) : lc;
  const _idx_t r0 = t_row * TILE_ROWS + wv * TRIPS;          // this wave's first row
  // (the same for all lanes of a wave: the lanes differ by `lc` alone)
  const ptrdiff_t at0 = ((ptrdiff_t)o * n + r0) * inner + (ptrdiff_t)cb * COLS_T;
  // ---- the lane's rows as loaded, all requested at once
  cupy::Vec<_in_t, VEC> raw[TRIPS];
#pragma unroll
  for (int t = 0; t < TRIPS; ++t) {
    if (has_cols && r0 + t < n) {
      raw[t] = cupy::load_vec<_in_t, VEC, NT_LOAD>(in + at0 + (ptrdiff_t)t * inner + lm);
    } else {
#pragma unroll
      for (int k = 0; k < VEC; ++k) raw[t].v[k] = _in_t();
    }
  }
  // ---- totals: of the lane, of the waves above it, of the tile
  _acc_t run[VEC];
#pragma unroll
  for (int k = 0; k < VEC; ++k) run[k] = SCAN_IDENTITY;
#pragma unroll
  for (int t = 0; t < TRIPS; ++t) {
    if (r0 + t < n) {
#pragma unroll
      for (int k = 0; k < VEC; ++k)
        run[k] = (t == 0) ? _load_value(raw[t].v[k]) : SCAN_OP(run[k], _load_value(raw[t].v[k]));
    }
  }
#pragma unroll
  for (int k = 0; k < VEC; ++k) sm_wave[wv][k * 64 + lane] = run[k];
  __syncthreads();
  _acc_t wave_before[VEC], tile_total[VEC];
#pragma unroll
  for (int k = 0; k < VEC; ++k) {
    wave_before[k] = SCAN_IDENTITY;
    tile_total[k] = sm_wave[0][k * 64 + lane];
#pragma unroll
    for (int w = 1; w < WAVES; ++w) {
      if (w == wv) wave_before[k] = tile_total[k];
      tile_total[k] = SCAN_OP(tile_total[k], sm_wave[w][k * 64 + lane]);
    }
  }
  // ---- what precedes the tile in its columns: the totals of the tiles above
  // it in its group and of the groups above its own.  The first half of the
  // waves shares out the former, the second half the latter (every wave a run
  // of consecutive ones), so that the trips to memory overlap; the partial
  // results are then combined in the order of the waves.
  const _idx_t g = t_row / group_tiles;
  const int t_group = (int)(t_row - g * group_tiles);
  const bool closes_group = (t_group == group_tiles - 1) || (t_row == row_tiles - 1);
  const ptrdiff_t tile_stride = (ptrdiff_t)col_blocks * COLS_T;   // values from a tile to the one below
  if (wv == 0 && has_cols) {
#pragma unroll
    for (int k = 0; k < VEC; ++k)
      _publish(tile_totals, tile * COLS_T + lane * VEC + k, tile_total[k], epoch);
  }
  const bool tiles_side = wv < HALF;
  const int side_count = tiles_side ? t_group : (int)g;
  const int per_wave = (side_count + HALF - 1) / HALF;
  {
    const int j0 = (tiles_side ? wv : wv - HALF) * per_wave;
    int mine = side_count - j0;
    mine = mine < 0 ? 0 : (mine > per_wave ? per_wave : mine);
    const ptrdiff_t first =
        (tiles_side ? (tile - (ptrdiff_t)t_group * col_blocks) * COLS_T
                    : (((ptrdiff_t)o * groups_per_col) * col_blocks + cb) * COLS_T)
        + lane * VEC + (ptrdiff_t)j0 * tile_stride;
    bool ok = true;
    _acc_t part[VEC];
    _await_fold_cols(tiles_side ? tile_totals : group_totals, first, tile_stride,
                     has_cols ? mine : 0, epoch, spin_limit, ok, part);
#pragma unroll
    for (int k = 0; k < VEC; ++k) sm_part[wv][k * 64 + lane] = part[k];
    if (!ok && lane == 0 && fault) *reinterpret_cast<volatile unsigned*>(fault) = 1u;
  }
  __syncthreads();
  const int per_tiles = (t_group + HALF - 1) / HALF;
  const int per_groups = ((int)g + HALF - 1) / HALF;
  const bool seeded = t_row > 0 || wv > 0;
#pragma unroll
  for (int k = 0; k < VEC; ++k) {
    _acc_t in_group = SCAN_IDENTITY, groups_before = SCAN_IDENTITY;
#pragma unroll
    for (int w = 0; w < HALF; ++w) {
      if (w * per_tiles < t_group)
        in_group = (w == 0) ? sm_part[w][k * 64 + lane] : SCAN_OP(in_group, sm_part[w][k * 64 + lane]);
      if (w * per_groups < (int)g)
        groups_before = (w == 0) ? sm_part[HALF + w][k * 64 + lane]
                                 : SCAN_OP(groups_before, sm_part[HALF + w][k * 64 + lane]);
    }
    if (wv == 0 && has_cols && closes_group)
      _publish(group_totals,
               (((ptrdiff_t)o * groups_per_col + g) * col_blocks + cb) * COLS_T + lane * VEC + k,
               (t_group > 0) ? SCAN_OP(in_group, tile_total[k]) : tile_total[k], epoch);
    _acc_t base = SCAN_IDENTITY;
    if (g > 0) base = groups_before;
    if (t_group > 0) base = (g > 0) ? SCAN_OP(base, in_group) : in_group;
    if (wv > 0) base = (t_row > 0) ? SCAN_OP(base, wave_before[k]) : wave_before[k];
    run[k] = base;
  }
  // ---- results
  if (!has_cols) return;
#pragma unroll
  for (int t = 0; t < TRIPS; ++t) {
    if (r0 + t < n) {
      cupy::Vec<_out_t, VEC> r;
#pragma unroll
      for (int k = 0; k < VEC; ++k) {
        const _acc_t x = _load_value(raw[t].v[k]);
        run[k] = (seeded || t > 0) ? SCAN_OP(run[k], x) : x;
        r.v[k] = static_cast<_out_t>(run[k]);
      }
      cupy::store_vec<_out_t, VEC, NT_STORE>(out + at0 + (ptrdiff_t)t * inner + lm, r);
    }
  }
}
""" % dict(in_t=in_t, out_t=out_t, acc_t=acc_t, idx_t='ptrdiff_t' if idx64 else 'int',
           op_c=op_c, ident=ident, start=_start_text(op, acc_t), vec=vec, trips=trips, conv=conv, block=waves * _WAVE,
           waves=waves, header=_CHAIN_HEADER_WORDS, sleep=sleep, ahead=ahead, bands=1 if bands else 0,
           ntl='true' if stream[0] else 'false', nts='true' if stream[1] else 'false')


def _module_chain_cols(in_dtype, out_dtype, op, skip_nan, vec, trips, idx64, waves, stream,
                       bands=False):
    sleep = _tuning.get('scan_chain_sleep')
    key = ('chain cols', _device.get_device_id(), in_dtype.char, out_dtype.char, op, skip_nan,
           vec, trips, idx64, waves, stream, sleep, bands)
    mod = _memo.get(key)
    if mod is None:
        # published totals a lane asks for at a time: what the registers of
        # a lane in a workgroup of 16 waves hold beside its rows
        ahead = 4 if (in_dtype.itemsize == 4 and _acc_dtype(out_dtype).itemsize * vec <= 8) else 2
        src = _emit_chain_cols(_get_typename(in_dtype), _get_typename(out_dtype), op, skip_nan,
                               vec, trips, idx64, waves, stream, sleep, ahead, bands)
        mod = compiler.compile_with_cache(src)
        with _lock:
            mod = _memo.setdefault(key, mod)
    return mod


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


def _chain_fault_word(dev_id):
    """Address of the word in pinned host memory a tile that gave up waiting
    writes to (0 where none could be allocated)."""
    return _giveup.word(dev_id, _giveup.SCAN)


_chain_arenas = {}       # (device id, stream) -> [slots array, number of the last launch]


def _chain_slots(dev_id, stream_ptr, words, mod):
    """Memory for the published totals of one launch on ``stream_ptr`` and the
    launch's number.  A stream keeps its array from call to call (launches on
    one stream run one after the other, and each marks what it publishes with
    its own number, so nothing needs clearing in between); the array is
    cleared when it is created, when it has to grow and when the numbers wrap
    around."""
    if stream_ptr is None:
        stream_ptr = _stream.get_current_stream_ptr()
    key = (dev_id, stream_ptr)
    with _lock:
        arena = _chain_arenas.get(key)
        if arena is None or arena[0].size < words or arena[1] >= 0xffffffff:
            if len(_chain_arenas) >= 64:
                _chain_arenas.clear()
            size = max(words, 1 << 16)
            if arena is not None:
                size = max(size, 2 * arena[0].size)
            desc = ndarray._new_contiguous((size,), numpy.dtype('uint32'))
            # (a kernel, not a memset: the caller may be capturing the stream)
            mod.get_function('cupy_scan_chain_clear').launch_packed(
                (max(1, min(1024, (size + _BLOCK - 1) // _BLOCK)), 1, 1), (_BLOCK, 1, 1),
                struct.pack('@PI', desc.data.ptr, size), 0, stream_ptr)
            arena = _chain_arenas[key] = [desc, 0]
        arena[1] += 1
        return arena[0], arena[1]


def _chain_ready():
    """(device id, address of the device's fault word) if the one-pass kernels
    may be used, else None."""
    if not _tuning.get('scan_chain'):
        return None
    dev_id = _device.get_device_id()
    if dev_id in _giveup.disabled[_giveup.SCAN]:
        return None
    if _stream.get_current_stream_ptr() == _stream.STREAM_PER_THREAD:
        # (one handle, a different stream in every thread: the published
        # totals of two threads' scans would share their memory)
        return None
    fault = _chain_fault_word(dev_id)
    # A tile of an earlier scan that gave up waiting for the tiles before it
    # left wrong results.  Not expected to happen: poll() says so, and the
    # kernels stay unused from there on.
    _giveup.poll(dev_id)
    return dev_id, fault


def _scan_chained(src, dst, n_rows, n, op, skip_nan, vec, idx64, stream, stream_ptr, inner=1):
    """The one-pass scan of a few long rows (``_emit_chain``) or, with
    ``inner`` > 1, of a few long slices of rows of ``inner`` elements scanned
    down their columns (``_emit_chain_tile``): input read once, output written
    once.  Returns False where it does not apply (the caller then takes the
    three-pass route)."""
    ready = _chain_ready()
    if ready is None:
        return False
    dev_id, fault = ready
    in_dtype, out_dtype = src.dtype, dst.dtype
    trips = 4
    waves, wide = _tuning.get('scan_chain_waves'), 1
    parts = _tuning.get('scan_chain_parts')
    if not parts:
        # Bigger tiles mean fewer waits per byte but fewer workgroups per CU;
        # measured on 2^20 .. 2^26 float32: 8 parts (128 KiB of input per tile)
        # are best from 64 MiB on, 4 from 16 MiB on
        # (with 8-byte and wider values 8 parts do not fit the registers of a lane)
        nbytes = n_rows * n * inner * in_dtype.itemsize
        parts = 8 if nbytes >= 64 << 20 else 4 if nbytes >= 16 << 20 else 2
        if max(in_dtype.itemsize, _acc_dtype(out_dtype).itemsize) > 4 or inner > 1:
            parts = min(parts, 4)
            if inner == 1 and parts == 4 and waves >= 2 * _CHAIN_WAVES:
                # (2^25 float64 in one row: 4 waves x 4 parts 122 us, 8 x 2 114,
                # 8 x 3 110, 16 x 2 112)
                parts = 6
        if 1 < inner <= 6:
            # (2^26 float32 as (n,3): 115 us with 2 parts, 123 with 4; as (n,5)
            # 133 / 138; as (n,12) 131 / 113; as (n,16) 128 / 120)
            parts = min(parts, 2)
    if inner > 1:
        vec = max(1, 16 // max(in_dtype.itemsize, out_dtype.itemsize))
        tile = _CHAIN_WAVES * parts * _tile_geometry(inner, vec, trips)[0]     # rows
        waves = _CHAIN_WAVES
    else:
        # No tile longer than a row; and rows of few tiles want small ones: a
        # tile then waits for few others, and there are many rows to go on
        # with (2^26 float32 over rotating buffers, 1 / 8 parts: 1024 rows of
        # 65536 93.5 / 101 us, 4096 rows of 16384 94.5 / 99; but 64 rows of
        # 2^20 183 / 102 and one row 138 / 104)
        base_tiles = n // (_BLOCK * vec * trips)
        if not _tuning.get('scan_chain_parts'):
            parts = min(parts, 1 if base_tiles <= 16 else 2 if base_tiles <= 64
                        else 4 if base_tiles <= 128 else 8)
        parts = max(1, min(parts, base_tiles))
        # the same tile from more waves with fewer vectors per lane
        while (_CHAIN_WAVES * wide < waves and parts % 2 == 0
               and parts > _tuning.get('scan_chain_min_parts')):
            parts //= 2
            wide *= 2
        waves = _CHAIN_WAVES * wide
        tile = waves * _WAVE * vec * trips * parts
    tiles_per_row = (n + tile - 1) // tile
    n_tiles = n_rows * tiles_per_row
    if n_tiles < 2 or n_tiles * max(_BLOCK, waves * _WAVE) > 0xffffffff or n < _BLOCK * vec * trips:
        return False
    if (inner == 1 and tiles_per_row * tile > _tuning.get('scan_chain_max_waste') * n
            and n_rows >= _device.get_compute_units(dev_id) * _tuning.get('scan_waves_per_cu')):
        # Many rows a little longer than a whole number of tiles: the last
        # tile of every row would be all but empty (rows of 4099 floats: two
        # tiles of 4096); a wave per row does better.
        return False
    # groups of about sqrt(tiles per row) tiles: a tile then reads about
    # 2 sqrt(tiles per row) published totals
    group_tiles = max(32, min(2048, internal.clp2(int(tiles_per_row ** 0.5))))
    groups_per_row = (tiles_per_row + group_tiles - 1) // group_tiles
    n_groups = n_rows * groups_per_row
    # every 32-bit word of a published total sits in a 64-bit slot beside its mark
    words_per_value = (_acc_dtype(out_dtype).itemsize + 3) // 4
    desc_words = _CHAIN_HEADER_WORDS + 2 * words_per_value * inner * (n_tiles + n_groups)
    if desc_words > 0xffffffff:
        return False
    if inner > 1:
        mod = _module_chain_tile(in_dtype, out_dtype, op, skip_nan, vec, trips, idx64, inner,
                                 stream, parts)
        name = 'cupy_scan_chain_tile'
    else:
        # Rows off the cache lines, enough of them for every die, two tiles to
        # a row: a die per row (8192 rows of 8191 float32: 101 -> 95 us; rows of
        # many tiles lose, their tiles wait for each other on one die: 1024 rows
        # of 65537 102 -> 131)
        mode = _tuning.get('scan_chain_xcd')
        bands = bool(mode) and n_rows >= 64 and tiles_per_row == 2 and (
            mode is True or (n * in_dtype.itemsize) % 128 != 0 or src.data.ptr % 128 != 0
            or (n * out_dtype.itemsize) % 128 != 0 or dst.data.ptr % 128 != 0)
        if bands:
            launched = 8 * ((n_rows + 7) // 8) * tiles_per_row
            if launched * waves * _WAVE > 0xffffffff:
                bands = False
        mod = _module_chain(in_dtype, out_dtype, op, skip_nan, vec, trips, idx64, stream,
                            n % vec != 0, parts, waves, bands)
        name = 'cupy_scan_chain'
        if bands:
            n_tiles = launched
    desc, epoch = _chain_slots(dev_id, stream_ptr, desc_words, mod)
    ic = 'q' if idx64 else 'i'
    blob = struct.pack('@PPP' + ic * 5 + 'IIP', src.data.ptr, dst.data.ptr, desc.data.ptr,
                       n_rows, n, tiles_per_row, group_tiles, groups_per_row, epoch,
                       _tuning.get('scan_chain_spin_limit'), fault)
    mod.get_function(name).launch_packed(
        (n_tiles, 1, 1), (waves * _WAVE if inner == 1 else _BLOCK, 1, 1), blob, 0, stream_ptr)
    return True


def _may_overlap(src, dst):
    """True if a scan from ``src`` into ``dst`` may read what it has written
    (in place, or views of one allocation whose byte ranges meet)."""
    from cupy_amd._core._carray import may_share_bounds
    return may_share_bounds(src, dst)


def _scan_chained_cols(src, dst, outer, n, inner, op, skip_nan, idx64, stream, stream_ptr):
    """The one-pass scan down many long columns (``_emit_chain_cols``).  Returns
    False where it does not apply."""
    if not _tuning.get('scan_chain_cols'):
        return False
    ready = _chain_ready()
    if ready is None:
        return False
    dev_id, fault = ready
    in_dtype, out_dtype = src.dtype, dst.dtype
    acc_item = _acc_dtype(out_dtype).itemsize
    # (a lane keeps its rows as loaded: the width of the accumulator, wider than
    # the values for float16, does not count)
    item = max(in_dtype.itemsize, out_dtype.itemsize)
    # Vectors of 8 bytes, or of 4 where those would leave many lanes of the
    # last block of columns idle; a workgroup of 16 waves, each lane keeping
    # 256 bytes of its columns.  (2^26 float32 over rotating buffers, us, for
    # 8192 x 8192 / 16 x 4096 x 1024 / 262144 x 256: 16 waves, 8-byte vectors,
    # 32 rows a lane 97 / 112 / 110; 8 waves 99 / 110 / 110; 4 waves 105 / 126
    # / 147; 16-byte vectors with 4 waves and 32 rows 122 / 152 / 188.  The
    # three-pass kernels: 145 / 149 / 169.)
    best = None
    forced = _tuning.get('scan_chain_cols_vec_bytes')
    for vec_bytes in ((forced,) if forced else (8, 4)):
        # (two columns a lane at most: every column has its running values and
        # its share of the look-back in registers)
        v = max(1, min(2, vec_bytes // item))
        # (rows of any length and arrays aligned for one element keep their
        # vectors where wide accesses need no more than that: the last vector
        # of a row then overlaps its neighbour, which in place would let one
        # lane read what another has already written)
        loose = (_tuning.get('unaligned_vectors') and _tuning.get('scan_chain_cols_unaligned')
                 and inner >= 2 * v and not _may_overlap(src, dst))
        while v > 1 and not loose and (
                not _aligned(src.data.ptr, v * in_dtype.itemsize)
                or not _aligned(dst.data.ptr, v * out_dtype.itemsize) or inner % v):
            v //= 2
        cols_t = _WAVE * v
        blocks = (inner + cols_t - 1) // cols_t
        used = inner / (blocks * cols_t)
        if best is None or used > best[0] + 0.1:
            best = (used, v, blocks)
    _, vec, col_blocks = best
    waves = max(2, min(16, _tuning.get('scan_chain_cols_waves')))
    # (values narrower than a register are unpacked: fewer rows then)
    trips = _tuning.get('scan_chain_cols_trips')
    if not trips:
        trips = max(4, min(64 if item >= 4 else 32, (256 if item < 16 else 128) // (vec * item)))
        # (columns of a few hundred rows: shorter tiles, so that there are at
        # least two down a column; 257 slices of 511 x 509 float32: 137 us with
        # 16 rows a lane, 149 with 8, 204 with 4)
        while trips > 16 and n < 2 * waves * trips:
            trips //= 2
    tile_rows = waves * trips
    row_tiles = (n + tile_rows - 1) // tile_rows
    n_tiles = outer * row_tiles * col_blocks
    if row_tiles < 2 or n_tiles * waves * _WAVE > 0xffffffff:
        return False
    # groups of about sqrt(tiles down a column) tiles
    group_tiles = max(2, 1 << (row_tiles.bit_length() // 2))
    groups_per_col = (row_tiles + group_tiles - 1) // group_tiles
    n_groups = outer * groups_per_col * col_blocks
    words_per_value = (acc_item + 3) // 4
    desc_words = _CHAIN_HEADER_WORDS + 2 * words_per_value * _WAVE * vec * (n_tiles + n_groups)
    if desc_words > 0x7fffffff:
        return False
    # Rows off the cache lines: tiles numbered band by band (see the kernel)
    mode = _tuning.get('scan_chain_cols_xcd')
    bands = bool(mode) and col_blocks >= 32 and (
        mode is True or (inner * in_dtype.itemsize) % 128 != 0 or src.data.ptr % 128 != 0
        or (inner * out_dtype.itemsize) % 128 != 0 or dst.data.ptr % 128 != 0)
    launched = n_tiles
    if bands:
        launched = 8 * outer * row_tiles * ((col_blocks + 7) // 8)
        if launched * waves * _WAVE > 0xffffffff:
            bands, launched = False, n_tiles
    mod = _module_chain_cols(in_dtype, out_dtype, op, skip_nan, vec, trips, idx64, waves, stream,
                             bands)
    desc, epoch = _chain_slots(dev_id, stream_ptr, desc_words, mod)
    ic = 'q' if idx64 else 'i'
    blob = struct.pack('@PPP' + ic * 7 + 'IIP', src.data.ptr, dst.data.ptr, desc.data.ptr,
                       outer, n, inner, col_blocks, row_tiles, group_tiles, groups_per_col,
                       epoch, _tuning.get('scan_chain_spin_limit'), fault)
    mod.get_function('cupy_scan_chain_cols').launch_packed(
        (launched, 1, 1), (waves * _WAVE, 1, 1), blob, 0, stream_ptr)
    return True


def _chunk_below(cus, n, want):
    """Number of slices below which the staged and the lane-interleaved kernels
    cut the slices into chunks.  Slices of fewer than 4096 rows are better off
    whole, a wave each, while there are four waves per CU: 2^26 floats in
    slices of 1024 x 16 143 us cut up, 114 whole; of 1024 x 36 148 -> 113, of
    512 x 64 142 -> 117, of 257 x 100 186 -> 132; with fewer waves than that
    whole slices lose (8192 x 16 from 512 waves: 186 against 105), and longer
    slices do well in the one-pass kernels (16384 x 3: 107 against 125)."""
    if n < 4096:
        return min(want, cus * _tuning.get('scan_whole_slices_waves_per_cu'))
    return want


def _scan_packed(src, dst, outer, n, inner, op, skip_nan, vec, trips, idx64, stream, stream_ptr,
                 cus):
    """Launches ``_emit_tile_packed`` where several slices fit a round: two for
    rows that are no whole vectors, else four (with two the plain kernels are
    as good there: 2^17 slices of 32 x 16 floats 86.6 us against 91.5).
    Returns False otherwise."""
    if outer < 2 or not _tuning.get('scan_tile_packed'):
        return False
    while _tile_geometry(inner, vec, trips)[2] > 32 and trips > 1:
        trips //= 2       # (a lane marks the slice starts among its rows in 64 bits)
    rows_t, _, lrows, _ = _tile_geometry(inner, vec, trips)
    # (rows that are whole vectors do as well a slice to a wave down to a third
    # of a round: 2^26 floats in slices of 24 x 16 88 us against 96 here; others
    # do not: 100 x 3 180 against 97, 60 x 5 241 against 95, 12 x 31 130
    # against 93, 10 x 33 176 against 98)
    least = _tuning.get('scan_tile_packed_min_slices')
    if not least:
        least = 4 if inner == 1 or inner % vec == 0 else 2
    if least * n > rows_t or lrows > 64:
        return False
    round_rows = rows_t // n * n
    mod = _module_tile_packed(src.dtype, dst.dtype, op, skip_nan, vec, trips, idx64, inner, stream)
    rounds = (outer * n + round_rows - 1) // round_rows
    per_block = _BLOCK // _WAVE
    grid = max(1, min((rounds + per_block - 1) // per_block,
                      cus * _tuning.get('scan_blocks_per_cu')))
    blob = struct.pack('@PP' + ('q' if idx64 else 'i') + 'ii', src.data.ptr, dst.data.ptr,
                       outer * n, n, round_rows)
    mod.get_function('cupy_scan_tile_packed').launch_packed(
        (grid, 1, 1), (_BLOCK, 1, 1), blob, 0, stream_ptr)
    return True


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
        # Inputs stream; results too once input and output together reach half
        # the memory-side cache.  (Measured over rotating buffer sets, so that
        # no call finds what an earlier one left behind: with non-temporal
        # stores 2^26 float32 along rows of 8192 take 104 us against 111, down
        # 64 long columns 97 against 104, in one dimension 102 against 107;
        # arrays of 64 and 128 MiB gain 2-5 %.  Repeated scans of ONE array of
        # 256 MiB look faster with plain stores, 85 us, only because the
        # cache absorbs the rewriting of the same lines.)
        stream = (True, total * (in_dtype.itemsize + out_dtype.itemsize)
                  >= _tuning.get('cache_bytes') // 2)
    else:
        stream = _tuning.stream_policy(setting, total * in_dtype.itemsize,
                                       total * out_dtype.itemsize)
    # A chunked scan reads its input twice.  While the input is not much larger
    # than the memory-side cache, the second reading starts where the first
    # ended and finds (part of) it there.
    reuse_ok = (_tuning.get('scan_chunk_reuse')
                and total * in_dtype.itemsize <= 2 * _tuning.get('cache_bytes'))
    if inner > 1 and n <= 256 and total * item <= _tuning.get('scan_whole_max_bytes'):
        # Small arrays scanned down short columns: three launches and a
        # temporary cost more than the few rounds of a single pass (us per
        # call, whole against cut: 128 x 128 floats along axis 0 13 / 36,
        # 256 x 256 25 / 40, 128 x 2048 16 / 39, 256 x 1024 29 / 40; longer
        # columns are better off cut: 1024 x 64 41 / 31).
        may_chunk = False
    if inner == 1:
        vec = max(1, 16 // item)
        # (rows of any length keep their vectors: wide accesses need the
        # alignment of an element only, and the kernels end every row element
        # by element; 2^26 floats as rows of 33: 294 us element-wide)
        loose = _tuning.get('unaligned_vectors') and _tuning.get('scan_rows_unaligned')
        if (n % vec and _tuning.get('scan_rows_packed')
                and _aligned(src.data.ptr, in_dtype.itemsize * vec)
                and _scan_packed(src, dst, outer, n, 1, op, skip_nan, vec, 4, idx64, stream,
                                 stream_ptr, cus)):
            # short rows that are no whole number of vectors: as slices of one
            # column, many to a wave (2^26 floats as rows of 33: 45 % of peak
            # with a lane group per row)
            return
        while vec > 1 and ((not loose and (
                not _aligned(src.data.ptr, vec * in_dtype.itemsize)
                or not _aligned(dst.data.ptr, vec * out_dtype.itemsize)
                or (outer > 1 and n % vec))) or n < vec):
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
        long_rows = n * in_dtype.itemsize >= _tuning.get('scan_chain_min_row_bytes')
        if (n_chunks > 1 or long_rows) and _scan_chained(
                src, dst, outer, n, op, skip_nan, vec, idx64, stream, stream_ptr):
            return
        chunk_len = (n + n_chunks - 1) // n_chunks
        chunk_len = (chunk_len + per_group - 1) // per_group * per_group
        n_chunks = (n + chunk_len - 1) // chunk_len
        mod = _module(in_dtype, out_dtype, op, skip_nan, vec, trips, idx64, group, stream,
                      ragged=n % vec != 0, reuse=n_chunks > 1 and reuse_ok)
        groups = outer * n_chunks
        per_block = _BLOCK // group
        grid = max(1, min((groups + per_block - 1) // per_block, cus * _tuning.get('scan_blocks_per_cu')))
        fmt = '@PPP' + ic * 4

        def launch(name, totals_ptr):
            blob = struct.pack(fmt, src.data.ptr, dst.data.ptr, totals_ptr, outer, n,
                               n_chunks, chunk_len)
            mod.get_function(name).launch_packed(
                (grid, 1, 1), (_BLOCK, 1, 1), blob, 0, stream_ptr)
        prefix = 'cupy_scan_rows'
        totals_shape = (outer, n_chunks, 1)
        middle_round = _WAVE * 4 * 4          # elements one wave takes per round
    elif (inner >= 2 and n >= 2 and _slab_pays(src, dst, n, inner, item)
          and _scan_slab(src, dst, outer, n, inner, op, skip_nan, idx64, stream, stream_ptr, cus)):
        return
    elif (inner > 64 and n >= 2
          and _scan_slab_long(src, dst, outer, n, inner, op, skip_nan, idx64, stream, stream_ptr,
                              cus)):
        return
    elif (2 <= inner <= (_tuning.get('scan_tile_max_inner') if n < 16384 else 32)
          and _tuning.get('scan_tile')):
        # (33 to 64 columns: a lane per column, half the wave idle while it
        # scans, but whole vectors both ways; 2^26 floats in slices of 16 x 33:
        # 51 -> 62 % of peak, of 100 x 63: 33 -> 56 %.  Long columns are better
        # off in the one-pass kernel for many columns.)
        vec = max(1, 16 // item)
        trips = 4
        rows_t, _, _, _ = _tile_geometry(inner, vec, trips)
        # Slices of few rows: many to a round.  (2^26 float32 as 2^22 slices of
        # 4 x 4: 1190 us with a wave per slice; 2^21 of 16 x 2: 697; 2^20 of
        # 2 x 32: 278)
        if _scan_packed(src, dst, outer, n, inner, op, skip_nan, vec, trips, idx64, stream,
                        stream_ptr, cus):
            return
        want = cus * _tuning.get('scan_waves_per_cu')
        n_chunks = 1
        if may_chunk and outer < _chunk_below(cus, n, want) and n > 2 * rows_t:
            n_chunks = min((want + outer - 1) // outer, (n + rows_t - 1) // rows_t)
        if n_chunks > 1 and _scan_chained(src, dst, outer, n, op, skip_nan, vec, idx64, stream,
                                          stream_ptr, inner=inner):
            return
        chunk_len = (n + n_chunks - 1) // n_chunks
        chunk_len = (chunk_len + rows_t - 1) // rows_t * rows_t
        n_chunks = (n + chunk_len - 1) // chunk_len
        mod = _module_tile(in_dtype, out_dtype, op, skip_nan, vec, trips, idx64, inner, stream,
                           n_chunks > 1 and reuse_ok)
        waves = outer * n_chunks
        per_block = _BLOCK // _WAVE
        grid = max(1, min((waves + per_block - 1) // per_block, cus * _tuning.get('scan_blocks_per_cu')))
        fmt = '@PPP' + ic * 4

        def launch(name, totals_ptr):
            blob = struct.pack(fmt, src.data.ptr, dst.data.ptr, totals_ptr, outer, n,
                               n_chunks, chunk_len)
            mod.get_function(name).launch_packed(
                (grid, 1, 1), (_BLOCK, 1, 1), blob, 0, stream_ptr)
        prefix = 'cupy_scan_tile'
        totals_shape = (outer, n_chunks, inner)
        middle_round = rows_t
    elif (_tuning.get('scan_lanes') and _lanes_geometry(src, dst, inner, item) is not None
          # (a slice with fewer rows than a wave takes per trip leaves most of
          # the wave idle: a thread per column vector instead; 2^19 slices of
          # 2 x 64 floats: 274 us here)
          and n > _WAVE // _lanes_geometry(src, dst, inner, item)[1]):
        vec, lstride = _lanes_geometry(src, dst, inner, item)
        trips = 4
        trip_rows = _WAVE // lstride
        per_wave = trip_rows * trips
        want = cus * _tuning.get('scan_waves_per_cu')
        n_chunks = 1
        if may_chunk and outer < _chunk_below(cus, n, want) and n > 2 * per_wave:
            n_chunks = min((want + outer - 1) // outer, (n + per_wave - 1) // per_wave)
        if n_chunks > 1 and _scan_chained_cols(src, dst, outer, n, inner, op, skip_nan, idx64,
                                               stream, stream_ptr):
            return
        chunk_len = (n + n_chunks - 1) // n_chunks
        chunk_len = (chunk_len + per_wave - 1) // per_wave * per_wave
        n_chunks = (n + chunk_len - 1) // chunk_len
        mod = _module_lanes(in_dtype, out_dtype, op, skip_nan, vec, trips, idx64, lstride,
                            stream)
        waves = outer * n_chunks
        per_block = _BLOCK // _WAVE
        grid = max(1, min((waves + per_block - 1) // per_block, cus * _tuning.get('scan_blocks_per_cu')))
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
        # A thread owns ``vec`` adjacent columns and walks down them, ``trips``
        # rows requested at a time.  Wide vectors need many columns to give
        # every CU its waves; narrower ones with more rows in flight keep a
        # narrow array in one pass (two transfers per element) where cutting
        # the rows into chunks costs three.  2^26 float32 over rotating
        # buffers, us: 64 x 2^20 16-byte vectors 32 rows 92 (16 rows 98, 4
        # rows 115); 256 x 2^18 8-byte vectors 32 rows 89 (16-byte 8 rows 95,
        # 32 rows 141, chunked 131); 1024 x 2^16 4-byte vectors 64 rows 104 (32
        # rows 125, chunked 128).  Below 256 threads per CU the rows are cut
        # into chunks: 4096 x 2^14 135 with 8 rows at a time.
        # (not in place: a thread would find its neighbour's results where it
        # expects the values of the columns they share)
        # (and rows of 128 columns or more: 2^26 floats in slices of 100 x 33
        # take 220 us element-wide, 280 with overlapping vectors; in slices of
        # 2 x 65537 89 us against 141)
        loose = (_tuning.get('unaligned_vectors') and _tuning.get('scan_cols_unaligned')
                 and src.data.ptr != dst.data.ptr and inner >= 128)

        def threads_with(vec_bytes):
            # (vectors need the alignment of an element only, and a row that
            # is no whole number of them ends with one that overlaps its
            # neighbour)
            v = max(1, vec_bytes // item)
            while v > 1 and (v > inner or (not loose and (
                    not _aligned(src.data.ptr, v * in_dtype.itemsize)
                    or not _aligned(dst.data.ptr, v * out_dtype.itemsize)
                    or inner % v))):
                v //= 2
            return v, outer * ((inner + v - 1) // v)
        forced = _tuning.get('scan_cols_vec_bytes')
        per_cu = _tuning.get('scan_cols_threads_per_cu')
        one_pass_trips = 0
        if forced:
            vec, threads = threads_with(forced)
        else:
            for vec_bytes, need, rows in ((16, 2 * per_cu, 32), (8, 2 * per_cu, 32),
                                          (max(4, min(item, 8)), per_cu, 64)):
                if vec_bytes < item and vec_bytes != 16:
                    continue
                vec, threads = threads_with(vec_bytes)
                # (8-byte vectors from three quarters of that on: 2^26 floats
                # in slices of 257 x 100, 130550 threads, 167 us against 204
                # element-wide)
                if threads >= cus * need * (0.75 if vec_bytes == 8 else 1):
                    one_pass_trips = rows
                    break
            else:
                vec, threads = threads_with(16)
        want = cus * per_cu
        n_chunks = 1
        if may_chunk and not one_pass_trips and threads < want and n >= 128:
            n_chunks = min((want + threads - 1) // threads, n // 64)
        # (slices with too few columns for wide vectors and rows that start off
        # the vectors' grid: the tiles of the one-pass kernel, with their
        # overlapping vectors, do better than a thread per column with single
        # elements; 257 slices of 511 x 509 float32: 232 -> 137 us, 64 of
        # 1024 x 1025: 160 -> 151.  With aligned rows the thread per column
        # wins: 128 slices of 512 x 1024 87 against 106)
        narrow_one_pass = (one_pass_trips == 64 and not forced and inner >= 128 and n >= 256
                           and outer >= 2 and (inner * item) % 16 != 0
                           and _tuning.get('scan_chain_cols_short'))
        if (n_chunks > 1 or narrow_one_pass) and _scan_chained_cols(
                src, dst, outer, n, inner, op, skip_nan, idx64, stream, stream_ptr):
            return
        chunk_len = (n + n_chunks - 1) // n_chunks
        n_chunks = (n + chunk_len - 1) // chunk_len
        trips = _tuning.get('scan_cols_trips')
        if not trips:
            if n_chunks > 1:
                trips = 8
            else:
                trips = one_pass_trips or 32
                while trips > 4 and trips > n:
                    trips //= 2
        mod = _module(in_dtype, out_dtype, op, skip_nan, vec, trips, idx64, 64, stream,
                      reuse=n_chunks > 1 and reuse_ok)
        work = threads * n_chunks
        grid = max(1, min((work + _BLOCK - 1) // _BLOCK, cus * 2 * _tuning.get('scan_blocks_per_cu')))
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
    skip_nan = skip_nan and src.dtype.kind in 'fc'
    if (op == _SUM and not skip_nan and src.dtype == numpy.complex128 and n >= 1024
            and src.dtype == result.dtype and _tuning.get('scan_complex_as_real')):
        # Sums of complex numbers are sums of their parts: long scans of
        # complex128 go over the array as a real one with twice the columns
        # (the same additions in the same order).  Values of 16 bytes leave the
        # one-pass kernels at 35-50 % of peak: 2^24 in one dimension 190 us, as
        # 2^24 x 2 doubles 118; 8192 rows of 2048 113-129 -> 101; 2^22 x 4 along
        # axis 0 136 -> 106.  (Short rows and complex64 are as fast or faster
        # as they are: 2^21 rows of 16 complex64 86 us, as 16 x 2 floats more.)
        part = numpy.dtype('float64')
        _scan_contiguous(src.reshape(-1).view(part), result.reshape(-1).view(part), outer, n,
                         inner * 2, op, False, stream_ptr)
    else:
        _scan_contiguous(src, result, outer, n, inner, op, skip_nan, stream_ptr)
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
