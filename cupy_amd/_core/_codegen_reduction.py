"""HIP source emitters for reduction kernels (gfx950, wave64).

A reduction is stated as in the reference (cupy/_core/_reduction.pyx:44-126):
``pre_map_expr`` over the input element(s), ``reduce_expr`` over ``a`` and
``b`` of type ``_type_reduce``, ``post_map_expr`` storing the final value, an
``identity``, and ``_J`` = position of the element along the reduced axes.
Where the reference has one template (strided per-thread accumulation followed
by an LDS tree with a barrier per level, one launch geometry formula), this
module has four kernels, chosen by the host from the canonical 2-d form
``in[i, j]`` (i = output index, j = reduce index) of the problem:

``rows``     the reduce axis is contiguous in memory.  A group of G lanes
             (G = 1..64, or a whole 256-thread workgroup) owns a row, reads it
             with 128-bit loads into per-lane accumulators and combines them
             with wave64 cross-lane exchanges -- no LDS and no barrier unless a
             workgroup shares the row.  Long rows with few outputs are split
             across workgroups (grid.y) into partial results.
``cols``     the output axis is contiguous (e.g. ``axis=0`` of a C-order
             matrix).  Threads own ``V`` adjacent output columns and walk down
             the reduce axis, TY row-slices per workgroup and grid.y slices per
             launch; slices are combined through cross-lane exchanges, LDS and,
             across workgroups, a partial-result buffer.  The same kernel
             takes a batch of such problems (reduction over a middle axis:
             ``in[b, j, c]`` to ``out[b, c]``).
``rows_flat`` short rows of odd length stored without gaps: a workgroup
             copies a run of whole rows into the LDS with full vector loads
             and lane groups reduce the rows from there.
``generic``  any strides: CIndexer addressing, same thread layout as ``cols``.

Partial results are combined by a second ``cols`` launch that reads
``_type_reduce`` values (``partial_in``) -- deterministic, no atomics.
"""
import re

BLOCK = 256
WAVE = 64


class RArg:
    """Kernel parameter of a reduction.

    kind     'in' (iterated input array), 'out' (output array), 'raw' (CArray
             passed through), 'scalar'
    name     identifier used by the expressions
    store_t  element type in memory / scalar type
    var_t    type of the variable the expressions see
    bcast_r  'in' only: the array does not vary along the reduce axis
    bcast_o  'in' only: the array does not vary along the output axis
    """

    def __init__(self, kind, name, store_t, var_t=None, is_const=True, ndim=0,
                 c_contiguous=False, index_32=True, bcast_r=False, bcast_o=False):
        self.kind = kind
        self.name = name
        self.store_t = store_t
        self.var_t = var_t or store_t
        self.is_const = is_const
        self.ndim = ndim
        self.c_contiguous = c_contiguous
        self.index_32 = index_32
        self.bcast_r = bcast_r
        self.bcast_o = bcast_o

    def key(self):
        return (self.kind, self.name, self.store_t, self.var_t, self.is_const,
                self.ndim, self.c_contiguous, self.index_32, self.bcast_r,
                self.bcast_o)


def _prologue(typedefs, preamble, reduce_type, reduce_expr, post_map_expr):
    return '''#include <cupy/carray.cuh>
%s
%s
#define REDUCE(a, b) (%s)
#define POST_MAP(a) (%s)
typedef %s _type_reduce;
// lets the host learn sizeof(_type_reduce) (size of this variable) when it has
// to allocate a buffer of partial results
__device__ __attribute__((used)) char _cupy_type_reduce_probe[sizeof(_type_reduce)];
struct _ReduceOp {
  __device__ __forceinline__ _type_reduce operator()(
      const _type_reduce& a, const _type_reduce& b) const {
    return REDUCE(a, b);
  }
};
''' % (typedefs, preamble, reduce_expr, post_map_expr, reduce_type)


# Finishing a split reduction inside the launch that produced the partial
# results.  Every workgroup publishes its partial result(s) in slots of 64 bits:
# a 32-bit word of the value beside the number of the launch (``epoch``), one
# relaxed device-scope store each, so that neither side needs a fence.  The
# workgroup of a column block (or row) that starts last -- the one with the
# highest number, workgroups start in the order of their numbers -- waits for
# the slots of the others, combines them in the order of their numbers and
# stores the result(s).  The number of the launch is kept in the memory the
# slots live in (word 0): every workgroup reads it at its start, and the very
# last workgroup of the grid advances it once every other finishing workgroup
# has reported (each reports after it has seen the partial results of all its
# workgroups, which therefore have all read the number).  Launches that share
# the memory must not overlap: the host keeps one such memory per stream.
# Every wait is bounded by ``_spin_limit`` polls; a workgroup that gives up
# says so in ``_fault`` and runs to its end all the same.
_SYNC_HELPERS = r"""
typedef unsigned long long _slot_t;
constexpr int _kWords = (sizeof(_type_reduce) + 3) / 4;
#define _SYNC_HEADER_WORDS 64
#define _SYNC_AHEAD %(ahead)d

// (the value by value: taken by reference, structures of four doubles went
// through the stack)
__device__ __forceinline__ void _sync_publish(_slot_t* slots, const ptrdiff_t i,
                                              const _type_reduce v, const unsigned epoch) {
  unsigned w[_kWords];
#pragma unroll
  for (int k = 0; k < _kWords; ++k) w[k] = 0u;
  __builtin_memcpy(w, &v, sizeof(_type_reduce));
#pragma unroll
  for (int k = 0; k < _kWords; ++k)
    __hip_atomic_store(slots + i * _kWords + k, ((_slot_t)epoch << 32) | w[k], __ATOMIC_RELAXED,
                       __HIP_MEMORY_SCOPE_AGENT);
}

// The values first, first + stride, ... (`count` of them), waited for and
// combined in that order onto `acc`.  Asks for _SYNC_AHEAD values at a time.
// Returns false if it gave up.
__device__ __forceinline__ bool _sync_fold(_slot_t* slots, const ptrdiff_t first,
                                           const ptrdiff_t stride, const int count,
                                           const unsigned epoch, const unsigned spin_limit,
                                           _type_reduce& acc) {
  int i = 0;
  unsigned spins = 0;
  while (i < count) {
    _slot_t x[_SYNC_AHEAD][_kWords];
#pragma unroll
    for (int a = 0; a < _SYNC_AHEAD; ++a) {
      // (past the last value: the last one again, not used)
      const int ia = (i + a < count) ? i + a : count - 1;
#pragma unroll
      for (int k = 0; k < _kWords; ++k)
        x[a][k] = __hip_atomic_load(slots + (first + (ptrdiff_t)ia * stride) * _kWords + k,
                                    __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    // (no early exit from the loop: it unrolls whole, and `x` stays in registers)
    bool stalled = false;
#pragma unroll
    for (int a = 0; a < _SYNC_AHEAD; ++a) {
      bool written = true;
      unsigned w[_kWords];
#pragma unroll
      for (int k = 0; k < _kWords; ++k) {
        written = written && (unsigned)(x[a][k] >> 32) == epoch;
        w[k] = (unsigned)x[a][k];
      }
      const bool due = !stalled && i < count;
      if (due && written) {
        _type_reduce v;
        __builtin_memcpy(&v, w, sizeof(_type_reduce));
        acc = REDUCE(acc, v);
        ++i;
      }
      stalled = stalled || (due && !written);
    }
    if (stalled) {
      if (spins >= spin_limit) return false;
      ++spins;
      __builtin_amdgcn_s_sleep(8);
    }
  }
  return true;
}

// Number of this launch, read by the first wave of every workgroup at its start.
__device__ __forceinline__ unsigned _sync_epoch(unsigned* sync) {
  return __hip_atomic_load(sync, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) + 1u;
}

// The finishing workgroup `x` of `n_finishers` reports; the last one waits
// for the reports of the others and advances the number of the launch.  One
// wave, all lanes call.  `done` are the slots after those of the partial
// results.
__device__ __forceinline__ void _sync_report(unsigned* sync, _slot_t* done, const ptrdiff_t x,
                                             const ptrdiff_t n_finishers, const unsigned epoch,
                                             const unsigned spin_limit, unsigned* fault,
                                             const ptrdiff_t all_slots) {
  const int lane = threadIdx.x & 63;
  if (lane == 0)
    __hip_atomic_store(done + x, ((_slot_t)epoch << 32), __ATOMIC_RELAXED,
                       __HIP_MEMORY_SCOPE_AGENT);
  if (x != n_finishers - 1) return;
  bool ok = true;
  unsigned spins = 0;
  for (ptrdiff_t i = lane; i < n_finishers - 1; i += 64) {
    for (;;) {
      const _slot_t v = __hip_atomic_load(done + i, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      if ((unsigned)(v >> 32) == epoch) break;
      if (spins >= spin_limit) { ok = false; break; }
      ++spins;
      __builtin_amdgcn_s_sleep(8);
    }
    if (!ok) break;
  }
  const bool all_ok = __ballot(!ok) == 0;
  if (!all_ok && lane == 0 && fault) *reinterpret_cast<volatile unsigned*>(fault) = 1u;
  unsigned next = epoch;
  if (epoch == 0xffffffffu) {
    // the numbers start over: nothing may be left that carries an old one
    _slot_t* slots = reinterpret_cast<_slot_t*>(sync + _SYNC_HEADER_WORDS);
    for (ptrdiff_t i = lane; i < all_slots; i += 64)
      __hip_atomic_store(slots + i, (_slot_t)0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    next = 0u;
  }
  if (lane == 0)
    __hip_atomic_store(sync, next, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
"""


def _sync_helpers(reduce_words_hint=2):
    # values a lane asks for at a time: what fits the registers beside the rest
    return _SYNC_HELPERS % dict(ahead=8 if reduce_words_hint <= 2 else 4)


def _raw_param(a):
    const = 'const ' if a.is_const else ''
    return '%sCArray<%s, %d, %d, %d> %s' % (
        const, a.store_t, a.ndim, a.c_contiguous, a.index_32, a.name)


def _fast_params(args, idx_t, partial_in, partial_out, finish=False):
    """Parameter list of the rows / cols kernels."""
    parts = []
    for a in args:
        if a.kind == 'in':
            if partial_in:
                parts.append('const _type_reduce* __restrict__ _p_%s' % a.name)
            else:
                parts.append('const %s* __restrict__ _p_%s' % (a.store_t, a.name))
        elif a.kind == 'out':
            parts.append('%s* __restrict__ _p_%s' % (a.store_t, a.name))
        elif a.kind == 'raw':
            parts.append(_raw_param(a))
        else:
            parts.append('const %s %s' % (a.store_t, a.name))
    parts.append('const %s _n_out' % idx_t)
    parts.append('const %s _n_red' % idx_t)
    parts.append('const long long _in_total')     # element count of the whole problem
    for a in args:
        if a.kind == 'in':
            parts.append('const %s _so_%s' % (idx_t, a.name))   # stride along i
            parts.append('const %s _sr_%s' % (idx_t, a.name))   # stride along j
        elif a.kind == 'out':
            parts.append('const %s _so_%s' % (idx_t, a.name))
    if partial_out and finish:
        # memory of the slots (see _SYNC_HELPERS), workgroups along the outputs
        parts.append('unsigned* _sync')
        parts.append('const unsigned _spin_limit')
        parts.append('unsigned* _fault')
        parts.append('const %s _gx' % idx_t)
    elif partial_out:
        parts.append('_type_reduce* __restrict__ _partials')
    return ', '.join(parts)


_SIZE_INDEXERS = ('  const SizeOnly _in_ind((ptrdiff_t)_in_total); '
                  'const SizeOnly _out_ind((ptrdiff_t)_n_out); (void)_in_ind; (void)_out_ind;')


def _identity_decl(identity):
    return '_type_reduce(%s)' % identity


def _finish(args, partial_out, pad, i_expr='_i', s_expr='_s', split_expr='blockIdx.y'):
    """Code storing one finished value: either into the partial buffer or
    through POST_MAP into the output element(s)."""
    lines = []
    if partial_out == 'publish':
        lines.append('%s_sync_publish(_slots, (ptrdiff_t)%s * _n_out + %s, %s, _epoch);' % (
            pad, split_expr, i_expr, s_expr))
    elif partial_out:
        lines.append('%s_partials[(ptrdiff_t)%s * _n_out + %s] = %s;' % (
            pad, split_expr, i_expr, s_expr))
    else:
        for a in args:
            if a.kind == 'out':
                lines.append('%s%s &%s = _p_%s[(ptrdiff_t)%s * _so_%s];' % (
                    pad, a.var_t, a.name, a.name, i_expr, a.name))
        lines.append('%sPOST_MAP(%s);' % (pad, s_expr))
    return lines


def emit_rows(name, args, identity, pre_map_expr, reduce_expr, post_map_expr,
              reduce_type, typedefs='', preamble='', group=64, vec=4,
              idx64=False, partial_out=False, stream_hint=False, unroll=2, block=BLOCK,
              finish=False, reduce_words=2):
    """Reduce-axis-contiguous kernel.  ``group`` lanes per row (power of two up
    to 64) or ``BLOCK`` for a workgroup (of ``block`` threads) per row.  With ``partial_out`` the reduce
    range is cut into gridDim.y chunks of ``_chunk`` elements (an extra kernel
    parameter) and each (chunk, row) writes one ``_type_reduce`` partial."""
    idx_t = 'ptrdiff_t' if idx64 else 'int'
    nt = 'true' if stream_hint else 'false'
    ins = [a for a in args if a.kind == 'in']
    finish = bool(finish and partial_out and group >= BLOCK)
    params = _fast_params(args, idx_t, False, partial_out, finish)
    if partial_out:
        params += ', const %s _chunk' % idx_t
    block_mode = group >= BLOCK
    wg = block if block_mode else BLOCK
    lanes = wg if block_mode else group
    src = [_prologue(typedefs, preamble, reduce_type, reduce_expr, post_map_expr)]
    if finish:
        src.append(_sync_helpers(reduce_words))
    src.append('extern "C" __global__ void __launch_bounds__(%d) %s(%s) {' % (
        wg, name, params))
    src.append(_SIZE_INDEXERS)
    split_of_block = 'blockIdx.y'
    if finish:
        # a grid of one dimension, numbered along the outputs first: the
        # workgroups of one output start in the order of their chunks
        src.append('  const %s _bx = (%s)(blockIdx.x %% (unsigned)_gx);' % (idx_t, idx_t))
        src.append('  const %s _by = (%s)(blockIdx.x / (unsigned)_gx);' % (idx_t, idx_t))
        src.append('  const %s _gy = (%s)(gridDim.x / (unsigned)_gx);' % (idx_t, idx_t))
        src.append('  _slot_t* _slots = reinterpret_cast<_slot_t*>(_sync + _SYNC_HEADER_WORDS);')
        # (asked for now, needed when the partial result is there: the first
        # wave alone uses it)
        src.append('  unsigned _epoch = 0u;')
        src.append('  if (threadIdx.x < %d) _epoch = _sync_epoch(_sync);' % WAVE)
        split_of_block = '_by'
    if block_mode:
        src.append('  __shared__ __attribute__((aligned(16))) char _sm_raw[%d * sizeof(_type_reduce)];' % (wg // WAVE))
        src.append('  _type_reduce* _sm = reinterpret_cast<_type_reduce*>(_sm_raw);')
        src.append('  const int _lane = threadIdx.x;')
        if finish:
            src.append('  const %s _first = _bx;' % idx_t)
            src.append('  const %s _step = _gx;' % idx_t)
        else:
            src.append('  const %s _first = blockIdx.x;' % idx_t)
            src.append('  const %s _step = gridDim.x;' % idx_t)
    else:
        src.append('  const int _lane = threadIdx.x %% %d;' % group)
        src.append('  const %s _first = ((%s)blockIdx.x * %d + threadIdx.x) / %d;' % (
            idx_t, idx_t, BLOCK, group))
        src.append('  const %s _step = (%s)gridDim.x * %d;' % (idx_t, idx_t, BLOCK // group))
    if partial_out:
        src.append('  const %s _j_begin = (%s)%s * _chunk;' % (idx_t, idx_t, split_of_block))
        src.append('  const %s _j_end = (_j_begin + _chunk < _n_red) ? (_j_begin + _chunk) : _n_red;' % idx_t)
    else:
        src.append('  const %s _j_begin = 0;' % idx_t)
        src.append('  const %s _j_end = _n_red;' % idx_t)
    # inputs that do not vary along the output axis keep the same per-lane
    # elements for every row when the row fits one trip: hoisting is left to
    # the compiler (the loads are loop-invariant and the pointers const).
    src.append('  for (%s _i = _first; _i < _n_out; _i += _step) {' % idx_t)
    for a in ins:
        src.append('    const %s* _row_%s = _p_%s + (ptrdiff_t)_i * _so_%s;' % (
            a.store_t, a.name, a.name, a.name))
    src.append('    _type_reduce _acc[%d];' % vec)
    src.append('#pragma unroll')
    src.append('    for (int _k = 0; _k < %d; ++_k) _acc[_k] = %s;' % (
        vec, _identity_decl(identity)))
    # (items that are a whole vector by themselves, or arrays aligned for no
    # more than one item, take the same loop: it is the one that keeps several
    # loads in flight per lane and marks them as streaming)
    preload = vec > 1
    if vec > 1 or unroll > 1:
        src.append('    const %s _j_vend = _j_begin + (_j_end - _j_begin) / %d * %d;' % (
            idx_t, vec, vec))
        if preload:
            # the elements after the last whole vector: a lane's first one,
            # asked for now (from a valid address whatever the lane)
            src.append('    const %s _jt = _j_vend + _lane;' % idx_t)
            src.append('    const bool _tail = _jt < _j_end;')
            for a in ins:
                if not a.bcast_r:
                    src.append('    const %s _t_%s = _row_%s[_tail ? _jt : _j_begin];' % (
                        a.store_t, a.name, a.name))
        stride = lanes * vec

        def loads(pad, j_expr, suffix):
            for a in ins:
                if a.bcast_r:
                    src.append('%sconst %s _b_%s%s = _row_%s[0];' % (
                        pad, a.store_t, a.name, suffix, a.name))
                else:
                    src.append('%sconst cupy::Vec<%s, %d> _l_%s%s = cupy::load_vec<%s, %d, %s>('
                               '_row_%s + (%s));' % (pad, a.store_t, vec, a.name, suffix,
                                                     a.store_t, vec, nt, a.name, j_expr))

        def accumulate(pad, j_expr, suffix):
            src.append('#pragma unroll')
            src.append('%sfor (int _k = 0; _k < %d; ++_k) {' % (pad, vec))
            src.append('%s  const IndexT _J = (%s) + _k;' % (pad, j_expr))
            for a in ins:
                val = ('_b_%s%s' % (a.name, suffix)) if a.bcast_r else (
                    '_l_%s%s.v[_k]' % (a.name, suffix))
                src.append('%s  const %s %s(%s);' % (pad, a.var_t, a.name, val))
            src.append('%s  _type_reduce _a = static_cast<_type_reduce>(%s);' % (
                pad, pre_map_expr))
            src.append('%s  _acc[_k] = REDUCE(_acc[_k], _a);' % pad)
            src.append('%s}' % pad)

        def masked_loads(pad, u, suffix):
            # a lane whose vector would lie past the whole vectors of the row
            # asks for the row's first one instead and does not use it
            src.append('%sconst bool _ok%s = _j + %d < _j_vend;' % (pad, suffix, u * stride))
            for a in ins:
                if a.bcast_r:
                    src.append('%sconst %s _b_%s%s = _row_%s[0];' % (
                        pad, a.store_t, a.name, suffix, a.name))
                else:
                    src.append('%sconst cupy::Vec<%s, %d> _l_%s%s = cupy::load_vec<%s, %d, %s>('
                               '_row_%s + (_ok%s ? _j + %d : _j_begin));' % (
                                   pad, a.store_t, vec, a.name, suffix, a.store_t, vec, nt,
                                   a.name, suffix, u * stride))

        def masked_block(pad, count, tag):
            for u in range(count):
                masked_loads(pad, u, '_%s%d' % (tag, u))
            for u in range(count):
                src.append('%sif (_ok_%s%d) {' % (pad, tag, u))
                accumulate(pad + '  ', '_j + %d' % (u * stride), '_%s%d' % (tag, u))
                src.append('%s}' % pad)

        # `_j0` is the position of lane 0 (the same for all lanes of the row:
        # every test on it is one the whole group agrees on)
        src.append('    %s _j0 = _j_begin;' % idx_t)
        src.append('    %s _j = _j_begin + _lane * %d;' % (idx_t, vec))
        if unroll > 1:
            # `unroll` vectors per lane and trip, every load issued before the
            # first value is used; these trips are whole for every lane
            src.append('    for (; _j0 + %d <= _j_vend; _j0 += %d, _j += %d) {' % (
                unroll * stride, unroll * stride, unroll * stride))
            for u in range(unroll):
                loads('      ', '_j + %d' % (u * stride), '_%d' % u)
            for u in range(unroll):
                accumulate('      ', '_j + %d' % (u * stride), '_%d' % u)
            src.append('    }')
            # What is left -- fewer trips than that, the last of them whole for
            # some lanes only -- is asked for in one go as well: every lane
            # takes part, the ones without a vector ask for the start of the
            # row and leave it unused.  (Left to a loop of its own, the lanes
            # that run out first make the group walk both paths one after the
            # other, and the last loads wait for everything before them: rows
            # of 1023 float32, a wave per row, variance 61 us against 46 for
            # rows of 1024.)  Two trips where two suffice.
            src.append('    if (_j0 < _j_vend) {')
            if unroll > 2:
                src.append('      if (_j0 + %d < _j_vend) {' % (2 * stride))
                masked_block('        ', unroll, 'm')
                src.append('      } else {')
                masked_block('        ', 2, 'n')
                src.append('      }')
            else:
                masked_block('      ', unroll, 'm')
            src.append('    }')
        else:
            src.append('    for (; _j < _j_vend; _j += %d) {' % stride)
            loads('      ', '_j', '')
            accumulate('      ', '_j', '')
            src.append('    }')
    else:
        src.append('    const %s _j_vend = _j_begin;' % idx_t)
    # ragged tail (and the whole row when vec == 1).  Its first element per
    # lane -- all of it, unless the row has fewer lanes than a vector has
    # elements -- was requested before the vector loop (see `preload`), so that
    # it does not cost a round trip of its own after the loop.
    if preload:
        src.append('    if (_tail) {')
        src.append('      const IndexT _J = _jt;')
        for a in ins:
            val = ('_row_%s[0]' % a.name) if a.bcast_r else ('_t_%s' % a.name)
            src.append('      const %s %s(%s);' % (a.var_t, a.name, val))
        src.append('      _type_reduce _a = static_cast<_type_reduce>(%s);' % pre_map_expr)
        src.append('      _acc[0] = REDUCE(_acc[0], _a);')
        src.append('    }')
    src.append('    for (%s _j = _j_vend + _lane%s; _j < _j_end; _j += %d) {' % (
        idx_t, (' + %d' % lanes) if preload else '', lanes))
    src.append('      const IndexT _J = _j;')
    for a in ins:
        val = ('_row_%s[0]' % a.name) if a.bcast_r else ('_row_%s[_j]' % a.name)
        src.append('      const %s %s(%s);' % (a.var_t, a.name, val))
    src.append('      _type_reduce _a = static_cast<_type_reduce>(%s);' % pre_map_expr)
    src.append('      _acc[0] = REDUCE(_acc[0], _a);')
    src.append('    }')
    src.append('    _type_reduce _s = _acc[0];')
    if vec > 1:
        src.append('#pragma unroll')
        src.append('    for (int _k = 1; _k < %d; ++_k) _s = REDUCE(_s, _acc[_k]);' % vec)
    if block_mode:
        src.append('    _s = cupy::group_allreduce<%d>(_s, _ReduceOp());' % WAVE)
        src.append('    if ((threadIdx.x %% %d) == 0) _sm[threadIdx.x / %d] = _s;' % (WAVE, WAVE))
        src.append('    __syncthreads();')
        src.append('    if (threadIdx.x == 0) {')
        src.append('      _s = _sm[0];')
        src.append('      for (int _w = 1; _w < %d; ++_w) _s = REDUCE(_s, _sm[_w]);' % (wg // WAVE))
        src.extend(_finish(args, 'publish' if finish else partial_out, '      ',
                           split_expr=split_of_block))
        src.append('    }')
        src.append('    __syncthreads();')
        if finish:
            # the workgroup of the last chunk of output _i finishes it: the
            # partial results of the chunks, a lane taking every 64th, then
            # across the lanes
            src.append('    if (_by == _gy - 1 && threadIdx.x < %d) {' % WAVE)
            src.append('      _type_reduce _t = %s;' % _identity_decl(identity))
            src.append('      const int _mine = (int)((_gy - threadIdx.x + %d) / %d);' % (WAVE - 1, WAVE))
            src.append('      const bool _ok = _sync_fold(_slots, (ptrdiff_t)threadIdx.x * _n_out + _i, '
                       '(ptrdiff_t)%d * _n_out, _mine, _epoch, _spin_limit, _t);' % WAVE)
            src.append('      if (__ballot(!_ok) != 0 && threadIdx.x == 0 && _fault) '
                       '*reinterpret_cast<volatile unsigned*>(_fault) = 1u;')
            # (lanes without a chunk hold the identity, as lanes without
            # elements do in the reduction proper)
            src.append('      _type_reduce _s = cupy::group_allreduce<%d>(_t, _ReduceOp());' % WAVE)
            src.append('      if (threadIdx.x == 0) {')
            src.extend(_finish(args, False, '        '))
            src.append('      }')
            src.append('      _sync_report(_sync, _slots + (ptrdiff_t)_gy * _n_out * _kWords, _i, _n_out, '
                       '_epoch, _spin_limit, _fault, (ptrdiff_t)_gy * _n_out * _kWords + _n_out);')
            src.append('    }')
    else:
        if group > 1:
            src.append('    _s = cupy::group_allreduce<%d>(_s, _ReduceOp());' % group)
        src.append('    if (_lane == 0) {')
        src.extend(_finish(args, partial_out, '      '))
        src.append('    }')
    src.append('  }')
    src.append('}')
    return '\n'.join(src) + '\n'


def emit_rows_batched(name, args, identity, pre_map_expr, reduce_expr, post_map_expr,
                      reduce_type, typedefs='', preamble='', group=32, vec=4, trips=1,
                      batch=4, idx64=False, stream_hint=False, exact=False):
    """Reduce-axis-contiguous kernel for short rows: a group of ``group`` lanes
    (power of two <= 64) covers a whole row in ``trips`` vector loads per lane
    (``n_red <= group * vec * trips``; ``exact``: equal).  To keep enough bytes
    in flight per wave, each group works on ``batch`` rows at a time: all their
    loads are issued first, then the ``batch`` independent cross-lane
    butterflies run interleaved.  Fewer lanes per row with more trips per lane
    trade cross-lane steps for in-lane accumulation.  Inputs that do not vary
    along the output axis (``bcast_o``) are loaded once, before the row loop.

    Every vector load is unconditional: a load under a branch makes the
    compiler wait for it at the end of the branch, one load at a time.  Lanes
    past the end of a row (or rows past the last one) load from a position that
    is known to be valid instead, and their values are left out of the
    accumulation by a select."""
    idx_t = 'ptrdiff_t' if idx64 else 'int'
    nt = 'true' if stream_hint else 'false'
    ins = [a for a in args if a.kind == 'in']
    params = _fast_params(args, idx_t, False, False)
    src = [_prologue(typedefs, preamble, reduce_type, reduce_expr, post_map_expr)]
    src.append('extern "C" __global__ void __launch_bounds__(%d) %s(%s) {' % (
        BLOCK, name, params))
    src.append(_SIZE_INDEXERS)
    src.append('  const int _lane = threadIdx.x %% %d;' % group)
    src.append('  const %s _first = ((%s)blockIdx.x * %d + threadIdx.x) / %d;' % (
        idx_t, idx_t, BLOCK, group))
    src.append('  const %s _step = (%s)gridDim.x * %d;' % (idx_t, idx_t, BLOCK // group))
    # trip t of this lane covers elements [_JV(t), _JV(t) + vec)
    src.append('#define _JV(t) ((%s)((t) * %d + _lane) * %d)' % (idx_t, group, vec))
    if exact:
        src.append('#define _JOK(t) true')
        src.append('#define _JC(t) _JV(t)')
    else:
        src.append('  const %s _j_vend = _n_red / %d * %d;' % (idx_t, vec, vec))
        src.append('#define _JOK(t) (_JV(t) < _j_vend)')
        # position 0 always holds a whole vector (the host guarantees n_red >= vec)
        src.append('#define _JC(t) (_JOK(t) ? _JV(t) : (%s)0)' % idx_t)
    for a in ins:
        if a.bcast_o and not a.bcast_r:
            src.append('  cupy::Vec<%s, %d> _h_%s[%d];' % (a.store_t, vec, a.name, trips))
            src.append('#pragma unroll')
            src.append('  for (int _t = 0; _t < %d; ++_t) '
                       '_h_%s[_t] = cupy::load_vec<%s, %d, false>(_p_%s + _JC(_t));' % (
                           trips, a.name, a.store_t, vec, a.name))
    src.append('  for (%s _i0 = _first; _i0 < _n_out; _i0 += _step * %d) {' % (idx_t, batch))
    for a in ins:
        if not a.bcast_o and not a.bcast_r:
            src.append('    cupy::Vec<%s, %d> _l_%s[%d][%d];' % (
                a.store_t, vec, a.name, batch, trips))
    src.append('#pragma unroll')
    src.append('    for (int _r = 0; _r < %d; ++_r) {' % batch)
    if batch > 1:
        # rows past the end re-read row _i0; their results are dropped below
        src.append('      const %s _i = (_i0 + _r * _step < _n_out) ? _i0 + _r * _step : _i0;'
                   % idx_t)
    else:
        src.append('      const %s _i = _i0;' % idx_t)
    src.append('#pragma unroll')
    src.append('      for (int _t = 0; _t < %d; ++_t) {' % trips)
    for a in ins:
        if not a.bcast_o and not a.bcast_r:
            src.append('        _l_%s[_r][_t] = cupy::load_vec<%s, %d, %s>('
                       '_p_%s + (ptrdiff_t)_i * _so_%s + _JC(_t));' % (
                           a.name, a.store_t, vec, nt, a.name, a.name))
    src.append('      }')
    src.append('    }')
    src.append('    _type_reduce _s[%d];' % batch)
    src.append('#pragma unroll')
    src.append('    for (int _r = 0; _r < %d; ++_r) {' % batch)
    if batch > 1:
        src.append('      const %s _i = (_i0 + _r * _step < _n_out) ? _i0 + _r * _step : _i0;'
                   % idx_t)
    else:
        src.append('      const %s _i = _i0;' % idx_t)
    src.append('      _type_reduce _acc = %s;' % _identity_decl(identity))
    src.append('#pragma unroll')
    src.append('      for (int _t = 0; _t < %d; ++_t) {' % trips)
    src.append('#pragma unroll')
    src.append('        for (int _k = 0; _k < %d; ++_k) {' % vec)
    src.append('          const IndexT _J = _JV(_t) + _k;')
    for a in ins:
        if a.bcast_r:
            val = '_p_%s[(ptrdiff_t)_i * _so_%s]' % (a.name, a.name)
        elif a.bcast_o:
            val = '_h_%s[_t].v[_k]' % a.name
        else:
            val = '_l_%s[_r][_t].v[_k]' % a.name
        src.append('          const %s %s(%s);' % (a.var_t, a.name, val))
    src.append('          _type_reduce _a = static_cast<_type_reduce>(%s);' % pre_map_expr)
    if exact:
        src.append('          _acc = REDUCE(_acc, _a);')
    else:
        src.append('          const _type_reduce _n = REDUCE(_acc, _a);')
        src.append('          _acc = cupy::select_value(_JOK(_t), _n, _acc);')
    src.append('        }')
    src.append('      }')
    if not exact:
        src.append('      for (%s _jt = _j_vend + _lane; _jt < _n_red; _jt += %d) {' % (
            idx_t, group))
        src.append('        const IndexT _J = _jt;')
        for a in ins:
            if a.bcast_r:
                val = '_p_%s[(ptrdiff_t)_i * _so_%s]' % (a.name, a.name)
            else:
                val = '_p_%s[(ptrdiff_t)_i * _so_%s + _jt]' % (a.name, a.name)
            src.append('        const %s %s(%s);' % (a.var_t, a.name, val))
        src.append('        _type_reduce _a = static_cast<_type_reduce>(%s);' % pre_map_expr)
        src.append('        _acc = REDUCE(_acc, _a);')
        src.append('      }')
    src.append('      _s[_r] = _acc;')
    src.append('    }')
    if group > 1:
        # the steps of the `batch` independent all-reduces side by side
        src.append('    cupy::batch_allreduce<%d>(_s, _ReduceOp());' % group)
    src.append('#pragma unroll')
    src.append('    for (int _r = 0; _r < %d; ++_r) {' % batch)
    src.append('      const %s _i = _i0 + _r * _step;' % idx_t)
    src.append('      if (_lane == 0 && _i < _n_out) {')
    src.extend(_finish(args, False, '        ', s_expr='_s[_r]'))
    src.append('      }')
    src.append('    }')
    src.append('  }')
    src.append('#undef _JV')
    src.append('#undef _JOK')
    src.append('#undef _JC')
    src.append('}')
    return '\n'.join(src) + '\n'


def emit_rows_flat(name, args, identity, pre_map_expr, reduce_expr, post_map_expr,
                   reduce_type, typedefs='', preamble='', width=3, group=1, rows=256,
                   stream_hint=False, inner=1):
    """Reduce-axis-contiguous kernel for short rows of ``width`` elements (a
    compile-time constant) that follow one another without gaps and whose
    length in bytes is not a multiple of a vector: a lane group per row would
    either leave lanes idle or load element by element.  A workgroup instead
    copies ``rows`` consecutive rows -- one contiguous run of memory -- into
    the LDS with full 16-byte loads on consecutive lanes, and then ``group``
    lanes per row (a power of two) read the row back from the LDS and reduce
    it.  Row r starts its walk ``r * group`` elements into the row (and wraps
    around), so that the lanes of a wave are spread over the LDS banks for
    even widths too.

    Every input must have element strides (width, 1), or (0, 1): one row that
    all outputs share (``bcast_o``), or a value per row (``bcast_r``), both
    read in place.  Same parameters as the rows kernel.

    ``inner`` > 1: a row is a slice of ``width / inner`` lines of ``inner``
    columns each, reduced down its columns (the reduction over the middle axis
    of (slices, lines, columns) with few columns): ``group`` lanes per slice
    and column, ``inner`` results per slice stored next to one another;
    ``_n_out`` counts the results.  Plain inputs only."""
    all_ins = [a for a in args if a.kind == 'in']
    ins = [a for a in all_ins if not (a.bcast_o or a.bcast_r)]
    assert ins and group in (1, 2, 4, 8, 16, 32, 64)
    assert inner == 1 and rows % (BLOCK // group) == 0 or (
        inner > 1 and width % inner == 0 and len(ins) == len(all_ins))
    nt = 'true' if stream_hint else 'false'
    params = _fast_params(args, 'ptrdiff_t', False, False)
    per_pass = BLOCK // group
    src = [_prologue(typedefs, preamble, reduce_type, reduce_expr, post_map_expr)]
    src.append('extern "C" __global__ void __launch_bounds__(%d) %s(%s) {' % (
        BLOCK, name, params))
    src.append(_SIZE_INDEXERS)
    src.append('  const ptrdiff_t _row0 = (ptrdiff_t)blockIdx.x * %d;' % rows)
    src.append('  const ptrdiff_t _n_rows_all = _n_out / %d;' % inner)
    src.append('  const int _nrows = (_n_rows_all - _row0 < %d) ? (int)(_n_rows_all - _row0) : %d;' % (rows, rows))
    src.append('  const int _count = _nrows * %d;' % width)
    vecs = {}
    for a in ins:
        # element size of the stored type is not known here: 16 bytes per lane
        src.append('  constexpr int _V_%s = 16 / sizeof(%s) > 0 ? 16 / sizeof(%s) : 1;' % (
            a.name, a.store_t, a.store_t))
        src.append('  constexpr int _T_%s = (%d + %d * _V_%s - 1) / (%d * _V_%s);' % (
            a.name, rows * width, BLOCK, a.name, BLOCK, a.name))
        src.append('  __shared__ __attribute__((aligned(16))) char _slab_raw_%s[(%d + _V_%s) * sizeof(%s)];' % (
            a.name, rows * width, a.name, a.store_t))
        src.append('  %s* _slab_%s = reinterpret_cast<%s*>(_slab_raw_%s);' % (
            a.store_t, a.name, a.store_t, a.name))
        src.append('  const %s* _src_%s = _p_%s + _row0 * %d;' % (a.store_t, a.name, a.name, width))
        src.append('  cupy::Vec<%s, _V_%s> _st_%s[_T_%s];' % (a.store_t, a.name, a.name, a.name))
    # every load is issued before the first store into the LDS
    for a in ins:
        src.append('#pragma unroll')
        src.append('  for (int _t = 0; _t < _T_%s; ++_t) {' % a.name)
        src.append('    const int _q = (_t * %d + threadIdx.x) * _V_%s;' % (BLOCK, a.name))
        src.append('    if (_q + _V_%s <= _count) _st_%s[_t] = cupy::load_vec<%s, _V_%s, %s>(_src_%s + _q);' % (
            a.name, a.name, a.store_t, a.name, nt, a.name))
        src.append('  }')
    # values per row are requested along with the rows and handed over through
    # the LDS as well: a load after the barrier would be waited for by itself
    row_vals = [a for a in all_ins if a.bcast_r]
    n_rv = (rows + BLOCK - 1) // BLOCK
    for a in row_vals:
        src.append('  __shared__ __attribute__((aligned(16))) char _rowv_raw_%s[%d * sizeof(%s)];' % (
            a.name, rows, a.store_t))
        src.append('  %s* _rowv_%s = reinterpret_cast<%s*>(_rowv_raw_%s);' % (
            a.store_t, a.name, a.store_t, a.name))
        src.append('  %s _rvst_%s[%d];' % (a.store_t, a.name, n_rv))
        src.append('#pragma unroll')
        src.append('  for (int _t = 0; _t < %d; ++_t) {' % n_rv)
        src.append('    const int _rr = _t * %d + threadIdx.x;' % BLOCK)
        src.append('    if (_rr < _nrows) _rvst_%s[_t] = _p_%s[(_row0 + _rr) * _so_%s];' % (
            a.name, a.name, a.name))
        src.append('  }')
    for a in row_vals:
        src.append('#pragma unroll')
        src.append('  for (int _t = 0; _t < %d; ++_t) {' % n_rv)
        src.append('    const int _rr = _t * %d + threadIdx.x;' % BLOCK)
        src.append('    if (_rr < _nrows) _rowv_%s[_rr] = _rvst_%s[_t];' % (a.name, a.name))
        src.append('  }')
    for a in ins:
        src.append('#pragma unroll')
        src.append('  for (int _t = 0; _t < _T_%s; ++_t) {' % a.name)
        src.append('    const int _q = (_t * %d + threadIdx.x) * _V_%s;' % (BLOCK, a.name))
        src.append('    if (_q + _V_%s <= _count) {' % a.name)
        src.append('      *reinterpret_cast<cupy::Vec<%s, _V_%s>*>(_slab_%s + _q) = _st_%s[_t];' % (
            a.store_t, a.name, a.name, a.name))
        src.append('    } else {')
        src.append('      for (int _k = 0; _k < _V_%s; ++_k) if (_q + _k < _count) _slab_%s[_q + _k] = _src_%s[_q + _k];' % (
            a.name, a.name, a.name))
        src.append('    }')
        src.append('  }')
    src.append('  __syncthreads();')
    src.append('  const int _g = threadIdx.x %% %d;' % group)
    if inner > 1:
        lines = width // inner
        src.append('  for (int _it = threadIdx.x / %d; _it < _nrows * %d; _it += %d) {' % (
            group, inner, per_pass))
        src.append('    const int _r = _it / %d;' % inner)
        src.append('    const int _c = _it - _r * %d;' % inner)
        src.append('    _type_reduce _s = %s;' % _identity_decl(identity))
        # slice r starts its walk r lines down (and wraps around): the lanes of
        # a wave, which hold the same column of consecutive slices, are then
        # spread over the LDS banks whatever the length of a slice
        # (only where slices start a multiple of 16 words apart: elsewhere the
        # banks are spread as it is, and the plain walk is quicker)
        rotate = width % 16 == 0
        src.append('    const int _rot = %s;' % (('_r %% %d' % lines) if rotate else '0'))
        if lines // group <= 32:
            src.append('#pragma unroll')
        src.append('    for (int _jq = _g; _jq < %d; _jq += %d) {' % (lines, group))
        if rotate:
            src.append('      const int _j = (_jq + _rot >= %d) ? (_jq + _rot - %d) : (_jq + _rot);' % (
                lines, lines))
        else:
            src.append('      const int _j = _jq;')
        src.append('      const IndexT _J = _j;')
        for a in all_ins:
            src.append('      const %s %s(_slab_%s[_r * %d + _j * %d + _c]);' % (
                a.var_t, a.name, a.name, width, inner))
        src.append('      _type_reduce _a = static_cast<_type_reduce>(%s);' % pre_map_expr)
        src.append('      _s = REDUCE(_s, _a);')
        src.append('    }')
        if group > 1:
            src.append('    _s = cupy::group_allreduce<%d>(_s, _ReduceOp());' % group)
            src.append('    if (_g == 0) {')
        else:
            src.append('    {')
        src.append('      const ptrdiff_t _i = (_row0 + _r) * %d + _c;' % inner)
        src.extend(_finish(args, False, '      '))
        src.append('    }')
        src.append('  }')
        src.append('}')
        return '\n'.join(src) + '\n'
    src.append('  for (int _r = threadIdx.x / %d; _r < _nrows; _r += %d) {' % (group, per_pass))
    src.append('    _type_reduce _s = %s;' % _identity_decl(identity))
    src.append('    const int _rot = (_r * %d) %% %d;' % (group, width))
    if width // group <= 32:
        src.append('#pragma unroll')
    src.append('    for (int _jq = _g; _jq < %d; _jq += %d) {' % (width, group))
    src.append('      const int _j = (_jq + _rot >= %d) ? (_jq + _rot - %d) : (_jq + _rot);' % (width, width))
    src.append('      const IndexT _J = _j;')
    for a in all_ins:
        if a.bcast_r:
            src.append('      const %s %s(_rowv_%s[_r]);' % (a.var_t, a.name, a.name))
        elif a.bcast_o:
            src.append('      const %s %s(_p_%s[_j]);' % (a.var_t, a.name, a.name))
        else:
            src.append('      const %s %s(_slab_%s[_r * %d + _j]);' % (a.var_t, a.name, a.name, width))
    src.append('      _type_reduce _a = static_cast<_type_reduce>(%s);' % pre_map_expr)
    src.append('      _s = REDUCE(_s, _a);')
    src.append('    }')
    if group > 1:
        src.append('    _s = cupy::group_allreduce<%d>(_s, _ReduceOp());' % group)
        src.append('    if (_g == 0) {')
    else:
        src.append('    {')
    src.append('      const ptrdiff_t _i = _row0 + _r;')
    src.extend(_finish(args, False, '      '))
    src.append('    }')
    src.append('  }')
    src.append('}')
    return '\n'.join(src) + '\n'


def emit_cols_flat(name, args, identity, pre_map_expr, reduce_expr, post_map_expr,
                   reduce_type, typedefs='', preamble='', width=3, vec=4, threads=255,
                   idx64=False, stream_hint=False, unroll=4, block=BLOCK, chunked=False):
    """Reduction down the columns of a NARROW dense matrix (``width`` columns,
    stored row after row, every input alike), partial results per workgroup.

    A workgroup per column block would leave most lanes idle (67 columns: 17 of
    32 lanes) and its vectors would start wherever the rows do.  Here the matrix
    is walked as the one contiguous piece of memory it is: lane ``t`` of the
    first ``threads`` lanes takes the vectors ``t``, ``t + threads``, ... of its
    workgroup's trips, all of them aligned.  ``threads * vec`` is a multiple of
    ``width``, so the columns a lane's ``vec`` elements fall into are the same
    on every trip -- element ``k`` of lane ``t`` always lies in column
    ``(t * vec + k) % width`` -- and a lane keeps one accumulator per element.
    At the end the accumulators of a column are combined through the LDS in a
    fixed order and written as the workgroup's partial result for that column.
    ``chunked``: a workgroup takes a run of consecutive trips, one contiguous
    piece of memory; otherwise trips ``blockIdx.x``, ``+ gridDim.x``, ..., the
    workgroups walking down the matrix side by side."""
    assert (threads * vec) % width == 0 and threads <= block
    idx_t = 'ptrdiff_t' if idx64 else 'int'
    nt = 'true' if stream_hint else 'false'
    ins = [a for a in args if a.kind == 'in']
    params = _fast_params(args, idx_t, False, True)
    src = [_prologue(typedefs, preamble, reduce_type, reduce_expr, post_map_expr)]
    src.append('extern "C" __global__ void __launch_bounds__(%d) %s(%s) {' % (block, name, params))
    src.append(_SIZE_INDEXERS)
    src.append('  __shared__ __attribute__((aligned(16))) char _sm_raw[%d * sizeof(_type_reduce)];'
               % (threads * vec))
    src.append('  _type_reduce* _sm = reinterpret_cast<_type_reduce*>(_sm_raw);')
    src.append('  const int _t = threadIdx.x;')
    src.append('  const ptrdiff_t _total = (ptrdiff_t)_n_red * %d;' % width)
    src.append('  _type_reduce _acc[%d];' % vec)
    src.append('#pragma unroll')
    src.append('  for (int _k = 0; _k < %d; ++_k) _acc[_k] = %s;' % (vec, _identity_decl(identity)))
    src.append('  if (_t < %d) {' % threads)
    if chunked:
        # a workgroup takes a run of consecutive trips: one contiguous piece of memory
        src.append('    const ptrdiff_t _trips = (_total + %d) / %d;' % (threads * vec - 1, threads * vec))
        src.append('    const ptrdiff_t _per = (_trips + gridDim.x - 1) / gridDim.x;')
        src.append('    const ptrdiff_t _q1 = ((ptrdiff_t)blockIdx.x + 1) * _per < _trips ? '
                   '((ptrdiff_t)blockIdx.x + 1) * _per : _trips;')
        src.append('    ptrdiff_t _e = ((ptrdiff_t)blockIdx.x * _per * %d + _t) * %d;' % (threads, vec))
        src.append('    const ptrdiff_t _step = %d;' % (threads * vec))
        src.append('    const ptrdiff_t _end = _q1 * %d < _total ? _q1 * %d : _total;' % (
            threads * vec, threads * vec))
    else:
        src.append('    ptrdiff_t _e = ((ptrdiff_t)blockIdx.x * %d + _t) * %d;' % (threads, vec))
        src.append('    const ptrdiff_t _step = (ptrdiff_t)gridDim.x * %d;' % (threads * vec))
        src.append('    const ptrdiff_t _end = _total;')
    # the row of element k of this lane's vector: a step is a whole number of
    # rows, so the rows advance by a constant from trip to trip and no element
    # needs a division of its own
    src.append('    const IndexT _jstep = (IndexT)(_step / %d);' % width)
    src.append('    IndexT _jb[%d];' % vec)
    src.append('#pragma unroll')
    src.append('    for (int _k = 0; _k < %d; ++_k) _jb[_k] = (IndexT)((_e + _k) / %d);' % (vec, width))

    def loads(pad, e_expr, suffix):
        for a in ins:
            src.append('%sconst cupy::Vec<%s, %d> _l_%s%s = cupy::load_vec<%s, %d, %s>(_p_%s + (%s));'
                       % (pad, a.store_t, vec, a.name, suffix, a.store_t, vec, nt, a.name, e_expr))

    def accumulate(pad, u, suffix):
        src.append('#pragma unroll')
        src.append('%sfor (int _k = 0; _k < %d; ++_k) {' % (pad, vec))
        src.append('%s  const IndexT _J = _jb[_k] + %d * _jstep; (void)_J;' % (pad, u))
        for a in ins:
            src.append('%s  const %s %s(_l_%s%s.v[_k]);' % (pad, a.var_t, a.name, a.name, suffix))
        src.append('%s  _type_reduce _a = static_cast<_type_reduce>(%s);' % (pad, pre_map_expr))
        src.append('%s  _acc[_k] = REDUCE(_acc[_k], _a);' % pad)
        src.append('%s}' % pad)

    if unroll > 1:
        src.append('    for (; _e + %d * _step + %d <= _end; _e += %d * _step) {' % (
            unroll - 1, vec, unroll))
        for u in range(unroll):
            loads('      ', '_e + %d * _step' % u, '_%d' % u)
        for u in range(unroll):
            accumulate('      ', u, '_%d' % u)
        src.append('#pragma unroll')
        src.append('      for (int _k = 0; _k < %d; ++_k) _jb[_k] += %d * _jstep;' % (vec, unroll))
        src.append('    }')
    src.append('    for (; _e + %d <= _end; _e += _step) {' % vec)
    loads('      ', '_e', '')
    accumulate('      ', 0, '')
    src.append('#pragma unroll')
    src.append('      for (int _k = 0; _k < %d; ++_k) _jb[_k] += _jstep;' % vec)
    src.append('    }')
    # the last vector of the matrix may be a partial one
    src.append('    if (_e < _end) {')
    src.append('#pragma unroll')
    src.append('      for (int _k = 0; _k < %d; ++_k) if (_e + _k < _end) {' % vec)
    src.append('        const IndexT _J = _jb[_k]; (void)_J;')
    for a in ins:
        src.append('        const %s %s(_p_%s[_e + _k]);' % (a.var_t, a.name, a.name))
    src.append('        _type_reduce _a = static_cast<_type_reduce>(%s);' % pre_map_expr)
    src.append('        _acc[_k] = REDUCE(_acc[_k], _a);')
    src.append('      }')
    src.append('    }')
    src.append('#pragma unroll')
    src.append('    for (int _k = 0; _k < %d; ++_k) _sm[_t * %d + _k] = _acc[_k];' % (vec, vec))
    src.append('  }')
    src.append('  __syncthreads();')
    # accumulator f of the workgroup (lane f / vec, element f % vec) belongs
    # to column f % width: the accumulators j = f / width of a column are
    # folded pairwise, j with j + m for m halving from the power of two below
    # their number -- a fixed order, every thread taking several pairs
    count = threads * vec // width
    m = 1
    while m * 2 < count:
        m *= 2
    while m >= 1 and count > 1:
        src.append('  for (int _p = _t; _p < %d; _p += %d) {' % (width * m, block))
        src.append('    const int _j = _p / %d;' % width)
        src.append('    if (_j + %d < %d) _sm[_p] = REDUCE(_sm[_p], _sm[_p + %d]);' % (
            m, count, m * width))
        src.append('  }')
        src.append('  __syncthreads();')
        count = min(count, m)
        m //= 2
    src.append('  for (int _c = _t; _c < %d; _c += %d)' % (width, block))
    src.append('    _partials[(ptrdiff_t)blockIdx.x * %d + _c] = _sm[_c];' % width)
    src.append('}')
    return '\n'.join(src) + '\n'


def emit_cols(name, args, identity, pre_map_expr, reduce_expr, post_map_expr,
              reduce_type, typedefs='', preamble='', tx=64, vec=4, idx64=False,
              partial_in=False, partial_out=False, stream_hint=False, unroll=4,
              solo=False, batched=False, clamp_tail=False, vec_out=False, solo_block=BLOCK,
              finish=False, reduce_words=2, xcd=False):
    """Output-axis-contiguous kernel.  Thread layout: ``tx`` threads across
    the output axis (each owning ``vec`` adjacent outputs) times 256/tx slices
    of the reduce axis; gridDim.y further slices.  ``partial_in``: the single
    input holds ``_type_reduce`` values that are combined as they are."""
    # ``solo``: every thread owns its columns for the whole reduce axis (a
    # handful of rows): nothing to combine across lanes or waves
    # ``batched``: the outputs form ``_n_out / _n_inner`` rows of ``_n_inner``
    # adjacent columns (stored one row after the other); row b of input x
    # starts ``_sb_x`` elements after row b - 1 and is reduced like the whole
    # problem of the plain kernel.  Column blocks do not straddle rows: block
    # ``_blk`` works on row ``_blk / _nbc``.
    # ``clamp_tail``: the thread whose vector would reach past the last column
    # loads the last full vector instead (overlapping its neighbour's) and
    # moves its own columns to the front of its accumulators at the end; no
    # lane then walks the reduce axis element by element.  Needs loads that
    # may start at any element.
    block = solo_block if solo else BLOCK
    if solo:
        tx = block
    clamp_tail = clamp_tail and vec > 1 and not partial_in
    assert tx in (1, 2, 4, 8, 16, 32, 64) or solo
    idx_t = 'ptrdiff_t' if idx64 else 'int'
    nt = 'true' if stream_hint else 'false'
    ins = [a for a in args if a.kind == 'in']
    ty = block // tx
    waves = block // WAVE
    finish = bool(finish and partial_out and not solo and not batched and not partial_in)
    params = _fast_params(args, idx_t, partial_in, partial_out, finish)
    if batched:
        assert not partial_in and not any(a.bcast_o for a in ins)
        for a in ins:
            params = re.sub(r'\b_p_%s\b' % a.name, '_q_%s' % a.name, params)
        params += ', const %s _n_inner, const %s _nbc' % (idx_t, idx_t)
        params += ''.join(', const %s _sb_%s' % (idx_t, a.name) for a in ins)
    src = [_prologue(typedefs, preamble, reduce_type, reduce_expr, post_map_expr)]
    if finish:
        src.append(_sync_helpers(reduce_words))
    src.append('extern "C" __global__ void __launch_bounds__(%d) %s(%s) {' % (
        block, name, params))
    src.append(_SIZE_INDEXERS)
    if not solo:
        src.append('  __shared__ __attribute__((aligned(16))) char _sm_raw[%d * sizeof(_type_reduce)];' % (
            waves * tx * vec))
        src.append('  _type_reduce* _sm = reinterpret_cast<_type_reduce*>(_sm_raw);')
    src.append('  const int _tx = threadIdx.x %% %d;' % tx)
    src.append('  const int _ty = threadIdx.x / %d;' % tx)
    if finish:
        # a grid of one dimension, numbered along the column blocks first: the
        # workgroups of one column block start in the order of their slices
        src.append('  const %s _blk = (%s)(blockIdx.x %% (unsigned)_gx);' % (idx_t, idx_t))
        src.append('  const %s _by = (%s)(blockIdx.x / (unsigned)_gx);' % (idx_t, idx_t))
        src.append('  const %s _gy = (%s)(gridDim.x / (unsigned)_gx);' % (idx_t, idx_t))
        src.append('  _slot_t* _slots = reinterpret_cast<_slot_t*>(_sync + _SYNC_HEADER_WORDS);')
        # (asked for now, needed when the partial results are there)
        src.append('  __shared__ unsigned _sh_epoch;')
        src.append('  unsigned _epoch0 = 0u;')
        src.append('  if (threadIdx.x == 0) _epoch0 = _sync_epoch(_sync);')
        by_expr, gy_expr = '_by', '_gy'
    elif xcd:
        # Workgroups are handed to the eight compute dies in turn (workgroup w
        # of the grid, counted along x first, goes to die w % 8), and every die
        # has a cache of its own.  Neighbouring column blocks share the cache
        # line their border falls into whenever the rows do not start on line
        # boundaries: numbered so that a die takes a run of consecutive column
        # blocks, the line is fetched from memory once instead of once per die
        # (grid.z is 1 here).
        src.append('  const unsigned _lin = blockIdx.y * gridDim.x + blockIdx.x;')
        src.append('  const unsigned _whole = (gridDim.x * gridDim.y) & ~7u;')
        src.append('  const unsigned _turn = _lin < _whole ? (_lin & 7u) * (_whole >> 3) + (_lin >> 3) : _lin;')
        src.append('  const %s _blk = (%s)(_turn %% gridDim.x);' % (idx_t, idx_t))
        src.append('  const %s _by = (%s)(_turn / gridDim.x);' % (idx_t, idx_t))
        by_expr, gy_expr = '_by', '(%s)gridDim.y' % idx_t
    else:
        # column blocks beyond the capacity of grid.x continue along grid.z
        src.append('  const %s _blk = (%s)blockIdx.z * gridDim.x + blockIdx.x;' % (idx_t, idx_t))
        by_expr, gy_expr = '(%s)blockIdx.y' % idx_t, '(%s)gridDim.y' % idx_t
    if batched:
        src.append('  const %s _b = _blk / _nbc;' % idx_t)
        src.append('  const %s _c = ((_blk - _b * _nbc) * %d + _tx) * %d;' % (idx_t, tx, vec))
        # blocks past the last row (grid rounded up along z) have no columns
        src.append('  const %s _ncol = ((ptrdiff_t)_b * _n_inner < _n_out) ? _n_inner : 0;' % idx_t)
        src.append('  const %s _i0 = _b * _n_inner;' % idx_t)
        for a in ins:
            src.append('  const %s* __restrict__ _p_%s = _q_%s + (ptrdiff_t)_b * _sb_%s;' % (
                a.store_t, a.name, a.name, a.name))
    else:
        src.append('  const %s _c = (_blk * %d + _tx) * %d;' % (idx_t, tx, vec))
        src.append('  const %s _ncol = _n_out;' % idx_t)
        src.append('  const %s _i0 = 0;' % idx_t)
    src.append('  _type_reduce _acc[%d];' % vec)
    src.append('#pragma unroll')
    src.append('  for (int _k = 0; _k < %d; ++_k) _acc[_k] = %s;' % (vec, _identity_decl(identity)))
    if clamp_tail:
        src.append('  const %s _cl = (_c + %d <= _ncol) ? _c : (_ncol - %d);' % (idx_t, vec, vec))
        src.append('  const int _shift = (int)(_c - _cl);')
    else:
        src.append('  const %s _cl = _c;' % idx_t)
    src.append('  if (_c < _ncol) {')
    if clamp_tail:
        src.append('    const bool _full = _ncol >= %d;' % vec)
    else:
        src.append('    const bool _full = _c + %d <= _ncol;' % vec)
    src.append('    if (_full) {')
    src.append('      const %s _jstep = %s * %d;' % (idx_t, gy_expr, ty))
    src.append('      %s _j = %s * %d + _ty;' % (idx_t, by_expr, ty))
    # operands that do not vary along the reduce axis are read once
    for a in ins:
        if a.bcast_r and not partial_in:
            if a.bcast_o:
                src.append('      const %s _r_%s = _p_%s[0];' % (a.store_t, a.name, a.name))
            else:
                src.append('      const cupy::Vec<%s, %d> _r_%s = cupy::load_vec<%s, %d, false>('
                           '_p_%s + _cl);' % (a.store_t, vec, a.name, a.store_t, vec, a.name))

    def loads(pad, j_expr, suffix):
        for a in ins:
            if a.bcast_r and not partial_in:
                continue
            if partial_in:
                # partial results may have any size: plain element reads
                src.append('%s_type_reduce _l_%s%s[%d];' % (pad, a.name, suffix, vec))
                src.append('#pragma unroll')
                src.append('%sfor (int _k = 0; _k < %d; ++_k) _l_%s%s[_k] = '
                           '_p_%s[(ptrdiff_t)(%s) * _sr_%s + _c + _k];' % (
                               pad, vec, a.name, suffix, a.name, j_expr, a.name))
            elif a.bcast_o:
                src.append('%sconst %s _b_%s%s = _p_%s[(ptrdiff_t)(%s) * _sr_%s];' % (
                    pad, a.store_t, a.name, suffix, a.name, j_expr, a.name))
            else:
                src.append('%sconst cupy::Vec<%s, %d> _l_%s%s = cupy::load_vec<%s, %d, %s>('
                           '_p_%s + (ptrdiff_t)(%s) * _sr_%s + _cl);' % (
                               pad, a.store_t, vec, a.name, suffix, a.store_t, vec, nt,
                               a.name, j_expr, a.name))

    def accumulate(pad, j_expr, suffix):
        src.append('%s{' % pad)
        src.append('%s  const IndexT _J = %s;' % (pad, j_expr))
        src.append('#pragma unroll')
        src.append('%s  for (int _k = 0; _k < %d; ++_k) {' % (pad, vec))
        if partial_in:
            a = ins[0]
            src.append('%s    _acc[_k] = REDUCE(_acc[_k], _l_%s%s[_k]);' % (pad, a.name, suffix))
        else:
            for a in ins:
                if a.bcast_r:
                    val = ('_r_%s' % a.name) if a.bcast_o else ('_r_%s.v[_k]' % a.name)
                else:
                    val = ('_b_%s%s' % (a.name, suffix)) if a.bcast_o else (
                        '_l_%s%s.v[_k]' % (a.name, suffix))
                src.append('%s    const %s %s(%s);' % (pad, a.var_t, a.name, val))
            src.append('%s    _type_reduce _a = static_cast<_type_reduce>(%s);' % (
                pad, pre_map_expr))
            src.append('%s    _acc[_k] = REDUCE(_acc[_k], _a);' % pad)
        src.append('%s  }' % pad)
        src.append('%s}' % pad)

    if unroll > 1:
        # `unroll` row-slices per trip: every load is issued before the first
        # value is used, so that many requests are in flight per lane
        src.append('      for (; _j + %d * _jstep < _n_red; _j += %d * _jstep) {' % (
            unroll - 1, unroll))
        for u in range(unroll):
            loads('        ', '_j + %d * _jstep' % u, '_%d' % u)
        for u in range(unroll):
            accumulate('        ', '_j + %d * _jstep' % u, '_%d' % u)
        src.append('      }')
    src.append('      for (; _j < _n_red; _j += _jstep) {')
    loads('        ', '_j', '')
    accumulate('        ', '_j', '')
    src.append('      }')
    src.append('    } else {')
    src.append('      for (%s _j = %s * %d + _ty; _j < _n_red; _j += %s * %d) {' % (
        idx_t, by_expr, ty, gy_expr, ty))
    src.append('        const IndexT _J = _j;')
    # a constant trip count with the bound tested inside: the accumulators are
    # then indexed by constants only and stay in registers whatever their type
    src.append('#pragma unroll')
    src.append('        for (int _k = 0; _k < %d; ++_k) if (_c + _k < _ncol) {' % vec)
    if partial_in:
        a = ins[0]
        src.append('          _acc[_k] = REDUCE(_acc[_k], _p_%s[(ptrdiff_t)_j * _sr_%s + _c + _k]);' % (
            a.name, a.name))
    else:
        for a in ins:
            if a.bcast_o:
                val = '_p_%s[(ptrdiff_t)_j * _sr_%s]' % (a.name, a.name)
            else:
                val = '_p_%s[(ptrdiff_t)_j * _sr_%s + _c + _k]' % (a.name, a.name)
            src.append('          const %s %s(%s);' % (a.var_t, a.name, val))
        src.append('          _type_reduce _a = static_cast<_type_reduce>(%s);' % pre_map_expr)
        src.append('          _acc[_k] = REDUCE(_acc[_k], _a);')
    src.append('        }')
    src.append('      }')
    src.append('    }')
    src.append('  }')
    if clamp_tail:
        src.append('  if (_c < _ncol && _ncol >= %d && _shift) {' % vec)
        src.append('#pragma unroll')
        src.append('    for (int _s = 1; _s < %d; ++_s) if (_shift == _s) {' % vec)
        src.append('#pragma unroll')
        src.append('      for (int _k = 0; _k < %d; ++_k) if (_k + _s < %d) _acc[_k] = _acc[_k + _s];' % (
            vec, vec))
        src.append('    }')
        src.append('  }')
    if solo:
        outs = [a for a in args if a.kind == 'out']
        if vec_out and vec > 1 and not partial_out:
            # outputs stored next to one another: the thread's results leave as
            # one vector per output (with few rows to reduce, the outputs are a
            # large share of the traffic)
            src.append('  if (_c + %d <= _ncol) {' % vec)
            for a in outs:
                src.append('    cupy::Vec<%s, %d> _o_%s;' % (a.store_t, vec, a.name))
            src.append('#pragma unroll')
            src.append('    for (int _k = 0; _k < %d; ++_k) {' % vec)
            src.append('      _type_reduce _s = _acc[_k];')
            src.append('      const %s _i = _i0 + _c + _k; (void)_i;' % idx_t)
            for a in outs:
                src.append('      %s &%s = _o_%s.v[_k];' % (a.var_t, a.name, a.name))
            src.append('      POST_MAP(_s);')
            src.append('    }')
            for a in outs:
                src.append('    cupy::store_vec<%s, %d, %s>(_p_%s + _i0 + _c, _o_%s);' % (
                    a.store_t, vec, nt, a.name, a.name))
            src.append('  } else')
        src.append('  if (_c < _ncol) {')
        src.append('#pragma unroll')
        src.append('    for (int _k = 0; _k < %d; ++_k) if (_c + _k < _ncol) {' % vec)
        src.append('      _type_reduce _s = _acc[_k];')
        src.append('      const %s _i = _i0 + _c + _k;' % idx_t)
        src.extend(_finish(args, partial_out, '      '))
        src.append('    }')
        src.append('  }')
        src.append('}')
        return '\n'.join(src) + '\n'
    # combine the row-slices held by the lanes of one wave, then the waves
    if tx < WAVE:
        src.append('#pragma unroll')
        src.append('  for (int _k = 0; _k < %d; ++_k) {' % vec)
        src.append('    _acc[_k] = cupy::strided_allreduce<%d>(_acc[_k], _ReduceOp());' % tx)
        src.append('  }')
    src.append('  const int _wave = threadIdx.x / %d;' % WAVE)
    src.append('  if ((threadIdx.x %% %d) < %d) {' % (WAVE, tx))
    src.append('#pragma unroll')
    src.append('    for (int _k = 0; _k < %d; ++_k) _sm[(_wave * %d + _tx) * %d + _k] = _acc[_k];' % (
        vec, tx, vec))
    src.append('  }')
    if finish:
        src.append('  if (threadIdx.x == 0) _sh_epoch = _epoch0;')
    src.append('  __syncthreads();')
    if finish:
        src.append('  const unsigned _epoch = _sh_epoch;')
    src.append('  if (threadIdx.x < %d && _c < _ncol) {' % tx)
    src.append('    for (int _k = 0; _k < %d && _c + _k < _ncol; ++_k) {' % vec)
    src.append('      _type_reduce _s = _sm[_tx * %d + _k];' % vec)
    src.append('      for (int _w = 1; _w < %d; ++_w) _s = REDUCE(_s, _sm[(_w * %d + _tx) * %d + _k]);' % (
        waves, tx, vec))
    src.append('      const %s _i = _i0 + _c + _k;' % idx_t)
    src.extend(_finish(args, 'publish' if finish else partial_out, '      ',
                       split_expr='_by' if (finish or xcd) else 'blockIdx.y'))
    src.append('    }')
    src.append('  }')
    if finish:
        # the workgroup of the last slice finishes the columns of its block: a
        # thread per column combines the partial results of the slices in
        # their order
        src.append('  if (_by == _gy - 1) {')
        src.append('    bool _ok = true;')
        src.append('    for (%s _c1 = _blk * %d + threadIdx.x; _c1 < (_blk + 1) * %d && _c1 < _ncol; '
                   '_c1 += %d) {' % (idx_t, tx * vec, tx * vec, block))
        src.append('      _type_reduce _s = %s;' % _identity_decl(identity))
        src.append('      _ok = _sync_fold(_slots, (ptrdiff_t)_i0 + _c1, (ptrdiff_t)_n_out, (int)_gy, '
                   '_epoch, _spin_limit, _s) && _ok;')
        src.append('      const %s _i = _i0 + _c1;' % idx_t)
        src.extend(_finish(args, False, '      '))
        src.append('    }')
        src.append('    if (!_ok && _fault) *reinterpret_cast<volatile unsigned*>(_fault) = 1u;')
        src.append('    __syncthreads();')
        src.append('    if (threadIdx.x < %d)' % WAVE)
        src.append('      _sync_report(_sync, _slots + (ptrdiff_t)_gy * _n_out * _kWords, _blk, _gx, '
                   '_epoch, _spin_limit, _fault, (ptrdiff_t)_gy * _n_out * _kWords + _gx);')
        src.append('  }')
    src.append('}')
    return '\n'.join(src) + '\n'


def emit_generic(name, args, identity, pre_map_expr, reduce_expr, post_map_expr,
                 reduce_type, typedefs='', preamble='', tx=64, in_ndim=1,
                 out_ndim=1, in_index_32=True, out_index_32=True,
                 partial_out=False, partial_in=False):
    """Any-stride kernel.  The inputs are views whose leading axes are the
    reduced ones; element (i, J) of the problem has linear index
    ``i + J * _out_ind.size()`` in ``_in_ind`` (the reference's convention,
    cupy/_core/_reduction.pyx:75-93), so expressions may also use ``_in_ind``,
    ``_out_ind``, ``_i`` and ``_j``."""
    assert tx in (1, 2, 4, 8, 16, 32, 64)
    ty = BLOCK // tx
    waves = BLOCK // WAVE
    parts = []
    for a in args:
        if a.kind in ('in', 'out'):
            const = 'const ' if (a.kind == 'in' and a.is_const) else ''
            parts.append('%sCArray<%s, %d, %d, %d> _raw_%s' % (
                const, a.store_t, a.ndim, a.c_contiguous, a.index_32, a.name))
        elif a.kind == 'raw':
            parts.append(_raw_param(a))
        else:
            parts.append('const %s %s' % (a.store_t, a.name))
    parts.append('CIndexer<%d, %d> _in_ind' % (in_ndim, in_index_32))
    parts.append('CIndexer<%d, %d> _out_ind' % (out_ndim, out_index_32))
    if partial_out:
        parts.append('_type_reduce* _partials')
    params = ', '.join(parts)
    src = [_prologue(typedefs, preamble, reduce_type, reduce_expr, post_map_expr)]
    src.append('extern "C" __global__ void __launch_bounds__(%d) %s(%s) {' % (
        BLOCK, name, params))
    src.append('  __shared__ __attribute__((aligned(16))) char _sm_raw[%d * sizeof(_type_reduce)];' % (
        waves * tx))
    src.append('  _type_reduce* _sm = reinterpret_cast<_type_reduce*>(_sm_raw);')
    src.append('  const int _tx = threadIdx.x %% %d;' % tx)
    src.append('  const int _ty = threadIdx.x / %d;' % tx)
    src.append('  const ptrdiff_t _n_out = _out_ind.size();')
    src.append('  const ptrdiff_t _n_red = _n_out ? _in_ind.size() / _n_out : 0;')
    src.append('  for (ptrdiff_t _i_base = (ptrdiff_t)blockIdx.x * %d; _i_base < _n_out; '
               '_i_base += (ptrdiff_t)gridDim.x * %d) {' % (tx, tx))
    src.append('    const ptrdiff_t _i = _i_base + _tx;')
    src.append('    _type_reduce _s = %s;' % _identity_decl(identity))
    src.append('    if (_i < _n_out) {')
    src.append('      for (ptrdiff_t _Jl = (ptrdiff_t)blockIdx.y * %d + _ty; _Jl < _n_red; '
               '_Jl += (ptrdiff_t)gridDim.y * %d) {' % (ty, ty))
    src.append('        const IndexT _J = _Jl;')
    src.append('        const ptrdiff_t _j = _i + _Jl * _n_out;')
    src.append('        _in_ind.set(_j);')
    for a in args:
        if a.kind == 'in':
            if a.is_const:
                src.append('        const %s %s(_raw_%s[_in_ind.get()]);' % (
                    a.var_t, a.name, a.name))
            else:
                src.append('        %s &%s = _raw_%s[_in_ind.get()];' % (
                    a.var_t, a.name, a.name))
    src.append('        _type_reduce _a = static_cast<_type_reduce>(%s);' % pre_map_expr)
    src.append('        _s = REDUCE(_s, _a);')
    src.append('      }')
    src.append('    }')
    if tx < WAVE:
        src.append('    _s = cupy::strided_allreduce<%d>(_s, _ReduceOp());' % tx)
    src.append('    if ((threadIdx.x %% %d) < %d) _sm[(threadIdx.x / %d) * %d + _tx] = _s;' % (
        WAVE, tx, WAVE, tx))
    src.append('    __syncthreads();')
    src.append('    if (threadIdx.x < %d && _i < _n_out) {' % tx)
    src.append('      _s = _sm[_tx];')
    src.append('      for (int _w = 1; _w < %d; ++_w) _s = REDUCE(_s, _sm[_w * %d + _tx]);' % (
        waves, tx))
    if partial_out:
        src.append('      _partials[(ptrdiff_t)blockIdx.y * _n_out + _i] = _s;')
    else:
        src.append('      _out_ind.set(_i);')
        for a in args:
            if a.kind == 'out':
                src.append('      %s &%s = _raw_%s[_out_ind.get()];' % (
                    a.var_t, a.name, a.name))
        src.append('      POST_MAP(_s);')
    src.append('    }')
    src.append('    __syncthreads();')
    src.append('  }')
    src.append('}')
    del partial_in
    return '\n'.join(src) + '\n'


def emit_finalize_generic(name, args, identity, reduce_expr, post_map_expr,
                          reduce_type, typedefs='', preamble='', out_ndim=1,
                          out_index_32=True):
    """Second pass after a split ``generic`` launch: combines
    ``_partials[s][i]`` over s and applies POST_MAP through the strided
    output views.  One thread per output."""
    parts = []
    for a in args:
        if a.kind == 'out':
            parts.append('CArray<%s, %d, %d, %d> _raw_%s' % (
                a.store_t, a.ndim, a.c_contiguous, a.index_32, a.name))
        elif a.kind == 'raw':
            parts.append(_raw_param(a))
        elif a.kind == 'scalar':
            parts.append('const %s %s' % (a.store_t, a.name))
    parts.append('CIndexer<%d, %d> _out_ind' % (out_ndim, out_index_32))
    parts.append('const _type_reduce* _partials')
    parts.append('const int _n_split')
    parts.append('const long long _in_total')     # element count of the whole problem
    params = ', '.join(parts)
    src = [_prologue(typedefs, preamble, reduce_type, reduce_expr, post_map_expr)]
    src.append('extern "C" __global__ void __launch_bounds__(%d) %s(%s) {' % (
        BLOCK, name, params))
    # post-maps ask the input indexer for its size only (a mean divides by
    # `_in_ind.size() / _out_ind.size()`)
    src.append('  const SizeOnly _in_ind((ptrdiff_t)_in_total); (void)_in_ind;')
    src.append('  const ptrdiff_t _n_out = _out_ind.size();')
    src.append('  CUPY_FOR(_i, _n_out) {')
    src.append('    _type_reduce _s = %s;' % _identity_decl(identity))
    src.append('    for (int _sp = 0; _sp < _n_split; ++_sp) '
               '_s = REDUCE(_s, _partials[(ptrdiff_t)_sp * _n_out + _i]);')
    src.append('    _out_ind.set(_i);')
    for a in args:
        if a.kind == 'out':
            src.append('    %s &%s = _raw_%s[_out_ind.get()];' % (a.var_t, a.name, a.name))
    src.append('    POST_MAP(_s);')
    src.append('  }')
    src.append('}')
    return '\n'.join(src) + '\n'
