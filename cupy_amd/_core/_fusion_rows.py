"""One kernel for fused functions whose reductions all run along the last axis.

Row-wise normalisations -- softmax, standardisation, a norm followed by a
division -- reduce every row of a matrix and combine the results with the row
again.  Cut at the reductions (``_fusion_split``) they become a sequence of
kernels that each read the matrix once more.  When a row is short enough to be
held in the registers of one workgroup, the whole function fits in ONE kernel:
a group of lanes loads a row, runs the reductions one after the other on the
registers (wave all-reduce, LDS across waves), evaluates the elementwise results
from the same registers and stores them.  The matrix is read once and written
once.  The reference has no counterpart on this platform: its general tracer
needs a grid-wide barrier (cupy/_core/_fusion_kernel.pyx:99-115).

The pieces of the function (one map-reduce function per reduction, one
elementwise function per result) come from ``_fusion_emit`` as bare device
functions; this module composes them.
"""
import numpy

from cupy_amd._core import _codegen_reduction as _cg
from cupy_amd._core import _fusion_emit
from cupy_amd._core import _launch_plan
from cupy_amd._core import _tuning
from cupy_amd._core import internal
from cupy_amd._core._kernel import _make_packer, _scalar_struct_code, _aligned
from cupy_amd._core._scalar import CScalar, get_typename
from cupy_amd._core.core import ndarray
from cupy_amd._core.fusion import _collect, _leaf_reader
from cupy_amd.cuda import compiler
from cupy_amd.cuda import device as _device
from cupy_amd.cuda import stream as _stream

BLOCK = 256
WAVE = 64
# registers (32-bit words) per lane that rows held in registers may take
_ROW_WORDS_PER_LANE = 64


class _Unsupported(Exception):
    pass


def _kind_of_leaf(shape, full):
    """How an argument of ``shape`` meets the rows of a ``full``-shaped array."""
    if shape is None or internal.prod(shape) == 1 and len(shape) <= len(full) \
            and all(s == 1 for s in shape):
        return 'uni'
    if tuple(shape) == tuple(full):
        return 'full'
    if len(full) >= 2 and tuple(shape) == tuple(full[:-1]) + (1,):
        return 'rowk'
    if len(shape) <= len(full) and shape[-1] == full[-1] and all(s == 1 for s in shape[:-1]):
        return 'col'
    raise _Unsupported('argument of shape %r against rows of %r' % (shape, full))


def _classify(nodes, full):
    """Kind of every recorded value: 'full' (one per element), 'col' (one per
    column), 'row' / 'rowk' (one per row, without / with the reduced axis kept),
    'uni' (one for all)."""
    kinds = {}
    last = len(full) - 1
    for n in nodes:
        if n.kind in ('array', 'scalar'):
            k = _kind_of_leaf(n.shape, full)
        elif n.kind == 'const':
            k = 'uni'
        elif n.kind == 'reduce':
            src = n.src
            if kinds.get(src.order) != 'full' or n.axes != (last,):
                raise _Unsupported('a reduction that is not along the last axis of a row')
            k = 'row'
        elif n.kind == 'keepdims':
            k = 'rowk'
        else:
            ks = set(kinds[a.order] for a in n.inputs)
            ks.discard('uni')
            if not ks:
                k = 'uni'
            elif 'row' in ks:
                # without the reduced axis NumPy would line such a value up with
                # the columns; only values of the same family may meet it
                if ks != {'row'} and len(full) > 1:
                    raise _Unsupported('a reduced value without keepdims meets an array')
                k = 'row' if ks == {'row'} else 'full'
            elif 'full' in ks or ks == {'rowk', 'col'}:
                k = 'full'
            else:
                k, = ks
        expect = {'full': tuple(full), 'row': tuple(full[:-1]),
                  'rowk': tuple(full[:-1]) + (1,)}.get(k)
        if n.kind not in ('array', 'scalar', 'const') and expect is not None \
                and n.shape is not None \
                and tuple(n.shape) != expect:
            raise _Unsupported('shape %r of a %s value' % (n.shape, k))
        kinds[n.order] = k
    return kinds


class RowPlan:
    """The fused function as one launch."""

    def __init__(self, fn, packer, grid, n_rows, in_slots, out_specs, returns, single):
        self.fn = fn
        self.packer = packer
        self.grid = grid
        self.n_rows = n_rows
        # per kernel argument (reader of the call's arguments, x); x is the
        # alignment in bytes required of an array's data, or the dtype of a scalar
        self.in_slots = tuple(in_slots)
        self.out_specs = tuple(out_specs)    # (shape, dtype) per output pointer
        self.returns = tuple(returns)        # as fusion._collect takes them
        self.store_positions = ()
        self.single = single
        self.fallback = None
        self.steps = (('kernel', self),)

    def run(self, *args):
        vals = []
        for read, descr in self.in_slots:
            v = read(args)
            if type(descr) is int:
                # an array: contiguous and aligned as the kernel's vector
                # accesses assume, or the call goes the general way
                ptr = v.data.ptr
                if not v._c_contiguous or not _aligned(ptr, descr):
                    return self.fallback.run(*args)
                vals.append(ptr)
            else:
                vals.append(_launch_plan.scalar_value(v, descr))
        outs = [ndarray._new_contiguous(shape, dtype) for shape, dtype in self.out_specs]
        vals.extend(o.data.ptr for o in outs)
        vals.append(self.n_rows)
        self.fn.launch_packed(self.grid, (BLOCK, 1, 1), self.packer.pack(*vals), 0,
                              _stream.get_current_stream_ptr())
        return _collect(self.returns, outs, args, self.single)


def build(nodes, pieces, returns, single, args, name):
    """RowPlan for the recorded function, or None when it does not have the
    row-wise form (the caller then launches the pieces one by one).

    ``nodes``: the values of the recording that the results depend on;
    ``pieces``: the ``Piece`` objects of ``_fusion_split`` in evaluation order;
    ``returns``: as ``fusion.Recording`` lists them."""
    if not _tuning.get('fused_rows'):
        return None
    try:
        return _build(nodes, pieces, returns, single, args, name)
    except _Unsupported:
        return None


class _RowPiece:
    """A piece of the row kernel: like ``_fusion_split.Piece`` without a kernel
    object; ``keep``: the target stays in registers for later pieces."""
    __slots__ = ('leaves', 'targets', 'reduce', 'keep')

    def __init__(self, leaves, targets, reduce=None, keep=False):
        self.leaves, self.targets, self.reduce, self.keep = leaves, targets, reduce, keep


def _with_kept_values(nodes, pieces, kinds, returns, full_leaves, row_words, lane_elems):
    from cupy_amd._core._fusion_split import leaves_of
    consumers = {}
    for n in nodes:
        for a in n.inputs:
            consumers.setdefault(a.order, []).append(n)
    keep = []
    for p in pieces:
        if p.reduce is None:
            continue
        src = p.reduce.src
        if src.kind != 'apply' or kinds.get(src.order) != 'full':
            continue
        if len(consumers.get(src.order, ())) < 2:
            continue
        keep.append(src)
    if not keep:
        return pieces
    # register budget: a kept array that replaces the row operands it came from
    # is free, any other counts like one more row operand
    later_roots = [v for kind, v in returns if kind == 'value']
    words = row_words
    accepted = []
    for src in keep:
        feeds = [l for l in leaves_of([src], set(n.order for n in full_leaves))]
        others = [n for n in nodes if n.order > src.order and n.kind in ('apply', 'reduce')
                  and not _depends_only_through(n, src, feeds)]
        replaces = bool(feeds) and not others
        cost = lane_elems * max(1, src.dtype.itemsize // 4)
        if replaces or words + cost <= _ROW_WORDS_PER_LANE:
            accepted.append(src)
            if not replaces:
                words += cost
    if not accepted:
        return pieces
    # the pieces again, with the kept values as starting points
    stored = set(n.order for n in nodes if n.kind in ('array', 'scalar'))
    out = []
    kept_orders = set(v.order for v in accepted)
    for p in pieces:
        if p.reduce is not None:
            src = p.reduce.src
            if src.order in kept_orders and src.order not in stored:
                out.append(_RowPiece(leaves_of([src], stored), [src], keep=True))
                stored.add(src.order)
            out.append(_RowPiece(leaves_of([src], stored), list(p.targets), reduce=p.reduce))
            stored.add(p.reduce.order)
            for n in nodes:
                if n.kind == 'keepdims' and n.src is p.reduce:
                    stored.add(n.order)
        else:
            out.append(_RowPiece(leaves_of(list(p.targets), stored), list(p.targets)))
    return out


def _depends_only_through(n, kept, feeds):
    """True unless ``n`` reads one of the row operands ``feeds`` by a path that
    does not pass through ``kept``."""
    feed_orders = set(f.order for f in feeds)
    stack = [n]
    seen = set()
    while stack:
        v = stack.pop()
        if v.order in seen or v is kept:
            continue
        seen.add(v.order)
        if v.order in feed_orders:
            return False
        stack.extend(v.inputs)
    return True


def _build(nodes, pieces, returns, single, args, name):
    reduces = [n for n in nodes if n.kind == 'reduce']
    if not reduces:
        raise _Unsupported('no reduction')
    full = tuple(reduces[0].src.shape)
    if len(full) < 1 or internal.prod(full) == 0:
        raise _Unsupported('empty')
    n_cols = full[-1]
    n_rows = internal.prod(full[:-1])
    kinds = _classify(nodes, full)

    # ---- the values every piece starts from --------------------------------------------
    leaf_value = {}
    leaf_nodes = [n for n in nodes if n.kind in ('array', 'scalar')]
    for n in leaf_nodes:
        leaf_value[n.order] = _leaf_reader(n)(args)
    for n in leaf_nodes:
        if kinds[n.order] != 'uni':
            a = leaf_value[n.order]
            if not isinstance(a, ndarray) or not a._c_contiguous:
                raise _Unsupported('operand that is not C-contiguous')
    full_leaves = [n for n in leaf_nodes if kinds[n.order] == 'full']
    col_leaves = [n for n in leaf_nodes if kinds[n.order] == 'col']
    if not full_leaves:
        raise _Unsupported('no full-size operand')

    # ---- geometry ----------------------------------------------------------------------
    items = [leaf_value[n.order].dtype.itemsize for n in full_leaves + col_leaves]
    vec = max(1, 16 // max(items))
    while vec > 1:
        # a row length that is not a whole number of vectors is fine where
        # vectors may start at any element: the last, partial vector of a row
        # is then read and written element by element
        ok = n_cols % vec == 0 or (_tuning.get('unaligned_vectors') and n_cols > vec)
        for n in full_leaves + col_leaves:
            a = leaf_value[n.order]
            ok = ok and _aligned(a.data.ptr, min(16, vec * a.dtype.itemsize))
        if ok:
            break
        vec //= 2
    def words_for(group):
        per_lane = (n_cols + group * vec - 1) // (group * vec)
        return sum(per_lane * vec * max(1, it // 4) for it in items)
    # a wave per row while the row fits its registers: no barrier, and every
    # lane keeps many loads in flight; a workgroup per row beyond that
    group = WAVE if words_for(WAVE) <= _tuning.get('fused_rows_wave_words') else BLOCK
    if group == WAVE:
        # short rows: several rows per wave, a few vectors of a row per lane
        n_vec = (n_cols + vec - 1) // vec
        per = max(1, _tuning.get('fused_rows_vectors_per_lane'))
        group = max(1, min(WAVE, internal.clp2((n_vec + per - 1) // per)))
    per_lane = (n_cols + group * vec - 1) // (group * vec)          # vectors per lane and operand
    words = words_for(group)
    # rows a group has in flight: `fused_rows_in_flight` where a lane holds one
    # vector of a row and the rows are enough for every CU to have several
    # workgroups (rows of 257 float32, two vectors per lane: a softmax gains
    # 8 us of 110 with two rows in flight, x / sqrt(sum(x * x)) loses 8 of 92)
    rows_in_flight = 1
    if group <= WAVE and per_lane == 1:
        cus_ = _device.get_compute_units(_device.get_device_id())
        rows_in_flight = max(1, _tuning.get('fused_rows_in_flight'))
        while rows_in_flight > 1 and n_rows < cus_ * 8 * (BLOCK // group) * rows_in_flight:
            rows_in_flight //= 2
    if words > _ROW_WORDS_PER_LANE or n_cols < 2:
        raise _Unsupported('row of %d elements does not fit the registers of a group' % n_cols)

    # ---- values kept in registers between pieces -------------------------------------------
    # The source of a reduction that later pieces need again (the exponentials
    # of a softmax: summed, then divided by the sum) is evaluated once, into a
    # register array of its own, instead of once per piece -- when that does not
    # raise the register count: the row operands it is computed from must not be
    # needed afterwards (the array then takes their place), or everything still
    # fits the budget of one row.
    pieces = _with_kept_values(nodes, pieces, kinds, returns, full_leaves,
                               words, per_lane * vec)

    # ---- every piece as device functions -------------------------------------------------
    dtype_of = dict((n.order, n.dtype) for n in nodes)
    described = []
    for p in pieces:
        if p.reduce is not None:
            described.append(_fusion_emit.describe_reduction(p.reduce, p.leaves))
        else:
            # values one row shares: a division by such a value goes through
            # its reciprocal, taken once per row
            shared = [l.order for l in p.leaves if kinds[l.order] in ('row', 'rowk', 'uni')]
            if not _tuning.get('fused_rows_reciprocal') or not any(
                    kinds[t.order] == 'full' for t in p.targets):
                shared = ()
            described.append(_fusion_emit.describe_elementwise(p.leaves, p.targets, shared))

    # ---- kernel parameters ---------------------------------------------------------------
    params = []
    fmt = ['@']
    in_slots = []
    cname = {}

    for n in leaf_nodes:
        v = leaf_value[n.order]
        read = _leaf_reader(n)
        if isinstance(v, ndarray):
            t = get_typename(v.dtype)
            params.append('const %s* __restrict__ _p%d' % (t, n.order))
            fmt.append('P')
            vector = kinds[n.order] in ('full', 'col')
            in_slots.append((read, min(16, vec * v.dtype.itemsize) if vector
                             else v.dtype.itemsize))
        else:
            s = CScalar(v)
            t = get_typename(s.descr)
            params.append('const %s _s%d' % (t, n.order))
            fmt.append(_scalar_struct_code(t))
            in_slots.append((read, s.descr))
            cname[n.order] = '_s%d' % n.order
    out_nodes = []
    out_returns = []
    for kind, n in returns:
        if kind != 'value':
            out_returns.append((kind, n))
            continue
        if not any(n is m for m in out_nodes):
            out_nodes.append(n)
        out_returns.append(('out', [m.order for m in out_nodes].index(n.order)))
    out_specs = []
    for n in out_nodes:
        if kinds[n.order] not in ('full', 'row', 'rowk'):
            raise _Unsupported('result that is neither per element nor per row')
        t = get_typename(dtype_of[n.order])
        params.append('%s* __restrict__ _o%d' % (t, n.order))
        fmt.append('P')
        out_specs.append((tuple(n.shape), dtype_of[n.order]))

    # ---- source --------------------------------------------------------------------------
    in_bytes = sum(leaf_value[n.order].nbytes for n in full_leaves)
    out_bytes = sum(internal.prod(s) * numpy.dtype(d).itemsize for s, d in out_specs)
    nt_l, nt_s = _tuning.stream_policy('auto', in_bytes, out_bytes)
    ntl = 'true' if nt_l else 'false'
    nts = 'true' if nt_s else 'false'
    idx_t = 'int' if n_rows * n_cols <= 0x7fffffff - (1 << 24) else 'ptrdiff_t'
    shared = []
    for d in described:
        for pre in d['preambles']:
            if pre and pre not in shared:
                shared.append(pre)
    src = ['#include <cupy/carray.cuh>', 'typedef int IndexT;']
    src.extend(shared)
    src.append('#define NCOLS %d' % n_cols)
    src.append('#define GROUP %d' % group)
    src.append('#define VEC %d' % vec)
    src.append('#define PER_LANE %d' % per_lane)
    src.append('#define ROWS %d' % rows_in_flight)
    # a vector of a row: whole where it lies within the row, element by element
    # where the row ends inside it (rows that are not a multiple of VEC long)
    src.append('''template <typename T, bool kStream>
__device__ __forceinline__ cupy::Vec<T, VEC> _row_vec(const T* row, int col) {
  if (NCOLS % VEC == 0 || col + VEC <= NCOLS) return cupy::load_vec<T, VEC, kStream>(row + col);
  cupy::Vec<T, VEC> v;
#pragma unroll
  for (int k = 0; k < VEC; ++k) v.v[k] = (col + k < NCOLS) ? row[col + k] : T();
  return v;
}
template <typename T, bool kStream>
__device__ __forceinline__ void _row_store(T* row, int col, const cupy::Vec<T, VEC>& v) {
  if (NCOLS % VEC == 0 || col + VEC <= NCOLS) { cupy::store_vec<T, VEC, kStream>(row + col, v); return; }
#pragma unroll
  for (int k = 0; k < VEC; ++k) if (col + k < NCOLS) row[col + k] = v.v[k];
}''')
    if any(d.get('reciprocals') for d in described):
        src.append(_fusion_emit.SHARED_RECIPROCAL)
    for k, (p, d) in enumerate(zip(pieces, described)):
        src.append('namespace piece%d {' % k)
        src.append(d['functions'])
        if d['kind'] == 'reduce':
            src.append('typedef %s reduce_t;' % d['reduce_ctype'])
            src.append('struct Op { __device__ __forceinline__ reduce_t operator()('
                       'const reduce_t& a, const reduce_t& b) const { return (%s); } };'
                       % d['reduce_expr'])
        src.append('}  // namespace piece%d' % k)
    params.append('const %s _n_rows' % idx_t)
    fmt.append('q' if idx_t == 'ptrdiff_t' else 'i')
    src.append('extern "C" __global__ void __launch_bounds__(%d) %s(%s) {' % (
        BLOCK, name, ', '.join(params)))
    if group == BLOCK:
        for k, d in enumerate(described):
            if d['kind'] == 'reduce':
                src.append('  __shared__ __attribute__((aligned(16))) char _sm_raw%d[%d * sizeof('
                           'piece%d::reduce_t)];' % (k, BLOCK // WAVE, k))
                src.append('  piece%d::reduce_t* _sm%d = reinterpret_cast<piece%d::reduce_t*>('
                           '_sm_raw%d);' % (k, k, k, k))
    src.append('  const int _lane = threadIdx.x % GROUP;')
    # values that do not depend on the row: one per column, one for all
    for n in col_leaves:
        t = get_typename(leaf_value[n.order].dtype)
        src.append('  cupy::Vec<%s, VEC> _c%d[PER_LANE];' % (t, n.order))
        src.append('#pragma unroll')
        src.append('  for (int _e = 0; _e < PER_LANE; ++_e) {')
        src.append('    const int _col = (_e * GROUP + _lane) * VEC;')
        src.append('    _c%d[_e] = _row_vec<%s, false>(_p%d, _col < NCOLS ? _col : 0);'
                   % (n.order, t, n.order))
        src.append('  }')
    for n in leaf_nodes:
        if kinds[n.order] == 'uni' and n.order not in cname:
            t = get_typename(leaf_value[n.order].dtype)
            src.append('  const %s _u%d = _p%d[0];' % (t, n.order, n.order))
            cname[n.order] = '_u%d' % n.order
    src.append('  const %s _rows_per_block = %d / GROUP;' % (idx_t, BLOCK))
    # Short rows: a group has ROWS rows in flight -- the loads of all of them
    # are issued before the first is worked on (a lane holds a few words of a
    # row: one row per pass leaves too few bytes on their way to hide the
    # memory's latency behind the arithmetic)
    src.append('  for (%s _row0 = (%s)blockIdx.x * (_rows_per_block * ROWS) + threadIdx.x / GROUP; '
               '_row0 < _n_rows; _row0 += (%s)gridDim.x * (_rows_per_block * ROWS)) {'
               % (idx_t, idx_t, idx_t))
    for n in full_leaves:
        t = get_typename(leaf_value[n.order].dtype)
        src.append('    cupy::Vec<%s, VEC> _fa%d[ROWS][PER_LANE];' % (t, n.order))
    src.append('#pragma unroll')
    src.append('    for (int _r = 0; _r < ROWS; ++_r) {')
    src.append('      const %s _rr = (_row0 + _r * _rows_per_block < _n_rows) ? '
               '(_row0 + _r * _rows_per_block) : (_n_rows - 1);' % idx_t)
    src.append('#pragma unroll')
    src.append('      for (int _e = 0; _e < PER_LANE; ++_e) {')
    src.append('        const int _col = (_e * GROUP + _lane) * VEC;')
    src.append('        const int _cc = _col < NCOLS ? _col : 0;')
    for n in full_leaves:
        t = get_typename(leaf_value[n.order].dtype)
        src.append('        _fa%d[_r][_e] = _row_vec<%s, %s>(_p%d + (ptrdiff_t)_rr * NCOLS, _cc);'
                   % (n.order, t, ntl, n.order))
    src.append('      }')
    src.append('    }')
    src.append('#pragma unroll')
    src.append('    for (int _r = 0; _r < ROWS; ++_r) {')
    src.append('    const %s _row = _row0 + _r * _rows_per_block;' % idx_t)
    # (a group's lanes share the row, so this is uniform over every set of
    # lanes that exchanges values below)
    src.append('    if (ROWS > 1 && _row >= _n_rows) break;')
    for n in full_leaves:
        t = get_typename(leaf_value[n.order].dtype)
        src.append('    cupy::Vec<%s, VEC> (&_f%d)[PER_LANE] = _fa%d[_r];' % (t, n.order, n.order))
    for n in leaf_nodes:
        if kinds[n.order] == 'rowk':
            t = get_typename(leaf_value[n.order].dtype)
            src.append('    const %s _r%d = _p%d[_row];' % (t, n.order, n.order))
            cname[n.order] = '_r%d' % n.order

    def operand(n):
        """Expression of a value inside the element loop (_e, _k) or, for
        values per row, anywhere in the row loop."""
        k = kinds[n.order]
        if n.order in cname:
            return cname[n.order]
        if n.kind == 'keepdims':
            return operand(n.src)
        if k == 'full' and n.kind == 'array':
            return '_f%d[_e].v[_k]' % n.order
        if k == 'full' and n.order in kept_names:
            return '_m%d[_e].v[_k]' % n.order
        if k == 'col' and n.kind == 'array':
            return '_c%d[_e].v[_k]' % n.order
        raise _Unsupported('value %d (%s, %s) is not available here' % (n.order, n.kind, k))

    kept_names = set()
    for k, (p, d) in enumerate(zip(pieces, described)):
        call_args = [operand(l) for l in p.leaves]
        for order in d.get('reciprocals', ()):
            (leaf,) = [l for l in p.leaves if l.order == order]
            src.append('    const float _rcp%d_%d = shared_reciprocal(%s);' % (k, order, operand(leaf)))
            call_args.append('_rcp%d_%d' % (k, order))
        if getattr(p, 'keep', False):
            (t,) = p.targets
            src.append('    cupy::Vec<%s, VEC> _m%d[PER_LANE];' % (
                get_typename(dtype_of[t.order]), t.order))
            src.append('#pragma unroll')
            src.append('    for (int _e = 0; _e < PER_LANE; ++_e) {')
            src.append('#pragma unroll')
            src.append('      for (int _k = 0; _k < VEC; ++_k) {')
            src.append('        piece%d::elementwise(%s);' % (
                k, ', '.join(call_args + ['_m%d[_e].v[_k]' % t.order])))
            src.append('      }')
            src.append('    }')
            kept_names.add(t.order)
            continue
        if d['kind'] == 'reduce':
            (target,) = p.targets
            ident = _cg._identity_decl(d['identity']).replace('_type_reduce', 'piece%d::reduce_t' % k)
            src.append('    piece%d::reduce_t _a%d = %s;' % (k, k, ident))
            src.append('#pragma unroll')
            src.append('    for (int _e = 0; _e < PER_LANE; ++_e) {')
            src.append('      const int _col = (_e * GROUP + _lane) * VEC;')
            # (rows of whole vectors: one test per vector instead of one per element)
            whole = n_cols % vec == 0
            if whole:
                src.append('      if (_col < NCOLS) {')
            src.append('#pragma unroll')
            src.append('      for (int _k = 0; _k < VEC; ++_k) %s{' % (
                '' if whole else 'if (_col + _k < NCOLS) '))
            src.append('        _a%d = piece%d::Op()(_a%d, piece%d::_fz_map(%s));' % (
                k, k, k, k, ', '.join(call_args)))
            src.append('      }')
            if whole:
                src.append('      }')
            src.append('    }')
            if group == 1:
                pass
            elif group <= WAVE:
                src.append('    _a%d = cupy::group_allreduce<GROUP>(_a%d, piece%d::Op());' % (k, k, k))
            else:
                src.append('    _a%d = cupy::group_allreduce<64>(_a%d, piece%d::Op());' % (k, k, k))
                src.append('    if ((threadIdx.x & 63) == 0) _sm%d[threadIdx.x >> 6] = _a%d;' % (k, k))
                src.append('    __syncthreads();')
                src.append('    _a%d = _sm%d[0];' % (k, k))
                src.append('    for (int _w = 1; _w < %d; ++_w) _a%d = piece%d::Op()(_a%d, _sm%d[_w]);'
                           % (BLOCK // WAVE, k, k, k, k))
                src.append('    __syncthreads();')
            t = get_typename(dtype_of[target.order])
            src.append('    %s _t%d;' % (t, target.order))
            src.append('    piece%d::_fz_finish(_a%d, _t%d);' % (k, k, target.order))
            cname[target.order] = '_t%d' % target.order
        else:
            target_kinds = set(kinds[t.order] for t in p.targets)
            if target_kinds <= {'row', 'rowk'}:
                if any(kinds[l.order] in ('full', 'col') for l in p.leaves):
                    raise _Unsupported('a value per row computed from values per element')
                for t in p.targets:
                    src.append('    %s _t%d;' % (get_typename(dtype_of[t.order]), t.order))
                    cname[t.order] = '_t%d' % t.order
                src.append('    piece%d::elementwise(%s);' % (
                    k, ', '.join(call_args + [cname[t.order] for t in p.targets])))
            elif target_kinds == {'full'}:
                src.append('#pragma unroll')
                src.append('    for (int _e = 0; _e < PER_LANE; ++_e) {')
                src.append('      const int _col = (_e * GROUP + _lane) * VEC;')
                for t in p.targets:
                    src.append('      cupy::Vec<%s, VEC> _v%d;' % (
                        get_typename(dtype_of[t.order]), t.order))
                src.append('#pragma unroll')
                src.append('      for (int _k = 0; _k < VEC; ++_k) {')
                src.append('        piece%d::elementwise(%s);' % (
                    k, ', '.join(call_args + ['_v%d.v[_k]' % t.order for t in p.targets])))
                src.append('      }')
                for t in p.targets:
                    if not any(t is m for m in out_nodes):
                        raise _Unsupported('elementwise value that is not a result')
                    src.append('      if (_col < NCOLS) _row_store<%s, %s>('
                               '_o%d + (ptrdiff_t)_row * NCOLS, _col, _v%d);' % (
                                   get_typename(dtype_of[t.order]), nts, t.order, t.order))
                src.append('    }')
            else:
                raise _Unsupported('results of mixed kinds in one piece')
    # results held per row
    for n in out_nodes:
        if kinds[n.order] in ('row', 'rowk'):
            src.append('    if (_lane == 0) _o%d[_row] = %s;' % (n.order, operand(n)))
    src.append('    }')
    src.append('  }')
    src.append('}')
    code = '\n'.join(src) + '\n'
    fn = compiler.compile_with_cache(code, ('-DCUPY_FUSED_ROWS',)).get_function(name)
    rows_per_block = BLOCK // group * rows_in_flight
    cus = _device.get_compute_units(_device.get_device_id())
    grid = max(1, min((n_rows + rows_per_block - 1) // rows_per_block,
                      cus * _tuning.get('fused_rows_blocks_per_cu')))
    return RowPlan(fn, _make_packer(fmt), (grid, 1, 1), n_rows, in_slots, out_specs,
                   out_returns, single)
