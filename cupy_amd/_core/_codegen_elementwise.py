"""HIP source emitters for elementwise kernels (gfx950).

Three kernel shapes are produced from one loop body:

``flat``     every array operand walks memory linearly (contiguous, or a single
             broadcast element): 128-bit vector loads/stores, grid-stride over
             vectors, scalar tail.
``tiled2d``  two-dimensional problems where each operand is contiguous along
             one of the two axes (row-major operands, row/column broadcasts and
             transposed operands): transposed operands go through an LDS tile
             so that every global access is coalesced.
``generic``  anything else: CIndexer/CArray addressing per element, the same
             semantics as the reference's kernel template
             (cupy/_core/_kernel.pyx:78-107,709-728) including ``continue`` in
             the body and outputs that are read before they are written.

The body sees the names the reference provides: the parameters, ``i`` (linear
index) and ``_ind``.
"""
import re

BLOCK = 256


class Operand:
    """One kernel parameter as the emitters see it.

    kind        'array' (broadcast, iterated), 'raw' (CArray handed to the body
                untouched), 'scalar' (by value) or 'indexer'
    name        identifier used by the body
    store_t     C type of an element in memory / of the scalar argument
    var_t       C type of the variable the body sees
    is_out      True for output arrays
    read_out    outputs only: load the old element before running the body
    cast_in     callable(expr) -> expr converting a loaded element to var_t
    cast_out    callable(expr) -> expr converting the variable to store_t
    ndim, c_contiguous, index_32   CArray template arguments (raw / generic)
    """

    def __init__(self, kind, name, store_t, var_t=None, is_out=False,
                 read_out=False, cast_in=None, cast_out=None, ndim=0,
                 c_contiguous=False, index_32=True, is_const=True):
        self.kind = kind
        self.name = name
        self.store_t = store_t
        self.var_t = var_t or store_t
        self.is_out = is_out
        self.read_out = read_out
        self.cast_in = cast_in or (lambda e: e)
        self.cast_out = cast_out or (lambda e: e)
        self.ndim = ndim
        self.c_contiguous = c_contiguous
        self.index_32 = index_32
        self.is_const = is_const

    def key(self):
        return (self.kind, self.name, self.store_t, self.var_t, self.is_out,
                self.read_out, self.ndim, self.c_contiguous, self.index_32,
                self.is_const, self.cast_in('@'), self.cast_out('@'))


_ident_cache = {}


def uses_identifier(code, ident):
    """True if ``ident`` appears in ``code`` as a whole word."""
    key = (code, ident)
    hit = _ident_cache.get(key)
    if hit is None:
        hit = re.search(r'(?<![A-Za-z0-9_])%s(?![A-Za-z0-9_])' % re.escape(ident),
                        code) is not None
        if len(_ident_cache) < 4096:
            _ident_cache[key] = hit
    return hit


def output_is_write_only(operation, name):
    """Conservative test that the body assigns ``name`` unconditionally before
    any other use: its first occurrence is ``name = ...`` as a statement at
    brace depth 0 that is not governed by ``if``/``else``/a loop.  Anything
    else (compound assignment, assignment inside a branch, a read) makes the
    emitter load the previous value first, which reproduces reference
    semantics where the variable is a reference to the element in memory."""
    m = re.search(r'(?<![A-Za-z0-9_])%s(?![A-Za-z0-9_])' % re.escape(name), operation)
    if m is None:
        return False
    head = operation[:m.start()]
    tail = operation[m.end():]
    if not re.match(r'\s*=(?!=)', tail):
        return False
    if head.count('{') != head.count('}'):
        return False
    if head.count('(') != head.count(')'):
        return False
    stmt_start = max(head.rfind(';'), head.rfind('}'))
    stmt_head = head[stmt_start + 1:]
    return stmt_head.strip() == ''


def body_needs_generic(operation):
    """Bodies that steer the element loop themselves need the one-element-per-
    iteration loop of the generic kernel."""
    return (uses_identifier(operation, 'continue')
            or uses_identifier(operation, 'return')
            or uses_identifier(operation, 'break')
            or uses_identifier(operation, 'goto'))


def _param_decl(op):
    if op.kind == 'array':
        const = 'const ' if (op.is_const and not op.is_out) else ''
        return '%s%s* _p_%s' % (const, op.store_t, op.name)
    if op.kind == 'raw':
        const = 'const ' if op.is_const else ''
        return '%sCArray<%s, %d, %d, %d> %s' % (
            const, op.store_t, op.ndim, op.c_contiguous, op.index_32, op.name)
    if op.kind == 'scalar':
        return 'const %s %s' % (op.store_t, op.name)
    if op.kind == 'indexer':
        return 'CIndexer<%d, %d> %s' % (op.ndim, op.index_32, op.name)
    raise AssertionError(op.kind)


def _header(typedefs, preamble):
    return ('#include <cupy/carray.cuh>\n' + typedefs + '\n' + preamble + '\n')


def _element_code(operands, operation, load_expr, store_stmt, indent):
    """Per-element code: declare the body variables from ``load_expr(op)``,
    run the body, hand results to ``store_stmt(op, value_expr)``."""
    pad = ' ' * indent
    lines = []
    for op in operands:
        if op.kind != 'array':
            continue
        if not op.is_out:
            lines.append('%sconst %s %s(%s);' % (
                pad, op.var_t, op.name, op.cast_in(load_expr(op))))
        elif op.read_out:
            lines.append('%s%s %s(%s);' % (
                pad, op.var_t, op.name, op.cast_in(load_expr(op))))
        else:
            lines.append('%s%s %s;' % (pad, op.var_t, op.name))
    lines.append('%s{ %s; }' % (pad, operation))
    for op in operands:
        if op.kind == 'array' and op.is_out:
            lines.append(pad + store_stmt(op, op.cast_out(op.name)))
    return '\n'.join(lines)


# A vector load whose value meets, at the end of a branch, one put together
# element by element: the compiler would take both apart into element loads
# (sixteen byte loads per lane for uint8; (4, 2^24) + row 63 us against 28).
# Passing the loaded registers through an empty statement keeps them whole.
_LOAD_WHOLE = """
template <int kBytes> struct _WholeRaw { typedef void type; };
template <> struct _WholeRaw<16> { typedef unsigned int __attribute__((ext_vector_type(4))) type; };
template <> struct _WholeRaw<8> { typedef unsigned int __attribute__((ext_vector_type(2))) type; };
template <> struct _WholeRaw<4> { typedef unsigned int type; };
template <> struct _WholeRaw<2> { typedef unsigned short type; };
template <typename T, int N>
__device__ __forceinline__ cupy::Vec<T, N> _load_whole(const T* p) {
  constexpr int kBytes = sizeof(T) * N;
  if constexpr (kBytes == 16 || kBytes == 8 || kBytes == 4 || kBytes == 2) {
    typedef typename _WholeRaw<kBytes>::type raw_t;
    typedef raw_t __attribute__((aligned(alignof(T)))) raw_at_t;
    raw_t r = *reinterpret_cast<const raw_at_t*>(p);
    asm("" : "+v"(r));
    cupy::Vec<T, N> out;
    __builtin_memcpy(&out, &r, kBytes);
    return out;
  } else {
    return cupy::load_vec<T, N, false>(p);
  }
}
"""


def emit_flat(name, operands, operation, typedefs='', preamble='',
              loop_prep='', after_loop='', vec=4, unroll=1, idx64=False,
              bcast=(), stream_hint=True, block=BLOCK, partial=None):
    """Kernel for operands that are all contiguous.

    ``bcast`` names array operands that hold a single element broadcast over
    the whole index space.  Trailing parameters of the kernel: the array
    pointers / scalars / raw arrays in operand order, then ``_n`` (element
    count) and, when the body uses it, ``_ind``.

    ``partial`` maps names of input arrays to 'row' or 'col' when the index
    space is a matrix of ``_nc`` columns stored row after row: a 'row' operand
    holds a value per row, a 'col' operand a value per column, ``_sb_<name>``
    elements apart ('col1': one element apart).  The other arrays are still walked with whole vectors;
    row and column of an element come from one division per vector.
    ``_nc`` and the ``_sb_`` strides follow ``_n``.
    """
    partial = partial or {}
    idx_t = 'ptrdiff_t' if idx64 else 'int'
    arrays = [op for op in operands if op.kind == 'array']
    iter_arrays = [op for op in arrays if op.name not in bcast and op.name not in partial]
    part_ops = [op for op in arrays if op.name in partial]
    for op in part_ops:
        assert not op.is_out
    needs_ind = any(op.kind == 'indexer' for op in operands)
    params = ', '.join([_param_decl(op) for op in operands if op.kind != 'indexer']
                       + ['const %s _n' % idx_t]
                       + (['const %s _nc' % idx_t] if partial else [])
                       + ['const %s _sb_%s' % (idx_t, op.name) for op in part_ops]
                       + [_param_decl(op) for op in operands if op.kind == 'indexer'])
    _nt_l, _nt_s = stream_hint if isinstance(stream_hint, tuple) else (stream_hint, stream_hint)
    ntl = 'true' if _nt_l else 'false'
    nts = 'true' if _nt_s else 'false'
    use_i = uses_identifier(operation, 'i')
    set_ind = '_ind.set(i);' if needs_ind and uses_identifier(operation, '_ind') else ''

    def bcast_decls():
        out = []
        for op in arrays:
            if op.name in bcast and not op.is_out:
                out.append('  const %s _b_%s = _p_%s[0];' % (
                    op.store_t, op.name, op.name))
        return '\n'.join(out)

    def part_expr(op):
        return '_p_%s[(ptrdiff_t)%s * _sb_%s]' % (
            op.name, '_rk' if partial[op.name] == 'row' else '_ck', op.name)

    row_ops = [op for op in part_ops if partial[op.name] == 'row']
    col_ops = [op for op in part_ops if partial[op.name] != 'row']

    def rc_init(pad, start, whole_vector=True):
        """Row and column of element ``start``; for a whole vector also the
        values of the per-row operands (reloaded when the vector runs into the
        next row) and a vector of the per-column operands (one load when the
        vector lies within a row and the operand is stored densely)."""
        if not partial:
            return []
        out = ['%s%s _rk = (%s) / _nc;' % (pad, idx_t, start),
               '%s%s _ck = (%s) - _rk * _nc;' % (pad, idx_t, start)]
        if not whole_vector:
            return out
        for op in row_ops:
            out.append('%s%s _pr_%s = %s;' % (pad, op.store_t, op.name, part_expr(op)))
        for op in col_ops:
            out.append('%scupy::Vec<%s, %d> _pc_%s;' % (pad, op.store_t, vec, op.name))
            gather = ('{ %s _cc = _ck;\n%s#pragma unroll\n%s  for (int _k = 0; _k < %d; ++_k) { '
                      '_pc_%s.v[_k] = _p_%s[(ptrdiff_t)_cc * _sb_%s]; if (++_cc == _nc) _cc = 0; } }' % (
                          idx_t, pad, pad, vec, op.name, op.name, op.name))
            if partial[op.name] == 'col1':
                out.append('%sif (_ck + %d <= _nc) _pc_%s = _load_whole<%s, %d>(_p_%s + _ck);' % (
                    pad, vec, op.name, op.store_t, vec, op.name))
                out.append('%selse %s' % (pad, gather))
            else:
                out.append('%s%s' % (pad, gather))
        return out

    def rc_step(pad):
        if not row_ops:
            return []
        reload = ' '.join('_pr_%s = %s;' % (op.name, part_expr(op)) for op in row_ops)
        return ['%sif (_k + 1 < %d) { if (++_ck == _nc) { _ck = 0; ++_rk; %s } }' % (
            pad, vec, reload)]

    def part_value(op):
        if partial[op.name] == 'row':
            return '_pr_%s' % op.name
        return '_pc_%s.v[_k]' % op.name

    def vec_load_expr(suffix):
        def f(op):
            if op.name in bcast:
                return '_b_%s' % op.name
            if op.name in partial:
                return part_value(op)
            return '_l_%s%s.v[_k]' % (op.name, suffix)
        return f

    def vec_store_stmt(suffix):
        def f(op, value):
            return '_l_%s%s.v[_k] = %s;' % (op.name, suffix, value)
        return f

    # --- vector part: `unroll` vectors per thread per trip -----------------------
    body = []
    body.append('  const %s _nvec = _n / %d;' % (idx_t, vec))
    body.append('  const %s _gstride = (%s)gridDim.x * %d;' % (idx_t, idx_t, block * unroll))
    body.append('  for (%s _v0 = (%s)blockIdx.x * %d + threadIdx.x; _v0 < _nvec; '
                '_v0 += _gstride) {' % (idx_t, idx_t, block * unroll))
    if unroll > 1:
        body.append('    if (_v0 + %d < _nvec) {' % ((unroll - 1) * block))
        # all loads first, so that `unroll` independent requests are in flight
        for u in range(unroll):
            for op in iter_arrays:
                if (not op.is_out) or op.read_out:
                    body.append(
                        '      cupy::Vec<%s, %d> _l_%s_%d = cupy::load_vec<%s, %d, %s>('
                        '_p_%s + (_v0 + %d) * %d);' % (
                            op.store_t, vec, op.name, u, op.store_t, vec, ntl,
                            op.name, u * block, vec))
                else:
                    body.append('      cupy::Vec<%s, %d> _l_%s_%d;' % (
                        op.store_t, vec, op.name, u))
        for u in range(unroll):
            body.append('      {')
            body.append('        const %s _base = (_v0 + %d) * %d;' % (idx_t, u * block, vec))
            body.extend(rc_init('        ', '_base'))
            body.append('#pragma unroll')
            body.append('        for (int _k = 0; _k < %d; ++_k) {' % vec)
            if use_i or set_ind:
                body.append('          const ptrdiff_t i = _base + _k; %s' % set_ind)
            body.append(_element_code(
                operands, operation, vec_load_expr('_%d' % u),
                vec_store_stmt('_%d' % u), 10))
            body.extend(rc_step('          '))
            body.append('        }')
            for op in iter_arrays:
                if op.is_out:
                    body.append(
                        '        cupy::store_vec<%s, %d, %s>(_p_%s + _base, _l_%s_%d);' % (
                            op.store_t, vec, nts, op.name, op.name, u))
            body.append('      }')
        body.append('    } else {')
        body.append('      for (%s _v = _v0; _v < _nvec; _v += %d) {' % (idx_t, block))
        inner_pad = 8
    else:
        body.append('    {')
        body.append('      const %s _v = _v0; {' % idx_t)
        inner_pad = 8
    pad = ' ' * inner_pad
    body.append('%sconst %s _base = _v * %d;' % (pad, idx_t, vec))
    for op in iter_arrays:
        if (not op.is_out) or op.read_out:
            body.append('%scupy::Vec<%s, %d> _l_%s = cupy::load_vec<%s, %d, %s>('
                        '_p_%s + _base);' % (pad, op.store_t, vec, op.name,
                                             op.store_t, vec, ntl, op.name))
        else:
            body.append('%scupy::Vec<%s, %d> _l_%s;' % (pad, op.store_t, vec, op.name))
    body.extend(rc_init(pad, '_base'))
    body.append('#pragma unroll')
    body.append('%sfor (int _k = 0; _k < %d; ++_k) {' % (pad, vec))
    if use_i or set_ind:
        body.append('%s  const ptrdiff_t i = _base + _k; %s' % (pad, set_ind))
    body.append(_element_code(operands, operation, vec_load_expr(''),
                              vec_store_stmt(''), inner_pad + 2))
    body.extend(rc_step(pad + '  '))
    body.append('%s}' % pad)
    for op in iter_arrays:
        if op.is_out:
            body.append('%scupy::store_vec<%s, %d, %s>(_p_%s + _base, _l_%s);' % (
                pad, op.store_t, vec, nts, op.name, op.name))
    body.append('      }')
    body.append('    }')
    body.append('  }')

    # --- scalar tail ----------------------------------------------------------------
    def tail_load(op):
        if op.name in bcast:
            return '_b_%s' % op.name
        if op.name in partial:
            return part_expr(op)
        return '_p_%s[_t]' % op.name

    def tail_store(op, value):
        return '_p_%s[_t] = %s;' % (op.name, value)

    tail = []
    tail.append('  for (%s _t = _nvec * %d + (%s)blockIdx.x * %d + threadIdx.x; _t < _n; '
                '_t += (%s)gridDim.x * %d) {' % (idx_t, vec, idx_t, block, idx_t, block))
    if use_i or set_ind:
        tail.append('    const ptrdiff_t i = _t; %s' % set_ind)
    tail.extend(rc_init('    ', '_t', whole_vector=False))
    tail.append(_element_code(operands, operation, tail_load, tail_store, 4))
    tail.append('  }')

    src = [_header(typedefs, preamble)]
    if any(kind == 'col1' for kind in partial.values()):
        src.append(_LOAD_WHOLE)
    src.append('extern "C" __global__ void __launch_bounds__(%d) %s(%s) {' % (
        block, name, params))
    src.append('  %s;' % loop_prep)
    b = bcast_decls()
    if b:
        src.append(b)
    # (vec == 1 -- items of 16 bytes, arrays aligned for no more than an item --
    # takes the same loop with vectors of one element: it is the one that marks
    # accesses as streaming and keeps several in flight per lane)
    src.extend(body)
    src.extend(tail)
    src.append('  %s;' % after_loop)
    src.append('}')
    return '\n'.join(src) + '\n'


def emit_generic(name, operands, operation, typedefs='', preamble='',
                 loop_prep='', after_loop='', block=128):
    """Reference-semantics kernel: one element per loop trip, operands
    addressed through CArray/CIndexer, body variables are references into
    memory (so ``continue``, partial writes and in-place reads all behave as
    in the reference)."""
    parts = []
    for op in operands:
        if op.kind == 'array':
            const = 'const ' if (op.is_const and not op.is_out) else ''
            parts.append('%sCArray<%s, %d, %d, %d> _raw_%s' % (
                const, op.store_t, op.ndim, op.c_contiguous, op.index_32, op.name))
        else:
            parts.append(_param_decl(op))
    params = ', '.join(parts)
    lines = []
    for op in operands:
        if op.kind != 'array':
            continue
        same = op.cast_in('@') == '@' and op.cast_out('@') == '@' and \
            op.store_t == op.var_t
        if same or op.var_t == op.store_t:
            if op.is_out:
                lines.append('    %s &%s = _raw_%s[_ind.get()];' % (
                    op.var_t, op.name, op.name))
            else:
                lines.append('    const %s &%s = _raw_%s[_ind.get()];' % (
                    op.var_t, op.name, op.name))
        elif op.is_out:
            if op.read_out:
                lines.append('    %s %s(%s);' % (op.var_t, op.name, op.cast_in(
                    '_raw_%s[_ind.get()]' % op.name)))
            else:
                lines.append('    %s %s;' % (op.var_t, op.name))
        else:
            lines.append('    const %s %s(%s);' % (op.var_t, op.name, op.cast_in(
                '_raw_%s[_ind.get()]' % op.name)))
    lines.append('    %s;' % operation)
    for op in operands:
        if op.kind == 'array' and op.is_out and op.var_t != op.store_t:
            lines.append('    _raw_%s[_ind.get()] = %s;' % (
                op.name, op.cast_out(op.name)))
    src = [_header(typedefs, preamble)]
    src.append('extern "C" __global__ void %s(%s) {' % (name, params))
    src.append('  %s;' % loop_prep)
    src.append('#pragma unroll 1')
    src.append('  CUPY_FOR(i, _ind.size()) {')
    src.append('    _ind.set(i);')
    src.extend(lines)
    src.append('  }')
    src.append('  %s;' % after_loop)
    src.append('}')
    return '\n'.join(src) + '\n'


def emit_rows2d(name, operands, operation, typedefs='', preamble='',
                loop_prep='', after_loop='', kinds=None, vec=4, idx64=False,
                stream_hint=True, block=BLOCK, outer=1):
    """Kernel for a matrix problem (rows r, columns c) none of whose arrays
    runs against the columns: every row is walked in vectors of ``vec``
    columns that start at column 0, 1 * vec, ... of that row, so that no
    vector reaches into the next row and rows may be spaced in any way.
    Consecutive lanes take consecutive vectors, across row ends.

    ``kinds[name]`` is
      'R'    unit stride along columns, any stride along rows: vector access;
      'row'  zero stride along columns: one value per row;
      'S'    anything else (every second column, columns backwards, ...):
             element-wise access.
    The last ``_nc % vec`` columns of a row are handled element by element by
    the lane that owns them.  Kernel parameters after the operands:
    ``_nr, _nc``, then per array its row stride and column stride in elements.

    ``outer`` > 1: the rows are the positions of ``outer`` axes (C order), each
    with a stride of its own per array -- a permutation of the leading axes of
    arrays whose last axis is contiguous.  ``_nr`` is still the number of rows;
    the extents of all but the first of those axes follow ``_nc``
    (``_ne1`` .. ), and every array brings one row stride per axis.
    """
    idx_t = 'ptrdiff_t' if idx64 else 'int'
    arrays = [op for op in operands if op.kind == 'array']
    _nt_l, _nt_s = stream_hint if isinstance(stream_hint, tuple) else (stream_hint, stream_hint)
    ntl = 'true' if _nt_l else 'false'
    nts = 'true' if _nt_s else 'false'
    use_i = uses_identifier(operation, 'i')
    parts = [_param_decl(op) for op in operands if op.kind != 'indexer']
    parts += ['const %s _nr' % idx_t, 'const %s _nc' % idx_t]
    parts += ['const %s _ne%d' % (idx_t, d) for d in range(1, outer)]
    for op in arrays:
        parts += ['const %s _sr_%s' % (idx_t, op.name)]
        parts += ['const %s _sr%d_%s' % (idx_t, d, op.name) for d in range(1, outer)]
        parts += ['const %s _sc_%s' % (idx_t, op.name)]
    assert not any(op.kind == 'indexer' for op in operands)
    params = ', '.join(parts)

    def addr(op, c):
        return '(_p_%s + _ro_%s + (ptrdiff_t)(%s) * _sc_%s)' % (op.name, op.name, c, op.name)

    src = [_header(typedefs, preamble)]
    src.append('extern "C" __global__ void __launch_bounds__(%d) %s(%s) {' % (
        block, name, params))
    src.append('  %s;' % loop_prep)
    src.append('  const %s _nvr = (_nc + %d) / %d;' % (idx_t, vec - 1, vec))
    src.append('  const %s _nv = _nr * _nvr;' % idx_t)
    src.append('  for (%s _v = (%s)blockIdx.x * %d + threadIdx.x; _v < _nv; '
               '_v += (%s)gridDim.x * %d) {' % (idx_t, idx_t, block, idx_t, block))
    src.append('    const %s _rk = _v / _nvr;' % idx_t)
    src.append('    const %s _ck = (_v - _rk * _nvr) * %d;' % (idx_t, vec))
    # where the row starts in every array
    if outer == 1:
        for op in arrays:
            src.append('    const ptrdiff_t _ro_%s = (ptrdiff_t)_rk * _sr_%s;' % (op.name, op.name))
    else:
        src.append('    %s _rest = _rk;' % idx_t)
        for d in range(outer - 1, 0, -1):
            src.append('    const %s _q%d = _rest / _ne%d;' % (idx_t, d, d))
            src.append('    const %s _i%d = _rest - _q%d * _ne%d;' % (idx_t, d, d, d))
            src.append('    _rest = _q%d;' % d)
        for op in arrays:
            terms = ['(ptrdiff_t)_rest * _sr_%s' % op.name]
            terms += ['(ptrdiff_t)_i%d * _sr%d_%s' % (d, d, op.name) for d in range(1, outer)]
            src.append('    const ptrdiff_t _ro_%s = %s;' % (op.name, ' + '.join(terms)))
    src.append('    if (_ck + %d <= _nc) {' % vec)
    for op in arrays:
        k = kinds[op.name]
        reads = (not op.is_out) or op.read_out
        if k == 'R':
            if reads:
                src.append('      cupy::Vec<%s, %d> _l_%s = cupy::load_vec<%s, %d, %s>(%s);' % (
                    op.store_t, vec, op.name, op.store_t, vec, ntl, addr(op, '_ck')))
            else:
                src.append('      cupy::Vec<%s, %d> _l_%s;' % (op.store_t, vec, op.name))
        elif k == 'row':
            if reads:
                src.append('      const %s _b_%s = *%s;' % (op.store_t, op.name, addr(op, '0')))
        else:
            src.append('      cupy::Vec<%s, %d> _l_%s;' % (op.store_t, vec, op.name))
            if reads:
                src.append('#pragma unroll')
                src.append('      for (int _k = 0; _k < %d; ++_k) _l_%s.v[_k] = *%s;' % (
                    vec, op.name, addr(op, '_ck + _k')))

    def full_load(op):
        if kinds[op.name] == 'row':
            return '_b_%s' % op.name
        return '_l_%s.v[_k]' % op.name

    def full_store(op, value):
        return '_l_%s.v[_k] = %s;' % (op.name, value)

    src.append('#pragma unroll')
    src.append('      for (int _k = 0; _k < %d; ++_k) {' % vec)
    if use_i:
        src.append('        const ptrdiff_t i = (ptrdiff_t)_rk * _nc + _ck + _k;')
    src.append(_element_code(operands, operation, full_load, full_store, 8))
    src.append('      }')
    for op in arrays:
        if op.is_out:
            if kinds[op.name] == 'R':
                src.append('      cupy::store_vec<%s, %d, %s>(%s, _l_%s);' % (
                    op.store_t, vec, nts, addr(op, '_ck'), op.name))
            else:
                src.append('#pragma unroll')
                src.append('      for (int _k = 0; _k < %d; ++_k) *%s = _l_%s.v[_k];' % (
                    vec, addr(op, '_ck + _k'), op.name))
    src.append('    } else {')
    # the last, partial vector of a row: the same three phases under a
    # per-element test, so that all loads are in flight together (a loop of
    # unknown length would wait for every element in turn)
    for op in arrays:
        k = kinds[op.name]
        reads = (not op.is_out) or op.read_out
        if k == 'row':
            if reads:
                src.append('      const %s _b_%s = *%s;' % (op.store_t, op.name, addr(op, '0')))
            continue
        src.append('      cupy::Vec<%s, %d> _l_%s;' % (op.store_t, vec, op.name))
        if reads:
            src.append('#pragma unroll')
            src.append('      for (int _k = 0; _k < %d; ++_k) if (_ck + _k < _nc) _l_%s.v[_k] = *%s;' % (
                vec, op.name, addr(op, '_ck + _k')))
    src.append('#pragma unroll')
    src.append('      for (int _k = 0; _k < %d; ++_k) if (_ck + _k < _nc) {' % vec)
    if use_i:
        src.append('        const ptrdiff_t i = (ptrdiff_t)_rk * _nc + _ck + _k;')
    src.append(_element_code(operands, operation, full_load, full_store, 8))
    src.append('      }')
    for op in arrays:
        if op.is_out:
            src.append('#pragma unroll')
            src.append('      for (int _k = 0; _k < %d; ++_k) if (_ck + _k < _nc) *%s = _l_%s.v[_k];' % (
                vec, addr(op, '_ck + _k'), op.name))
    src.append('    }')
    src.append('  }')
    src.append('  %s;' % after_loop)
    src.append('}')
    return '\n'.join(src) + '\n'


def _die_by_die(index, total, idx_t, enabled):
    """Expression that renumbers work item ``index`` of ``total`` so that each
    of the eight compute dies, which take the workgroups of a grid in turn
    (workgroup w goes to die w % 8), works on a run of consecutive items: the
    items whose borders share cache lines then meet in one die's cache.  The
    last ``total % 8`` items keep their numbers."""
    if not enabled:
        return index
    return ('((%s) < ((%s) & ~(%s)7) ? ((%s) & 7) * (((%s) & ~(%s)7) >> 3) + ((%s) >> 3) : (%s))'
            % (index, total, idx_t, index, total, idx_t, index, index))


def emit_tiled2d(name, operands, operation, typedefs='', preamble='',
                 loop_prep='', after_loop='', layouts=None, vec=4, tile_r=64,
                 tile_c=64, threads=256, idx64=False, stream_hint=True, batched=False,
                 batch_first=False, svec=None, flat_stage=0, xcd=False, strip=16):
    """Kernel for a 2-d index space (rows r, columns c) where every array
    operand is contiguous along one of the axes.

    ``batched``: ``_nbt`` such index spaces, numbered b = b0 * ``_nb1`` + b1;
    array x starts ``b0 * _sb0_x + b1 * _sb1_x`` elements further on in space b
    (the two slowest axes of a 3-d or 4-d problem whose arrays are permuted
    differently).  These parameters follow the strides.  The element index
    ``i`` is not available then.

    ``layouts[name]`` is
      'R'   unit stride along columns, any stride (also 0) along rows;
      'R0'  zero stride along columns (a value per row, broadcast over columns);
      'C'   unit stride along rows, any stride along columns: a transposed
            operand.  Inputs only.
    'C' inputs are staged through an LDS tile: the tile is read from memory
    along rows (coalesced) and consumed along columns.

    Work split: a workgroup of ``threads`` threads owns a ``tile_r`` x ``tile_c``
    block; tiles are visited in diagonal order.  Every thread handles ``vec``
    consecutive elements (along rows when staging, along columns otherwise).
    Interior tiles take an unguarded, fully vectorised path, edge tiles a guarded
    scalar one.  Kernel parameters after the operands: ``_nr, _nc``, then per
    array its row stride and column stride in elements.
    """
    idx_t = 'ptrdiff_t' if idx64 else 'int'
    arrays = [op for op in operands if op.kind == 'array']
    needs_ind = any(op.kind == 'indexer' for op in operands)
    _nt_l, _nt_s = stream_hint if isinstance(stream_hint, tuple) else (stream_hint, stream_hint)
    ntl = 'true' if _nt_l else 'false'
    nts = 'true' if _nt_s else 'false'
    use_i = uses_identifier(operation, 'i')
    set_ind = '_ind.set(i);' if needs_ind and uses_identifier(operation, '_ind') else ''
    # ``svec``: elements per staging access of the transposed operands (along
    # the rows), where that differs from the ``vec`` of the accesses along the
    # columns: a narrow array has room or alignment for vectors one way only
    if svec is None:
        svec = vec
    assert tile_r % svec == 0 and tile_c % vec == 0
    n_stage = (tile_r // svec) * tile_c         # staging vectors per tile
    n_work = tile_r * (tile_c // vec)           # compute vectors per tile
    assert n_stage % threads == 0 and n_work % threads == 0
    pitch = tile_c + 1                          # odd pitch: column walks spread over banks

    parts = [_param_decl(op) for op in operands if op.kind != 'indexer']
    parts += ['const %s _nr' % idx_t, 'const %s _nc' % idx_t]
    for op in arrays:
        parts += ['const %s _sr_%s' % (idx_t, op.name),
                  'const %s _sc_%s' % (idx_t, op.name)]
    if batched:
        assert not (use_i or set_ind) and not needs_ind
        parts += ['const %s _nbt' % idx_t, 'const %s _nb1' % idx_t]
        for op in arrays:
            parts += ['const %s _sb0_%s' % (idx_t, op.name),
                      'const %s _sb1_%s' % (idx_t, op.name)]
    parts += [_param_decl(op) for op in operands if op.kind == 'indexer']
    params = ', '.join(parts)

    c_ops = [op for op in arrays if layouts[op.name] == 'C']
    for op in c_ops:
        assert not op.is_out, 'transposed outputs are not handled by tiled2d'

    def gaddr(op, r, c):
        return '(_p_%s + %s(ptrdiff_t)(%s) * _sr_%s + (ptrdiff_t)(%s) * _sc_%s)' % (
            op.name, ('_o_%s + ' % op.name) if batched else '', r, op.name, c, op.name)

    src = [_header(typedefs, preamble)]
    src.append('extern "C" __global__ void __launch_bounds__(%d) %s(%s) {' % (
        threads, name, params))
    src.append('  %s;' % loop_prep)
    for op in c_ops:
        src.append('  __shared__ %s _t_%s[%d];' % (op.store_t, op.name, tile_r * pitch))
    src.append('  const %s _ntr = (_nr + %d) / %d;' % (idx_t, tile_r - 1, tile_r))
    src.append('  const %s _ntc = (_nc + %d) / %d;' % (idx_t, tile_c - 1, tile_c))
    if batched:
        src.append('  const %s _nt2 = _ntr * _ntc;' % idx_t)
        src.append('  for (%s _tile_q = blockIdx.x; _tile_q < _nt2 * _nbt; _tile_q += gridDim.x) {' % idx_t)
        src.append('    const %s _tile_b = %s;' % (idx_t, _die_by_die('_tile_q', '_nt2 * _nbt', idx_t, xcd)))
        if batch_first:
            # consecutive workgroups take the same tile of consecutive batch
            # entries: where those lie closer together in memory than the rows
            # of a tile, workgroups that run side by side share DRAM pages
            src.append('    const %s _tile = _tile_b / _nbt;' % idx_t)
            src.append('    const %s _bt = _tile_b - _tile * _nbt;' % idx_t)
        else:
            src.append('    const %s _bt = _tile_b / _nt2;' % idx_t)
            src.append('    const %s _tile = _tile_b - _bt * _nt2;' % idx_t)
        src.append('    const %s _b0 = _bt / _nb1;' % idx_t)
        src.append('    const %s _b1 = _bt - _b0 * _nb1;' % idx_t)
        for op in arrays:
            src.append('    const ptrdiff_t _o_%s = (ptrdiff_t)_b0 * _sb0_%s + (ptrdiff_t)_b1 * _sb1_%s;' % (
                op.name, op.name, op.name))
    else:
        src.append('  for (%s _tile_q = blockIdx.x; _tile_q < _ntr * _ntc; _tile_q += gridDim.x) {' % idx_t)
        src.append('    const %s _tile = %s;' % (idx_t, _die_by_die('_tile_q', '_ntr * _ntc', idx_t, xcd)))
    # Diagonal tile order: consecutive workgroups differ in both the row block
    # and the column block.  With power-of-two pitches, walking along one axis
    # only would keep the low address bits of either the transposed reads or the
    # row-major accesses identical across all concurrently running workgroups,
    # and with them the memory channel.
    if xcd and not batched:
        # Operands off the cache lines (odd pitches): neighbouring tiles share
        # the lines at their borders, along the rows in one operand and along
        # the columns in another.  A die walks strips `strip` tiles wide row by
        # row, so that the tiles it works on at one time are neighbours both
        # ways (odd pitches spread over the memory channels by themselves).
        src.append('    const %s _strip = _tile / (_ntr * %d);' % (idx_t, strip))
        src.append('    const %s _sw = (_ntc - _strip * %d < %d) ? (_ntc - _strip * %d) : %d;' % (
            idx_t, strip, strip, strip, strip))
        src.append('    const %s _sv = _tile - _strip * (_ntr * %d);' % (idx_t, strip))
        src.append('    const %s _tr = _sv / _sw;' % idx_t)
        src.append('    const %s _r0 = _tr * %d;' % (idx_t, tile_r))
        src.append('    const %s _c0 = (_strip * %d + (_sv - _tr * _sw)) * %d;' % (idx_t, strip, tile_c))
    else:
        src.append('    const %s _tr = _tile %% _ntr;' % idx_t)
        src.append('    const %s _r0 = _tr * %d;' % (idx_t, tile_r))
        src.append('    const %s _c0 = ((_tile / _ntr + _tr) %% _ntc) * %d;' % (idx_t, tile_c))
    src.append('    const bool _interior = (_r0 + %d <= _nr) && (_c0 + %d <= _nc);' % (
        tile_r, tile_c))
    # Row-major inputs of an interior tile are requested first of all, for every
    # trip of the consume loop at once: they are in flight while the transposed
    # operands are staged, and none of them waits behind a store.
    n_it = n_work // threads
    pre_ops = [op for op in arrays
               if layouts[op.name] == 'R' and ((not op.is_out) or op.read_out)]
    row_ops = [op for op in arrays
               if layouts[op.name] == 'R0' and ((not op.is_out) or op.read_out)]
    for op in pre_ops:
        src.append('    cupy::Vec<%s, %d> _pre_%s[%d];' % (op.store_t, vec, op.name, n_it))
    # per-row values travel with them: a load left to the consume loop would
    # only be issued after the wait for the vectors
    for op in row_ops:
        src.append('    %s _prer_%s[%d];' % (op.store_t, op.name, n_it))
    if pre_ops or row_ops:
        src.append('    if (_interior) {')
        src.append('#pragma unroll')
        src.append('      for (int _it = 0; _it < %d; ++_it) {' % n_it)
        src.append('        const int _w = threadIdx.x + _it * %d;' % threads)
        src.append('        const %s _r = _r0 + _w / %d;' % (idx_t, tile_c // vec))
        src.append('        const %s _c = _c0 + (_w %% %d) * %d;' % (idx_t, tile_c // vec, vec))
        for op in pre_ops:
            src.append('        _pre_%s[_it] = cupy::load_vec<%s, %d, %s>(%s);' % (
                op.name, op.store_t, vec, ntl, gaddr(op, '_r', '_c')))
        for op in row_ops:
            src.append('        _prer_%s[_it] = *%s;' % (op.name, gaddr(op, '_r', '0')))
        src.append('      }')
        src.append('    }')
    if c_ops and flat_stage:
        # ---- stage transposed operands whose tile is ONE contiguous piece of
        # memory (the tile spans their whole fast extent, and their lines follow
        # one another without gaps): vectors of ``flat_stage`` elements over the
        # piece, whatever the length of a line; element _f of the piece is row
        # _f %% tile_r of column _f / tile_r
        n_flat = -(-(tile_r * tile_c) // (flat_stage * threads))
        src.append('    {')
        src.append('      const int _limit = ((_nc - _c0 < %d) ? (int)(_nc - _c0) : %d) * %d;' % (
            tile_c, tile_c, tile_r))
        src.append('#pragma unroll')
        src.append('      for (int _it = 0; _it < %d; ++_it) {' % n_flat)
        src.append('        const int _f = (threadIdx.x + _it * %d) * %d;' % (threads, flat_stage))
        src.append('        if (_f + %d <= _limit) {' % flat_stage)
        for op in c_ops:
            src.append('          { const cupy::Vec<%s, %d> _lv = cupy::load_vec<%s, %d, %s>(%s + _f);' % (
                op.store_t, flat_stage, op.store_t, flat_stage, ntl, gaddr(op, '0', '_c0')))
            src.append('#pragma unroll')
            src.append('            for (int _k = 0; _k < %d; ++_k) { const int _lc = (_f + _k) / %d; '
                       '_t_%s[(_f + _k - _lc * %d) * %d + _lc] = _lv.v[_k]; } }' % (
                           flat_stage, tile_r, op.name, tile_r, pitch))
        src.append('        } else {')
        src.append('#pragma unroll')
        src.append('          for (int _k = 0; _k < %d; ++_k) if (_f + _k < _limit) {' % flat_stage)
        src.append('            const int _lc = (_f + _k) / %d;' % tile_r)
        for op in c_ops:
            src.append('            _t_%s[(_f + _k - _lc * %d) * %d + _lc] = (%s)[_f + _k];' % (
                op.name, tile_r, pitch, gaddr(op, '0', '_c0')))
        src.append('          }')
        src.append('        }')
        src.append('      }')
        src.append('    }')
        src.append('    __syncthreads();')
    elif c_ops:
        # ---- stage transposed operands: rows are the fast direction -------------------
        src.append('    if (_interior) {')
        src.append('#pragma unroll')
        src.append('      for (int _it = 0; _it < %d; ++_it) {' % (n_stage // threads))
        src.append('        const int _v = threadIdx.x + _it * %d;' % threads)
        src.append('        const int _lr = (_v %% %d) * %d;' % (tile_r // svec, svec))
        src.append('        const int _lc = _v / %d;' % (tile_r // svec))
        for op in c_ops:
            src.append('        { const cupy::Vec<%s, %d> _lv = cupy::load_vec<%s, %d, %s>(%s);' % (
                op.store_t, svec, op.store_t, svec, ntl, gaddr(op, '_r0 + _lr', '_c0 + _lc')))
            src.append('#pragma unroll')
            src.append('          for (int _k = 0; _k < %d; ++_k) '
                       '_t_%s[(_lr + _k) * %d + _lc] = _lv.v[_k]; }' % (svec, op.name, pitch))
        src.append('      }')
        src.append('    } else {')
        # edge tile: the same vectors where they lie inside the array, element by
        # element (under a test each) where they cross its border
        src.append('#pragma unroll')
        src.append('      for (int _it = 0; _it < %d; ++_it) {' % (n_stage // threads))
        src.append('        const int _v = threadIdx.x + _it * %d;' % threads)
        src.append('        const int _lr = (_v %% %d) * %d;' % (tile_r // svec, svec))
        src.append('        const int _lc = _v / %d;' % (tile_r // svec))
        src.append('        if (_c0 + _lc < _nc) {')
        src.append('          if (_r0 + _lr + %d <= _nr) {' % svec)
        for op in c_ops:
            src.append('            { const cupy::Vec<%s, %d> _lv = cupy::load_vec<%s, %d, %s>(%s);' % (
                op.store_t, svec, op.store_t, svec, ntl, gaddr(op, '_r0 + _lr', '_c0 + _lc')))
            src.append('#pragma unroll')
            src.append('              for (int _k = 0; _k < %d; ++_k) '
                       '_t_%s[(_lr + _k) * %d + _lc] = _lv.v[_k]; }' % (svec, op.name, pitch))
        src.append('          } else {')
        src.append('#pragma unroll')
        src.append('            for (int _k = 0; _k < %d; ++_k) if (_r0 + _lr + _k < _nr) {' % svec)
        for op in c_ops:
            src.append('              _t_%s[(_lr + _k) * %d + _lc] = *%s;' % (
                op.name, pitch, gaddr(op, '_r0 + _lr + _k', '_c0 + _lc')))
        src.append('            }')
        src.append('          }')
        src.append('        }')
        src.append('      }')
        src.append('    }')
        src.append('    __syncthreads();')

    # ---- consume: columns are the fast direction ----------------------------------------
    def full_load(op):
        lay = layouts[op.name]
        if lay == 'C':
            return '_t_%s[_lr * %d + _lc + _k]' % (op.name, pitch)
        if lay == 'R0':
            return '_b_%s' % op.name
        return '_l_%s.v[_k]' % op.name

    def full_store(op, value):
        return '_l_%s.v[_k] = %s;' % (op.name, value)

    src.append('    if (_interior) {')
    src.append('#pragma unroll')
    src.append('      for (int _it = 0; _it < %d; ++_it) {' % (n_work // threads))
    src.append('        const int _w = threadIdx.x + _it * %d;' % threads)
    src.append('        const int _lc = (_w %% %d) * %d;' % (tile_c // vec, vec))
    src.append('        const int _lr = _w / %d;' % (tile_c // vec))
    src.append('        const %s _r = _r0 + _lr;' % idx_t)
    src.append('        const %s _c = _c0 + _lc;' % idx_t)
    for op in arrays:
        lay = layouts[op.name]
        if lay == 'R':
            if (not op.is_out) or op.read_out:
                src.append('        cupy::Vec<%s, %d> _l_%s = _pre_%s[_it];' % (
                    op.store_t, vec, op.name, op.name))
            else:
                src.append('        cupy::Vec<%s, %d> _l_%s;' % (op.store_t, vec, op.name))
        elif lay == 'R0':
            if (not op.is_out) or op.read_out:
                src.append('        const %s _b_%s = _prer_%s[_it];' % (op.store_t, op.name, op.name))
            else:
                src.append('        const %s _b_%s = *%s;' % (
                    op.store_t, op.name, gaddr(op, '_r', '0')))
    src.append('#pragma unroll')
    src.append('        for (int _k = 0; _k < %d; ++_k) {' % vec)
    if use_i or set_ind:
        src.append('          const ptrdiff_t i = (ptrdiff_t)_r * _nc + _c + _k; %s' % set_ind)
    src.append(_element_code(operands, operation, full_load, full_store, 10))
    src.append('        }')
    for op in arrays:
        if op.is_out:
            src.append('        cupy::store_vec<%s, %d, %s>(%s, _l_%s);' % (
                op.store_t, vec, nts, gaddr(op, '_r', '_c'), op.name))
    src.append('      }')
    src.append('    } else {')

    def edge_load(op):
        lay = layouts[op.name]
        if lay == 'C':
            return '_t_%s[_lr * %d + _lc + _k]' % (op.name, pitch)
        return '(*%s)' % gaddr(op, '_r', '_c + _k')

    def edge_store(op, value):
        return '*%s = %s;' % (gaddr(op, '_r', '_c + _k'), value)

    src.append('#pragma unroll')
    src.append('      for (int _it = 0; _it < %d; ++_it) {' % (n_work // threads))
    src.append('        const int _w = threadIdx.x + _it * %d;' % threads)
    src.append('        const int _lc = (_w %% %d) * %d;' % (tile_c // vec, vec))
    src.append('        const int _lr = _w / %d;' % (tile_c // vec))
    src.append('        const %s _r = _r0 + _lr;' % idx_t)
    src.append('        const %s _c = _c0 + _lc;' % idx_t)
    src.append('        if (_r < _nr && _c + %d <= _nc) {' % vec)
    for op in arrays:
        lay = layouts[op.name]
        reads = (not op.is_out) or op.read_out
        if lay == 'R':
            if reads:
                src.append('          cupy::Vec<%s, %d> _l_%s = cupy::load_vec<%s, %d, %s>(%s);' % (
                    op.store_t, vec, op.name, op.store_t, vec, ntl, gaddr(op, '_r', '_c')))
            else:
                src.append('          cupy::Vec<%s, %d> _l_%s;' % (op.store_t, vec, op.name))
        elif lay == 'R0':
            src.append('          const %s _b_%s = *%s;' % (op.store_t, op.name, gaddr(op, '_r', '0')))
    src.append('#pragma unroll')
    src.append('          for (int _k = 0; _k < %d; ++_k) {' % vec)
    if use_i or set_ind:
        src.append('            const ptrdiff_t i = (ptrdiff_t)_r * _nc + _c + _k; %s' % set_ind)
    src.append(_element_code(operands, operation, full_load, full_store, 12))
    src.append('          }')
    for op in arrays:
        if op.is_out:
            src.append('          cupy::store_vec<%s, %d, %s>(%s, _l_%s);' % (
                op.store_t, vec, nts, gaddr(op, '_r', '_c'), op.name))
    src.append('        } else if (_r < _nr) {')
    src.append('#pragma unroll')
    src.append('          for (int _k = 0; _k < %d; ++_k) if (_c + _k < _nc) {' % vec)
    if use_i or set_ind:
        src.append('            const ptrdiff_t i = (ptrdiff_t)_r * _nc + _c + _k; %s' % set_ind)
    src.append(_element_code(operands, operation, edge_load, edge_store, 12))
    src.append('          }')
    src.append('        }')
    src.append('      }')
    src.append('    }')
    if c_ops:
        src.append('    __syncthreads();')
    src.append('  }')
    src.append('  %s;' % after_loop)
    src.append('}')
    return '\n'.join(src) + '\n'


def emit_packed(name, operands, operation, typedefs='', preamble='',
                loop_prep='', after_loop='', tile=(), in_order=(), staged=(),
                zero_last=(), zero_moving=(), vec=1, svec=1, group=1, ogroup=1,
                unit_first=True, threads=256, idx64=False, stream_hint=True, xcd=False, tile_order=None):
    """Kernel for an index space of ``len(tile)`` axes whose arrays are
    permuted differently, with a tile that spans SEVERAL axes: as many of the
    last axes as give the outputs a long contiguous run, and as many of the
    axes the ``staged`` inputs run fastest along (``in_order``, fastest first)
    as give those a long run too.  Small trailing axes -- a (B, 4, 3) array
    copied as (B, 3, 4), pairs or quadruples kept together under a
    permutation of the leading axes -- are then part of every tile instead of
    being its edges.

    A workgroup takes a tile in two passes.  First it reads the staged inputs in
    THEIR order, ``svec`` elements per access, and puts them into an LDS image
    of the tile that is laid out in the order of the outputs (padded so that
    lanes side by side spread over the banks).  Then it goes through the tile in
    the order of the outputs, ``vec`` elements per access: the other arrays
    (unit stride along the last axis, or zero for the inputs named in
    ``zero_last``; any stride along the others) come straight from memory, the
    staged ones from the image.

    ``group``: how many of the first axes of ``in_order`` lie in the staged
    inputs as ONE contiguous piece within a tile (each but the last of them
    spanned whole, each starting where the one before ends): the accesses of
    ``svec`` elements then run over that piece as a whole, whatever the extents
    of its axes, and every element finds its own place in the image.
    ``unit_first``: every staged input has unit stride along ``in_order[0]``
    (else ``svec`` and ``group`` are 1 and the stride is applied).  ``ogroup``:
    the same for the last axes and the arrays of the second pass; the inputs of
    ``zero_last`` give one value per access, those also named in
    ``zero_moving`` (a value per row under a piece of several rows) one per
    element.  At the border of
    the array a piece is shorter, never split: only its last axis can be cut.

    ``tile[a]`` elements along axis a; tiles are numbered along the axes of
    ``tile_order``, fastest first (default: the order of the outputs; ``xcd``:
    die by die, see ``_die_by_die``).  Kernel parameters after the operands: the
    extents ``_e<a>``, then per array its strides ``_s<a>_<name>`` in elements.
    The element index ``i`` and the indexer are not available.
    """
    nd = len(tile)
    idx_t = 'ptrdiff_t' if idx64 else 'int'
    arrays = [op for op in operands if op.kind == 'array']
    assert not any(op.kind == 'indexer' for op in operands)
    _nt_l, _nt_s = stream_hint if isinstance(stream_hint, tuple) else (stream_hint, stream_hint)
    ntl = 'true' if _nt_l else 'false'
    nts = 'true' if _nt_s else 'false'
    s_ops = [op for op in arrays if op.name in staged]
    d_ops = [op for op in arrays if op.name not in staged]
    for op in s_ops:
        assert not op.is_out
    assert unit_first or (svec == 1 and group == 1)
    volume = 1
    for t in tile:
        volume *= t
    out_order = list(range(nd - 1, -1, -1))
    # position of an element in the image: its number in the order of the outputs
    lds_step = [1] * nd
    for a in range(nd - 2, -1, -1):
        lds_step[a] = lds_step[a + 1] * tile[a + 1]
    # Lanes side by side in the first pass are ``quantum`` words apart in the
    # image (the step of the axis they differ in): a step that is a multiple of
    # eight gets one pad word per step, which makes it odd and spreads the lanes
    # over the banks
    quantum = 0
    if s_ops:
        for n, a in enumerate(in_order):
            if tile[a] > (svec if n == 0 else 1):
                step = lds_step[a] * (svec if n == 0 and tile[a] % svec == 0 else 1)
                if step % 8 == 0:
                    quantum = step
                break
    padded = volume + (volume // quantum if quantum else 0) + 1

    def pad(expr):
        if not quantum:
            return '(%s)' % expr
        return '((%s) + (%s) / %d)' % (expr, expr, quantum)

    def unroll(trips):
        return '#pragma unroll' if trips <= 16 else '#pragma unroll 4'

    parts = [_param_decl(op) for op in operands]
    parts += ['const %s _e%d' % (idx_t, a) for a in range(nd)]
    for op in arrays:
        parts += ['const %s _s%d_%s' % (idx_t, a, op.name) for a in range(nd)]
    src = [_header(typedefs, preamble)]
    src.append('extern "C" __global__ void __launch_bounds__(%d) %s(%s) {' % (
        threads, name, ', '.join(parts)))
    src.append('  %s;' % loop_prep)
    for op in s_ops:
        src.append('  __shared__ %s _t_%s[%d];' % (op.store_t, op.name, padded))
    for a in range(nd):
        src.append('  const %s _nt%d = (_e%d + %d) / %d;' % (idx_t, a, a, tile[a] - 1, tile[a]))
    src.append('  const %s _ntiles = %s;' % (idx_t, ' * '.join('_nt%d' % a for a in range(nd))))
    src.append('  for (%s _tile = blockIdx.x; _tile < _ntiles; _tile += gridDim.x) {' % idx_t)
    src.append('    %s _q = %s;' % (idx_t, _die_by_die('_tile', '_ntiles', idx_t, xcd)))
    tile_order = list(tile_order) if tile_order else out_order
    for a in tile_order[:-1]:
        src.append('    const %s _o%d = (_q %% _nt%d) * %d; _q /= _nt%d;' % (idx_t, a, a, tile[a], a))
    src.append('    const %s _o%d = _q * %d;' % (idx_t, tile_order[-1], tile[tile_order[-1]]))
    src.append('    const bool _interior = %s;' % ' && '.join(
        '(_o%d + %d <= _e%d)' % (a, tile[a], a) for a in range(nd)))
    for op in arrays:
        src.append('    %s%s* const _b_%s = _p_%s + %s;' % (
            'const ' if (op.is_const and not op.is_out) else '', op.store_t, op.name, op.name,
            ' + '.join('(ptrdiff_t)_o%d * _s%d_%s' % (a, a, op.name) for a in range(nd))))

    def one_pass(order, n_group, width, prefix):
        """Code that numbers the accesses of a pass: ``_g`` where an access
        starts within the contiguous piece of the first ``n_group`` axes of
        ``order``, ``<prefix><a>`` the index along each other axis, ``_len``
        the length of the piece in this tile.  Returns (axes of the piece,
        other axes, slots, trips)."""
        g_axes = list(order[:n_group])
        rest = list(order[n_group:])
        g_len = 1
        for a in g_axes:
            g_len *= tile[a]
        # (a piece that is no whole number of accesses ends in a partial one,
        # which goes element by element like those at the border of the array)
        per = -(-g_len // width)
        slots = (volume // g_len) * per
        trips = -(-slots // threads)
        cut = g_axes[-1]
        src.append('    const int _len%s = %d * (int)((_e%d - _o%d < %d) ? (_e%d - _o%d) : %d);' % (
            prefix, g_len // tile[cut], cut, cut, tile[cut], cut, cut, tile[cut]))
        src.append(unroll(trips))
        src.append('    for (int _it = 0; _it < %d; ++_it) {' % trips)
        src.append('      const int _v = threadIdx.x + _it * %d;' % threads)
        src.append('      const int _g = (_v %% %d) * %d; int _r = _v / %d;' % (per, width, per))
        src.append('      const int _first = _r * %d + _g;' % g_len)
        for n, a in enumerate(rest):
            if tile[a] == 1:
                src.append('      const int %s%d = 0;' % (prefix, a))
            elif n == len(rest) - 1:
                src.append('      const int %s%d = _r;' % (prefix, a))
            else:
                src.append('      const int %s%d = _r %% %d; _r /= %d;' % (prefix, a, tile[a], tile[a]))
        return g_axes, rest, slots, trips

    def split(g_axes, expr):
        """Indices along the axes of a piece of its element number ``expr``."""
        out = {}
        left = expr
        for n, a in enumerate(g_axes):
            if tile[a] == 1:
                out[a] = '0'
            elif n == len(g_axes) - 1:
                out[a] = '(%s)' % left
            else:
                out[a] = '((%s) %% %d)' % (left, tile[a])
                left = '(%s) / %d' % (left, tile[a])
        return out

    def rest_offset(op, rest, prefix):
        terms = ['(ptrdiff_t)%s%d * _s%d_%s' % (prefix, a, a, op.name) for a in rest if tile[a] > 1]
        return ' + '.join(terms) if terms else '0'

    def rest_inside(rest, prefix):
        return ' && '.join('(_o%d + %s%d < _e%d)' % (a, prefix, a, a)
                           for a in rest if tile[a] > 1) or 'true'

    if s_ops:
        # ---- first pass: the staged inputs in their own order --------------------------------
        g_axes, rest, slots, trips = one_pass(in_order, group, svec, '_i')
        src.append('      const int _pos = %s;' % (
            ' + '.join('_i%d * %d' % (a, lds_step[a]) for a in rest if tile[a] > 1) or '0'))

        def image(expr):
            idx = split(g_axes, expr)
            terms = ['%s * %d' % (idx[a], lds_step[a]) for a in g_axes if tile[a] > 1]
            return pad(' + '.join(['_pos'] + terms))

        def within(op, expr):
            if unit_first:
                return expr
            idx = split(g_axes, expr)
            return ' + '.join('(ptrdiff_t)%s * _s%d_%s' % (idx[a], a, op.name)
                              for a in g_axes if tile[a] > 1) or '0'
        guard = '' if slots % threads == 0 else '_v < %d && ' % slots
        src.append('      if (%s(_interior || (%s))) {' % (guard, rest_inside(rest, '_i')))
        src.append('        if (_g + %d <= _len_i) {' % svec)
        for op in s_ops:
            src.append('          { const cupy::Vec<%s, %d> _lv = cupy::load_vec<%s, %d, %s>(%s + %s + %s);' % (
                op.store_t, svec, op.store_t, svec, ntl, '_b_' + op.name,
                rest_offset(op, rest, '_i'), within(op, '_g')))
            src.append('#pragma unroll')
            src.append('            for (int _k = 0; _k < %d; ++_k) _t_%s[%s] = _lv.v[_k]; }' % (
                svec, op.name, image('_g + _k')))
        if svec > 1:
            src.append('        } else {')
            src.append('#pragma unroll')
            src.append('          for (int _k = 0; _k < %d; ++_k) if (_g + _k < _len_i) {' % svec)
            for op in s_ops:
                src.append('            _t_%s[%s] = (%s + %s)[%s];' % (
                    op.name, image('_g + _k'), '_b_' + op.name, rest_offset(op, rest, '_i'),
                    within(op, '_g + _k')))
            src.append('          }')
        src.append('        }')
        src.append('      }')
        src.append('    }')
        src.append('    __syncthreads();')

    # ---- second pass: the tile in the order of the outputs ---------------------------------------
    g_axes, rest, slots, trips = one_pass(out_order, ogroup, vec, '_j')
    src.append('      const int _pos = _first;')
    guard = '' if slots % threads == 0 else '_v < %d && ' % slots

    def address(op):
        return '(_b_%s + %s)' % (op.name, rest_offset(op, rest, '_j'))

    # inputs with zero stride along the last axis: one value per access where
    # they do not move along the other axes of the piece either (``_s<a>`` may
    # be anything there: the host says which), else one per element
    def zero_value(op):
        if op.name not in zero_moving:
            return '_z_%s' % op.name
        idx = split(g_axes, '_g + _k')
        terms = ['(ptrdiff_t)%s * _s%d_%s' % (idx[a], a, op.name)
                 for a in g_axes[1:] if tile[a] > 1]
        return '%s[%s]' % (address(op), ' + '.join(terms) or '0')

    def full_load(op):
        if op.name in staged:
            return '_t_%s[%s]' % (op.name, pad('_pos + _k'))
        if op.name in zero_last:
            return zero_value(op)
        return '_l_%s.v[_k]' % op.name

    def full_store(op, value):
        return '_l_%s.v[_k] = %s;' % (op.name, value)

    def edge_load(op):
        if op.name in staged:
            return '_t_%s[%s]' % (op.name, pad('_pos + _k'))
        if op.name in zero_last:
            return zero_value(op)
        return '%s[_g + _k]' % address(op)

    def edge_store(op, value):
        return '%s[_g + _k] = %s;' % (address(op), value)

    src.append('      if (%s(_interior || (%s))) {' % (guard, rest_inside(rest, '_j')))
    for op in d_ops:
        if op.name in zero_last and op.name not in zero_moving:
            src.append('        const %s _z_%s = *%s;' % (op.store_t, op.name, address(op)))
    src.append('        if (_g + %d <= _len_j) {' % vec)
    for op in d_ops:
        if op.name in zero_last:
            continue
        if (not op.is_out) or op.read_out:
            src.append('          cupy::Vec<%s, %d> _l_%s = cupy::load_vec<%s, %d, %s>(%s + _g);' % (
                op.store_t, vec, op.name, op.store_t, vec, ntl, address(op)))
        else:
            src.append('          cupy::Vec<%s, %d> _l_%s;' % (op.store_t, vec, op.name))
    src.append('#pragma unroll')
    src.append('          for (int _k = 0; _k < %d; ++_k) {' % vec)
    src.append(_element_code(operands, operation, full_load, full_store, 12))
    src.append('          }')
    for op in d_ops:
        if op.is_out:
            src.append('          cupy::store_vec<%s, %d, %s>(%s + _g, _l_%s);' % (
                op.store_t, vec, nts, address(op), op.name))
    if vec > 1:
        src.append('        } else {')
        src.append('#pragma unroll')
        src.append('          for (int _k = 0; _k < %d; ++_k) if (_g + _k < _len_j) {' % vec)
        src.append(_element_code(operands, operation, edge_load, edge_store, 12))
        src.append('          }')
    src.append('        }')
    src.append('      }')
    src.append('    }')
    if s_ops:
        src.append('    __syncthreads();')
    src.append('  }')
    src.append('  %s;' % after_loop)
    src.append('}')
    return '\n'.join(src) + '\n'
