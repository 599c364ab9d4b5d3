"""ElementwiseKernel, ufunc and their shared host machinery.

Public behaviour follows the reference's cupy/_core/_kernel.pyx
(ParameterInfo :464-525, type resolution :557-604, broadcasting :607-640,
output handling :646-706, ElementwiseKernel :743-1002, ufunc :1147-1493,
loop selection :1532-1753); what happens below the call surface -- stride
canonicalisation into launch plans, the HIP emitters, argument packing -- is
specific to this implementation.
"""
import math
import struct
import threading
import warnings

import numpy

from cupy_amd._core import _carray
from cupy_amd._core import _codegen_elementwise as _cg
from cupy_amd._core import _fusion_thread_local
from cupy_amd._core import _launch_plan
from cupy_amd._core import _scalar
from cupy_amd._core import _tuning
from cupy_amd._core import internal
from cupy_amd._core._dtype import get_dtype, _raise_if_invalid_cast
from cupy_amd._core._scalar import CScalar, get_typename as _get_typename
from cupy_amd._core.core import ndarray, _convert_from_cupy_like
from cupy_amd.cuda import compiler
from cupy_amd.cuda import device as _device
from cupy_amd.cuda import stream as _stream

_INT32_MAX = (1 << 31) - 1


# ---------------------------------------------------------------------------------
# parameters and type placeholders
# ---------------------------------------------------------------------------------

class ParameterInfo:
    """One entry of an ``in_params`` / ``out_params`` string:
    ``[raw] [_non_const] <dtype name | single-letter placeholder> <name>``
    (reference: cupy/_core/_kernel.pyx:464-518; same attributes, same errors)."""

    # what a leading keyword sets
    _KEYWORDS = {'raw': ('raw', True), '_non_const': ('is_const', False)}

    def __init__(self, param, is_const):
        words = param.split()
        if len(words) < 2:
            raise Exception('Syntax error: %s' % param)
        *keywords, type_word, self.name = words
        self.dtype, self.ctype = self._read_type(type_word)
        self.raw = False
        self.is_const = is_const
        for word in keywords:
            if word not in self._KEYWORDS:
                raise Exception('Unknown keyword "%s"' % word)
            attribute, value = self._KEYWORDS[word]
            setattr(self, attribute, value)

    @staticmethod
    def _read_type(word):
        """(dtype, C type name) of the type word: the indexer pseudo-type has
        neither, a single letter is a placeholder bound at call time, anything
        else names a dtype."""
        if word == 'CIndexer':
            return None, None
        if len(word) == 1:
            return None, word
        dtype = get_dtype(word)
        return dtype, _get_typename(dtype)

    def _key(self):
        return (self.name, self.dtype, self.ctype, self.raw, self.is_const)

    def __hash__(self):
        return hash(self._key())

    def __eq__(self, other):
        return isinstance(other, ParameterInfo) and self._key() == other._key()

    def __repr__(self):
        return '<ParameterInfo name=%r dtype=%r ctype=%r raw=%r is_const=%r>' % (
            self._key())


_param_info_memo = {}


def _get_param_info(s, is_const):
    """Tuple of ParameterInfo for a comma-separated parameter string (memoised)."""
    try:
        return _param_info_memo[s, is_const]
    except KeyError:
        pass
    entries = s.strip().split(',') if s else ()
    infos = _param_info_memo[s, is_const] = tuple(
        ParameterInfo(entry, is_const) for entry in entries)
    return infos


class _TypeMap:
    """Resolved type placeholders: pairs (placeholder, dtype)."""

    def __init__(self, pairs):
        self._pairs = tuple(pairs)

    def __hash__(self):
        return hash(self._pairs)

    def __eq__(self, other):
        return isinstance(other, _TypeMap) and self._pairs == other._pairs

    def __str__(self):
        return '<_TypeMap {}>'.format(self._pairs)

    def get_typedef_code(self):
        return ''.join('typedef %s %s;\n' % (_get_typename(t), name)
                       for name, t in self._pairs)


def _decide_params_type_core(in_params, out_params, in_args_dtype, out_args_dtype):
    """Binds single-letter type placeholders from the dtypes of the array
    arguments (outputs first) and checks fixed-dtype parameters (reference:
    cupy/_core/_kernel.pyx:557-604; same error texts)."""
    bound = {}

    def settle(param, given, as_dtype):
        # a parameter of fixed dtype only has to agree with the argument; a
        # placeholder takes the first dtype it meets and must meet no other
        if param.dtype is not None:
            if as_dtype(given) != as_dtype(param.dtype):
                raise TypeError('Type is mismatched. %s %s %s' % (
                    param.name, given, param.dtype))
            return
        known = bound.setdefault(param.ctype, given)
        if as_dtype(known) != as_dtype(given):
            raise TypeError('Type is mismatched. %s %s %s %s' % (
                param.name, given, known, param.ctype))

    if out_args_dtype:
        assert len(out_params) == len(out_args_dtype)
        for param, given in zip(out_params, out_args_dtype):
            if given is None:
                raise TypeError('Output arguments must be cupy.ndarray')
            settle(param, given, get_dtype)
    assert len(in_params) == len(in_args_dtype)
    for param, given in zip(in_params, in_args_dtype):
        if given is not None:           # (scalars take the type they are given)
            settle(param, given, numpy.dtype)

    def resolved(params):
        return tuple(bound[p.ctype] if p.dtype is None else p.dtype for p in params)
    return resolved(in_params), resolved(out_params), _TypeMap(sorted(bound.items()))


_decide_memo = {}


def _decide_params_type(in_params, out_params, in_args_dtype, out_args_dtype):
    key = (in_params, out_params, in_args_dtype, out_args_dtype)
    ret = _decide_memo.get(key)
    if ret is None:
        ret = _decide_params_type_core(
            in_params, out_params, in_args_dtype, out_args_dtype)
        _decide_memo[key] = ret
    return ret


# ---------------------------------------------------------------------------------
# argument handling
# ---------------------------------------------------------------------------------

def _check_peer_access(arr, device_id):
    if arr.data.device_id == device_id:
        return
    raise ValueError(
        'The device where the array resides ({}) is different from the current '
        'device ({}). Peer access is unavailable between these devices.'.format(
            arr.data.device_id, device_id))


def _preprocess_arg(dev_id, arg):
    if type(arg) is ndarray:
        s = arg
    else:
        s = _convert_from_cupy_like(arg, error=False)
    if s is not None:
        if s.data.device_id != dev_id:
            _check_peer_access(s, dev_id)
        return s
    return CScalar(arg)


def _preprocess_args(dev_id, args):
    return [_preprocess_arg(dev_id, a) for a in args]


def _preprocess_optional_args(dev_id, args):
    return [None if a is None else _preprocess_arg(dev_id, a) for a in args]


def _broadcast(args, params, use_size):
    """Broadcasts the arrays of ``args`` that take part in the loop (arrays of
    parameters not marked ``raw``) against each other; everything else passes
    through.  Returns (new args, loop shape).  ``use_size``: the caller gave
    ``size=``, which is allowed exactly when no array takes part (reference:
    cupy/_core/_kernel.pyx:607-640)."""
    looped = [i for i, (a, p) in enumerate(zip(args, params))
              if isinstance(a, ndarray) and not p.raw]
    if use_size and looped:
        raise ValueError('Specified \'size\' can be used only '
                         'if all of the ndarray are \'raw\'.')
    if not use_size and not looped:
        raise ValueError('Loop size is undecided.')
    views = [None] * len(args)
    for i in looped:
        views[i] = args[i]
    shape = internal._broadcast_core(views)      # (replaces the arrays by views)
    return [a if v is None else v for a, v in zip(args, views)], shape


def _get_out_args_from_optionals(subtype, out_args, out_types, out_shape, casting, obj):
    out_args = list(out_args)
    while len(out_args) < len(out_types):
        out_args.append(None)
    for i, a in enumerate(out_args):
        if a is None:
            arr = ndarray._new_contiguous(out_shape, out_types[i])
            if subtype is not ndarray:
                arr = arr._retype(subtype, obj)
            out_args[i] = arr
            continue
        if not isinstance(a, ndarray):
            raise TypeError('Output arguments type must be cupy.ndarray')
        if a._shape != out_shape:
            raise ValueError('Out shape is mismatched')
        out_type = get_dtype(out_types[i])
        _raise_if_invalid_cast(out_type, a.dtype, casting, 'output operand')
    return out_args


def _copy_in_args_if_needed(in_args, out_args):
    """Inputs that overlap an explicit output (without being that very array)
    are copied first, so the kernel never reads what it has already written."""
    for i, a in enumerate(in_args):
        if isinstance(a, ndarray):
            for out in out_args:
                if a is not out and _carray.may_share_bounds(a, out):
                    in_args[i] = a.copy()
                    break


def _get_out_args_with_params(out_args, out_types, out_shape, out_params,
                              is_size_specified):
    if not out_args:
        for p in out_params:
            if p.raw and not is_size_specified:
                raise ValueError('Output array size is Undecided')
        return [ndarray._new_contiguous(out_shape, t) for t in out_types]
    for a, p in zip(out_args, out_params):
        if not isinstance(a, ndarray):
            raise TypeError('Output arguments type must be cupy.ndarray')
        if not p.raw and a._shape != out_shape:
            raise ValueError('Out shape is mismatched')
    return out_args


# ---------------------------------------------------------------------------------
# launch plans
# ---------------------------------------------------------------------------------

def _canonical_dims(arrays, shape):
    """Merges axes that every array walks back to back and drops unit axes.
    Returns (shape, [strides per array]) of the equivalent smaller problem."""
    return _merge_axes(shape, [a._strides for a in arrays])


def _merge_axes(shape, strides):
    """``_canonical_dims`` for a shape and the strides of every array along it."""
    cshape = []
    cstrides = [[] for _ in strides]
    for d, ext in enumerate(shape):
        if ext == 1:
            continue
        if cshape:
            for cs, st in zip(cstrides, strides):
                if cs[-1] != st[d] * ext:
                    break
            else:
                cshape[-1] *= ext
                for cs, st in zip(cstrides, strides):
                    cs[-1] = st[d]
                continue
        cshape.append(ext)
        for cs, st in zip(cstrides, strides):
            cs.append(st[d])
    return tuple(cshape), [tuple(cs) for cs in cstrides]


def _max_vector_width(itemsizes):
    """Elements per thread such that the narrowest operand moves 16 bytes and
    the widest at most 64."""
    v = 16 // min(itemsizes)
    while v > 1 and v * max(itemsizes) > 64:
        v //= 2
    return max(v, 1)


def _aligned(value, nbytes):
    """Whether vector accesses of ``nbytes`` may start at the address (or be
    spaced by the byte stride) ``value``.  The device takes such accesses at
    the alignment of one element, which every array has."""
    return value % nbytes == 0 or _tuning.get('unaligned_vectors')


_grid_limit_memo = {}


def _grid_limit(dev_id, blocks_per_cu):
    key = (dev_id, blocks_per_cu)
    g = _grid_limit_memo.get(key)
    if g is None:
        g = _device.get_compute_units(dev_id) * blocks_per_cu
        _grid_limit_memo[key] = g
    return g


def _off_lines(arrays, strides):
    """Whether an array starts inside a 128-byte line, or has a stride of more
    than a line that is no whole number of lines: tiles then share the lines at
    their borders."""
    return any(
        a.data.ptr % 128 or any(abs(c) >= 128 and c % 128 for c in cs)
        for a, cs in zip(arrays, strides))


def _max_blocks(block):
    """Most workgroups of ``block`` work-items one grid dimension may hold: a
    dispatch carries its size in work-items in 32 bits per dimension."""
    return min(0x7fffffff, 0xffffffff // block)


class _ElementwisePlanner:
    """Builds, memoises and launches the kernels of one elementwise operation
    (an ElementwiseKernel, or one loop of a ufunc)."""

    def __init__(self, name, params, operation, preamble, loop_prep, after_loop,
                 options, is_ufunc):
        self.name = name
        self.params = params          # ParameterInfo of inputs + outputs
        self.operation = operation
        self.preamble = preamble
        self.loop_prep = loop_prep
        self.after_loop = after_loop
        self.options = tuple(options)
        self.is_ufunc = is_ufunc
        self._memo = {}
        self._codes = {}
        self._lock = threading.Lock()
        self._force_generic = _cg.body_needs_generic(operation) or \
            _cg.body_needs_generic(loop_prep) or _cg.body_needs_generic(after_loop)
        self._uses_ind = _cg.uses_identifier(operation, '_ind') or \
            _cg.uses_identifier(loop_prep, '_ind') or \
            _cg.uses_identifier(after_loop, '_ind')
        self._uses_i = _cg.uses_identifier(operation, 'i')
        # False: the kernel sees the axes of the broadcast arguments as they
        # are (``reduce_dims=False``): no axes are merged, ``_ind`` and the
        # arrays keep their number of dimensions
        self.reduce_dims = True

    # One operand description per kernel parameter -------------------------------------
    def _make_operands(self, args, nin, var_types, casts, force_read_out):
        ops = []
        for idx, (p, a) in enumerate(zip(self.params, args)):
            is_out = idx >= nin
            if isinstance(a, ndarray):
                store_t = _get_typename(a.dtype)
                if p.raw:
                    ops.append(_cg.Operand(
                        'raw', p.name, store_t, ndim=a.ndim,
                        c_contiguous=a._c_contiguous, index_32=a._index_32_bits,
                        is_const=p.is_const, is_out=is_out))
                else:
                    cast_in, cast_out = casts[idx] if casts else (None, None)
                    read_out = False
                    if is_out:
                        read_out = force_read_out or not _cg.output_is_write_only(
                            self.operation, p.name)
                    elif not p.is_const:
                        # a `_non_const` input is written by the body
                        is_out = True
                        read_out = True
                    ops.append(_cg.Operand(
                        'array', p.name, store_t, var_types[idx], is_out=is_out,
                        read_out=read_out, cast_in=cast_in, cast_out=cast_out,
                        ndim=a.ndim, c_contiguous=a._c_contiguous,
                        index_32=a._index_32_bits, is_const=p.is_const))
            else:
                ops.append(_cg.Operand(
                    'scalar', p.name, _get_typename(a.descr), is_const=True))
        return ops

    def launch(self, dev_id, args, nin, shape, var_types, typedefs, casts=None,
               force_generic=False, force_read_out=False, stream=None,
               block_size=None, kernel_name=None, rec=None):
        """Plans and launches.  ``args``: preprocessed inputs then outputs
        (ndarrays already broadcast to ``shape``, CScalars already typed).
        ``rec``: optional recorder of the launch; argument ``i`` is ref ``i``."""
        params = self.params
        arrays = [a for a, p in zip(args, params)
                  if isinstance(a, ndarray) and not p.raw]
        size = internal.prod(shape)
        stream_ptr = _stream.get_current_stream_ptr() if stream is None else stream.ptr
        mode = 'generic'
        cshape = cstrides = None
        if arrays and any(a.dtype.kind == 'V' for a in arrays):
            # elements that are structures go one by one through the indexer
            # kernel (the vector helpers want element sizes that are powers of two)
            force_generic = True
        if not self.reduce_dims:
            force_generic = True
        if not (force_generic or self._force_generic) and arrays:
            cshape, cstrides = _canonical_dims(arrays, shape)
            nd = len(cshape)
            if nd >= 3 and not self._uses_i and not self._uses_ind and _tuning.get(
                    'order_by_outputs'):
                # An elementwise operation may visit its elements in any order:
                # the axes are taken in the order the OUTPUTS are stored in, so
                # that a permuted destination (dst.transpose(...)[...] = x) is
                # the array that is walked along its memory, and x the permuted one
                outs = args[nin:]
                ref = next((cs for a, cs in zip(arrays, cstrides)
                            if any(a is o for o in outs)), None)
                if ref is not None:
                    order = sorted(range(nd), key=lambda ax: -abs(ref[ax]))
                    if order != list(range(nd)):
                        cshape, cstrides = _merge_axes(
                            [cshape[ax] for ax in order],
                            [[cs[ax] for ax in order] for cs in cstrides])
                        nd = len(cshape)
            if nd <= 1:
                ok = True
                for a, cs in zip(arrays, cstrides):
                    if nd == 1 and cs[0] != a.dtype.itemsize and cs[0] != 0:
                        ok = False
                        break
                if ok:
                    mode = 'flat'
                elif not self._uses_ind:
                    # one axis with a stride: a matrix of one row
                    plan = self._plan_rows2d(
                        arrays, (1, cshape[0]), [(0, cs[0]) for cs in cstrides], args, nin)
                    if plan is not None and plan[0][0] == 1:
                        return self._launch_rows2d(
                            dev_id, args, nin, arrays, plan, var_types, typedefs, casts,
                            force_read_out, stream_ptr, kernel_name, rec)
            elif nd == 2 and not self._uses_ind:
                part = self._plan_flat_bcast(arrays, cshape, cstrides, args, nin)
                if part is not None:
                    return self._launch_flat(
                        dev_id, args, nin, arrays, cstrides, size, var_types, typedefs,
                        casts, force_read_out, stream_ptr, kernel_name, rec,
                        partial=part, nc=cshape[1])
                # rows of a few one- or two-byte elements that do not follow one
                # another without gaps (windows of narrow matrices): tiles of many
                # rows, the inputs staged through the LDS, the outputs written as
                # one piece (float16 (11184809, 6), x[:-1, :-1] - x[1:, 1:]: 99 us
                # row by row, 65 so; four- and eight-byte elements gain nothing)
                if (not self._uses_i and _tuning.get('packed_tiles')
                        and min(a.dtype.itemsize for a in arrays) < 4
                        and cshape[1] * max(a.dtype.itemsize for a in arrays)
                        < _tuning.get('packed_short_rows_bytes')):
                    packed = self._plan_packed(arrays, cshape, cstrides, args, nin)
                    if packed is not None:
                        return self._launch_packed(
                            dev_id, args, nin, arrays, cshape, cstrides, packed, var_types,
                            typedefs, casts, force_read_out, stream_ptr, kernel_name, rec)
                plan = self._plan_rows2d(arrays, cshape, cstrides, args, nin)
                if plan is not None:
                    return self._launch_rows2d(
                        dev_id, args, nin, arrays, plan, var_types, typedefs, casts,
                        force_read_out, stream_ptr, kernel_name, rec)
                mode = self._classify_2d(arrays, cstrides, args, nin)
            elif 3 <= nd <= 6 and not self._uses_ind and not self._uses_i:
                plan = None
                if nd <= 4:
                    plan = self._plan_rows_nd(arrays, cshape, cstrides, args, nin)
                    if plan is not None:
                        return self._launch_rows2d(
                            dev_id, args, nin, arrays, plan, var_types, typedefs, casts,
                            force_read_out, stream_ptr, kernel_name, rec)
                    plan = self._plan_batched(arrays, cshape, cstrides, args, nin)
                # Tiles over several axes (emit_packed) where tiles of two axes
                # would be small or narrow: those are mostly edge, or one tile per
                # small matrix (2^26 float32 over rotating buffers, us, tiles of
                # two axes / of several: (2^20, 8, 8) with its matrices transposed
                # 1591 / 86; (2^18, 16, 16) 340 / 86; (4, 2^22, 4) reversed
                # 6271 / 102; large tiles of two axes stay ahead: (256, 512, 512)
                # as (0, 2, 1) 87 / 94, as (2, 1, 0) 94 / 112)
                mode_p = _tuning.get('packed_tiles')
                # (rows shorter than a tile of two axes is wide make every such
                # tile an edge tile, which goes element by element)
                if mode_p and not (mode_p == 'auto' and plan is not None
                                   and plan[0][0] * plan[0][1] >= _tuning.get('packed_tiles_below')
                                   and min(plan[0]) >= 16 and plan[0][1] >= 64):
                    packed = self._plan_packed(arrays, cshape, cstrides, args, nin)
                    if packed is not None:
                        return self._launch_packed(
                            dev_id, args, nin, arrays, cshape, cstrides, packed, var_types,
                            typedefs, casts, force_read_out, stream_ptr, kernel_name, rec)
                if plan is not None:
                    done = self._launch_tiled(
                        dev_id, args, nin, arrays, plan[0], plan[1], var_types, typedefs,
                        casts, force_read_out, stream_ptr, kernel_name, False, rec,
                        batch=plan[2])
                    if done is not None:
                        return
        if mode == 'flat':
            return self._launch_flat(
                dev_id, args, nin, arrays, cstrides, size, var_types, typedefs,
                casts, force_read_out, stream_ptr, kernel_name, rec)
        if mode in ('tiled', 'tiled_t'):
            done = self._launch_tiled(
                dev_id, args, nin, arrays, cshape, cstrides, var_types, typedefs,
                casts, force_read_out, stream_ptr, kernel_name, mode == 'tiled_t',
                rec)
            if done is not None:
                return
        return self._launch_generic(
            dev_id, args, nin, shape, var_types, typedefs, casts, force_read_out,
            stream_ptr, block_size or 128, kernel_name, rec)

    def _plan_flat_bcast(self, arrays, cshape, cstrides, args, nin):
        """Matrix problem whose full-size arrays are all stored row after row
        without gaps and whose other arrays hold a value per row or a value per
        column: {parameter name: ('row' | 'col', byte stride)} for the latter,
        None when the problem is not of this kind."""
        if not _tuning.get('flat_bcast'):
            return None
        nc = cshape[1]
        names = [p.name for a, p in zip(args, self.params)
                 if isinstance(a, ndarray) and not p.raw]
        outs = args[nin:]
        part = {}
        n_full = 0
        for a, cs, nm in zip(arrays, cstrides, names):
            item = a.dtype.itemsize
            if cs[1] == item and cs[0] == nc * item:
                n_full += 1
                continue
            if any(a is o for o in outs) or cs[0] % item or cs[1] % item:
                return None
            if cs[1] == 0:
                kind = ('row', cs[0])
            elif cs[0] == 0:
                kind = ('col1' if cs[1] == item else 'col', cs[1])
            else:
                return None
            if part.get(nm, kind) != kind:
                return None       # the same parameter name twice: not expected
            part[nm] = kind
        if not n_full or not part:
            return None
        return part

    def _plan_rows2d(self, arrays, cshape, cstrides, args, nin):
        """Matrix problem in which no array runs against the columns: every
        output has unit stride along the columns, every input unit, zero or a
        small stride.  Returns (shape, strides per array, kinds per parameter
        name), with the two axes swapped when that is what makes it fit (all
        arrays stored column after column), or None."""
        if not _tuning.get('rows2d'):
            return None
        names = [p.name for a, p in zip(args, self.params)
                 if isinstance(a, ndarray) and not p.raw]
        outs = args[nin:]
        for swap in ((False, True) if not self._uses_i else (False,)):
            kinds = {}
            ok = True
            for a, cs, nm in zip(arrays, cstrides, names):
                sr, sc = (cs[1], cs[0]) if swap else cs
                item = a.dtype.itemsize
                is_out = any(a is o for o in outs)
                if sr % item or sc % item:
                    ok = False
                elif sc == item:
                    kind = 'R'
                elif is_out:
                    ok = False
                elif sc == 0:
                    kind = 'row'
                elif abs(sc) <= 4 * item and (sr == 0 or abs(sr) >= abs(sc)):
                    kind = 'S'
                else:
                    ok = False
                if not ok or kinds.get(nm, kind) != kind:
                    ok = False
                    break
                kinds[nm] = kind
            if ok and any(k == 'R' for k in kinds.values()):
                if swap:
                    return ((cshape[1], cshape[0]), [(cs[1], cs[0]) for cs in cstrides], kinds)
                return cshape, cstrides, kinds
        return None

    def _plan_rows_nd(self, arrays, cshape, cstrides, args, nin):
        """Problem of three or four axes in which every array runs along the
        last axis with unit stride (or repeats one value along it): a
        permutation of the leading axes, (B, S, H, D) -> (B, H, S, D), a
        value per row.  The row kernel then takes the leading axes as ONE run
        of rows whose start it finds from one stride per axis and array.
        Returns ((rows, columns), [(row strides per leading axis, column
        stride) per array], kinds, extents of the leading axes) or None."""
        if not _tuning.get('rows2d'):
            return None
        names = [p.name for a, p in zip(args, self.params)
                 if isinstance(a, ndarray) and not p.raw]
        outs = args[nin:]
        kinds = {}
        for a, cs, nm in zip(arrays, cstrides, names):
            item = a.dtype.itemsize
            if any(s % item for s in cs):
                return None
            if cs[-1] == item:
                kind = 'R'
            elif cs[-1] == 0 and not any(a is o for o in outs):
                kind = 'row'
            else:
                return None
            if kinds.get(nm, kind) != kind:
                return None
            kinds[nm] = kind
        if not any(k == 'R' for k in kinds.values()):
            return None
        lead = tuple(cshape[:-1])
        # rows of a vector or two leave most lanes of a wave on different rows
        # with nothing gained over the tiled kernel
        if cshape[-1] * max(a.dtype.itemsize for a in arrays) < 256:
            return None
        return ((internal.prod(lead), cshape[-1]),
                [(tuple(cs[:-1]), cs[-1]) for cs in cstrides], kinds, lead)

    def _launch_rows2d(self, dev_id, args, nin, arrays, plan, var_types, typedefs, casts,
                       force_read_out, stream_ptr, kernel_name, rec):
        if len(plan) == 4:
            (nr, nc), nd_strides, kinds, lead = plan
        else:
            (nr, nc), cstrides, kinds = plan
            nd_strides = [((cs[0],), cs[1]) for cs in cstrides]
            lead = (nr,)
        outer = len(lead)
        vec = max(1, 16 // max(a.dtype.itemsize for a in arrays))
        if _tuning.get('rows2d_narrow_vec') and nc < 12 * vec:
            # few vectors per row: a partial one at every row end would split
            # the lanes of a wave between two code paths
            while vec > 1 and nc % vec:
                vec //= 2
        span = max(sum(abs(s) * e for s, e in zip(rs, lead)) + abs(sc) * nc
                   for rs, sc in nd_strides)
        nvr = (nc + vec - 1) // vec
        idx64 = span > _INT32_MAX or nr * nvr * vec > _INT32_MAX - (1 << 24)
        operands = self._make_operands(args, nin, var_types, casts, force_read_out)
        names = [p.name for a, p in zip(args, self.params)
                 if isinstance(a, ndarray) and not p.raw]
        # a value per row, or one row repeated: not counted as streamed traffic
        light = [n for n, (rs, sc) in zip(names, nd_strides)
                 if sc == 0 or all(r == 0 for r in rs)]
        in_bytes, out_bytes = self._traffic(args, nin, light)
        stream_hint = _tuning.stream_policy(_tuning.get('tiled_stream'), in_bytes, out_bytes)
        if (stream_hint[0] and nin > 1 and _tuning.get('tiled_stream') == 'auto'
                and self._inputs_overlap(args, nin)):
            stream_hint = (False, stream_hint[1])
        block = 256
        key = ('rows2d', tuple(o.key() for o in operands), typedefs, vec, idx64,
               tuple(sorted(kinds.items())), dev_id, stream_hint, block, outer)
        entry = self._memo.get(key)
        if entry is None:
            name = kernel_name or self.name
            code = _cg.emit_rows2d(
                name, operands, self.operation, typedefs, self.preamble,
                self.loop_prep, self.after_loop, kinds=kinds, vec=vec, idx64=idx64,
                stream_hint=stream_hint, block=block, outer=outer)
            fn = compiler.compile_with_cache(code, self.options).get_function(name)
            ic = 'q' if idx64 else 'i'
            fmt = ['@']
            for o in operands:
                if o.kind == 'array':
                    fmt.append('P')
                elif o.kind == 'raw':
                    fmt.append('P' + 'q' * (1 + 2 * o.ndim))
                elif o.kind == 'scalar':
                    fmt.append(_scalar_struct_code(o.store_t))
            fmt.append(ic * (2 + (outer - 1) + (outer + 1) * len(arrays)))
            entry = (fn, _make_packer(fmt), code)
            with self._lock:
                entry = self._memo.setdefault(key, entry)
            self._remember_code(args, entry[2])
        fn, packer, _ = entry
        block_args = self._flat_values(args)
        block_args.const(nr, nc, *lead[1:])
        for a, (rs, sc) in zip(arrays, nd_strides):
            item = a.dtype.itemsize
            block_args.const(*([r // item for r in rs] + [sc // item]))
        grid = max(1, min((nr * nvr + block - 1) // block,
                          _grid_limit(dev_id, _tuning.get('flat_blocks_per_cu')) * 4))
        _launch_plan.launch(rec, fn, (grid, 1, 1), (block, 1, 1), packer, block_args,
                            stream_ptr)

    # -- flat ---------------------------------------------------------------------------
    def _launch_flat(self, dev_id, args, nin, arrays, cstrides, size, var_types,
                     typedefs, casts, force_read_out, stream_ptr, kernel_name, rec,
                     partial=None, nc=None):
        params = self.params
        bcast = []
        itemsizes = []
        ai = 0
        for a, p in zip(args, params):
            if isinstance(a, ndarray) and not p.raw:
                cs = cstrides[ai]
                ai += 1
                if partial and p.name in partial:
                    continue
                if size > 1 and (len(cs) == 1 and cs[0] == 0):
                    bcast.append(p.name)
                else:
                    itemsizes.append(a.dtype.itemsize)
        if not itemsizes:
            itemsizes = [arrays[0].dtype.itemsize]
        vec = _max_vector_width(itemsizes)
        mixed = False
        if _tuning.get('flat_vec_by') == 'wide' and max(itemsizes) != min(itemsizes):
            vec = max(1, 16 // max(itemsizes))
            mixed = True
        # every iterated array must sit on a boundary of its vector
        ai = 0
        for a, p in zip(args, params):
            if isinstance(a, ndarray) and not p.raw:
                if p.name not in bcast and not (partial and p.name in partial):
                    while vec > 1 and not _aligned(
                            a.data.ptr, min(16, vec * a.dtype.itemsize)):
                        vec //= 2
                ai += 1
        if size < vec * 64:
            vec = 1
        idx64 = size > _INT32_MAX - (1 << 24)
        unroll = _tuning.get('flat_unroll') if vec > 1 else 1
        if mixed and vec > 1:
            unroll = _tuning.get('flat_mixed_unroll') if len(itemsizes) <= 2 else 1
        block = _tuning.get('flat_block')
        in_bytes, out_bytes = self._traffic(args, nin, bcast + list(partial or ()))
        # nothing streams in (a fill): full-size workgroups and four times the
        # usual grid, so that a thread stores a few vectors only (2^28 float32:
        # 197 -> 174 us)
        write_only = in_bytes == 0
        if write_only:
            block = _tuning.get('flat_fill_block')
        if len(itemsizes) <= 2 and block > 512 and not write_only:
            # one stream in, one out: measured 2 % faster with smaller
            # workgroups (the grid cap below keeps threads per CU the same)
            block = 512
        stream_hint = _tuning.stream_policy(
            _tuning.get('flat_stream'), in_bytes, out_bytes)
        if (stream_hint[0] and nin > 1 and _tuning.get('flat_stream') == 'auto'
                and self._inputs_overlap(args, nin)):
            stream_hint = (False, stream_hint[1])
        operands = self._make_operands(args, nin, var_types, casts, force_read_out)
        if self._uses_ind:
            operands.append(_cg.Operand('indexer', '_ind', '', ndim=1,
                                        index_32=not idx64))
        part_kinds = tuple(sorted((n, k[0]) for n, k in partial.items())) if partial else ()
        key = ('flat', tuple(o.key() for o in operands), typedefs, vec, unroll,
               idx64, tuple(bcast), dev_id, block, stream_hint, part_kinds)
        entry = self._memo.get(key)
        if entry is None:
            name = kernel_name or self.name
            code = _cg.emit_flat(
                name, operands, self.operation, typedefs, self.preamble,
                self.loop_prep, self.after_loop, vec=vec, unroll=unroll,
                idx64=idx64, bcast=tuple(bcast), stream_hint=stream_hint, block=block,
                partial=dict(part_kinds))
            fn = compiler.compile_with_cache(code, self.options).get_function(name)
            fmt = self._arg_format(operands, 'q' if idx64 else 'i', flat=True,
                                   extra=(1 + len(part_kinds)) if partial else 0)
            entry = (fn, _make_packer(fmt), code)
            with self._lock:
                entry = self._memo.setdefault(key, entry)
            self._remember_code(args, entry[2])
        fn, packer, _ = entry
        block_args = self._flat_values(args)
        block_args.const(size)
        if partial:
            block_args.const(nc)
            for a, p in zip(args, params):
                if isinstance(a, ndarray) and not p.raw and p.name in partial:
                    block_args.const(partial[p.name][1] // a.dtype.itemsize)
        if self._uses_ind:
            block_args.const(size, size, 0)
        nvec = size // vec
        per_block = block * unroll
        grid = max(1, min((max(nvec, size - nvec * vec) + per_block - 1) // per_block,
                          _grid_limit(dev_id, _tuning.get('flat_blocks_per_cu'))
                          * (_tuning.get('flat_block') // block) * (4 if write_only else 1)))
        _launch_plan.launch(rec, fn, (grid, 1, 1), (block, 1, 1), packer, block_args,
                            stream_ptr)

    def _inputs_overlap(self, args, nin):
        """True if two different input arrays of the call overlap in memory
        (``x[1:] + x[:-1]``, windows of one matrix): each cache line is then
        asked for twice, and loads without the non-temporal hint let the second
        request find it in the cache (2^26 float32 over rotating buffers:
        91.2 -> 87.4 us; windows of 8190 x 8190: 95.9 -> 93.1 us)."""
        ins = [a for a, p in zip(args[:nin], self.params)
               if isinstance(a, ndarray) and not p.raw and a.size]
        for k, a in enumerate(ins):
            for b in ins[k + 1:]:
                if (a is not b and a.data.mem.ptr == b.data.mem.ptr
                        and _carray.may_share_bounds(a, b)):
                    return True
        return False

    def _traffic(self, args, nin, bcast_names):
        """Bytes a launch reads and writes (broadcast operands and raw arrays
        not counted; an array passed twice counted once)."""
        in_bytes = out_bytes = 0
        seen = set()
        for idx, (a, p) in enumerate(zip(args, self.params)):
            if not isinstance(a, ndarray) or p.raw or p.name in bcast_names:
                continue
            if id(a) in seen:
                continue
            seen.add(id(a))
            nbytes = a.dtype.itemsize
            for ext, st in zip(a._shape, a._strides):
                if st != 0:
                    nbytes *= ext
            if idx >= nin:
                out_bytes += nbytes
            else:
                in_bytes += nbytes
        return in_bytes, out_bytes

    def _flat_values(self, args):
        """Argument values for kernels that take plain pointers: data pointer
        per iterated array, CArray fields per raw array, scalar values."""
        out = _launch_plan.ArgBlock()
        for ref, (a, p) in enumerate(zip(args, self.params)):
            if isinstance(a, ndarray):
                out.ptr(ref, a.data.ptr)
                if p.raw:
                    out.const(a.size, *a._shape)
                    out.const(*a._strides)
            else:
                out.scalar(ref, a)
        return out

    def _arg_format(self, operands, idx_code, flat, extra=0):
        """struct format of the kernel's argument block (``extra`` more index
        values after the element count)."""
        fmt = ['@']
        for o in operands:
            if o.kind == 'array':
                fmt.append('P' if flat else 'PP')
            elif o.kind == 'raw':
                fmt.append('P' + 'q' * (1 + 2 * o.ndim))
            elif o.kind == 'scalar':
                fmt.append(_scalar_struct_code(o.store_t))
        fmt.append(idx_code * (1 + extra))
        for o in operands:
            if o.kind == 'indexer':
                fmt.append('q' * (1 + 2 * o.ndim))
        return ''.join(fmt)

    # -- tiled 2-d -----------------------------------------------------------------------
    def _classify_2d(self, arrays, cstrides, args, nin):
        """'tiled' if every array is contiguous (or broadcast) along the
        columns, 'tiled_t' if that holds after swapping the two axes,
        'generic' otherwise.  Transposed ('C') operands are allowed as inputs."""
        def classify(swap):
            ok = True
            any_c = False
            for a, cs in zip(arrays, cstrides):
                s0, s1 = (cs[1], cs[0]) if swap else cs
                item = a.dtype.itemsize
                if s1 == item or s1 == 0:
                    if s0 % item:
                        ok = False
                elif s0 == item and s1 % item == 0:
                    any_c = True
                    if any(a is o for o in args[nin:]):
                        ok = False
                else:
                    ok = False
                if not ok:
                    break
            return ok, any_c
        ok, _ = classify(False)
        if ok:
            # outputs must be unit stride along columns
            for o in args[nin:]:
                for a, cs in zip(arrays, cstrides):
                    if a is o and cs[1] != a.dtype.itemsize:
                        ok = False
            if ok:
                return 'tiled'
        if self._uses_i:
            return 'generic'
        ok, _ = classify(True)
        if ok:
            for o in args[nin:]:
                for a, cs in zip(arrays, cstrides):
                    if a is o and cs[0] != a.dtype.itemsize:
                        ok = False
            if ok:
                return 'tiled_t'
        return 'generic'

    def _plan_batched(self, arrays, cshape, cstrides, args, nin):
        """Splits the axes of a 3-d or 4-d problem into batch axes and the two
        axes of the tiled kernel: columns = the axis every output (and every
        array that is not transposed) runs along with unit stride, rows = the
        axis the transposed inputs run along, or the innermost other axis.
        Returns ((nr, nc), [(sr, sc) per array], (batch shape, [batch strides
        per array])) or None."""
        nd = len(cshape)
        outs = args[nin:]
        is_out = [any(a is o for o in outs) for a in arrays]
        col = None
        for ax in range(nd - 1, -1, -1):
            if all(cs[ax] == a.dtype.itemsize
                   for a, cs, o in zip(arrays, cstrides, is_out) if o):
                col = ax
                break
        if col is None or not any(is_out):
            return None
        row = None
        for a, cs, o in zip(arrays, cstrides, is_out):
            item = a.dtype.itemsize
            if any(s % item for s in cs):
                return None
            if cs[col] == item or cs[col] == 0:
                continue
            if o:
                return None
            unit = [ax for ax in range(nd) if ax != col and cs[ax] == item]
            if not unit or (row is not None and row not in unit):
                return None
            row = unit[0] if row is None else row
        if row is None:
            row = max(ax for ax in range(nd) if ax != col)
        rest = [ax for ax in range(nd) if ax not in (row, col)]
        shape2 = (cshape[row], cshape[col])
        strides2 = [(cs[row], cs[col]) for cs in cstrides]
        bshape = tuple(cshape[ax] for ax in rest)
        bstrides = [tuple(cs[ax] for ax in rest) for cs in cstrides]
        if len(rest) == 1:
            bshape = bshape + (1,)
            bstrides = [bs + (0,) for bs in bstrides]
        return shape2, strides2, (bshape, bstrides)

    def _plan_packed(self, arrays, cshape, cstrides, args, nin):
        """Tiles over several axes (``emit_packed``) for a problem of three or
        more axes.  Arrays whose walk in the order of the outputs gives runs of
        64 bytes or more (unit stride along the last axis), or one value per
        vector (zero stride along it), are read straight from memory; the
        other inputs are staged through the LDS in their own order.  Returns
        (tile, order of the axes for staging, staged names, zero-stride names,
        those of them that move within a piece, vec, svec, axes of the
        contiguous pieces of the two passes, unit stride along the first axis
        of the staging?) or None."""
        nd = len(cshape)
        names = [p.name for a, p in zip(args, self.params)
                 if isinstance(a, ndarray) and not p.raw]
        outs = args[nin:]
        kinds = {}
        first_staged = None
        lds_item = 0
        max_item = max(a.dtype.itemsize for a in arrays)
        for a, cs, nm in zip(arrays, cstrides, names):
            item = a.dtype.itemsize
            if any(s % item for s in cs):
                return None
            is_out = any(a is o for o in outs)
            if cs[-1] == item:
                # how far the walk in the order of the outputs stays contiguous
                run = item
                for ax in range(nd - 1, -1, -1):
                    if cs[ax] != run:
                        break
                    run *= cshape[ax]
                kind = 'D' if (is_out or run >= 64) else 'S'
            elif cs[-1] == 0 and not is_out:
                kind = 'Z'
            elif not is_out:
                kind = 'S'
            else:
                return None
            if kinds.get(nm, kind) != kind:
                return None
            if kind == 'S' and nm not in kinds:
                lds_item += item
                if first_staged is None:
                    first_staged = cs
            kinds[nm] = kind
        if 'D' not in kinds.values():
            return None
        staged = tuple(sorted(n for n, k in kinds.items() if k == 'S'))
        zero_last = tuple(sorted(n for n, k in kinds.items() if k == 'Z'))
        out_order = list(range(nd - 1, -1, -1))
        if first_staged is not None:
            in_order = sorted(range(nd), key=lambda ax: (
                first_staged[ax] == 0, abs(first_staged[ax])))
        else:
            in_order = out_order
        first = in_order[0]
        direct = [(a, cs) for a, cs, nm in zip(arrays, cstrides, names) if kinds[nm] == 'D']
        s_arrays = [(a, cs) for a, cs, nm in zip(arrays, cstrides, names) if kinds[nm] == 'S']
        unit_first = all(cs[first] == a.dtype.itemsize for a, cs in s_arrays)
        # elements of a tile: what the LDS image of the staged inputs allows, and
        # enough for a few accesses per thread
        limit = 32768 // max_item
        max_v = limit if not lds_item else min(limit, (48 * 1024) // lds_item)
        want = min(max_v, _tuning.get('packed_tile_bytes') // max_item)
        run = max(32, 256 // max_item)
        while True:
            tile = [1] * nd

            def grow(order):
                have = 1
                for ax in order:
                    if have >= run:
                        break
                    tile[ax] = max(tile[ax], min(cshape[ax], -(-run // have)))
                    have *= tile[ax]
                    if tile[ax] < cshape[ax]:
                        break
            grow(out_order)
            grow(in_order)
            if internal.prod(tile) <= max_v or run <= 1:
                break
            run //= 2
        if internal.prod(tile) > max_v:
            return None
        turn = 0
        while internal.prod(tile) * 2 <= want:
            for k in range(2):
                order = (out_order, in_order)[(turn + k) % 2]
                ax = next((x for x in order if tile[x] < cshape[x]), None)
                if ax is not None:
                    tile[ax] = min(cshape[ax], tile[ax] * 2)
                    turn = (turn + k + 1) % 2
                    break
            else:
                break
        # an axis cut in two unequal parts: whole if there is room, else in
        # equal parts
        for ax in range(nd):
            if 1 < tile[ax] < cshape[ax]:
                if cshape[ax] < 2 * tile[ax] and (
                        internal.prod(tile) // tile[ax] * cshape[ax] <= max_v):
                    tile[ax] = cshape[ax]
                else:
                    parts = -(-cshape[ax] // tile[ax])
                    tile[ax] = min(tile[ax], -(-cshape[ax] // parts))

        def piece_axes(order, members, others):
            """How many of the first axes of ``order`` lie in ``members`` as one
            contiguous piece within a tile (``others`` do not move along them)."""
            count = 1
            while count < nd:
                a, b = order[count - 1], order[count]
                if tile[a] != cshape[a] or tile[b] == 1 or not all(
                        cs[b] == cs[a] * cshape[a] for arr, cs in members) or any(
                        cs[b] for arr, cs in others):
                    break
                count += 1
            return count

        def widen(order, count, members, item):
            """Widest access that divides the piece, the axis that cuts the piece
            made a multiple of what that takes where it is not spanned whole."""
            width = max(1, 16 // item)
            cut = order[count - 1]
            inner = internal.prod(tile[ax] for ax in order[:count - 1])
            while width > 1:
                step = width // math.gcd(inner, width)
                if tile[cut] < cshape[cut] and tile[cut] % step:
                    up = -(-tile[cut] // step) * step
                    down = tile[cut] // step * step
                    room = internal.prod(tile) // tile[cut]
                    if up <= cshape[cut] and room * up <= max_v:
                        tile[cut] = up
                    elif down:
                        tile[cut] = down
                # (a piece of several accesses may end in a partial one)
                ok = (inner * tile[cut]) % width == 0 or inner * tile[cut] >= 4 * width
                for arr, cs in members:
                    nb = width * arr.dtype.itemsize
                    if not _aligned(arr.data.ptr, nb) or not all(
                            _aligned(cs[ax], nb) for ax in order[count:]):
                        ok = False
                if ok:
                    break
                width //= 2
            return width

        group, svec = 1, 1
        if s_arrays and unit_first:
            group = piece_axes(in_order, s_arrays, ())
            svec = widen(in_order, group, s_arrays, max(a.dtype.itemsize for a, cs in s_arrays))
        # Inputs with a value per row: pieces of whole rows where a row is a
        # long enough run by itself (the value is then read once per access),
        # pieces of several rows with the value looked up per element where rows
        # are a few elements (float16 (171840, 5, 78) with a value per middle
        # index: 160 us per element, rows of 7 float32 the other way round)
        zeros = [(a, cs) for a, cs, nm in zip(arrays, cstrides, names) if kinds[nm] == 'Z']
        ogroup = piece_axes(out_order, direct, zeros)
        if zeros and internal.prod(tile[ax] for ax in out_order[:ogroup]) * min(
                a.dtype.itemsize for a, cs in direct) < 64:
            ogroup = piece_axes(out_order, direct, ())
        zero_moving = tuple(sorted(
            nm for (a, cs, nm) in zip(arrays, cstrides, names)
            if kinds[nm] == 'Z' and any(cs[ax] for ax in out_order[1:ogroup])))
        vec = widen(out_order, ogroup, direct, max_item)
        # (the second widening may have moved the axis the first one relied on)
        if s_arrays and unit_first:
            piece = internal.prod(tile[ax] for ax in in_order[:group])
            while svec > 1 and piece % svec and piece < 4 * svec:
                svec //= 2
        return (tuple(tile), tuple(in_order), staged, zero_last, zero_moving, vec, svec, group,
                ogroup, unit_first)

    def _launch_packed(self, dev_id, args, nin, arrays, cshape, cstrides, plan, var_types,
                       typedefs, casts, force_read_out, stream_ptr, kernel_name, rec):
        (tile, in_order, staged, zero_last, zero_moving, vec, svec, group, ogroup,
         unit_first) = plan
        nd = len(cshape)
        threads = _tuning.get('packed_threads')
        ntiles = 1
        span = 0
        for e, t in zip(cshape, tile):
            ntiles *= (e + t - 1) // t
        for a, cs in zip(arrays, cstrides):
            span = max(span, sum(abs(c) // a.dtype.itemsize * (e + t)
                                 for c, e, t in zip(cs, cshape, tile)))
        idx64 = span > _INT32_MAX or ntiles * internal.prod(tile) > _INT32_MAX
        operands = self._make_operands(args, nin, var_types, casts, force_read_out)
        stream_hint = _tuning.stream_policy(
            _tuning.get('tiled_stream'), *self._traffic(args, nin, ()))
        if _tuning.get('tiled_stream') == 'auto':
            # tiles share the cache lines at their borders wherever a run is no
            # whole number of lines: plain accesses let the cache put them together
            item = min(a.dtype.itemsize for a in arrays)
            aligned = not _off_lines(arrays, cstrides)
            piece_in = internal.prod(tile[ax] for ax in in_order[:group]) * item
            piece_out = internal.prod(tile[ax] for ax in range(nd - ogroup, nd)) * item
            stream_hint = (stream_hint[0] and aligned and piece_in % 128 == 0,
                           stream_hint[1] and aligned and piece_out % 128 == 0)
        # tiles whose borders fall inside cache lines: neighbours on one die
        mode = _tuning.get('packed_xcd')
        xcd = bool(mode) and (mode is True or _off_lines(arrays, cstrides))
        tile_order = None
        if staged and _tuning.get('packed_order') == 'in':
            tile_order = in_order
        key = ('packed', tile_order, tuple(o.key() for o in operands), typedefs, tile, in_order, staged,
               zero_last, zero_moving, vec, svec, group, ogroup, unit_first, idx64, dev_id,
               stream_hint, threads, xcd)
        entry = self._memo.get(key)
        if entry is None:
            name = kernel_name or self.name
            code = _cg.emit_packed(
                name, operands, self.operation, typedefs, self.preamble,
                self.loop_prep, self.after_loop, tile=tile, in_order=in_order,
                staged=staged, zero_last=zero_last, zero_moving=zero_moving, vec=vec, svec=svec,
                group=group, ogroup=ogroup, unit_first=unit_first, threads=threads, idx64=idx64, stream_hint=stream_hint,
                xcd=xcd, tile_order=tile_order)
            fn = compiler.compile_with_cache(code, self.options).get_function(name)
            ic = 'q' if idx64 else 'i'
            fmt = ['@']
            for o in operands:
                if o.kind == 'array':
                    fmt.append('P')
                elif o.kind == 'raw':
                    fmt.append('P' + 'q' * (1 + 2 * o.ndim))
                elif o.kind == 'scalar':
                    fmt.append(_scalar_struct_code(o.store_t))
            fmt.append(ic * (nd * (1 + len(arrays))))
            entry = (fn, _make_packer(fmt), code)
            with self._lock:
                entry = self._memo.setdefault(key, entry)
            self._remember_code(args, entry[2])
        fn, packer, _ = entry
        block_args = self._flat_values(args)
        block_args.const(*cshape)
        for a, cs in zip(arrays, cstrides):
            item = a.dtype.itemsize
            block_args.const(*(c // item for c in cs))
        grid = max(1, min(ntiles, _max_blocks(threads)))
        _launch_plan.launch(rec, fn, (grid, 1, 1), (threads, 1, 1), packer, block_args,
                            stream_ptr)
        return True

    @staticmethod
    def _flat_stage_width(arrays, cstrides, names, layouts, nr):
        """Elements per access with which the staged operands of a tile that
        spans their ``nr`` contiguous elements per line can be read as one
        piece (their lines follow one another without gaps), or 0."""
        if not _tuning.get('tiled_flat_stage'):
            return 0
        staged = [(a, cs) for a, cs, nm in zip(arrays, cstrides, names) if layouts[nm] == 'C']
        if not staged or not all(cs[0] == a.dtype.itemsize and cs[1] == nr * a.dtype.itemsize
                                 for a, cs in staged):
            return 0
        width = min(4, 16 // max(a.dtype.itemsize for a, cs in staged))
        return width if width >= 2 else 0

    def _launch_tiled(self, dev_id, args, nin, arrays, cshape, cstrides, var_types,
                      typedefs, casts, force_read_out, stream_ptr, kernel_name, swap,
                      rec, batch=None):
        params = self.params
        if swap:
            cshape = (cshape[1], cshape[0])
            cstrides = [(cs[1], cs[0]) for cs in cstrides]
        nr, nc = cshape
        layouts = {}
        itemsizes = [a.dtype.itemsize for a in arrays]
        # the widest operand moves 16 bytes per thread, narrower ones less
        vec = max(1, 16 // max(itemsizes))
        names = [p.name for a, p in zip(args, params)
                 if isinstance(a, ndarray) and not p.raw]
        n_transposed = 0
        lds_item = 0
        for a, cs, nm in zip(arrays, cstrides, names):
            item = a.dtype.itemsize
            if cs[1] == item:
                layouts[nm] = 'R'
            elif cs[1] == 0:
                layouts[nm] = 'R0'
            else:
                layouts[nm] = 'C'
                n_transposed += 1
                lds_item += item
        # Alignment of every vector access: along the columns (``vec``) for the
        # row-major operands, along the rows (``svec``) for the staged ones.
        # Wide accesses need the alignment of an element only; unaligned ones
        # cost a few per cent, element-wide ones most of the bandwidth.
        loose = _tuning.get('unaligned_vectors') and _tuning.get('tiled_unaligned')

        def widest(kinds, limit):
            v = max(1, 16 // max(itemsizes))
            while v > 1:
                ok = v <= limit
                for a, cs, nm in zip(arrays, cstrides, names):
                    if layouts[nm] not in kinds or loose:
                        continue
                    nb = v * a.dtype.itemsize
                    if not _aligned(a.data.ptr, nb) or not _aligned(
                            cs[0] if layouts[nm] == 'R' else cs[1], nb):
                        ok = False
                if ok:
                    break
                v //= 2
            return v
        vec = widest(('R',), nc)
        svec = widest(('C',), nr) if n_transposed else vec
        # Large tiles give long contiguous runs in memory on both the transposed
        # and the row-major side; they need the LDS for the staged operands.
        big_min = _tuning.get('tiled_big_min')
        if (nr >= big_min and nc >= big_min and lds_item * 128 * 129 <= 140 * 1024
                and ((nr + 127) // 128) * ((nc + 127) // 128) * (
                    batch[0][0] * batch[0][1] if batch else 1) >= 512):
            tile_r = tile_c = 128
            threads = 1024
        else:
            tile_r = tile_c = 64
            threads = 256
        narrow = n_transposed and min(nr, nc) <= 32 and _tuning.get('tiled_narrow')
        if narrow:
            # A narrow array (points as rows of three coordinates, say, to or
            # from three long rows): tiles as narrow as the array and long the
            # other way, so that no tile has an edge along the narrow side and
            # both sides move in long contiguous runs.  (2^26 floats over
            # rotating buffers, (n, 3) to (3, n): 1215 us with square tiles, 118
            # so; back: 531 -> 108; (n, 2): 1243 -> 105; (n, 15): 340 -> 161.
            # Tiles of about 1536 elements: of 4096 (n, 3) takes 214 us, of
            # 12288 615: few workgroups per CU then, each busy with one phase.)
            # the workgroup is a whole number of lines of the narrow side, so
            # that both loops of the kernel come out in whole trips
            want = _tuning.get('tiled_narrow_elements')
            if not want:
                # (widths that are no power of two want longer tiles, i.e.
                # longer runs per line of the other side: (n, 24) to (24, n)
                # 184 us with 1536 elements, 118 with 6144; (n, 20) 163 -> 116;
                # (n, 26) 187 -> 138 with 3072; odd widths and powers of two
                # are best at 1536)
                narrow_side = min(nr, nc)
                if narrow_side % 2 and narrow_side > 9 and nr <= 32 and self._flat_stage_width(
                        arrays, cstrides, names, layouts, nr):
                    # (odd widths whose staged tile is read as one piece, see
                    # below: (n, 13) 126 -> 114, (n, 19) 159 -> 123, (n, 31)
                    # 184 -> 125)
                    want = 3072 if narrow_side < 25 else 6144
                elif narrow_side & (narrow_side - 1) == 0 or narrow_side % 2:
                    want = 1536
                elif narrow_side % 4:
                    want = 3072
                else:
                    want = 6144
            want = max(512, min(want, (48 * 1024) // max(1, lds_item)))
            if nr <= 32:
                tile_r = nr
                while svec > 1 and tile_r % svec:
                    svec //= 2
                # (a power of two of lines: tiles then start on whole cache lines)
                per = internal.flp2(256 // tile_r)
                threads = tile_r * per
                m = 1
                while (vec * m) % svec or threads * vec * m < want:
                    m += 1
                tile_c = vec * per * m
            else:
                tile_c = nc
                while vec > 1 and tile_c % vec:
                    vec //= 2
                q = tile_c // vec
                per = internal.flp2(256 // q)
                threads = q * per
                m = 1
                while ((vec * m) % svec or (per * m) % svec or (per * m) % 32
                       or threads * vec * m < want):
                    m += 1
                tile_r = per * m
            if lds_item * tile_r * (tile_c + 1) > 64 * 1024:
                tile_r = tile_c = 64        # (many wide staged operands: square tiles)
                threads = 256
                vec = min(vec, svec)
                svec = vec
        forced = _tuning.get('tiled_tile')
        if forced and n_transposed:
            tile_r, tile_c, threads = forced
        if n_transposed == 0:
            # Nothing is staged: every operand runs along the columns, so the
            # tile is made as wide as divides the row length (up to one vector
            # per thread) and a few rows high -- long contiguous runs, like the
            # flat kernel, with the per-row operands read once per row.
            wide = threads * vec
            while wide > tile_c and nc % wide:
                wide //= 2
            if wide > tile_c:
                tile_r = tile_r * tile_c // wide
                tile_c = wide
        if lds_item * tile_r * (tile_c + 1) > 150 * 1024:
            return None       # too many staged operands for the LDS
        span = 0
        for a, cs in zip(arrays, cstrides):
            span = max(span, abs(cs[0]) * nr + abs(cs[1]) * nc)
        nbt = 1
        if batch:
            bshape, bstrides = batch
            nbt = bshape[0] * bshape[1]
            for k, bs in enumerate(bstrides):
                cs = cstrides[k]
                span = max(span, abs(cs[0]) * nr + abs(cs[1]) * nc
                           + abs(bs[0]) * bshape[0] + abs(bs[1]) * bshape[1])
            # the tile counter runs over whole tiles, edge tiles included
            span = max(span, nbt * (nr + tile_r) * (nc + tile_c))
        idx64 = span > _INT32_MAX or nr * nc > _INT32_MAX
        operands = self._make_operands(args, nin, var_types, casts, force_read_out)
        stream_hint = _tuning.stream_policy(
            _tuning.get('tiled_stream'),
            *self._traffic(args, nin, [n for n, l in layouts.items() if l == 'R0']))
        if stream_hint[1] and n_transposed and _tuning.get('tiled_stream') == 'auto':
            # a tile row is a short run of the output (256-512 bytes), written
            # by a few lanes while neighbouring tiles write the rest of the same
            # cache lines later: plain stores let the cache put the lines together
            # (transposed copy of 4099 x 16363 float32: 183 us with non-temporal
            # stores, 116 us without; C2a within the benchmark step 84.6 -> 80.8 us)
            # (batches of aligned tiles measure 2-6 % better with the hint)
            unaligned = any(
                any(a is o for o in args[nin:]) and (a.data.ptr % 128 or cs[0] % 128)
                for a, cs in zip(arrays, cstrides))
            if not batch or unaligned:
                stream_hint = (stream_hint[0], False)
        if narrow and _tuning.get('tiled_stream') == 'auto' and stream_hint[0]:
            # (tiles that span the narrow side share no lines along it: both
            # ways past the cache, (n, 3) to (3, n) 114 -> 105 us)
            stream_hint = (True, True)
        elif stream_hint[0] and n_transposed and _tuning.get('tiled_stream') == 'auto':
            # staged operands whose columns do not start on whole cache lines:
            # neighbouring tiles share the lines at their borders, and plain
            # loads let the second one find them in the cache (transposed copy
            # of 8191 x 8193 float32: 179 -> 157 us, of 4099 x 16363: 184 -> 157)
            if any(layouts[nm] == 'C' and (a.data.ptr % 128 or cs[1] % 128)
                   for a, cs, nm in zip(arrays, cstrides, names)):
                stream_hint = (False, stream_hint[1])
        # The order the tiles of a batch are visited in: batch entries that lie
        # closer together than the rows of a tile go first (see emit_tiled2d)
        batch_first = False
        if batch and _tuning.get('tiled_batch_first'):
            inner_batch = [abs(bs[1] if bshape[1] > 1 else bs[0]) for bs in bstrides]
            pitch = [max(abs(cs[0]), abs(cs[1])) for cs in cstrides]
            batch_first = all(b and b < p for b, p in zip(inner_batch, pitch))
        # Staged operands whose lines are no whole vectors (3, 7, 17, 31 ...
        # elements) and follow one another without gaps: a tile that spans the
        # lines is one contiguous piece of memory and is read with full vectors
        # all the same ((n, 17) to (17, n): 183 us element by element).
        flat_stage = 0
        if narrow and nr <= 32 and tile_r == nr and svec == 1 and n_transposed:
            flat_stage = self._flat_stage_width(arrays, cstrides, names, layouts, nr)
        # Tiles numbered so that neighbours run on one compute die, where
        # their borders do not fall on cache-line boundaries
        mode = _tuning.get('tiled_xcd')
        xcd = bool(mode) and (mode is True or any(
            a.data.ptr % 128 or any(
                abs(c) > a.itemsize and abs(c) % 128 for c in cs[:2])
            for a, cs in zip(arrays, cstrides)))
        key = ('tiled', tuple(o.key() for o in operands), typedefs, vec, idx64,
               tuple(sorted(layouts.items())), dev_id, stream_hint, tile_r, tile_c,
               threads, bool(batch), batch_first, svec, flat_stage, xcd,
               _tuning.get('tiled_xcd_strip'))
        entry = self._memo.get(key)
        if entry is None:
            name = kernel_name or self.name
            code = _cg.emit_tiled2d(
                name, operands, self.operation, typedefs, self.preamble,
                self.loop_prep, self.after_loop, layouts=layouts, vec=vec,
                tile_r=tile_r, tile_c=tile_c, threads=threads, idx64=idx64,
                stream_hint=stream_hint, batched=bool(batch), batch_first=batch_first,
                svec=svec, flat_stage=flat_stage, xcd=xcd,
                strip=_tuning.get('tiled_xcd_strip'))
            fn = compiler.compile_with_cache(code, self.options).get_function(name)
            ic = 'q' if idx64 else 'i'
            fmt = ['@']
            for o in operands:
                if o.kind == 'array':
                    fmt.append('P')
                elif o.kind == 'raw':
                    fmt.append('P' + 'q' * (1 + 2 * o.ndim))
                elif o.kind == 'scalar':
                    fmt.append(_scalar_struct_code(o.store_t))
            fmt.append(ic * (2 + 2 * len(arrays)))
            if batch:
                fmt.append(ic * (2 + 2 * len(arrays)))
            entry = (fn, _make_packer(fmt), code)
            with self._lock:
                entry = self._memo.setdefault(key, entry)
            self._remember_code(args, entry[2])
        fn, packer, _ = entry
        block_args = self._flat_values(args)
        block_args.const(nr, nc)
        for a, cs in zip(arrays, cstrides):
            item = a.dtype.itemsize
            block_args.const(cs[0] // item, cs[1] // item)
        if batch:
            block_args.const(nbt, bshape[1])
            for a, bs in zip(arrays, bstrides):
                item = a.dtype.itemsize
                block_args.const(bs[0] // item, bs[1] // item)
        ntiles = ((nr + tile_r - 1) // tile_r) * ((nc + tile_c - 1) // tile_c) * nbt
        grid = max(1, min(ntiles, _max_blocks(threads)))
        _launch_plan.launch(rec, fn, (grid, 1, 1), (threads, 1, 1), packer, block_args,
                            stream_ptr)
        return True

    # -- generic ---------------------------------------------------------------------------
    def _launch_generic(self, dev_id, args, nin, shape, var_types, typedefs, casts,
                        force_read_out, stream_ptr, block_size, kernel_name, rec):
        params = self.params
        arrays_idx = [i for i, (a, p) in enumerate(zip(args, params))
                      if isinstance(a, ndarray) and not p.raw]
        args = list(args)
        if arrays_idx and self.reduce_dims:
            arrays = [args[i] for i in arrays_idx]
            cshape, cstrides = _canonical_dims(arrays, shape)
            if len(cshape) != len(shape):
                if len(cshape) == 0:
                    cshape = (1,)
                    cstrides = [(a.dtype.itemsize,) for a in arrays]
                for i, cs in zip(arrays_idx, cstrides):
                    args[i] = args[i]._view(cshape, cs)
                shape = cshape
        indexer = _carray.Indexer(shape)
        operands = self._make_operands(args, nin, var_types, casts, force_read_out)
        operands.append(_cg.Operand('indexer', '_ind', '', ndim=indexer.ndim,
                                    index_32=indexer._index_32_bits))
        key = ('generic', tuple(o.key() for o in operands), typedefs, dev_id)
        entry = self._memo.get(key)
        if entry is None:
            name = kernel_name or self.name
            code = _cg.emit_generic(
                name, operands, self.operation, typedefs, self.preamble,
                self.loop_prep, self.after_loop)
            fn = compiler.compile_with_cache(code, self.options).get_function(name)
            fmt = ['@']
            for o in operands:
                if o.kind in ('array', 'raw'):
                    fmt.append('P' + 'q' * (1 + 2 * o.ndim))
                elif o.kind == 'scalar':
                    fmt.append(_scalar_struct_code(o.store_t))
                else:
                    fmt.append('q' * (1 + 2 * o.ndim))
            entry = (fn, _make_packer(fmt), code)
            with self._lock:
                entry = self._memo.setdefault(key, entry)
            self._remember_code(args, entry[2])
        fn, packer, _ = entry
        block_args = _launch_plan.ArgBlock()
        for ref, a in enumerate(args):
            if isinstance(a, ndarray):
                block_args.ptr(ref, a.data.ptr)
                block_args.const(a.size, *a._shape)
                block_args.const(*a._strides)
            else:
                block_args.scalar(ref, a)
        block_args.const(indexer.size, *indexer.shape)
        block_args.const(*((0,) * indexer.ndim))
        size = indexer.size
        block = max(1, min(block_size, size))
        # enough workgroups to fill the device several times over; the kernel
        # loops over what is left
        grid = max(1, min((size + block - 1) // block,
                          _grid_limit(dev_id, 32) * max(1, 256 // block)))
        _launch_plan.launch(rec, fn, (grid, 1, 1), (block, 1, 1), packer, block_args,
                            stream_ptr)

    def _remember_code(self, args, code):
        in_types = tuple(a.dtype for a in args if isinstance(a, ndarray))
        if in_types not in self._codes:
            self._codes[in_types] = code


_SCALAR_CODES = {
    'bool': '?', 'signed char': 'b', 'unsigned char': 'B', 'short': 'h',
    'unsigned short': 'H', 'int': 'i', 'unsigned int': 'I', 'long long': 'q',
    'unsigned long long': 'Q', 'float16': '2s', 'float': '4s', 'double': '8s',
    'complex<float>': 'F', 'complex<double>': 'D',
}


def _scalar_struct_code(ctype):
    """struct code for a by-value scalar; floats travel as their bytes with an
    explicit alignment pad handled by the native-alignment '@' mode."""
    code = _SCALAR_CODES[ctype]
    if code == '2s':
        return 'e'
    if code == '4s':
        return 'f'
    if code == '8s':
        return 'd'
    return code


class _ComplexPacker:
    """``struct.Struct`` stand-in for argument blocks that hold complex
    scalars: each takes one value on the way in and is laid out as two floats
    at the alignment of the kernel's ``complex<T>`` (twice the part's size)."""
    __slots__ = ('_struct', '_slots', 'size')

    def __init__(self, fmt):
        out = []
        slots = []
        n_values = 0
        for ch in fmt:
            if ch in 'FD':
                part = 'f' if ch == 'F' else 'd'
                align = 8 if ch == 'F' else 16
                here = struct.calcsize(''.join(out))
                out.append('x' * (-here % align) + part * 2)
                slots.append(n_values)
                n_values += 1
            else:
                out.append(ch)
                if ch == '?' or (ch.isalpha() and ch != 'x'):
                    n_values += 1
        self._struct = struct.Struct(''.join(out))
        self._slots = tuple(reversed(slots))
        self.size = self._struct.size

    def pack(self, *vals):
        vals = list(vals)
        for i in self._slots:
            v = complex(vals[i])
            vals[i:i + 1] = (v.real, v.imag)
        return self._struct.pack(*vals)


def _make_packer(fmt):
    """Packer of an argument block from a struct format (string or list of
    pieces) in which 'F' / 'D' stand for complex64 / complex128 scalars."""
    if not isinstance(fmt, str):
        fmt = ''.join(fmt)
    if 'F' in fmt or 'D' in fmt:
        return _ComplexPacker(fmt)
    return struct.Struct(fmt)


# ---------------------------------------------------------------------------------
# ElementwiseKernel
# ---------------------------------------------------------------------------------

class ElementwiseKernel:
    """User-defined elementwise kernel.

    The loop body ``operation`` is HIP C++ operating on one element; array
    parameters are broadcast against each other unless marked ``raw``.  The
    kernel is generated and compiled for gfx950 on first use for each
    combination of argument types and memory layouts, cached in the process and
    on disk.

    Args:
        in_params (str): Input argument list, e.g. ``'float32 x, T y'``.
        out_params (str): Output argument list.
        operation (str): The body of the loop.
        name (str): Name of the kernel function (shows up in profiles).
        reduce_dims (bool): Merge contiguous axes before launching.
        preamble (str): Code inserted before the kernel.
        no_return (bool): ``__call__`` returns ``None``.
        return_tuple (bool): ``__call__`` always returns a tuple.
        options (tuple): Extra hiprtc options.
        loop_prep (str): Code run by every thread before the loop.
        after_loop (str): Code run by every thread after the loop.
    """

    def __init__(self, in_params, out_params, operation, name='kernel',
                 reduce_dims=True, preamble='', no_return=False,
                 return_tuple=False, **kwargs):
        if not compiler.is_valid_kernel_name(name):
            raise ValueError('Invalid kernel name: "%s"' % name)
        self.name = self.__name__ = name
        self.operation = operation
        self.preamble = preamble
        self.reduce_dims = reduce_dims
        self.no_return = no_return
        self.return_tuple = return_tuple
        self.kwargs = dict(kwargs)
        extras = dict(options=(), loop_prep='', after_loop='')
        unknown = {k: v for k, v in kwargs.items() if k not in extras}
        if unknown:
            raise TypeError('Wrong arguments %s' % unknown)
        extras.update(kwargs)

        self.in_params = _get_param_info(in_params, True)
        self.out_params = _get_param_info(out_params, False)
        declared = self.in_params + self.out_params
        self.nin, self.nout, self.nargs = len(self.in_params), len(self.out_params), len(declared)
        # (the loop index `i` belongs to the generated loop)
        if any(p.name == 'i' for p in declared):
            raise ValueError('Can not use \'i\' as a parameter name')
        # what broadcasting sees: the declared parameters and the indexer
        self.params = declared + _get_param_info('CIndexer _ind', False)
        self._params_type_memo = {}
        self._planner = _ElementwisePlanner(
            name, declared, operation, preamble, extras['loop_prep'], extras['after_loop'],
            extras['options'], is_ufunc=False)
        self._planner.reduce_dims = bool(reduce_dims)
        self._cached_codes = self._planner._codes
        self._fast_calls = {}

    def _result(self, out_args, as_refs=False):
        """What a call hands back from its output arrays: nothing, the one
        array, or a tuple (``as_refs``: their positions among the arguments)."""
        if self.no_return:
            return None
        outs = tuple(range(self.nin, self.nargs)) if as_refs else tuple(out_args)
        if self.nout == 1 and not self.return_tuple:
            return outs[0]
        return outs

    def __call__(self, *args, **kwargs):
        """Compiles (if needed) and launches the kernel.

        Args:
            args: Inputs, optionally followed by the outputs.
            size (int): Number of loop iterations; required if and only if no
                non-raw array is among the arguments.
            stream: Stream to launch on (default: current stream).
            block_size (int): Threads per workgroup of the strided fallback
                kernel (default 128).
        """
        if not kwargs and len(args) == self.nargs:
            # the common call, seen before: straight to its recorded launches
            fast_key = _launch_plan.call_signature(args, _device.get_device_id())
            if fast_key is not None:
                fast = self._fast_calls.get(fast_key)
                if fast is not None:
                    return fast.run(args)
        options = dict(size=-1, stream=None, block_size=128)
        unknown = {k: v for k, v in kwargs.items() if k not in options}
        if unknown:
            raise TypeError('Wrong arguments %s' % unknown)
        options.update(kwargs)
        size, stream, block_size = options['size'], options['stream'], options['block_size']
        if block_size <= 0:
            raise ValueError('block_size must be greater than zero')
        n_args = len(args)
        if n_args not in (self.nin, self.nargs):
            raise TypeError(
                'Wrong number of arguments for {!r}. '
                'It must be either {} or {} (with outputs), '
                'but given {}.'.format(self.name, self.nin, self.nargs, n_args))
        dev_id = _device.get_device_id()
        # A call that looks like an earlier one replays that call's launch.
        fast_key = rec = None
        if size == -1 and stream is None and block_size == 128:
            fast_key = _launch_plan.call_signature(args, dev_id)
            if fast_key is not None:
                fast = self._fast_calls.get(fast_key)
                if fast is not None:
                    return fast.run(args)
                rec = _launch_plan.Recorder(self.nargs)
        for arg in args:
            if hasattr(arg, '__cupy_override_elementwise_kernel__'):
                return arg.__cupy_override_elementwise_kernel__(
                    self, *args, size=size, stream=stream, block_size=block_size)
        arg_list = _preprocess_args(dev_id, args)
        out_args = arg_list[self.nin:]
        bargs, shape = _broadcast(arg_list, self.params, size != -1)
        in_args = bargs[:self.nin]

        def array_dtypes(arguments):
            return tuple(a.dtype if isinstance(a, ndarray) else None for a in arguments)
        in_types, out_types, type_map = self._decide_params_type(
            array_dtypes(in_args), array_dtypes(out_args))

        size_given = size != -1
        if size_given:
            shape = (int(size),)
        out_args = _get_out_args_with_params(
            out_args, out_types, shape, self.out_params, size_given)
        ret = self._result(out_args)
        if 0 in shape:
            return ret

        for i, x in enumerate(in_args):
            if type(x) is CScalar:
                x.apply_dtype(in_types[i])

        inout_args = in_args + out_args
        var_types = [p.ctype for p in self.in_params + self.out_params]
        self._planner.launch(
            dev_id, inout_args, self.nin, shape, var_types,
            type_map.get_typedef_code(), stream=stream, block_size=block_size,
            rec=rec)
        if rec is not None and len(rec.launches) == 1:
            ret_refs = self._result(None, as_refs=True)
            out_specs = () if n_args == self.nargs else tuple(
                (shape, o.dtype) for o in out_args)
            _launch_plan.remember(
                self._fast_calls, fast_key,
                _launch_plan.FastCall(n_args, out_specs, rec, ret_refs))
        return ret

    def _decide_params_type(self, in_args_dtype, out_args_dtype):
        key = (in_args_dtype, out_args_dtype)
        ret = self._params_type_memo.get(key)
        if ret is None:
            ret = _decide_params_type_core(
                self.in_params, self.out_params, in_args_dtype, out_args_dtype)
            self._params_type_memo[key] = ret
        return ret

    @property
    def cached_codes(self):
        """dict: input dtypes -> generated source (for debugging)."""
        if len(self._cached_codes) == 0:
            warnings.warn(
                'No codes are cached because compilation is deferred until '
                'the first function call.')
        return dict(self._cached_codes.items())

    @property
    def cached_code(self):
        """``next(iter(self.cached_codes.values()))``."""
        codes = self._cached_codes
        if len(codes) > 1:
            warnings.warn(
                'The input types of the kernel could not be inferred. '
                'Please use `.cached_codes` instead.')
        return next(iter(codes.values()))


# ---------------------------------------------------------------------------------
# ufunc
# ---------------------------------------------------------------------------------

def fix_cast_expr(src_type, dst_type, expr):
    """Expression converting ``expr`` of ``src_type`` for use as ``dst_type``."""
    src_kind = get_dtype(src_type).kind
    dst_kind = get_dtype(dst_type).kind
    if src_kind == dst_kind:
        return expr
    if src_kind == 'b':
        if dst_kind == 'c':
            return 'static_cast<%s>((%s) ? 1 : 0)' % (_get_typename(dst_type), expr)
        return '((%s) ? 1 : 0)' % expr
    if src_kind == 'c':
        # to bool: NumPy's truth value; to a real type: the real part
        return 'static_cast<%s>(%s)' % (_get_typename(dst_type), expr)
    if dst_kind == 'c':
        return 'static_cast<%s>(%s)' % (_get_typename(dst_type), expr)
    return expr


_KIND_LADDER = ((numpy.bool_,), (numpy.integer, int), (numpy.inexact, float, complex))


def _get_kind_score(kind):
    """0 for booleans, 1 for integers, 2 for floating and complex types, 3 for
    anything else."""
    for score, kinds in enumerate(_KIND_LADDER):
        if issubclass(kind, kinds):
            return score
    return len(_KIND_LADDER)


def _check_should_use_weak_scalar(in_types, weaks):
    """With the first-matching-loop strategy a weak Python scalar may only take
    part in loop selection when it is not of a higher kind than the arrays
    (so that ``uint8 array + 0.`` does not pick up a float64 loop by way of
    the scalar alone)."""
    if weaks is None:
        return False
    max_array_kind = -1
    max_scalar_kind = -1
    for in_t, w_t in zip(in_types, weaks):
        if w_t:
            max_scalar_kind = max(max_scalar_kind, _get_kind_score(w_t))
        else:
            max_array_kind = max(max_array_kind, _get_kind_score(in_t.type))
    all_scalars_or_arrays = max_scalar_kind == -1 or max_array_kind == -1
    return not all_scalars_or_arrays and max_array_kind >= max_scalar_kind


class _Op:
    """One typed loop of a ufunc / reduction: input and output dtypes plus the
    routine (code) or an ``error_func`` raising for a forbidden combination."""

    def __init__(self, in_types, out_types, routine, error_func):
        # a loop either has code or refuses its type combination
        assert callable(error_func) if error_func is not None else routine is not None
        self.in_types, self.out_types = in_types, out_types
        self.nin, self.nout = len(in_types), len(out_types)
        self.routine, self.error_func = routine, error_func
        self._in_dtypes = tuple(map(get_dtype, in_types))
        self._out_dtypes = tuple(map(get_dtype, out_types))

    @staticmethod
    def _from(typ, routine, error_func):
        """From a signature such as ``'ff->f'``; a signature without an arrow
        gives the outputs the inputs' types."""
        ins, arrow, outs = typ.partition('->')
        in_types = tuple(get_dtype(c).type for c in ins)
        out_types = tuple(get_dtype(c).type for c in outs) if arrow else in_types
        return _Op(in_types, out_types, routine, error_func)

    def check_valid(self):
        if self.error_func is not None:
            self.error_func()

    def resolve_dtypes(self, in_args, out_args):
        return self._in_dtypes, self._out_dtypes

    def __repr__(self):
        return '_Op(%s -> %s)' % (self.in_types, self.out_types)


class _Ops:

    def __init__(self, ops):
        assert len(ops) > 0
        self.ops = ops
        self.nin, self.nout = ops[0].nin, ops[0].nout
        for op in ops:
            if (op.nin, op.nout) != (self.nin, self.nout):
                raise ValueError(f'invalid op {op}, wrong nin or nout.')

    @staticmethod
    def from_tuples(ops, routine):
        """Loop table from the entries ``create_ufunc`` / ``create_reduction_func``
        take (reference: cupy/_core/_kernel.pyx:1622-1650)."""
        return _Ops(tuple(_Op._from(*_read_loop_entry(entry, routine)) for entry in ops))

    def guess_routine(self, name, cache, in_args, dtype, out_ops):
        """The loop for these inputs, or for ``dtype=`` if given; memoised in
        ``cache`` (reference: cupy/_core/_kernel.pyx:1652-1706)."""
        if dtype is None:
            in_types, weaks = _loop_selection_types(in_args)
            key, asked = (in_types, weaks), in_types
            search, what = self._guess_routine_from_in_types, (in_types, weaks)
        else:
            key = asked = dtype
            search, what = (out_ops or self)._guess_routine_from_dtype, (dtype,)
        try:
            op = cache[key]
        except KeyError:
            op = cache[key] = search(*what)
        if op is None:
            raise TypeError('Wrong type (%s) of arguments for %s' % (asked, name))
        op.check_valid()        # (raises for a combination the ufunc forbids)
        return op

    def _guess_routine_from_in_types(self, in_types, weaks=None):
        """First loop every input can be safely cast to.  A weak Python scalar
        that cannot be cast safely is still accepted when it would not change
        the loop's type under NumPy's promotion (NEP 50)."""
        if weaks is None:
            weaks = (False,) * len(in_types)
        for op in self.ops:
            if all(_input_fits(given, wanted, weak)
                   for given, wanted, weak in zip(in_types, op.in_types, weaks)):
                return op
        return None

    def _guess_routine_from_dtype(self, dtype):
        """First loop all of whose outputs have ``dtype``."""
        for op in self.ops:
            if all(t == dtype for t in op.out_types):
                return op
        return None


def _read_loop_entry(entry, default):
    """``(signature, routine, error function)`` of one loop-table entry.  A
    bare signature takes the table's default routine; a pair may bring its own
    routine, a tuple of routines whose gaps the default fills, or a callable
    that raises for a forbidden type combination."""
    if not isinstance(entry, tuple):
        if not isinstance(entry, str):
            raise ValueError(f'invalid op {entry}, expected string')
        return entry, default, None
    signature, own = entry
    if own is None:
        return signature, default, None
    if isinstance(own, tuple):
        return signature, tuple(mine or theirs for mine, theirs in zip(own, default)), None
    if isinstance(own, str):
        return signature, own, None
    if not callable(own):
        raise ValueError(f'invalid op {entry}, expected callable {own}')
    return signature, None, own


def _weak_int_misfits(op, in_args):
    """Whether a weak Python integer among the inputs lies outside the
    integer type of its loop input while the loop's result is of another kind
    than integer (for loops with integer results NumPy raises, and so does the
    conversion of the scalar later on)."""
    if op.out_types and numpy.dtype(op.out_types[0]).kind in 'iu':
        return False
    for x, t in zip(in_args, op.in_types):
        if type(x) is CScalar and x.weak_t is int:
            t = numpy.dtype(t)
            if t.kind in 'iu':
                info = numpy.iinfo(t)
                if not info.min <= x.value <= info.max:
                    return True
    return False


def _loop_selection_types(in_args):
    """``(dtypes, weak types or None)`` of preprocessed inputs, as loop selection
    sees them: a Python scalar counts as weak only where
    ``_check_should_use_weak_scalar`` lets it."""
    in_types = []
    weaks = []
    for arg in in_args:
        if type(arg) is CScalar:
            in_types.append(arg.descr)
            weaks.append(arg.weak_t)
        elif isinstance(arg, ndarray):
            in_types.append(arg.dtype)
            weaks.append(False)
        else:
            raise RuntimeError(f'Need array or CScalar got {type(arg)}')
    in_types = tuple(in_types)
    weaks = tuple(weaks) if any(w is not False for w in weaks) else None
    if not _check_should_use_weak_scalar(in_types, weaks):
        weaks = (False,) * len(in_types)
    return in_types, weaks


def _input_fits(given, wanted, weak):
    """Whether an input of dtype ``given`` may feed a loop input of dtype
    ``wanted``; ``weak`` is the Python type of a weak scalar or False."""
    if numpy.can_cast(given, wanted):
        return True
    if not weak:
        return False
    try:
        # a weak scalar that would promote the loop's type cannot use it
        return numpy.result_type(weak(0), wanted) == wanted
    except TypeError:
        return False


_UFUNC_KEYWORDS = frozenset(('out', '_where', 'where', 'dtype', 'casting'))


def _preprocess_where(dev_id, where):
    """The ``_where=`` argument as a one-element argument list: a boolean
    array, or a scalar taken by its truth value."""
    where_args = _preprocess_args(dev_id, (where,))
    mask = where_args[0]
    if not isinstance(mask, ndarray):
        where_args[0] = CScalar(bool(mask.value))
    elif mask.dtype != bool:
        raise TypeError(
            f'Cannot cast array data from {mask.dtype!r} to '
            f'{get_dtype(bool)!r} according to the rule \'safe\'')
    return where_args


class ufunc:
    """Universal function: typed loops selected the way NumPy selects them,
    broadcasting, ``out=``, ``dtype=``, ``casting=`` and ``_where=``.

    Attributes:
        name (str), nin (int), nout (int), nargs (int), types (list of str)
    """

    def __init__(self, name, nin, nout, ops, preamble='', loop_prep='', doc='',
                 default_casting=None, *, out_ops=None, cutensor_op=None,
                 scatter_op=None):
        self.name = self.__name__ = name
        self._doc = self.__doc__ = doc
        self.nin, self.nout, self.nargs = nin, nout, nin + nout
        self._ops, self._out_ops = ops, out_ops
        self._preamble, self._loop_prep = preamble, loop_prep
        self._default_casting = default_casting or 'same_kind'
        self._scatter_op = scatter_op
        _in_params = tuple(ParameterInfo('T in%d' % i, True) for i in range(nin))
        _out_params = tuple(ParameterInfo('T out%d' % i, False) for i in range(nout))
        self._params = _in_params + _out_params
        self._params_with_where = (
            _in_params + (ParameterInfo('T _where', True),) + _out_params)
        self._routine_cache = {}
        self._planners = {}
        self._kernel_memo = self._planners
        self._fast_calls = {}

    def __repr__(self):
        return '<ufunc \'%s\'>' % self.name

    @property
    def types(self):
        """Type signatures ``'ff->f'`` of the loops, in selection order."""
        types = []
        for op in self._ops.ops:
            in_str = ''.join(get_dtype(t).char for t in op.in_types)
            out_str = ''.join(get_dtype(t).char for t in op.out_types)
            types.append('%s->%s' % (in_str, out_str))
        return types

    def _split_arguments(self, args, kwargs):
        """``(inputs, outputs, where, dtype, casting)`` of a call; outputs may
        come after the inputs or through ``out=`` (an array, or a tuple with
        one entry per output).  Checks follow the reference's order and texts
        (cupy/_core/_kernel.pyx:1268-1305)."""
        unknown = {k: v for k, v in kwargs.items() if k not in _UFUNC_KEYWORDS}
        dtype = kwargs.get('dtype')
        if dtype is not None:
            dtype = get_dtype(dtype).type
        if unknown:
            raise TypeError('Wrong arguments %s' % unknown)
        given = len(args)
        if given < self.nin or given > self.nargs:
            raise TypeError(
                'Wrong number of arguments for {!r}. '
                'It must be either {} or {} (with outputs), '
                'but given {}.'.format(self.name, self.nin, self.nargs, given))
        inputs, outputs = args[:self.nin], args[self.nin:]
        out = kwargs.get('out')
        if out is not None:
            if outputs:
                raise ValueError('Cannot specify \'out\' as both '
                                 'a positional and keyword argument')
            as_tuple = isinstance(out, tuple)
            outputs = out if as_tuple else (out,)
            if len(outputs) != self.nout:
                raise ValueError(
                    "The 'out' tuple must have exactly one entry per ufunc output"
                    if as_tuple else "'out' must be a tuple of arrays")
        where = kwargs.get('_where')
        if where is None:
            # NumPy's spelling; True, its default, selects every element
            where = kwargs.get('where')
            if where is True:
                where = None
        return (inputs, outputs, where, dtype,
                kwargs.get('casting', self._default_casting))

    def __call__(self, *args, **kwargs):
        """Applies the function elementwise.

        Args:
            args: Inputs (arrays or scalars), optionally followed by outputs.
            out (cupy.ndarray or tuple): Output array(s).
            dtype: Selects the loop by its output type.
            casting (str): Rule for casting results into given outputs
                (default ``'same_kind'``).
        """
        if _fusion_thread_local.recording and _fusion_thread_local.is_fusing():
            for arg in args:
                if hasattr(arg, '__cupy_override_elementwise_kernel__'):
                    return arg.__cupy_override_elementwise_kernel__(
                        self, *args, **kwargs)
            return _fusion_thread_local.call_ufunc(self, *args, **kwargs)

        # A call that looks like an earlier one replays that call's launch.
        # (Only plain arrays and scalars have a signature, and calls with
        # structured arrays are never recorded, so a hit needs none of the
        # checks below.)
        fast_key = rec = fast_args = extra = None
        nk = len(kwargs)
        if nk == 0:
            fast_args = args
        else:
            # (``out``, ``casting`` and ``dtype``: the casting rule only decides
            # whether the types of the call, which the signature holds, may be
            # cast, and the dtype selects the loop: both join the key.  astype,
            # copies and fills pass the rule.  Keywords given as None --
            # wrappers hand ``out=None, dtype=None`` on -- count as absent.)
            o = kwargs.get('out')
            known = 0 if o is None else 1
            value = kwargs.get('casting')
            if type(value) is str:
                known += 1
                extra = value
            value = kwargs.get('dtype')
            if value is not None:
                try:
                    extra = (extra, get_dtype(value).char)
                    known += 1
                except TypeError:
                    pass
            live = 0
            for value in kwargs.values():
                if value is not None:
                    live += 1
            if known == live:
                if o is None:
                    fast_args = args
                elif len(args) == self.nin:
                    fast_args = args + (o if type(o) is tuple else (o,))
        if fast_args is not None and self.nin <= len(fast_args) <= self.nargs:
            fast_key = _launch_plan.call_signature(fast_args, _device.get_device_id())
            if fast_key is not None:
                if extra is not None:
                    fast_key = fast_key + (extra,)
                fast = self._fast_calls.get(fast_key)
                if fast is not None:
                    ret = fast.run(fast_args)
                    if ret is not NotImplemented:
                        return ret
                    fast_key = None
        for arg in args:
            if hasattr(arg, '__cupy_override_elementwise_kernel__'):
                return arg.__cupy_override_elementwise_kernel__(
                    self, *args, **kwargs)
        for arg in args:
            if type(arg) is ndarray and arg.dtype.kind == 'V':
                return _call_structured(self, args, kwargs)
        if fast_key is not None:
            rec = _launch_plan.Recorder(self.nargs)

        in_args, out_args, where, dtype, casting = self._split_arguments(args, kwargs)
        has_where = where is not None

        dev_id = _device.get_device_id()
        in_args = _preprocess_args(dev_id, in_args)
        out_args = _preprocess_optional_args(dev_id, out_args)
        given_out_args = [o for o in out_args if o is not None]
        where_args = _preprocess_where(dev_id, where) if has_where else []

        if rec is not None:
            before = list(in_args)
        _copy_in_args_if_needed(in_args, given_out_args)
        _copy_in_args_if_needed(where_args, given_out_args)
        if rec is not None and any(a is not b for a, b in zip(before, in_args)):
            rec = None          # an input was copied: nothing to replay
        inout_args = in_args + where_args + given_out_args
        shape = internal._broadcast_core(inout_args)
        n_in = len(in_args)
        in_args = inout_args[:n_in]
        where_args = inout_args[n_in:n_in + len(where_args)]

        op = self._ops.guess_routine(
            self.name, self._routine_cache, in_args, dtype, self._out_ops)
        if dtype is not None:
            # several loops may give that result type (every comparison gives
            # bool): NumPy takes the first one the arrays can be cast to safely
            same_result = [o for o in (self._out_ops or self._ops).ops
                           if all(t == dtype for t in o.out_types)]
            if len(same_result) > 1:
                for candidate in same_result:
                    if all(not isinstance(x, ndarray) or numpy.can_cast(x.dtype, t, 'safe')
                           for x, t in zip(in_args, candidate.in_types)):
                        op = candidate
                        op.check_valid()
                        break
            # the loop was chosen by its result: the arrays must be castable
            # to its inputs under the rule, as NumPy demands (a complex array
            # does not silently lose its imaginary part to ``dtype=float``)
            for i, (x, t) in enumerate(zip(in_args, op.in_types)):
                if isinstance(x, ndarray) and not numpy.can_cast(x.dtype, t, casting):
                    raise TypeError(
                        "Cannot cast ufunc '%s' input %d from %r to %r with casting rule '%s'"
                        % (self.name.replace('cupy_', ''), i, x.dtype, numpy.dtype(t), casting))
        if dtype is None and _weak_int_misfits(op, in_args):
            # a Python integer outside the integer type the arrays chose, in a
            # loop that answers in another kind (a comparison, a true division,
            # a logical function): NumPy computes with the integer's value, so
            # it counts as a 64-bit integer of its own instead of wrapping or
            # raising (``uint8_array == -1`` is all False, ``uint8_array / -1``
            # is negative)
            in_args = [CScalar(x.value, x.descr) if type(x) is CScalar and x.weak_t is int
                       else x for x in in_args]
            op = self._ops.guess_routine(
                self.name, self._routine_cache, in_args, dtype, self._out_ops)

        # outputs are of the first array subclass among the inputs
        template = next((a for a in in_args
                         if type(a) is not ndarray and isinstance(a, ndarray)), None)
        subtype = ndarray if template is None else type(template)

        core_in_dtypes, core_out_dtypes = op.resolve_dtypes(in_args, out_args)
        out_args = _get_out_args_from_optionals(
            subtype, out_args, core_out_dtypes, shape, casting, template)
        ret = out_args[0] if self.nout == 1 else tuple(out_args)
        if 0 in shape:
            return ret

        if has_where and any(o.dtype != t for o, t in zip(out_args, core_out_dtypes)):
            # The kernel keeps what a masked-out element held by reading it as
            # the loop's result type, which cannot hold every value of another
            # type (a comparison into an integer array turned every skipped
            # element into 0 or 1).  Such a call computes into arrays of the
            # loop's types, converts them, and copies under the mask between
            # arrays of ONE type.
            from cupy_amd._core._ufuncs import elementwise_copy
            plain = {k: v for k, v in kwargs.items() if k in ('dtype', 'casting')}
            fresh = self(*args[:self.nin], **plain)
            for o, r in zip(out_args, fresh if self.nout > 1 else (fresh,)):
                elementwise_copy(r.astype(o.dtype, copy=False), o, _where=where)
            return ret

        for i, t in enumerate(core_in_dtypes):
            if type(in_args[i]) is CScalar:
                in_args[i].apply_dtype(t)

        planner = self._get_planner(op, has_where)
        all_args = in_args + where_args + out_args
        nin_total = n_in + len(where_args)
        # Body variables carry the loop's types; elements are converted on load
        # and store when the array's dtype differs.
        var_types = ['in%d_type' % i for i in range(n_in)]
        casts = []
        for i, a in enumerate(in_args):
            if isinstance(a, ndarray):
                lt = core_in_dtypes[i]
                casts.append((_make_cast(a.dtype, lt), None))
            else:
                casts.append((None, None))
        if has_where:
            var_types.append('bool')
            casts.append((None, None))
        for i, a in enumerate(out_args):
            var_types.append('out%d_type' % i)
            lt = core_out_dtypes[i]
            casts.append((_make_cast(a.dtype, lt), _make_cast(lt, a.dtype)))
        typedefs = ''.join(
            ['typedef %s in%d_type;\n' % (_get_typename(t), i)
             for i, t in enumerate(core_in_dtypes)]
            + ['typedef %s out%d_type;\n' % (_get_typename(t), i)
               for i, t in enumerate(core_out_dtypes)])
        planner.launch(
            dev_id, all_args, nin_total, shape, var_types, typedefs, casts=casts,
            force_generic=False, force_read_out=has_where,
            kernel_name=self._get_name_with_type(all_args, has_where), rec=rec)
        # (a cast that warns -- complex to real under 'unsafe' -- warns every time)
        warns = casting == 'unsafe' and any(
            get_dtype(lt).kind == 'c' and a.dtype.kind in 'iuf'
            for a, lt in zip(out_args, core_out_dtypes))
        if rec is not None and len(rec.launches) == 1 and not warns:
            n_user = len(fast_args)
            n_given = n_user - self.nin
            ret_refs = self.nin if self.nout == 1 else tuple(range(self.nin, self.nargs))
            out_specs = tuple((shape, o.dtype) for o in out_args[n_given:])
            overlap = [(i, self.nin + j) for j in range(n_given)
                       for i in range(self.nin) if isinstance(in_args[i], ndarray)]
            _launch_plan.remember(
                self._fast_calls, fast_key,
                _launch_plan.FastCall(n_user, out_specs, rec, ret_refs, overlap))
        return ret

    def _get_planner(self, op, has_where):
        key = (op, has_where)
        planner = self._planners.get(key)
        if planner is None:
            routine = op.routine
            if has_where:
                # masked-out elements keep the previous contents of the output
                names = ['out%d' % i for i in range(self.nout)]
                saves = ' '.join('const out%d_type _keep%d = %s;' % (i, i, n)
                                 for i, n in enumerate(names))
                restores = ' '.join('%s = _keep%d;' % (n, i)
                                    for i, n in enumerate(names))
                routine = '%s %s; if (!_where) { %s }' % (saves, routine, restores)
                params = self._params_with_where
            else:
                params = self._params
            planner = _ElementwisePlanner(
                self.name, params, routine, self._preamble, self._loop_prep, '',
                (), is_ufunc=True)
            planner = self._planners.setdefault(key, planner)
        return planner

    def _get_name_with_type(self, args, has_where):
        name = self.name
        if has_where:
            name += '_where'
        words = []
        for a in args:
            if isinstance(a, ndarray):
                words.append(a.dtype.name)
            else:
                words.append(a.descr.name.rstrip('0123456789'))
        return '{}__{}'.format(name, '_'.join(words))

    def outer(self, A, B, **kwargs):
        """Applies the ufunc to all pairs of elements of ``A`` and ``B``."""
        from cupy_amd._core.core import array
        A = array(A, copy=False)
        B = array(B, copy=False)
        A = A.reshape(A.shape + (1,) * B.ndim)
        B = B.reshape((1,) * (A.ndim - B.ndim) + B.shape) if B.ndim else B
        return self(A, B, **kwargs)

    def at(self, a, indices, b=None):
        """Applies the operation in place at ``a[indices]``, once per
        occurrence of an index (``numpy.ufunc.at``); available for the ufuncs
        that carry a scatter operation: add, subtract, maximum, minimum,
        bitwise_and / or / xor (cupy/_core/_kernel.pyx:1447-1456)."""
        if self._scatter_op is None:
            raise NotImplementedError(f'`{self.name}.at` is not supported yet')
        if b is None:
            raise ValueError('second operand needed for ufunc')
        from cupy_amd._core import _scatter
        _scatter.scatter_op(a, indices, b, self._scatter_op)

    # reductions and scans exist for the two ufuncs whose reduction is an
    # ndarray method (cupy/_core/_kernel.pyx:1452-1483)
    _REDUCE_METHODS = {'cupy_add': 'sum', 'cupy_multiply': 'prod'}
    _ACCUMULATE_METHODS = {'cupy_add': 'cumsum', 'cupy_multiply': 'cumprod'}

    def reduce(self, array, axis=0, dtype=None, out=None, keepdims=False):
        method = self._REDUCE_METHODS.get(self.name)
        if method is None:
            raise NotImplementedError(f'`{self.name}.reduce` is not supported yet')
        return getattr(array, method)(axis, dtype, out, keepdims)

    def accumulate(self, array, axis=0, dtype=None, out=None):
        method = self._ACCUMULATE_METHODS.get(self.name)
        if method is None:
            raise NotImplementedError(f'`{self.name}.accumulate` is not supported yet')
        return getattr(array, method)(axis, dtype, out)

    def reduceat(self, array, indices, axis=0, dtype=None, out=None):
        """``numpy.ufunc.reduceat`` for add (cupy/_core/_kernel.pyx:1485-1493)."""
        if self.name == 'cupy_add':
            from cupy_amd._core import _scatter
            return _scatter.add_reduceat(array, indices, axis, dtype, out)
        raise NotImplementedError(
            f'`{self.name}.reduceat` is not supported yet')


_struct_kernels = {}


def _call_structured(ufunc_obj, args, kwargs):
    """Copy and (in)equality of arrays whose elements are structures: the
    loops the reference has for them (cupy/_core/_routines_logic.pyx:76-117,
    field-wise assignment in include/cupy/structview.cuh)."""
    from cupy_amd._core import _structured
    from cupy_amd._core.core import array
    out = kwargs.pop('out', None)
    kwargs.pop('casting', None)
    if kwargs:
        raise TypeError('Wrong arguments %s' % kwargs)
    name = ufunc_obj.name
    if name not in ('cupy_copy', 'cupy_equal', 'cupy_not_equal'):
        raise TypeError('ufunc %r is not supported for structured dtypes' % name)
    args = list(args)
    if len(args) == ufunc_obj.nin + 1 and out is None:
        out = args.pop()
    if len(args) != ufunc_obj.nin:
        raise TypeError('Wrong number of arguments for %r' % name)
    if isinstance(out, tuple):
        (out,) = out
    ins = [a if isinstance(a, ndarray) else array(a) for a in args]
    if name == 'cupy_copy':
        (src,) = ins
        if out is None:
            out = ndarray._new_contiguous(src.shape, src.dtype)
        if src.dtype.fields is not None and out.dtype.fields is not None and \
                not numpy.can_cast(src.dtype, out.dtype, 'unsafe'):
            raise TypeError(f'Cannot cast array data from {src.dtype!r} to {out.dtype!r}')
        if src.dtype.fields is not None and out.dtype.fields is None:
            raise TypeError(f'Cannot cast array data from {src.dtype!r} to {out.dtype!r}')
        if out.dtype.kind == 'V' and out.dtype.fields is None and src.dtype != out.dtype:
            raise TypeError('raw bytes are only copied between arrays of the same dtype, '
                            f'not from {src.dtype!r} to {out.dtype!r}')
        kern = _struct_kernels.get('copy')
        if kern is None:
            kern = _struct_kernels['copy'] = ElementwiseKernel(
                'X x', 'Y y', 'y = x', 'cupy_copy_struct')
        if out.size:
            kern(src, out)
        return out
    a, b = ins
    common = _structured.comparison_dtype(a.dtype, b.dtype)
    if any(f[0].subdtype is not None for f in (common.fields or {}).values()):
        raise ValueError('comparison of structured arrays with subarray dtypes is not supported')
    # both sides in the common dtype first, as the reference's loop resolution
    # has it: field values are then compared like with like
    if a.dtype != common:
        a = a.astype(common)
    if b.dtype != common:
        b = b.astype(common)
    key = 'eq' if name == 'cupy_equal' else 'ne'
    kern = _struct_kernels.get(key)
    if kern is None:
        kern = _struct_kernels[key] = ElementwiseKernel(
            'X a, Y b', 'bool z', 'z = (a %s b)' % ('==' if key == 'eq' else '!='),
            'cupy_%s_struct' % ('equal' if key == 'eq' else 'not_equal'))
    if out is None:
        return kern(a, b)
    return kern(a, b, out)


def _make_cast(src_dtype, dst_dtype):
    """Callable(expr) applying the conversion quirks between two dtypes, or
    None when a plain C++ conversion does."""
    src = get_dtype(src_dtype)
    dst = get_dtype(dst_dtype)
    if src.kind == dst.kind or (src.kind != 'b' and 'c' not in (src.kind, dst.kind)):
        return None
    return lambda e: fix_cast_expr(src, dst, e)


def create_ufunc(name, ops, routine=None, preamble='', doc='',
                 default_casting=None, loop_prep='', out_ops=None,
                 cutensor_op=None, scatter_op=None, promote_types=None):
    """Builds a ufunc from loop signatures (``'ff->f'`` or
    ``('ff->f', routine)``) and a default routine."""
    ops_ = _Ops.from_tuples(ops, routine)
    _out_ops = None if out_ops is None else _Ops.from_tuples(out_ops, routine)
    return ufunc(name, ops_.nin, ops_.nout, ops_, preamble, loop_prep, doc,
                 default_casting=default_casting, out_ops=_out_ops,
                 cutensor_op=cutensor_op, scatter_op=scatter_op)
