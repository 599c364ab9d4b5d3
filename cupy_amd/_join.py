"""Joining, splitting, tiling and rolling arrays.  Splits are views; the others
allocate the result once and fill it piece by piece with the package's own
copy kernel (each piece is a strided window of the result, which the
elementwise planner turns into rows or tiles), so every element is read once
and written once.  Each function cites the reference function whose
arguments and errors it keeps."""
import functools
import itertools
import operator
import struct

import numpy

from cupy_amd._core import internal
from cupy_amd._core import _dtype
from cupy_amd._core import _tuning
from cupy_amd._core.core import ndarray, asarray
from cupy_amd._core._ufuncs import elementwise_copy


def _window(arr, axis, start, stop):
    return arr[tuple(slice(start, stop) if ax == axis else slice(None) for ax in range(arr.ndim))]


# ---------------------------------------------------------------------------------
# the pieces of a concatenation in one launch
# ---------------------------------------------------------------------------------
# Seen from the joined axis, a piece whose trailing axes are stored one after
# the other is a matrix: rows = the axes before the joined one, a row = one
# contiguous run of (extent along the axis) x (elements behind it), and its
# place in the result is the same matrix with the result's row pitch.  One
# kernel copies up to _MAX_PIECES such matrices: workgroups are dealt out to
# the pieces in proportion to their sizes (a table of first workgroups in the
# argument block), a thread moves a vector or a few, all requested before the
# first is stored; a row's last vector may be a partial one, done element by
# element.  A launch per piece costs a ramp and a tail each: two
# windows of 128 MiB took 95.7 us in two launches.

_MAX_PIECES = 8
_NARROW_PIECE_BYTES = 1 << 20

_PIECES_SOURCE = r"""
#include <cupy/carray.cuh>
struct Piece {
  const ITEM_T* src;
  ITEM_T* dst;
  long long src_pitch;      // elements between rows
  long long dst_pitch;
  unsigned int vecs_per_row;  // the last vector of a row may be a partial one
  unsigned int n_vecs;      // rows * vecs_per_row
  unsigned int first_block;
  unsigned int n_rep;       // copies of the piece in the result ...
  long long rep_step;       // ... this many elements apart
  unsigned int row_len;     // elements per row
  unsigned int pad;
};
struct Pieces { Piece p[MAX_PIECES]; };

extern "C" __global__ void __launch_bounds__(BLOCK)
cupy_concatenate_pieces(const Pieces ps, const int n_pieces) {
  int k = 0;
#pragma unroll
  for (int j = 1; j < MAX_PIECES; ++j)
    if (j < n_pieces && blockIdx.x >= ps.p[j].first_block) k = j;
  const Piece pc = ps.p[k];
  const unsigned int base = (blockIdx.x - pc.first_block) * (BLOCK * UNROLL) + threadIdx.x;
  cupy::Vec<ITEM_T, NV> v[UNROLL];
  long long to[UNROLL];
  unsigned int have[UNROLL];    // elements of the vector inside the row
#pragma unroll
  for (int u = 0; u < UNROLL; ++u) {
    const unsigned int i = base + u * BLOCK;
    have[u] = 0;
    if (i < pc.n_vecs) {
      const unsigned int r = i / pc.vecs_per_row;
      const unsigned int c = (i - r * pc.vecs_per_row) * NV;
      const ITEM_T* from = pc.src + r * pc.src_pitch + c;
      to[u] = r * pc.dst_pitch + c;
      have[u] = pc.row_len - c < NV ? pc.row_len - c : NV;
      if (have[u] == NV) {
        v[u] = cupy::load_vec<ITEM_T, NV, STREAM_IN>(from);
      } else {
#pragma unroll
        for (int e = 0; e < NV; ++e) if (e < have[u]) v[u].v[e] = from[e];
      }
    }
  }
#pragma unroll
  for (int u = 0; u < UNROLL; ++u) {
    if (have[u] == 0) continue;
    for (unsigned int j = 0; j < pc.n_rep; ++j) {
      ITEM_T* at = pc.dst + to[u] + j * pc.rep_step;
      if (have[u] == NV) {
        cupy::store_vec<ITEM_T, NV, STREAM_OUT>(at, v[u]);
      } else {
#pragma unroll
        for (int e = 0; e < NV; ++e) if (e < have[u]) at[e] = v[u].v[e];
      }
    }
  }
}
"""

_PIECE_STRUCT = struct.Struct('<QQqqIIIIqII')  # struct Piece of the kernel source


class _ArgBytes:
    """Bytes passed by value as one kernel argument."""

    def __init__(self, data):
        self._data = data

    def _kernel_arg_bytes(self):
        return self._data


_ITEM_TYPES = {1: 'unsigned char', 2: 'unsigned short', 4: 'unsigned int',
               8: 'unsigned long long'}

_pieces_kernels = {}


def _geometry():
    """(threads per workgroup, vectors per thread) of the kernel."""
    return _tuning.get('concatenate_block'), _tuning.get('concatenate_unroll')


def _pieces_kernel(itemsize, nv, stream_in, stream_out):
    _BLOCK, _UNROLL = _geometry()
    key = (itemsize, nv, stream_in, stream_out, _BLOCK, _UNROLL)
    ker = _pieces_kernels.get(key)
    if ker is None:
        from cupy_amd._core.raw import RawKernel
        defines = (('ITEM_T', 'item_t'), ('NV', nv), ('MAX_PIECES', _MAX_PIECES),
                   ('BLOCK', _BLOCK), ('UNROLL', _UNROLL),
                   ('STREAM_IN', 'true' if stream_in else 'false'),
                   ('STREAM_OUT', 'true' if stream_out else 'false'))
        source = 'typedef %s item_t;\n' % _ITEM_TYPES[itemsize] + _PIECES_SOURCE
        ker = _pieces_kernels[key] = RawKernel(
            source, 'cupy_concatenate_pieces', tuple('-D%s=%s' % d for d in defines))
    return ker


def _as_rows(shape, strides, item, lead):
    """(rows, elements per row, elements between rows) of a layout whose axes
    from ``lead`` on are stored one after the other and whose axes before it
    step evenly and forwards; None for any other layout."""
    run = item
    for k in range(len(shape) - 1, lead - 1, -1):
        if shape[k] != 1 and strides[k] != run:
            return None
        run *= shape[k]
    rows, pitch = 1, run
    for k in range(lead - 1, -1, -1):
        ext = shape[k]
        if ext == 1:
            continue
        st = strides[k]
        if rows == 1:
            if st < run or st % item:
                return None
            pitch = st
        elif st != pitch * rows:
            return None
        rows *= ext
    return rows, run // item, pitch // item


def _plan_pieces(pieces, dtype, copies=1, copy_step=0):
    """What the one-launch kernel needs to copy ``pieces``, a list of (shape,
    strides and address of the source, strides and address of its place in
    the result), all of element type ``dtype``, each to ``copies`` places
    ``copy_step`` bytes apart: (bytes per word, words per vector, [(source
    address, destination address, rows, words per row, words between the rows
    of the source, of the destination, copies, words between them)]), or None
    if a piece does not fit the kernel (a layout that is no matrix of
    contiguous rows, many rows of a few elements, 2**31 words or more)."""
    if len(pieces) * copies < 2 or dtype.fields is not None:
        return None
    item = dtype.itemsize
    # 16-byte elements travel as pairs of 8-byte words
    word, words = (8, 2) if item == 16 else (item, 1)
    if word not in _ITEM_TYPES:
        return None
    nv = 16 // word
    if copy_step % word:
        return None
    forms = []
    for shape, sstrides, sptr, dstrides, dptr in pieces:
        # the longest rows both sides have
        for lead in range(len(shape) + 1):
            fs = _as_rows(shape, sstrides, item, lead)
            if fs is None:
                continue
            fd = _as_rows(shape, dstrides, item, lead)
            if fd is not None:
                break
        else:
            return None
        rows, row = fs[0], fs[1] * words
        if rows > 1 and row * word < 64 and rows * row * word > _NARROW_PIECE_BYTES:
            # a few elements per row, and many rows: the tiled kernels do these better
            return None
        sp, dp = fs[2] * words, fd[2] * words
        if sp == row and dp == row:
            # rows follow each other on both sides: one long row
            rows, row = 1, rows * row
            sp = dp = row
        if rows * ((row + nv - 1) // nv) * nv >= 1 << 31:
            return None
        forms.append((sptr, dptr, rows, row, sp, dp, copies, copy_step // word))
    return word, nv, forms


def _piece_tables(nv, forms):
    """The argument tables of the launches that copy ``forms``, eight pieces a
    launch: [(table bytes, pieces in it, workgroups)]."""
    block, unroll = _geometry()
    per_block = block * unroll
    launches = []
    for lo in range(0, len(forms), _MAX_PIECES):
        batch = forms[lo:lo + _MAX_PIECES]
        table = bytearray(_MAX_PIECES * _PIECE_STRUCT.size)
        blocks = 0
        for k, (sptr, dptr, rows, row, sp, dp, copies, step) in enumerate(batch):
            vecs_per_row = (row + nv - 1) // nv
            n_vecs = rows * vecs_per_row
            _PIECE_STRUCT.pack_into(table, k * _PIECE_STRUCT.size, sptr, dptr, sp, dp,
                                    vecs_per_row, n_vecs, blocks, copies, step, row, 0)
            blocks += (n_vecs + per_block - 1) // per_block
        launches.append((bytes(table), len(batch), blocks))
    return launches


def _copy_pieces(pieces, dtype, nbytes, copies=1, copy_step=0):
    """Copies the pieces (``nbytes`` in all), each to ``copies`` places, with
    the one-launch kernel; False, with nothing done, if they do not fit it."""
    plan = _plan_pieces(pieces, dtype, copies, copy_step)
    if plan is None:
        return False
    word, nv, forms = plan
    stream_in, stream_out = _tuning.stream_policy(
        _tuning.get('flat_stream'), nbytes, nbytes * copies)
    ker = _pieces_kernel(word, nv, stream_in, stream_out)
    block = _geometry()[0]
    for table, n_pieces, blocks in _piece_tables(nv, forms):
        ker((blocks,), (block,), (_ArgBytes(table), numpy.int32(n_pieces)))
    return True


def _concatenate(arrays, axis, out, dtype, casting):
    """reference: cupy/_core/_routines_manipulation.pyx:652-760 (concatenate_method)"""
    arrays = list(arrays)
    if not arrays:
        raise ValueError('Cannot concatenate from empty tuple')
    for a in arrays:
        if not isinstance(a, ndarray):
            raise TypeError('Only cupy arrays can be concatenated')
    for a in arrays:
        if a.ndim == 0:
            raise TypeError('zero-dimensional arrays cannot be concatenated')
    first = arrays[0]
    nd = first.ndim
    if any(a.ndim != nd for a in arrays):
        raise ValueError('All arrays to concatenate must have the same ndim')
    axis = internal._normalize_axis_index(axis, nd)
    shape = list(first.shape)
    for a in arrays[1:]:
        if any(ax != axis and shape[ax] != a.shape[ax] for ax in range(nd)):
            raise ValueError('All arrays must have same shape except the axis to concatenate')
        shape[axis] += a.shape[axis]
    shape = tuple(shape)
    if out is None:
        if dtype is None:
            kinds = {a.dtype for a in arrays}
            dtype = first.dtype if len(kinds) == 1 else functools.reduce(numpy.promote_types, kinds)
        else:
            dtype = _dtype.get_dtype(dtype)
    else:
        if dtype is not None:
            raise TypeError('concatenate() only takes `out` or `dtype` as an '
                            'argument, but both were provided.')
        dtype = out.dtype
    for a in arrays:
        _dtype._raise_if_invalid_cast(a.dtype, dtype, casting)
    if out is None:
        out = ndarray(shape, dtype)
    else:
        if out.ndim != nd:
            raise ValueError('Output array has wrong dimensionality')
        if out.shape != shape:
            raise ValueError('Output array is the wrong shape')
    # (source, first index along the axis) of the pieces that hold anything
    placed, at = [], 0
    for a in arrays:
        if a.size:
            placed.append((a, at))
        at += a.shape[axis]
    if not placed:
        return out
    step = out.strides[axis]
    same_type = all(a.dtype == dtype for a, _ in placed)
    if same_type and _tuning.get('concatenate_one_launch') and _copy_pieces(
            [(a.shape, a.strides, a.data.ptr, out.strides, out.data.ptr + at * step)
             for a, at in placed], dtype, sum(a.nbytes for a, _ in placed)):
        return out
    for a, at in placed:
        elementwise_copy(a, _window(out, axis, at, at + a.shape[axis]), casting=casting)
    return out


def concatenate(tup, axis=0, out=None, *, dtype=None, casting='same_kind'):
    """Joins arrays along an existing axis (``axis=None``: their flattened forms)
    (reference: cupy/_manipulation/join.py:39-64)."""
    if axis is None:
        tup = [a.ravel() if isinstance(a, ndarray) else a for a in tup]
        axis = 0
    return _concatenate(tup, axis, out, dtype, casting)


def stack(tup, axis=0, out=None, *, dtype=None, casting='same_kind'):
    """Joins arrays along a new axis (reference: cupy/_manipulation/join.py:147-170)."""
    tup = list(tup)
    for a in tup:
        if not isinstance(a, ndarray):
            raise TypeError('Only cupy arrays can be stacked')
    if tup and any(a.shape != tup[0].shape for a in tup):
        raise ValueError('all input arrays must have the same shape')
    if tup:
        axis = internal._normalize_axis_index(axis, tup[0].ndim + 1)
    from cupy_amd._manipulation import expand_dims
    return _concatenate([expand_dims(a, axis) for a in tup], axis, out, dtype, casting)


def hstack(tup, *, dtype=None, casting='same_kind'):
    """reference: cupy/_manipulation/join.py:83-108"""
    from cupy_amd._manipulation import atleast_1d
    arrs = [atleast_1d(a) for a in tup]
    axis = 0 if arrs and arrs[0].ndim == 1 else 1
    return _concatenate(arrs, axis, None, dtype, casting)


def vstack(tup, *, dtype=None, casting='same_kind'):
    """reference: cupy/_manipulation/join.py:111-134"""
    from cupy_amd._manipulation import atleast_2d
    return _concatenate([atleast_2d(a) for a in tup], 0, None, dtype, casting)


row_stack = vstack


def dstack(tup):
    """reference: cupy/_manipulation/join.py:67-80"""
    from cupy_amd._manipulation import atleast_3d
    return _concatenate([atleast_3d(a) for a in tup], 2, None, None, 'same_kind')


def column_stack(tup):
    """1-d arrays become the columns of a matrix, 2-d arrays are joined as
    they are (reference: cupy/_manipulation/join.py:9-36)."""
    if any(not isinstance(a, ndarray) for a in tup):
        raise TypeError('Only cupy arrays can be column stacked')
    cols = []
    for a in tup:
        if a.ndim == 1:
            a = a[:, None]
        elif a.ndim != 2:
            raise ValueError('Only 1 or 2 dimensional arrays can be column stacked')
        cols.append(a)
    return _concatenate(cols, 1, None, None, 'same_kind')


# ---------------------------------------------------------------------------------
# splitting: views
# ---------------------------------------------------------------------------------

def array_split(ary, indices_or_sections, axis=0):
    """Views of consecutive pieces of one axis; a count that does not divide
    the axis gives the first pieces one element more
    (reference: cupy/_core/_routines_manipulation.pyx `array_split`)."""
    nd = ary.ndim
    if not -nd <= axis < nd:
        raise IndexError('Axis exceeds ndim')
    axis %= nd
    size = ary.shape[axis]
    if numpy.isscalar(indices_or_sections):
        sections = operator.index(indices_or_sections)
        if sections <= 0:
            raise ValueError('number sections must be larger than 0.')
        each, extra = divmod(size, sections)
        cuts = list(itertools.accumulate([each + 1] * extra + [each] * (sections - extra)))[:-1]
    else:
        cuts = [operator.index(i) for i in indices_or_sections]
    pieces, prev = [], 0
    for cut in cuts + [size]:
        # NumPy's slicing rules: negative cuts count from the end, cuts out of
        # range or out of order give empty pieces
        piece = _window(ary, axis, prev, cut)
        pieces.append(piece)
        prev = cut
    return pieces


def split(ary, indices_or_sections, axis=0):
    """reference: cupy/_manipulation/split.py:51-80"""
    if ary.ndim <= axis:
        raise IndexError('Axis exceeds ndim')
    if numpy.isscalar(indices_or_sections):
        if ary.shape[axis] % indices_or_sections != 0:
            raise ValueError(
                'indices_or_sections must divide the size along the axes.\n'
                'If you want to split the array into non-equally-sized '
                'arrays, use array_split instead.')
    return array_split(ary, indices_or_sections, axis)


def hsplit(ary, indices_or_sections):
    """reference: cupy/_manipulation/split.py:34-48"""
    if ary.ndim == 0:
        raise ValueError('Cannot hsplit a zero-dimensional array')
    return split(ary, indices_or_sections, 0 if ary.ndim == 1 else 1)


def vsplit(ary, indices_or_sections):
    """reference: cupy/_manipulation/split.py:83-94"""
    if ary.ndim <= 1:
        raise ValueError('Cannot vsplit an array with less than 2 dimensions')
    return split(ary, indices_or_sections, 0)


def dsplit(ary, indices_or_sections):
    """reference: cupy/_manipulation/split.py:21-31"""
    if ary.ndim <= 2:
        raise ValueError('Cannot dsplit an array with less than 3 dimensions')
    return split(ary, indices_or_sections, 2)


# ---------------------------------------------------------------------------------
# tiling
# ---------------------------------------------------------------------------------

def tile(A, reps):
    """The array repeated ``reps`` times along each axis: ONE broadcast copy
    into a result seen as (rep, extent) pairs of axes
    (reference: cupy/_manipulation/tiling.py:7-55)."""
    reps = tuple(reps) if isinstance(reps, (tuple, list)) else (reps,)
    reps = tuple(operator.index(r) for r in reps)
    a = asarray(A)
    nd = max(a.ndim, len(reps))
    if all(r == 1 for r in reps):
        return a.reshape((1,) * (nd - a.ndim) + a.shape).copy()
    shape = (1,) * (nd - a.ndim) + a.shape
    reps = (1,) * (nd - len(reps)) + reps
    out = ndarray(tuple(s * r for s, r in zip(shape, reps)), a.dtype)
    if out.size == 0:
        return out
    a = a.reshape(shape)
    # result axis k of extent r*s is the pair (r, s); the source has a step of 0 over r
    pair_shape = tuple(itertools.chain.from_iterable(zip(reps, shape)))
    paired = out.reshape(pair_shape)
    if _tuning.get('concatenate_one_launch') and _tile_pieces(a, paired, reps):
        return out
    src = a._view(pair_shape, tuple(itertools.chain.from_iterable((0, st) for st in a.strides)))
    elementwise_copy(src, paired)
    return out


def _tile_pieces(a, paired, reps):
    """The tiles written by the kernel that copies pieces: the source is read
    once per tile along all axes but the one with most repetitions, whose
    tiles are stored from the same registers."""
    most = max(range(len(reps)), key=lambda k: reps[k])
    others = [range(r) if k != most else range(1) for k, r in enumerate(reps)]
    if internal.prod([len(o) for o in others]) > 64:
        return False
    rep_strides, own_strides = paired.strides[0::2], paired.strides[1::2]
    pieces = [(a.shape, a.strides, a.data.ptr, own_strides,
               paired.data.ptr + sum(i * st for i, st in zip(combo, rep_strides)))
              for combo in itertools.product(*others)]
    return _copy_pieces(pieces, a.dtype, a.nbytes * len(pieces), reps[most], rep_strides[most])


def repeat(a, repeats, axis=None):
    """Every element repeated: one count for all (a broadcast copy) or a count
    per element given on the host (a copy per run)
    (reference: cupy/_manipulation/tiling.py:58-75,
    cupy/_core/_routines_manipulation.pyx `_repeat`)."""
    if isinstance(repeats, ndarray):
        raise ValueError('cupy.ndaray cannot be specified as `repeats` argument.')
    if axis is None:
        a = a.ravel()
        axis = 0
    else:
        axis = internal._normalize_axis_index(axis, a.ndim)
    if isinstance(repeats, (int, numpy.integer)):
        counts = [operator.index(repeats)]
    else:
        counts = [operator.index(r) for r in repeats]
    if any(c < 0 for c in counts):
        raise ValueError("'repeats' should not be negative: {}".format(repeats))
    n = a.shape[axis]
    if len(counts) == 1:
        r = counts[0]
        shape = a.shape[:axis] + (n * r,) + a.shape[axis + 1:]
        out = ndarray(shape, a.dtype)
        if out.size:
            paired = out.reshape(a.shape[:axis] + (n, r) + a.shape[axis + 1:])
            own = paired.strides[:axis + 1] + paired.strides[axis + 2:]
            if not (_tuning.get('concatenate_one_launch') and _copy_pieces(
                    [(a.shape, a.strides, a.data.ptr, own, paired.data.ptr)], a.dtype, a.nbytes,
                    r, paired.strides[axis + 1])):
                src = a._view(paired.shape,
                              a.strides[:axis] + (a.strides[axis], 0) + a.strides[axis + 1:])
                elementwise_copy(src, paired)
        return out
    if len(counts) != n:
        raise ValueError("'repeats' and 'axis' of 'a' should be same length: {} != {}".format(
            n, len(counts)))
    shape = a.shape[:axis] + (sum(counts),) + a.shape[axis + 1:]
    out = ndarray(shape, a.dtype)
    at = 0
    for i, c in enumerate(counts):
        if c and out.size:
            dst = _window(out, axis, at, at + c)
            src = _window(a, axis, i, i + 1)
            elementwise_copy(src._view(dst.shape, src.strides[:axis] + (0,) + src.strides[axis + 1:]), dst)
        at += c
    return out


# ---------------------------------------------------------------------------------
# rolling and quarter turns
# ---------------------------------------------------------------------------------

def roll(a, shift, axis=None):
    """Elements shifted along the axes, those pushed out re-enter at the other
    end; shifts are host integers (reference: cupy/_manipulation/rearrange.py:75-147)."""
    if isinstance(shift, ndarray):
        raise NotImplementedError('roll with a device array of shifts is not part of this build')
    if axis is None:
        return roll(a.ravel(), shift, 0).reshape(a.shape)
    axes = (axis,) if numpy.isscalar(axis) else tuple(axis)
    axes = tuple(internal._normalize_axis_index(ax, a.ndim) for ax in axes)
    pairs = numpy.broadcast(shift, axes)
    if pairs.nd > 1:
        raise ValueError("'shift' and 'axis' should be scalars or 1D sequences")
    total = dict.fromkeys(range(a.ndim), 0)
    for sh, ax in pairs:
        total[ax] += int(sh)
    # per axis: the (source, destination) windows the shift cuts it into
    cuts = []
    for ax in range(a.ndim):
        off = total[ax] % (a.shape[ax] or 1)
        if off:
            cuts.append(((slice(None, -off), slice(off, None)), (slice(-off, None), slice(None, off))))
        else:
            cuts.append(((slice(None), slice(None)),))
    out = ndarray(a.shape, a.dtype)
    if out.size == 0:
        return out
    moves = []
    for combo in itertools.product(*cuts):
        src, dst = zip(*combo)
        moves.append((a[src], out[dst]))
    if not (_tuning.get('concatenate_one_launch') and _copy_pieces(
            [(s.shape, s.strides, s.data.ptr, d.strides, d.data.ptr) for s, d in moves],
            a.dtype, a.nbytes)):
        for s, d in moves:
            elementwise_copy(s, d)
    return out


def rot90(a, k=1, axes=(0, 1)):
    """View turned by quarter turns in the plane of two axes
    (reference: cupy/_manipulation/rearrange.py:150-193)."""
    nd = a.ndim
    if nd < 2:
        raise ValueError('Input must be >= 2-d')
    axes = tuple(axes)
    if len(axes) != 2:
        raise ValueError('len(axes) must be 2')
    if axes[0] == axes[1] or abs(axes[0] - axes[1]) == nd:
        raise ValueError('axes must be different')
    if not (-nd <= axes[0] < nd and -nd <= axes[1] < nd):
        raise ValueError('axes must be >= %d and < %d' % (-nd, nd))
    from cupy_amd._manipulation import flip
    k %= 4
    if k == 0:
        return a[:]
    if k == 2:
        return flip(a, axes)
    order = list(range(nd))
    order[axes[0]], order[axes[1]] = order[axes[1]], order[axes[0]]
    if k == 1:
        return flip(a, axes[1]).transpose(order)
    return flip(a.transpose(order), axes[1])
