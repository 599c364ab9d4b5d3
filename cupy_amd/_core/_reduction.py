"""ReductionKernel, simple reductions (sum, argmax, ...) and their launch
planning.

The call surface and semantics follow the reference's
cupy/_core/_reduction.pyx (axis handling :147-176, ``_call`` :309-427,
``create_reduction_func`` / ``_SimpleReductionKernel`` :557-708,
``ReductionKernel`` :716-917).  The geometry is not the reference's
``_get_block_specs`` (:239-253): the problem is brought into a canonical
``(n_out, n_red)`` form and one of the kernels of ``_codegen_reduction`` is
launched, split over the grid with a second combining pass when there are too
few outputs to fill 256 CUs.
"""
import re
import struct
import threading
import warnings

import numpy

from cupy_amd import _dryrun
from cupy_amd._core import _carray
from cupy_amd._core import _codegen_reduction as _cg
from cupy_amd._core import _kernel
from cupy_amd._core import _launch_plan
from cupy_amd._core import _reduce_sync
from cupy_amd._core import _tuning
from cupy_amd._core import internal
from cupy_amd._core._codegen_elementwise import uses_identifier
from cupy_amd._core._dtype import get_dtype
from cupy_amd._core._kernel import (
    _get_param_info, _decide_params_type, _preprocess_args, _broadcast,
    _get_out_args_from_optionals, _get_out_args_with_params,
    _check_peer_access, _scalar_struct_code, _make_packer, _max_blocks, _max_vector_width, _aligned)
from cupy_amd._core._scalar import CScalar, get_typename as _get_typename
from cupy_amd._core.core import ndarray, _ascontiguous, _convert_from_cupy_like
from cupy_amd.cuda import compiler
from cupy_amd.cuda import device as _device
from cupy_amd.cuda import memory as _memory
from cupy_amd.cuda import stream as _stream

_INT32_MAX = (1 << 31) - 1


def _get_axis(axis, ndim):
    """(reduce axes, remaining axes), each sorted ascending."""
    if axis is None:
        return tuple(range(ndim)), ()
    if isinstance(axis, (tuple, list)):
        axis = tuple(axis)
    else:
        axis = axis,
    reduce_axis = tuple(sorted(
        internal._normalize_axis_index(dim, ndim) for dim in axis))
    out_axis = tuple(dim for dim in range(ndim) if dim not in reduce_axis)
    if len(reduce_axis) + len(out_axis) != ndim:
        raise ValueError("duplicate value in 'axis'")
    return reduce_axis, out_axis


def _get_out_shape(shape, reduce_axis, out_axis, keepdims):
    if keepdims:
        out_shape = list(shape)
        for i in reduce_axis:
            out_shape[i] = 1
        return tuple(out_shape)
    return tuple(shape[i] for i in out_axis)


def _sort_axis(axis, strides):
    """Axes in decreasing order of |stride| (stable)."""
    return tuple(sorted(axis, key=lambda i: -abs(strides[i])))


def _merge_dims(shape, strides_list):
    """Like ``_kernel._canonical_dims`` for explicit stride lists."""
    cshape = []
    cstrides = [[] for _ in strides_list]
    for d, ext in enumerate(shape):
        if ext == 1:
            continue
        if cshape:
            for cs, st in zip(cstrides, strides_list):
                if cs[-1] != st[d] * ext:
                    break
            else:
                cshape[-1] *= ext
                for cs, st in zip(cstrides, strides_list):
                    cs[-1] = st[d]
                continue
        cshape.append(ext)
        for cs, st in zip(cstrides, strides_list):
            cs.append(st[d])
    return cshape, cstrides


_known_type_sizes = {
    'bool': 1, 'signed char': 1, 'unsigned char': 1, 'short': 2,
    'unsigned short': 2, 'int': 4, 'unsigned int': 4, 'long long': 8,
    'unsigned long long': 8, 'float16': 2, 'float': 4, 'double': 8,
}


_TYPEDEF = re.compile(r'typedef\s+(.+?)\s+(\w+)\s*;')
_WRAPPED = re.compile(r'(mm_val|arg_state|var_st)\s*<\s*([^,>]+(?:<[^>]*>)?)\s*(?:,[^>]*)?>(?:::type)?')


def _reduce_type_bytes(reduce_type, typedefs):
    """Upper bound of ``sizeof`` of a reduction type, from its name alone
    (the same with and without a device): exact for the arithmetic types, the
    complex types and the structures of the min/max, argmin/argmax and
    variance reductions, 64 for anything else."""
    names = dict((name, what) for what, name in _TYPEDEF.findall(typedefs))

    def plain(t):
        t = names.get(t.strip(), t.strip())
        size = _known_type_sizes.get(t)
        if size is None:
            size = {'complex<float>': 8, 'complex<double>': 16}.get(t.replace(' ', ''))
        return size

    size = plain(reduce_type)
    if size is not None:
        return size
    m = _WRAPPED.fullmatch(reduce_type.strip())
    inner = plain(m.group(2)) if m else None
    if inner is None:
        return 64
    if m.group(1) == 'mm_val':
        return inner
    if m.group(1) == 'var_st':
        return 4 * inner
    # argmin / argmax: values of 4 bytes at most with 32-bit indices travel as
    # one 64-bit key, the others as (value, index of 8 bytes)
    if inner <= 4 and names.get('IndexT', '').strip() == 'int' and 'complex' not in (
            names.get(m.group(2).strip(), m.group(2))):
        return 8
    return 8 + (inner + 7) // 8 * 8


_SIZE_CALL = re.compile(r'\b_(?:in|out)_ind\s*\.\s*size\s*\(\s*\)')


class _AbstractReductionKernel:

    def __init__(self, name, identity, in_params, out_params):
        assert name is not None
        assert identity is not None
        self.name = name
        self.__name__ = name
        self.identity = identity
        self.in_params = _get_param_info(in_params, True)
        self.out_params = _get_param_info(out_params, False)
        self._cached_codes = {}
        self._memo = {}
        self._lock = threading.Lock()
        self._fast_calls = {}

    # Hooks of the concrete classes -----------------------------------------------------
    def _get_expressions_and_types(self, in_args, out_args, dtype):
        raise NotImplementedError

    def _get_out_args(self, out_args, out_types, out_shape):
        raise NotImplementedError

    def _get_preamble_options(self):
        raise NotImplementedError

    def _in_var_type(self, index, param):
        raise NotImplementedError

    # -----------------------------------------------------------------------------------
    def _call(self, in_args, out_args, a_shape, axis, dtype, keepdims, reduce_dims,
              device_id, stream, sort_reduce_axis=True, rec=None):
        if dtype is not None:
            dtype = get_dtype(dtype).type
        (map_expr, reduce_expr, post_map_expr, in_types, out_types, reduce_type,
         type_pairs) = self._get_expressions_and_types(in_args, out_args, dtype)

        ndim = len(a_shape)
        reduce_axis, out_axis = _get_axis(axis, ndim)
        if (len(in_args) == 1 and sort_reduce_axis
                and isinstance(in_args[0], ndarray)
                and not in_args[0]._c_contiguous):
            # sums do not care about the order: walking the reduced axes from
            # the largest stride to the smallest lets them merge
            reduce_axis = _sort_axis(reduce_axis, in_args[0]._strides)

        out_shape = _get_out_shape(a_shape, reduce_axis, out_axis, keepdims)
        out_args = self._get_out_args(out_args, out_types, out_shape)
        ret = out_args[0]
        if ret.size == 0:
            return ret
        if self.identity == '' and 0 in a_shape:
            raise ValueError(('zero-size array to reduction operation'
                              ' %s which has no identity') % self.name)

        in_size = internal.prod(a_shape)
        out_size = internal.prod(out_shape)
        index_t = 'long long' if in_size // max(out_size, 1) > _INT32_MAX else 'int'
        for x, t in zip(in_args, in_types):
            if type(x) is CScalar:
                x.apply_dtype(t)

        typedefs = ''.join('typedef %s %s;\n' % (_get_typename(t), n)
                           for n, t in type_pairs)
        typedefs += 'typedef %s IndexT;\n' % index_t

        self._launch(in_args, out_args, a_shape, reduce_axis, out_axis, keepdims,
                     map_expr, reduce_expr, post_map_expr, reduce_type, typedefs,
                     device_id, stream, rec)
        return ret

    def _fast_lookup(self, fast_args, extra, dev_id):
        """Replays an earlier call with the same argument signature.  Returns
        (done, result, key, recorder)."""
        key = _launch_plan.call_signature(fast_args, dev_id)
        if key is None:
            return False, None, None, None
        try:
            key = key + extra
            fast = self._fast_calls.get(key)
        except TypeError:       # unhashable axis / dtype argument
            return False, None, None, None
        if fast is not None and fast.stream is not None:
            # A record that finishes the reduction inside its one launch names
            # memory of the stream it was made on: other streams keep records
            # of their own under the key extended by the stream.  Once a
            # kernel of that kind gave up a wait on the device none of them is
            # replayed; the full path reports it and records over them.
            cur = _stream.get_current_stream_ptr()
            if fast.stale():
                fast = None
            elif fast.stream != cur:
                key = key + (cur,)
                fast = self._fast_calls.get(key)
                if fast is not None and fast.stale():
                    fast = None
        if fast is not None:
            ret = fast.run(fast_args)
            if ret is not NotImplemented:
                return True, ret, None, None
            return False, None, None, None
        nargs = len(self.in_params) + len(self.out_params)
        return False, None, key, _launch_plan.Recorder(nargs)

    def _fast_remember(self, key, rec, fast_args, ret):
        if rec is None or not rec.launches or ret is None:
            return
        nin = len(self.in_params)
        n_given = len(fast_args) - nin
        out_specs = ()
        if n_given == 0:
            if len(self.out_params) != 1:
                return
            out_specs = ((ret._shape, ret.dtype),)
        _launch_plan.remember(
            self._fast_calls, key,
            _launch_plan.FastCall(len(fast_args), out_specs, rec, nin))

    # -- planning ---------------------------------------------------------------------------
    def _launch(self, in_args, out_args, a_shape, reduce_axis, out_axis, keepdims,
                map_expr, reduce_expr, post_map_expr, reduce_type, typedefs,
                device_id, stream, rec=None):
        stream_ptr = _stream.get_current_stream_ptr() if stream is None else stream.ptr
        in_params = self.in_params
        out_params = self.out_params
        n_r = len(reduce_axis)
        perm = reduce_axis + out_axis
        need_perm = any(i != p for i, p in enumerate(perm))
        has_raw = any(p.raw for p in in_params + out_params)
        if need_perm and has_raw:
            raise NotImplementedError('Illegal conditions')

        red_shape = tuple(a_shape[i] for i in reduce_axis)
        kept_shape = tuple(a_shape[i] for i in out_axis)
        in_arr_idx = [i for i, (a, p) in enumerate(zip(in_args, in_params))
                      if isinstance(a, ndarray) and not p.raw]
        out_arr_idx = [i for i, (a, p) in enumerate(zip(out_args, out_params))
                       if not p.raw]
        # strides of every iterated array along the reduced / kept axes
        in_red_strides = []
        in_kept_strides = []
        for i in in_arr_idx:
            st = in_args[i]._strides
            in_red_strides.append(tuple(st[d] for d in reduce_axis))
            in_kept_strides.append(tuple(st[d] for d in out_axis))
        out_kept_strides = []
        for i in out_arr_idx:
            o = out_args[i]
            st = o._strides
            if keepdims:
                st = tuple(st[d] for d in out_axis)
            out_kept_strides.append(tuple(st))

        rshape, rstrides = _merge_dims(red_shape, in_red_strides)
        oshape, ostrides = _merge_dims(kept_shape, in_kept_strides + out_kept_strides)
        o_in = ostrides[:len(in_arr_idx)]
        o_out = ostrides[len(in_arr_idx):]

        exprs = (map_expr, reduce_expr, post_map_expr)
        # `_in_ind.size()` / `_out_ind.size()` are available everywhere; any
        # other use of the indexers needs the kernel that has them
        needs_indexers = any(
            uses_identifier(_SIZE_CALL.sub('', e), n)
            for e in exprs + (self._get_preamble_options()[0],)
            for n in ('_in_ind', '_out_ind', '_i', '_j'))
        canonical = (len(rshape) <= 1 and len(oshape) <= 1 and not has_raw
                     and not needs_indexers and in_arr_idx)
        if canonical:
            n_red = rshape[0] if rshape else 1
            n_out = oshape[0] if oshape else 1
            ins = [in_args[i] for i in in_arr_idx]
            outs = [out_args[i] for i in out_arr_idx]
            sr = [(rs[0] if rs else 0) for rs in rstrides]
            so_in = [(os_[0] if os_ else 0) for os_ in o_in]
            so_out = [(os_[0] if os_ else 0) for os_ in o_out]
            rows_ok = n_red > 1 and all(
                s == a.dtype.itemsize or s == 0 for s, a in zip(sr, ins)) and all(
                s % a.dtype.itemsize == 0 for s, a in zip(so_in, ins)) and all(
                s % a.dtype.itemsize == 0 for s, a in zip(so_out, outs))
            cols_ok = all(
                s == a.dtype.itemsize or s == 0 or n_out == 1
                for s, a in zip(so_in, ins)) and all(
                s == a.dtype.itemsize or n_out == 1
                for s, a in zip(so_out, outs)) and all(
                s % a.dtype.itemsize == 0 for s, a in zip(sr, ins))
            plan_args = (in_args, out_args, in_arr_idx, out_arr_idx, n_out, n_red,
                         so_in, sr, so_out, map_expr, reduce_expr, post_map_expr,
                         reduce_type, typedefs, device_id, stream_ptr, rec)
            if rows_ok:
                return self._launch_rows(*plan_args)
            if cols_ok:
                return self._launch_cols(*plan_args)
        # reduction over a middle axis: in[b, j, c] -> out[b, c] with c adjacent
        # in memory everywhere and the outputs stored row after row
        if (len(rshape) <= 1 and len(oshape) == 2 and not has_raw and not needs_indexers
                and in_arr_idx):
            ins = [in_args[i] for i in in_arr_idx]
            outs = [out_args[i] for i in out_arr_idx]
            n_batch, n_inner = oshape
            sr = [(rs[0] if rs else 0) for rs in rstrides]
            if (all(os_[1] == a.dtype.itemsize and os_[0] % a.dtype.itemsize == 0
                    for os_, a in zip(o_in, ins))
                    and all(tuple(os_) == (n_inner * a.dtype.itemsize, a.dtype.itemsize)
                            for os_, a in zip(o_out, outs))
                    and all(s % a.dtype.itemsize == 0 for s, a in zip(sr, ins))):
                n_red = rshape[0] if rshape else 1
                if (all(tuple(os_) == (n_red * n_inner * a.dtype.itemsize, a.dtype.itemsize)
                        and s == n_inner * a.dtype.itemsize
                        for os_, s, a in zip(o_in, sr, ins))
                        and self._launch_mid_flat(
                            in_args, out_args, in_arr_idx, out_arr_idx, n_batch, n_red, n_inner,
                            map_expr, reduce_expr, post_map_expr, reduce_type, typedefs,
                            device_id, stream_ptr, rec)):
                    return
                return self._launch_cols(
                    in_args, out_args, in_arr_idx, out_arr_idx, n_batch * n_inner,
                    rshape[0] if rshape else 1, [a.dtype.itemsize for a in ins], sr,
                    [a.dtype.itemsize for a in outs], map_expr, reduce_expr,
                    post_map_expr, reduce_type, typedefs, device_id, stream_ptr, rec,
                    batch=(n_batch, n_inner, [os_[0] for os_ in o_in]))
        # Kept and reduced axes interleaved with an innermost axis of a few
        # elements: the indexer kernel would walk the input in pieces of a few
        # bytes, and the staged form below would fold very many partial results
        # per output.  The input is copied once with the reduced axes last --
        # the permuted copy runs near the streaming rate -- and reduced row by
        # row: three passes over the data, and still ahead (us, before / so:
        # any over axes (1, 3) of 833 x 126 x 80 x 4 int32 149 / 61; sum over
        # (0, 3) of 1000 x 64 x 256 x 3 float16 133 / 52).  Longer innermost
        # axes are better off as they are (sum over (1, 3) of 64 x 100 x 64 x 100
        # float32 63 / 85), and so are one-byte elements (their copies are slow).
        if (in_arr_idx and len(in_arr_idx) == 1 and not has_raw and not needs_indexers
                and n_r and out_axis and _tuning.get('reduce_via_copy')
                and not any(uses_identifier(e, '_J') for e in exprs)):
            src = in_args[in_arr_idx[0]]
            size = internal.prod(a_shape)
            item = src.dtype.itemsize
            special = len(rshape) <= 1 and len(oshape) <= 2
            if (not special and item >= 2 and a_shape[-1] * item < 64
                    and tuple(src._shape) == tuple(a_shape)
                    and _tuning.get('reduce_via_copy_min') <= size
                    and src.nbytes <= (8 << 30)):
                perm = tuple(out_axis) + tuple(reduce_axis)
                try:
                    if stream is None:
                        tmp = _ascontiguous(src.transpose(perm))
                    else:
                        with stream:
                            tmp = _ascontiguous(src.transpose(perm))
                except MemoryError:
                    tmp = None        # no room for the copy: the input as it is
            else:
                tmp = None
            if tmp is not None:
                new_in = list(in_args)
                new_in[in_arr_idx[0]] = tmp
                new_out = list(out_args)
                if keepdims:
                    for i in out_arr_idx:
                        o = out_args[i]
                        new_out[i] = o._view(kept_shape, tuple(o._strides[d] for d in out_axis))
                n_k = len(out_axis)
                return self._launch(
                    new_in, new_out, tuple(a_shape[p] for p in perm),
                    tuple(range(n_k, len(perm))), tuple(range(n_k)), False,
                    map_expr, reduce_expr, post_map_expr, reduce_type, typedefs,
                    device_id, stream, None)
        # reduction over an outer and the innermost axis, in[r0, c, r1] -> out[c]
        # (e.g. per-channel statistics of a batch of images): the rows kernel
        # reduces r1 for every (r0, c) into partial results, which the combine
        # kernel reduces over r0
        if (len(rshape) == 2 and len(oshape) == 1 and not has_raw and not needs_indexers
                and in_arr_idx and not any(uses_identifier(e, '_J') for e in exprs)):
            ins = [in_args[i] for i in in_arr_idx]
            n_outer, n_inner = rshape
            n_keep = oshape[0]
            if all(rs[1] == a.dtype.itemsize and os_[0] % a.dtype.itemsize == 0
                   and rs[0] == n_keep * os_[0] and os_[0] >= n_inner * a.dtype.itemsize
                   for rs, os_, a in zip(rstrides, o_in, ins)) and n_inner > 1 and (
                       n_outer * n_keep * n_inner >= 1 << 16):     # else one launch is quicker
                return self._launch_rows(
                    in_args, out_args, in_arr_idx, out_arr_idx, n_outer * n_keep, n_inner,
                    [os_[0] for os_ in o_in], [rs[1] for rs in rstrides],
                    [os_[0] for os_ in o_out], map_expr, reduce_expr, post_map_expr,
                    reduce_type, typedefs, device_id, stream_ptr, rec,
                    stage=(n_outer, n_keep))
        # generic: views with the reduced axes in front, merged where possible
        g_in = list(in_args)
        for k, i in enumerate(in_arr_idx):
            shape = tuple(rshape) + tuple(oshape)
            strides = tuple(rstrides[k]) + tuple(o_in[k])
            g_in[i] = in_args[i]._view(shape, strides)
        g_out = list(out_args)
        for k, i in enumerate(out_arr_idx):
            g_out[i] = out_args[i]._view(tuple(oshape), tuple(o_out[k]))
        in_shape = tuple(rshape) + tuple(oshape)
        if not in_arr_idx:
            in_shape = red_shape + kept_shape
            oshape = kept_shape
        return self._launch_generic(
            g_in, g_out, in_shape, tuple(oshape), internal.prod(rshape) if in_arr_idx
            else internal.prod(red_shape), map_expr, reduce_expr, post_map_expr,
            reduce_type, typedefs, device_id, stream_ptr, rec)

    # -- helpers ----------------------------------------------------------------------------
    def _rargs(self, in_args, out_args, bcast_r=None, bcast_o=None):
        rargs = []
        k = 0
        for idx, (a, p) in enumerate(zip(in_args, self.in_params)):
            if isinstance(a, ndarray):
                st = _get_typename(a.dtype)
                if p.raw:
                    rargs.append(_cg.RArg(
                        'raw', p.name, st, is_const=p.is_const, ndim=a.ndim,
                        c_contiguous=a._c_contiguous, index_32=a._index_32_bits))
                else:
                    rargs.append(_cg.RArg(
                        'in', p.name, st, self._in_var_type(idx, p),
                        is_const=p.is_const, ndim=a.ndim,
                        c_contiguous=a._c_contiguous, index_32=a._index_32_bits,
                        bcast_r=bool(bcast_r and bcast_r[k]),
                        bcast_o=bool(bcast_o and bcast_o[k])))
                    k += 1
            else:
                rargs.append(_cg.RArg('scalar', p.name, _get_typename(a.descr)))
        for idx, (a, p) in enumerate(zip(out_args, self.out_params)):
            st = _get_typename(a.dtype)
            if p.raw:
                rargs.append(_cg.RArg(
                    'raw', p.name, st, is_const=False, ndim=a.ndim,
                    c_contiguous=a._c_contiguous, index_32=a._index_32_bits))
            else:
                rargs.append(_cg.RArg(
                    'out', p.name, st, self._out_var_type(idx, p), is_const=False,
                    ndim=a.ndim, c_contiguous=a._c_contiguous,
                    index_32=a._index_32_bits))
        return rargs

    def _out_var_type(self, index, param):
        return param.ctype

    def _compile(self, key, emit, in_args):
        """Memoised (function, module, code) for a kernel variant."""
        entry = self._memo.get(key)
        if entry is None:
            name, code = emit()
            preamble, options = self._get_preamble_options()
            mod = compiler.compile_with_cache(code, options)
            fn = mod.get_function(name)
            entry = (fn, mod, code)
            with self._lock:
                entry = self._memo.setdefault(key, entry)
            in_types = tuple(a.dtype.char for a in in_args if isinstance(a, ndarray))
            if in_types not in self._cached_codes:
                self._cached_codes[in_types] = code
        return entry

    def _reduce_type_size(self, reduce_type, mod):
        size = _known_type_sizes.get(reduce_type)
        if size is not None:
            return size
        if _dryrun.enabled():
            return 64
        _, nbytes = mod.get_global_var('_cupy_type_reduce_probe')
        return nbytes

    @staticmethod
    def _fast_format(rargs, ic, extra=''):
        fmt = ['@']
        for a in rargs:
            if a.kind in ('in', 'out'):
                fmt.append('P')
            elif a.kind == 'raw':
                fmt.append('P' + 'q' * (1 + 2 * a.ndim))
            else:
                fmt.append(_scalar_struct_code(a.store_t))
        fmt.append(ic * 2 + 'q')
        for a in rargs:
            if a.kind == 'in':
                fmt.append(ic * 2)
            elif a.kind == 'out':
                fmt.append(ic)
        fmt.append(extra)
        return ''.join(fmt)

    def _fast_values(self, in_args, out_args, n_out, n_red, so_in, sr, so_out):
        vals = _launch_plan.ArgBlock()
        nin = len(self.in_params)
        for ref, a in enumerate(in_args):
            if isinstance(a, ndarray):
                vals.ptr(ref, a.data.ptr)
            else:
                vals.scalar(ref, a)
        for j, a in enumerate(out_args):
            vals.ptr(nin + j, a.data.ptr)
        vals.const(n_out, n_red, n_out * n_red)
        k = 0
        for a, p in zip(in_args, self.in_params):
            if isinstance(a, ndarray) and not p.raw:
                item = a.dtype.itemsize
                vals.const(so_in[k] // item, sr[k] // item)
                k += 1
        for k, a in enumerate(out_args):
            vals.const(so_out[k] // a.dtype.itemsize)
        return vals

    def _finalize_partials(self, partials, n_split, out_args, out_arr_idx, n_out,
                           so_out, in_args, reduce_expr, post_map_expr, reduce_type,
                           typedefs, device_id, stream_ptr, rec, partials_ref, in_total):
        """Second pass: combine ``partials[s][i]`` over s, then POST_MAP."""
        preamble, _ = self._get_preamble_options()
        # lanes across the outputs, the rest of the workgroup down the partials:
        # with many partials per output few lanes go across, so that no lane
        # walks a long dependent chain of (cache-resident) loads
        tx = max(1, min(64, internal.clp2(n_out), internal.flp2(max(1, 4096 // n_split))))
        rargs = [_cg.RArg('in', '_partial_in', '_type_reduce')]
        rargs += [r for r in self._rargs(in_args, out_args) if r.kind in ('scalar', 'out')]
        idx64 = n_split * n_out > _INT32_MAX
        key = ('final', tuple(r.key() for r in rargs), typedefs, reduce_expr,
               post_map_expr, reduce_type, tx, idx64, device_id)

        def emit():
            name = self.name + '_combine'
            return name, _cg.emit_cols(
                name, rargs, self.identity, '_partial_in', reduce_expr,
                post_map_expr, reduce_type, typedefs, preamble, tx=tx, vec=1,
                idx64=idx64, partial_in=True)
        fn, _, _ = self._compile(key, emit, in_args)
        ic = 'q' if idx64 else 'i'
        fmt = ['@P']
        vals = _launch_plan.ArgBlock()
        vals.ptr(partials_ref, partials.ptr)
        nin = len(self.in_params)
        for ref, a in enumerate(in_args):
            if not isinstance(a, ndarray):
                fmt.append(_scalar_struct_code(_get_typename(a.descr)))
                vals.scalar(ref, a)
        for j, a in enumerate(out_args):
            fmt.append('P')
            vals.ptr(nin + j, a.data.ptr)
        fmt.append(ic * 2 + 'q' + ic * 2)
        vals.const(n_out, n_split, in_total, 1, n_out)
        for k, a in enumerate(out_args):
            fmt.append(ic)
            vals.const(so_out[k] // a.dtype.itemsize)
        grid = (n_out + tx - 1) // tx
        gz = (grid + _max_blocks(_cg.BLOCK) - 1) // _max_blocks(_cg.BLOCK)
        grid = (grid + gz - 1) // gz
        _launch_plan.launch(rec, fn, (grid, 1, gz), (_cg.BLOCK, 1, 1),
                            _make_packer(fmt), vals, stream_ptr)

    # -- short rows through the LDS -----------------------------------------------------------
    def _rows_flat_geometry(self, ins, n_out, n_red, so_in, sr):
        """(lanes per row, rows per workgroup) for the kernel that stages whole
        rows in the LDS, or None when the rows are not short, not stored back
        to back, or served as well by a lane group per row."""
        mode = _tuning.get('rows_flat')
        if not mode or n_red < 3 or n_out < 4096:
            return None
        items = [a.dtype.itemsize for a in ins]
        if n_red * max(items) > _tuning.get('rows_flat_max_bytes'):
            return None
        dense = 0
        for a, s_o, s_r in zip(ins, so_in, sr):
            if s_r == 0 and s_o % a.dtype.itemsize == 0:
                continue              # a value per row, read in place
            if s_r != a.dtype.itemsize:
                return None
            if s_o == n_red * a.dtype.itemsize:
                dense += 1
            elif s_o != 0:            # one row shared by all outputs is read in place
                return None
        if not dense:
            return None
        items = [a.dtype.itemsize for a, s_o, s_r in zip(ins, so_in, sr) if s_o and s_r]
        if mode == 'auto':
            # a lane group per row does as well when a row is a whole number
            # of vectors that fills a power-of-two group of lanes, or three
            # quarters of one from 384 bytes per row
            vec = _max_vector_width(items)
            lanes = (n_red + vec - 1) // vec
            full = internal.clp2(lanes)
            if n_red % vec == 0 and (lanes == full or (
                    lanes * 4 >= full * 3 and n_red * min(items) >= 384)):
                return None
        group = min(64, internal.clp2((n_red + 23) // 24))
        per_pass = _cg.BLOCK // group
        pass_bytes = per_pass * n_red * sum(items)
        if pass_bytes > 48 * 1024:
            return None
        k = max(1, min(8, (24 * 1024) // pass_bytes))
        rows = per_pass * k
        if (n_out + rows - 1) // rows > _max_blocks(_cg.BLOCK):
            return None
        return group, rows

    def _launch_rows_flat(self, geometry, in_args, out_args, in_arr_idx, out_arr_idx,
                          n_out, n_red, so_in, sr, so_out, map_expr, reduce_expr,
                          post_map_expr, reduce_type, typedefs, device_id, stream_ptr,
                          rec=None):
        preamble, _ = self._get_preamble_options()
        ins = [in_args[i] for i in in_arr_idx]
        group, rows = geometry
        rargs = self._rargs(in_args, out_args, bcast_r=[s == 0 for s in sr],
                            bcast_o=[s_o == 0 and s_r != 0 for s_o, s_r in zip(so_in, sr)])
        stream_hint = _tuning.stream_policy(
            _tuning.get('rows_stream'), self._read_bytes(ins, n_out, n_red, so_in, sr), 0)[0]
        key = ('rows_flat', tuple(r.key() for r in rargs), typedefs, map_expr, reduce_expr,
               post_map_expr, reduce_type, n_red, group, rows, device_id, stream_hint)

        def emit():
            return self.name, _cg.emit_rows_flat(
                self.name, rargs, self.identity, map_expr, reduce_expr, post_map_expr,
                reduce_type, typedefs, preamble, width=n_red, group=group, rows=rows,
                stream_hint=stream_hint)
        fn, _, _ = self._compile(key, emit, in_args)
        vals = self._fast_values(in_args, out_args, n_out, n_red, so_in, sr, so_out)
        _launch_plan.launch(
            rec, fn, ((n_out + rows - 1) // rows, 1, 1), (_cg.BLOCK, 1, 1),
            _make_packer(self._fast_format(rargs, 'q')), vals, stream_ptr)

    def _launch_mid_flat(self, in_args, out_args, in_arr_idx, out_arr_idx, n_batch, n_red,
                         n_inner, map_expr, reduce_expr, post_map_expr, reduce_type, typedefs,
                         device_id, stream_ptr, rec=None):
        """Reduction over the middle axis of dense (n_batch, n_red, n_inner)
        inputs whose slices are short and have few columns: workgroups stage
        runs of whole slices in the LDS (``emit_rows_flat`` with ``inner``).
        Returns False where that does not apply."""
        ins = [in_args[i] for i in in_arr_idx]
        items = [a.dtype.itemsize for a in ins]
        width = n_red * n_inner
        if (not _tuning.get('mid_flat') or n_inner > 1024 or n_red < 2 or n_batch < 1024
                or width * sum(items) > 32 * 1024):
            return False
        # a lane per slice and column for up to 32 lines, more lanes beyond
        # (states that are expensive to merge, like those of the variance,
        # want long walks and few lanes: 130561 slices of 257 x 2 floats, var:
        # 31 % of peak with 8 lines per lane, 58 % with 32; sums do not care)
        per_lane = _tuning.get('mid_flat_lines_per_lane')
        group = min(64, internal.clp2((n_red + per_lane - 1) // per_lane))
        rows = max(1, min((24 * 1024) // (width * sum(items)), 65536))
        if (n_batch + rows - 1) // rows > _max_blocks(_cg.BLOCK):
            return False
        preamble, _ = self._get_preamble_options()
        rargs = self._rargs(in_args, out_args)
        stream_hint = _tuning.stream_policy(
            _tuning.get('rows_stream'), sum(a.nbytes for a in ins), 0)[0]
        key = ('mid_flat', tuple(r.key() for r in rargs), typedefs, map_expr, reduce_expr,
               post_map_expr, reduce_type, width, n_inner, group, rows, device_id, stream_hint)

        def emit():
            return self.name, _cg.emit_rows_flat(
                self.name, rargs, self.identity, map_expr, reduce_expr, post_map_expr,
                reduce_type, typedefs, preamble, width=width, group=group, rows=rows,
                stream_hint=stream_hint, inner=n_inner)
        fn, _, _ = self._compile(key, emit, in_args)
        n_out = n_batch * n_inner
        vals = self._fast_values(
            in_args, out_args, n_out, n_red, [width * i for i in items],
            [n_inner * i for i in items],
            [out_args[i].dtype.itemsize for i in out_arr_idx])
        _launch_plan.launch(
            rec, fn, ((n_batch + rows - 1) // rows, 1, 1), (_cg.BLOCK, 1, 1),
            _make_packer(self._fast_format(rargs, 'q')), vals, stream_ptr)
        return True

    # -- rows ---------------------------------------------------------------------------------
    def _launch_rows(self, in_args, out_args, in_arr_idx, out_arr_idx, n_out, n_red,
                     so_in, sr, so_out, map_expr, reduce_expr, post_map_expr,
                     reduce_type, typedefs, device_id, stream_ptr, rec=None, stage=None):
        """``stage`` = (n_outer, n_keep): the ``n_out = n_outer * n_keep`` rows
        are not the final outputs; their results are partial results that a
        second launch combines over ``n_outer`` into ``n_keep`` outputs."""
        preamble, _ = self._get_preamble_options()
        ins = [in_args[i] for i in in_arr_idx]
        flat = None if stage else self._rows_flat_geometry(ins, n_out, n_red, so_in, sr)
        if flat is not None:
            return self._launch_rows_flat(
                flat, in_args, out_args, in_arr_idx, out_arr_idx, n_out, n_red, so_in,
                sr, so_out, map_expr, reduce_expr, post_map_expr, reduce_type, typedefs,
                device_id, stream_ptr, rec)
        cus = _device.get_compute_units(device_id)
        vec = _max_vector_width([a.dtype.itemsize for a in ins])
        while vec > 1:
            ok = True
            for a, s_o, s_r in zip(ins, so_in, sr):
                if s_r == 0:
                    continue
                nb = min(16, vec * a.dtype.itemsize)
                if not _aligned(a.data.ptr, nb) or (n_out > 1 and not _aligned(s_o, nb)):
                    ok = False
            if ok and n_red >= vec:
                break
            vec //= 2
        bcast_r = [s == 0 for s in sr]
        max_item = max(a.dtype.itemsize for a in ins)
        lanes_needed = (n_red + vec - 1) // vec
        # geometry
        if n_red * max_item >= _tuning.get('rows_block_mode_bytes'):
            group = _cg.BLOCK
        else:
            group = max(1, min(64, internal.clp2(lanes_needed)))
        n_split = 1
        chunk = n_red
        wg = _tuning.get('rows_block') if group == _cg.BLOCK else _cg.BLOCK
        # (a second launch costs about 8 us: below 128 KiB per row a workgroup
        # on its own is quicker)
        if (group == _cg.BLOCK and n_out < cus * _tuning.get('min_blocks_per_cu')
                and (n_red * max_item >= 128 * 1024 or stage)):
            trip = wg * vec
            want = (cus * (_tuning.get('rows_target_blocks_per_cu')
                           or _tuning.get('target_blocks_per_cu')) + n_out - 1) // n_out
            most = max(1, n_red // (trip * _tuning.get('rows_split_min_trips')))
            n_split = max(1, min(want, most, 65535))
            if n_split > 1:
                chunk = (n_red + n_split - 1) // n_split
                chunk = (chunk + trip - 1) // trip * trip
                n_split = (n_red + chunk - 1) // chunk
        partial = n_split > 1 or bool(stage)
        span = max([abs(s_o) * n_out + abs(s_r) * n_red for s_o, s_r in zip(so_in, sr)]
                   + [abs(s) * n_out for s in so_out] + [n_red + chunk])
        idx64 = span > _INT32_MAX - (1 << 24)
        finish, words_hint = None, 2
        if n_split > 1 and not stage and n_out <= _max_blocks(wg):
            words_hint, finish = self._finish_memory(
                ins, n_out, n_red, so_in, sr, reduce_type, typedefs,
                lambda words: n_split * n_out * words + n_out, (n_split + 63) // 64,
                False, device_id, stream_ptr)
        batch = _tuning.get('rows_batch')
        trips = 1
        batched = (group < _cg.BLOCK and batch >= 1 and n_red <= group * vec and not stage
                   and n_out >= 4 * batch and _tuning.get('rows_trips') >= 1)
        if batched:
            # Fewer lanes per row with several loads per lane shorten the
            # cross-lane butterfly; several rows per group keep loads in
            # flight.  Both are bounded by a budget of bytes (registers) per
            # lane.
            per_trip = sum(vec * a.dtype.itemsize for a, s_o in zip(ins, so_in)
                           if not (s_o == 0 and n_out > 1))
            budget = _tuning.get('rows_lane_bytes')
            min_group = max(1, _tuning.get('rows_min_group_bytes') // (vec * max_item))
            while (trips * 2 <= _tuning.get('rows_trips') and group >= 2 * min_group
                   and per_trip * trips * 2 <= budget):
                trips *= 2
                group //= 2
            batch = max(1, min(batch, budget // max(1, per_trip * trips)))
        bcast_o = [(s == 0 and n_out > 1) for s in so_in] if batched else None
        exact = batched and n_red == group * vec * trips
        if exact and n_red * max_item >= 256:
            # rows that fill their lanes' vectors exactly, of 256 bytes and more:
            # one row at a time per group does better (2^20 rows of 128 int32,
            # sum / argmax: 77 / 78 us against 81 / 82 with two; rows of 32 or 16
            # float32 and rows of 100 or 200 want two: 83 against 88, 66 against 67)
            batch = 1
        stream_hint = _tuning.stream_policy(
            _tuning.get('rows_stream'), self._read_bytes(ins, n_out, n_red, so_in, sr), 0)[0]
        rargs = self._rargs(in_args, out_args, bcast_r=bcast_r, bcast_o=bcast_o)
        key = ('rows', tuple(r.key() for r in rargs), typedefs, map_expr, reduce_expr,
               post_map_expr, reduce_type, group, vec, idx64, partial, device_id,
               batched, trips, exact, stream_hint, wg, bool(finish), _tuning.signature())

        def emit():
            if batched:
                return self.name, _cg.emit_rows_batched(
                    self.name, rargs, self.identity, map_expr, reduce_expr,
                    post_map_expr, reduce_type, typedefs, preamble, group=group,
                    vec=vec, trips=trips, batch=batch, idx64=idx64,
                    stream_hint=stream_hint, exact=exact)
            return self.name, _cg.emit_rows(
                self.name, rargs, self.identity, map_expr, reduce_expr,
                post_map_expr, reduce_type, typedefs, preamble, group=group,
                vec=vec, idx64=idx64, partial_out=partial,
                stream_hint=stream_hint,
                unroll=_tuning.get('rows_unroll'), block=wg,
                finish=bool(finish), reduce_words=words_hint)
        fn, mod, _ = self._compile(key, emit, in_args)
        ic = 'q' if idx64 else 'i'
        vals = self._fast_values(in_args, out_args, n_out, n_red, so_in, sr, so_out)
        if group == _cg.BLOCK:
            gx = min(n_out, _max_blocks(wg))
            cap = _tuning.get('rows_block_grid_per_cu')
            if cap and n_split == 1:
                gx = min(gx, cus * cap)
        else:
            rows_per_block = _cg.BLOCK // group * (batch if batched else 1)
            gx = min((n_out + rows_per_block - 1) // rows_per_block,
                     cus * _tuning.get('rows_group_rows_per_lane'))
        if finish:
            # one launch: the workgroup of the last chunk of every row combines
            # the partial results of the others
            if rec is not None:
                rec.bind_stream(stream_ptr, device_id)
            vals.const(finish[0], _tuning.get('reduce_finish_spin_limit'), finish[1], gx, chunk)
            _launch_plan.launch(
                rec, fn, (gx * n_split, 1, 1), (wg, 1, 1),
                _make_packer(self._fast_format(rargs, ic, 'PIP' + ic + ic)), vals, stream_ptr)
        elif partial:
            rsize = self._reduce_type_size(reduce_type, mod)
            partials, pref = self._alloc_partials(rec, rsize * n_split * n_out)
            vals.ptr(pref, partials.ptr)
            vals.const(chunk)
            _launch_plan.launch(
                rec, fn, (gx, n_split, 1), (wg, 1, 1),
                _make_packer(self._fast_format(rargs, ic, 'P' + ic)), vals, stream_ptr)
            if stage:
                n_split, n_final = n_split * stage[0], stage[1]
            else:
                n_final = n_out
            self._finalize_partials(
                partials, n_split, out_args, out_arr_idx, n_final, so_out, in_args,
                reduce_expr, post_map_expr, reduce_type, typedefs, device_id,
                stream_ptr, rec, pref, n_out * n_red)
        else:
            _launch_plan.launch(
                rec, fn, (gx, 1, 1), (wg, 1, 1),
                _make_packer(self._fast_format(rargs, ic)), vals, stream_ptr)

    @staticmethod
    def _read_bytes(ins, n_out, n_red, so_in, sr):
        """Bytes the iterated inputs of a canonical (n_out, n_red) problem
        occupy (broadcast axes not counted)."""
        total = 0
        for a, s_o, s_r in zip(ins, so_in, sr):
            total += a.dtype.itemsize * (n_out if s_o else 1) * (n_red if s_r else 1)
        return total

    def _finish_memory(self, ins, n_out, n_red, so_in, sr, reduce_type, typedefs, n_slots_of,
                       per_lane, by_thread, device_id, stream_ptr):
        """Decides whether a split reduction finishes inside its one launch.
        Returns ``(hint, None)`` or ``(hint, (block address, fault address))``:
        ``hint`` tells whether the reduction type fits two 32-bit words, as far
        as its name tells (2 or 4: it selects how many partial results a lane
        asks for at a time), the pair
        names the memory of the slots.  ``n_slots_of(words)`` gives the slots
        the launch needs for a type of that many words, ``per_lane`` is the
        number of partial results the busiest lane of a finishing workgroup
        combines; ``by_thread`` says that a thread does so for a column on its
        own (no other lanes share the work: the words it has to fetch are
        limited as well)."""
        words = (_reduce_type_bytes(reduce_type, typedefs) + 3) // 4
        hint = 2 if words <= 2 else 4
        if self._read_bytes(ins, n_out, n_red, so_in, sr) > _tuning.get('reduce_finish_max_bytes'):
            return hint, None
        # a lane asks for 8 partial results at a time (4 of the wider types)
        # and waits for them: beyond a few such round trips the second launch
        # is quicker
        if per_lane > _tuning.get('reduce_finish_round_trips') * (8 if hint == 2 else 4):
            return hint, None
        if by_thread and per_lane * words > 32:
            return hint, None
        got = _reduce_sync.acquire(device_id, stream_ptr, _stream.get_current_stream_ptr(),
                                   n_slots_of(words))
        return hint, got

    @staticmethod
    def _alloc_partials(rec, nbytes):
        """Temporary for partial results and its ref number for replays."""
        partials = _memory.alloc(nbytes)
        return partials, (rec.temp(nbytes) if rec is not None else -1)

    # -- narrow matrices, down the columns -----------------------------------------------------
    def _cols_flat_geometry(self, ins, n_out, n_red, so_in, sr, so_out, outs, vec, exprs,
                            state_bytes):
        """(vector width, active lanes) for the kernel that walks a narrow dense
        matrix as one piece of memory, or None where the column kernel serves:
        inputs that are not all the same dense matrix, rows that are whole
        vectors and fill a power-of-two group of lanes, wide or short matrices."""
        if not _tuning.get('cols_flat') or n_out < 2 or n_out > 256:
            return None
        items = set(a.dtype.itemsize for a in ins)
        if len(items) != 1:
            return None
        (item,) = items
        if any(s_o != item or s_r != n_out * item for s_o, s_r in zip(so_in, sr)):
            return None
        if n_out * n_red * item < _tuning.get('cols_flat_min_bytes'):
            return None
        vec = max(1, 16 // item)
        if any(not _aligned(a.data.ptr, min(16, vec * item)) for a in ins):
            return None
        import math
        period = n_out // math.gcd(n_out, vec)       # lanes after which the columns repeat
        if period > 1024:
            return None
        if _tuning.get('cols_flat') != 'always':
            # Measured over 2^26 float32 / 2^25 float64 / 2^27 float16 (us, this
            # kernel / the column kernel, combine launch included): 33 columns
            # 44 / 48, 67: 45 / 49, 100: 43 / 48, 129: 44 / 73, 200: 43 / 57; 3, 5,
            # 40, 80 columns: 43-45 either way; variances gain most (33: 48 / 59,
            # float16 x 67: 80 / 114).  Two exceptions.  Rows whose period divides
            # the workgroup (whole vectors that fill a power-of-two group of lanes:
            # 32, 64, 128, 256 float32 columns) are what the column kernel is made
            # for, and here every workgroup's piece would start on a multiple of
            # 4 KiB: 47 against 42.  Reductions that carry the position over
            # one-byte items pay more for it than they gain (int8 x 255 argmax:
            # 69 against 62).
            if _cg.BLOCK % period == 0:
                return None
            if item < 2 and any(uses_identifier(e, '_J') for e in exprs):
                return None
        # a lane keeps `vec` states, and the workgroup lays all of them out in
        # the LDS: wide states of narrow items (the variance of int8: 16 states
        # of four doubles per lane) stay with the column kernel.  The active
        # lanes are a whole number of periods of a workgroup of 256: larger
        # workgroups would leave fewer lanes idle (67 columns: 201 of 256, 469
        # of 512, 1005 of 1024; 129 columns: 129, 387, 903) and are slower all
        # the same (2^26 float32 with 67 / 129 / 255 columns: 45 / 46 / 47 us
        # with 256 threads, 47 / 49 / 50 with 512, 53 / 55 / 56 with 1024)
        block = _tuning.get('cols_flat_block') or _cg.BLOCK
        threads = period * (block // period)
        if threads == 0 or threads * vec * state_bytes > 32 * 1024:
            return None
        return vec, threads, block

    def _launch_cols_flat(self, geometry, in_args, out_args, in_arr_idx, out_arr_idx, n_out,
                          n_red, so_in, sr, so_out, map_expr, reduce_expr, post_map_expr,
                          reduce_type, typedefs, device_id, stream_ptr, rec=None):
        preamble, _ = self._get_preamble_options()
        ins = [in_args[i] for i in in_arr_idx]
        vec, threads, block = geometry
        cus = _device.get_compute_units(device_id)
        rargs = self._rargs(in_args, out_args)
        stream_hint = _tuning.stream_policy(
            _tuning.get('cols_stream'), self._read_bytes(ins, n_out, n_red, so_in, sr), 0)[0]
        unroll = 4
        idx64 = n_out * n_red > _INT32_MAX - (1 << 24)
        key = ('cols_flat', tuple(r.key() for r in rargs), typedefs, map_expr, reduce_expr,
               post_map_expr, reduce_type, n_out, vec, threads, idx64, device_id, stream_hint,
               unroll, block, _tuning.get('cols_flat_chunked'))

        def emit():
            return self.name, _cg.emit_cols_flat(
                self.name, rargs, self.identity, map_expr, reduce_expr, post_map_expr,
                reduce_type, typedefs, preamble, width=n_out, vec=vec, threads=threads,
                idx64=idx64, stream_hint=stream_hint, unroll=unroll, block=block,
                chunked=_tuning.get('cols_flat_chunked'))
        fn, mod, _ = self._compile(key, emit, in_args)
        trips = (n_out * n_red + threads * vec - 1) // (threads * vec)
        grid = max(1, min(cus * _tuning.get('cols_flat_blocks_per_cu') * _cg.BLOCK // block,
                          trips // unroll))
        ic = 'q' if idx64 else 'i'
        vals = self._fast_values(in_args, out_args, n_out, n_red, so_in, sr, so_out)
        rsize = self._reduce_type_size(reduce_type, mod)
        partials, pref = self._alloc_partials(rec, rsize * grid * n_out)
        vals.ptr(pref, partials.ptr)
        _launch_plan.launch(
            rec, fn, (grid, 1, 1), (block, 1, 1),
            _make_packer(self._fast_format(rargs, ic, 'P')), vals, stream_ptr)
        self._finalize_partials(
            partials, grid, out_args, out_arr_idx, n_out, so_out, in_args, reduce_expr,
            post_map_expr, reduce_type, typedefs, device_id, stream_ptr, rec, pref, n_out * n_red)

    # -- cols ---------------------------------------------------------------------------------
    def _launch_cols(self, in_args, out_args, in_arr_idx, out_arr_idx, n_out, n_red,
                     so_in, sr, so_out, map_expr, reduce_expr, post_map_expr,
                     reduce_type, typedefs, device_id, stream_ptr, rec=None, batch=None):
        """``batch`` = (rows of outputs, columns per row, byte stride of every
        input from row to row) for the reduction over a middle axis; ``n_out``
        is then the total number of outputs."""
        preamble, _ = self._get_preamble_options()
        ins = [in_args[i] for i in in_arr_idx]
        cus = _device.get_compute_units(device_id)
        vec = _max_vector_width([a.dtype.itemsize for a in ins])
        # A lane keeps one state per column of its vector: 16 one-byte values
        # with the four doubles of a variance each would be 512 bytes of
        # registers, and 128 KiB of LDS for the fold across the waves
        # (var over the middle axis of 2647 x 14 x 1780 int8: 435 us)
        state_bytes = _reduce_type_bytes(reduce_type, typedefs)
        while vec > 1 and vec * state_bytes > _tuning.get('cols_state_bytes_per_lane'):
            vec //= 2
        if not batch and len(ins) == len([a for a in in_args if isinstance(a, ndarray)]):
            flat = self._cols_flat_geometry(
                ins, n_out, n_red, so_in, sr, so_out, [out_args[i] for i in out_arr_idx], vec,
                (map_expr, reduce_expr, post_map_expr), state_bytes)
            if flat is not None:
                return self._launch_cols_flat(
                    flat, in_args, out_args, in_arr_idx, out_arr_idx, n_out, n_red, so_in, sr,
                    so_out, map_expr, reduce_expr, post_map_expr, reduce_type, typedefs,
                    device_id, stream_ptr, rec)
        bcast_o = [(s == 0 and n_out > 1) for s in so_in]
        n_batch, n_cols, sb = batch if batch else (1, n_out, None)
        while vec > 1:
            ok = n_cols >= vec
            for a, s_o, s_r in zip(ins, so_in, sr):
                if s_o == 0 and n_out > 1:
                    continue
                nb = min(16, vec * a.dtype.itemsize)
                if not _aligned(a.data.ptr, nb) or (n_red > 1 and not _aligned(s_r, nb)):
                    ok = False
            if batch and not all(_aligned(s, min(16, vec * a.dtype.itemsize))
                                 for s, a in zip(sb, ins)):
                ok = False
            if ok:
                break
            vec //= 2
        # narrower workgroups where the reduce axis will be split (few column
        # blocks for the device); with column blocks in plenty 64 lanes across
        # do better (sum of 33 x 65 x 31277 over its middle axis: 46 us against 51)
        # (rows that do not start on cache lines: a column block of 64 lanes
        # has 9 lines to fetch per row where it would have 8, one of 32 lanes 5
        # for 4; sum over axis 0 of 8191 x 8193 float32 50.7 -> 47.6 us, of
        # 4099 x 16363 48.6 -> 45.5)
        off_lines = any(s_r % 128 or a.data.ptr % 128 for a, s_r in zip(ins, sr))
        tx = 64
        if not off_lines and (n_cols + 64 * vec - 1) // (64 * vec) * n_batch < cus * _tuning.get(
                'cols_target_blocks_per_cu'):
            tx = _tuning.get('cols_tx')
        tx = max(1, min(tx, internal.clp2((n_cols + vec - 1) // vec)))
        # a handful of rows and plenty of columns: a thread per column vector
        solo_block = _tuning.get('cols_solo_block')
        solo = (n_red <= 8 and n_out >= cus * solo_block * vec
                and n_cols >= solo_block * vec)
        block = solo_block if solo else _cg.BLOCK
        if solo:
            tx = block
        ty = block // tx
        nbc = (n_cols + tx * vec - 1) // (tx * vec)
        gx = nbc * n_batch
        # the kernel does not loop over column blocks: beyond what grid.x may
        # hold they continue along grid.z
        gz = (gx + _max_blocks(block) - 1) // _max_blocks(block)
        gx = (gx + gz - 1) // gz
        want = (cus * (_tuning.get('cols_target_blocks_per_cu')
                       or _tuning.get('target_blocks_per_cu')) + gx * gz - 1) // (gx * gz)
        most = max(1, n_red // (ty * 8))
        n_split = max(1, min(want, most, 65535))
        if 1 < n_split and cus * 8 < gx * gz * n_split:
            # (never a few workgroups more than the device holds at once)
            n_split = max(1, cus * 8 // (gx * gz))
        partial = n_split > 1
        span = max([abs(s_o) * n_out + abs(s_r) * n_red for s_o, s_r in zip(so_in, sr)]
                   + [abs(s) * n_out for s in so_out] + [n_red + n_split * ty])
        if batch:
            span = max([span, gx * gz * tx * vec] + [
                abs(s_b) * n_batch + abs(s_r) * n_red + s_o * n_cols
                for s_b, s_r, s_o in zip(sb, sr, so_in)])
        idx64 = span > _INT32_MAX - (1 << 24)
        finish, words_hint = None, 2
        if partial and not batch and not solo and gz == 1:
            words_hint, finish = self._finish_memory(
                ins, n_out, n_red, so_in, sr, reduce_type, typedefs,
                lambda words: n_split * n_out * words + gx, n_split, True, device_id,
                stream_ptr)
        rargs = self._rargs(in_args, out_args, bcast_r=[s == 0 for s in sr], bcast_o=bcast_o)
        clamp = bool(n_cols % vec and n_cols >= vec and _tuning.get('unaligned_vectors'))
        outs = [out_args[i] for i in out_arr_idx]
        vec_out = bool(solo and all(s == a.dtype.itemsize for s, a in zip(so_out, outs)))
        if solo:
            # all rows of a column are requested together
            unroll = max(1, min(4, internal.flp2(n_red)))
        elif partial and all(s % 128 == 0 for s in sr):
            unroll = _tuning.get('cols_unroll')
        else:
            unroll = _tuning.get('cols_unroll_near')
        stream_hint = _tuning.stream_policy(
            _tuning.get('cols_stream'), self._read_bytes(ins, n_out, n_red, so_in, sr), 0)[0]
        # Column blocks numbered so that neighbours run on one compute die,
        # where their borders do not fall on cache-line boundaries
        mode = _tuning.get('cols_xcd')
        xcd = bool(mode) and gz == 1 and not finish and gx > 1 and (mode is True or off_lines)
        key = ('cols', tuple(r.key() for r in rargs), typedefs, map_expr, reduce_expr,
               post_map_expr, reduce_type, tx, vec, idx64, partial, device_id,
               stream_hint, solo, bool(batch), clamp, unroll, vec_out, block, bool(finish),
               xcd, _tuning.signature())

        def emit():
            return self.name, _cg.emit_cols(
                self.name, rargs, self.identity, map_expr, reduce_expr,
                post_map_expr, reduce_type, typedefs, preamble, tx=tx, vec=vec,
                idx64=idx64, partial_out=partial,
                stream_hint=stream_hint, unroll=unroll, solo=solo,
                batched=bool(batch), clamp_tail=clamp, vec_out=vec_out, solo_block=solo_block,
                finish=bool(finish), reduce_words=words_hint, xcd=xcd)
        fn, mod, _ = self._compile(key, emit, in_args)
        ic = 'q' if idx64 else 'i'
        vals = self._fast_values(in_args, out_args, n_out, n_red, so_in, sr, so_out)
        tail = ''
        if batch:
            tail = ic * (2 + len(ins))
            batch_vals = [n_cols, nbc] + [s // a.dtype.itemsize for s, a in zip(sb, ins)]
        if finish:
            # one launch: the workgroup of the last slice of every column block
            # combines the partial results of the others
            if rec is not None:
                rec.bind_stream(stream_ptr, device_id)
            vals.const(finish[0], _tuning.get('reduce_finish_spin_limit'), finish[1], gx)
            _launch_plan.launch(
                rec, fn, (gx * n_split, 1, 1), (block, 1, 1),
                _make_packer(self._fast_format(rargs, ic, 'PIP' + ic)), vals, stream_ptr)
        elif partial:
            rsize = self._reduce_type_size(reduce_type, mod)
            partials, pref = self._alloc_partials(rec, rsize * n_split * n_out)
            vals.ptr(pref, partials.ptr)
            if batch:
                vals.const(*batch_vals)
            _launch_plan.launch(
                rec, fn, (gx, n_split, gz), (block, 1, 1),
                _make_packer(self._fast_format(rargs, ic, 'P' + tail)), vals, stream_ptr)
            self._finalize_partials(
                partials, n_split, out_args, out_arr_idx, n_out, so_out, in_args,
                reduce_expr, post_map_expr, reduce_type, typedefs, device_id,
                stream_ptr, rec, pref, n_out * n_red)
        else:
            if batch:
                vals.const(*batch_vals)
            _launch_plan.launch(
                rec, fn, (gx, 1, gz), (block, 1, 1),
                _make_packer(self._fast_format(rargs, ic, tail)), vals, stream_ptr)

    # -- generic ------------------------------------------------------------------------------
    def _launch_generic(self, in_args, out_args, in_shape, out_shape, n_red,
                        map_expr, reduce_expr, post_map_expr, reduce_type, typedefs,
                        device_id, stream_ptr, rec=None):
        preamble, _ = self._get_preamble_options()
        cus = _device.get_compute_units(device_id)
        n_out = internal.prod(out_shape)
        in_ind = _carray.Indexer(in_shape)
        out_ind = _carray.Indexer(out_shape)
        # threads across the output index: as many as the innermost kept axis
        # is contiguous for, but no more than needed to leave every thread a
        # few elements of the reduce axis
        contiguous = 1
        nd_in = len(in_shape)
        nd_out = len(out_shape)
        for a, p in zip(in_args, self.in_params):
            if not isinstance(a, ndarray) or p.raw:
                continue
            run = 1
            for j in range(nd_out):
                if a._strides[nd_in - j - 1] != run * a.dtype.itemsize:
                    break
                run *= out_shape[nd_out - j - 1]
            contiguous = max(contiguous, run)
        tx = max(min(contiguous, 64), _cg.BLOCK // max(1, n_red))
        tx = max(1, min(64, internal.flp2(tx), internal.clp2(n_out)))
        ty = _cg.BLOCK // tx
        gx = min((n_out + tx - 1) // tx, _max_blocks(_cg.BLOCK))
        want = (cus * _tuning.get('target_blocks_per_cu') + gx - 1) // gx
        most = max(1, n_red // (ty * 8))
        n_split = max(1, min(want, most, 65535))
        partial = n_split > 1
        rargs = self._rargs(in_args, out_args)
        key = ('generic', tuple(r.key() for r in rargs), typedefs, map_expr,
               reduce_expr, post_map_expr, reduce_type, tx, in_ind.ndim,
               out_ind.ndim, in_ind._index_32_bits, out_ind._index_32_bits,
               partial, device_id)

        def emit():
            return self.name, _cg.emit_generic(
                self.name, rargs, self.identity, map_expr, reduce_expr,
                post_map_expr, reduce_type, typedefs, preamble, tx=tx,
                in_ndim=in_ind.ndim, out_ndim=out_ind.ndim,
                in_index_32=in_ind._index_32_bits,
                out_index_32=out_ind._index_32_bits, partial_out=partial)
        fn, mod, _ = self._compile(key, emit, in_args)
        fmt = ['@']
        vals = _launch_plan.ArgBlock()
        nin = len(self.in_params)

        def put(ref, a):
            if isinstance(a, ndarray):
                fmt.append('P' + 'q' * (1 + 2 * a.ndim))
                vals.ptr(ref, a.data.ptr)
                vals.const(a.size, *a._shape)
                vals.const(*a._strides)
            else:
                fmt.append(_scalar_struct_code(_get_typename(a.descr)))
                vals.scalar(ref, a)
        for ref, a in enumerate(in_args):
            put(ref, a)
        for j, a in enumerate(out_args):
            put(nin + j, a)
        for ind in (in_ind, out_ind):
            fmt.append('q' * (1 + 2 * ind.ndim))
            vals.const(ind.size, *ind.shape)
            vals.const(*((0,) * ind.ndim))
        if not partial:
            _launch_plan.launch(rec, fn, (gx, 1, 1), (_cg.BLOCK, 1, 1),
                                _make_packer(fmt), vals, stream_ptr)
            return
        rsize = self._reduce_type_size(reduce_type, mod)
        partials, pref = self._alloc_partials(rec, rsize * n_split * n_out)
        fmt.append('P')
        vals.ptr(pref, partials.ptr)
        _launch_plan.launch(rec, fn, (gx, n_split, 1), (_cg.BLOCK, 1, 1),
                            _make_packer(fmt), vals, stream_ptr)
        # second pass through the strided output views
        frargs = [r for r in rargs if r.kind in ('out', 'raw', 'scalar')]
        fkey = ('generic_final', tuple(r.key() for r in frargs), typedefs,
                reduce_expr, post_map_expr, reduce_type, out_ind.ndim,
                out_ind._index_32_bits, device_id)

        def emit_final():
            name = self.name + '_combine'
            return name, _cg.emit_finalize_generic(
                name, frargs, self.identity, reduce_expr, post_map_expr,
                reduce_type, typedefs, preamble, out_ndim=out_ind.ndim,
                out_index_32=out_ind._index_32_bits)
        ffn, _, _ = self._compile(fkey, emit_final, in_args)
        fmt = ['@']
        vals = _launch_plan.ArgBlock()
        # parameter order of emit_finalize_generic: out / raw / scalar in the
        # order they appear in `frargs`
        for ref, (a, p) in enumerate(zip(in_args, self.in_params)):
            if not isinstance(a, ndarray) or p.raw:
                put(ref, a)
        for j, a in enumerate(out_args):
            put(nin + j, a)
        fmt.append('q' * (1 + 2 * out_ind.ndim))
        vals.const(out_ind.size, *out_ind.shape)
        vals.const(*((0,) * out_ind.ndim))
        fmt.append('Piq')
        vals.ptr(pref, partials.ptr)
        vals.const(n_split, in_ind.size)
        grid = max(1, min((n_out + _cg.BLOCK - 1) // _cg.BLOCK, cus * 8))
        _launch_plan.launch(rec, ffn, (grid, 1, 1), (_cg.BLOCK, 1, 1),
                            _make_packer(fmt), vals, stream_ptr)

    # -- debugging aids ------------------------------------------------------------------------
    @property
    def cached_codes(self):
        """dict: input dtype characters -> generated source."""
        if len(self._cached_codes) == 0:
            warnings.warn(
                'No codes are cached because compilation is deferred until '
                'the first function call.')
        return dict(self._cached_codes.items())

    @property
    def cached_code(self):
        codes = self._cached_codes
        if len(codes) > 1:
            warnings.warn(
                'The input types of the kernel could not be inferred. '
                'Please use `.cached_codes` instead.')
        return next(iter(codes.values()))


# ---------------------------------------------------------------------------------
# create_reduction_func
# ---------------------------------------------------------------------------------

def create_reduction_func(name, ops, routine=None, identity=None, preamble='',
                          sort_reduce_axis=True):
    """Builds a one-input reduction from loop signatures and a routine
    ``(map_expr, reduce_expr, post_map_expr, reduce_type)``."""
    ops = _kernel._Ops.from_tuples(ops, routine)
    return _SimpleReductionKernel(name, ops, identity, preamble, sort_reduce_axis)


class _SimpleReductionKernel(_AbstractReductionKernel):

    def __init__(self, name, ops, identity, preamble, sort_reduce_axis=True):
        super().__init__(name, '' if identity is None else str(identity),
                         'T in0', 'T out0')
        self._ops = ops
        self.preamble = preamble
        self.nin = 1
        self.nout = 1
        self._routine_cache = {}
        self._sort_reduce_axis = sort_reduce_axis

    def __call__(self, a, axis=None, dtype=None, out=None, keepdims=False):
        if hasattr(a, '__cupy_override_reduction_kernel__'):
            return a.__cupy_override_reduction_kernel__(
                self, axis, dtype, out, keepdims)
        dev_id = _device.get_device_id()
        fast_args = (a,) if out is None else (a, out)
        done, ret, key, rec = self._fast_lookup(
            fast_args, (axis, dtype, keepdims), dev_id)
        if done:
            return ret
        arr = _convert_from_cupy_like(a, error="Argument 'a'")
        _check_peer_access(arr, dev_id)
        if out is None:
            out_args = []
        else:
            if not isinstance(out, ndarray):
                raise TypeError("Argument 'out' has incorrect type")
            _check_peer_access(out, dev_id)
            out_args = [out]
        ret = self._call([arr], out_args, arr._shape, axis, dtype, keepdims,
                         True, dev_id, None, self._sort_reduce_axis, rec)
        self._fast_remember(key, rec, fast_args, ret)
        return ret

    def _get_expressions_and_types(self, in_args, out_args, dtype):
        op = self._ops.guess_routine(
            self.name, self._routine_cache, in_args, dtype, self._ops)
        map_expr, reduce_expr, post_map_expr, reduce_type = op.routine
        if reduce_type is None:
            reduce_type = _get_typename(op.out_types[0])
        if out_args:
            out_type = out_args[0].dtype.type
        else:
            out_type = op.out_types[0]
        type_pairs = (('type_in0_raw', in_args[0].dtype.type),
                      ('type_out0_raw', out_type))
        return (map_expr, reduce_expr, post_map_expr, op.in_types, op.out_types,
                reduce_type, type_pairs)

    def _get_out_args(self, out_args, out_types, out_shape):
        return _get_out_args_from_optionals(
            ndarray, out_args, out_types, out_shape, 'unsafe', None)

    def _get_preamble_options(self):
        return self.preamble, ()

    def _in_var_type(self, index, param):
        return 'type_in0_raw'

    def _out_var_type(self, index, param):
        return 'type_out0_raw'


# ---------------------------------------------------------------------------------
# ReductionKernel
# ---------------------------------------------------------------------------------

class ReductionKernel(_AbstractReductionKernel):
    """User-defined reduction kernel.

    Args:
        in_params (str): Input argument list.
        out_params (str): Output argument list.
        map_expr (str): Expression applied to each input element (or tuple of
            elements of the broadcast inputs).
        reduce_expr (str): Combines ``a`` and ``b``.
        post_map_expr (str): Statement storing the reduced value ``a`` into the
            output parameter.
        identity (str): Initial value of the reduction.
        name (str): Kernel name.
        reduce_type (str): Type of ``a`` / ``b`` (default: first output type).
        reduce_dims (bool): Merge contiguous axes before launching.
        preamble (str): Code inserted before the kernel.
        options (tuple of str): Extra hiprtc options.
    """

    def __init__(self, in_params, out_params, map_expr, reduce_expr,
                 post_map_expr, identity, name='reduce_kernel', reduce_type=None,
                 reduce_dims=True, preamble='', options=()):
        if not compiler.is_valid_kernel_name(name):
            raise ValueError('Invalid kernel name: "%s"' % name)
        super().__init__(name, '' if identity is None else str(identity),
                         in_params, out_params)
        self.nin = len(self.in_params)
        self.nout = len(self.out_params)
        self.nargs = self.nin + self.nout
        self.reduce_expr = reduce_expr
        self.map_expr = map_expr
        self.post_map_expr = post_map_expr
        self.options = tuple(options)
        self.reduce_dims = reduce_dims
        if reduce_type is None:
            self.reduce_type = self.out_params[0].ctype
        else:
            self.reduce_type = reduce_type
        self.preamble = preamble

    def __call__(self, *args, **kwargs):
        """Compiles (if needed) and launches the reduction.

        Args:
            args: Inputs, optionally followed by the outputs.
            out (cupy.ndarray): Output array (not together with a positional one).
            axis (int or tuple of ints): Axes to reduce (default: all).
            keepdims (bool): Keep reduced axes with length one.
            stream: Stream to launch on.
        """
        out = kwargs.pop('out', None)
        axis = kwargs.pop('axis', None)
        keepdims = kwargs.pop('keepdims', False)
        stream = kwargs.pop('stream', None)
        if kwargs:
            raise TypeError('Wrong arguments %s' % kwargs)
        n_args = len(args)
        if n_args != self.nin and n_args != self.nargs:
            raise TypeError('Wrong number of arguments for %s' % self.name)
        out_args = list(args[self.nin:])
        if out is not None:
            if self.nout != 1:
                raise NotImplementedError('')
            if len(out_args) != 0:
                raise ValueError("cannot specify 'out' as both "
                                 "a positional and keyword argument")
            out_args = [out]
        dev_id = _device.get_device_id()
        key = rec = None
        if stream is None:
            fast_args = tuple(args[:self.nin]) + tuple(out_args)
            done, ret, key, rec = self._fast_lookup(
                fast_args, (axis, keepdims), dev_id)
            if done:
                return ret
        in_args = _preprocess_args(dev_id, args[:self.nin])
        out_args = _preprocess_args(dev_id, out_args)
        in_args, broad_shape = _broadcast(in_args, self.in_params, False)
        ret = self._call(in_args, out_args, broad_shape, axis, None, keepdims,
                         self.reduce_dims, dev_id, stream, True, rec)
        if rec is not None:
            self._fast_remember(key, rec, fast_args, ret)
        return ret

    def _get_expressions_and_types(self, in_args, out_args, dtype):
        in_ndarray_types = tuple(
            a.dtype.type if isinstance(a, ndarray) else None for a in in_args)
        out_ndarray_types = tuple(
            a.dtype.type if isinstance(a, ndarray) else None for a in out_args)
        in_types, out_types, type_map = _decide_params_type(
            self.in_params, self.out_params, in_ndarray_types, out_ndarray_types)
        return (self.map_expr, self.reduce_expr, self.post_map_expr, in_types,
                out_types, self.reduce_type, type_map._pairs)

    def _get_out_args(self, out_args, out_types, out_shape):
        return _get_out_args_with_params(
            out_args, out_types, out_shape, self.out_params, False)

    def _get_preamble_options(self):
        return self.preamble, self.options

    def _in_var_type(self, index, param):
        return param.ctype
