"""Replay of kernel launches for calls whose arguments look like an earlier call's.

Everything the host path decides for a call of an ElementwiseKernel, a ufunc, a
reduction or a fused function -- the loop's types, broadcasting, the merged
axes, the kernel variant, its launch geometry, the layout of its argument
block, the shapes and types of the outputs and of temporaries -- is a function
of the arguments' *signature*: for arrays the dtype, shape, strides, device and
the alignment of the data pointer, for scalars their Python or NumPy type.
Only data pointers and scalar values change from call to call.  The first call
with a signature goes through the full path and records what it launched; later
calls with the same signature patch pointers and scalar values into the recorded
argument blocks and launch.

The reference repeats its whole per-call path on every call
(cupy/_core/_kernel.pyx:870-935 for ElementwiseKernel, :1241-1330 for ufuncs,
cupy/_core/_reduction.pyx:309-427 for reductions); its kernel memo
(_kernel.pyx:948-975) saves only the compilation.
"""
import struct

import numpy

from cupy_amd import _dryrun
from cupy_amd import _rt
from cupy_amd._core import _carray
from cupy_amd._core import _tuning
from cupy_amd._core._scalar import CScalar
from cupy_amd.cuda import _giveup
from cupy_amd.cuda import memory as _memory
from cupy_amd.cuda import stream as _stream


_float64 = numpy.dtype('float64')
_float32 = numpy.dtype('float32')
_bool = numpy.dtype('bool')
_INT_LIMITS = {
    numpy.dtype(t): (int(numpy.iinfo(t).min), int(numpy.iinfo(t).max))
    for t in ('int8', 'int16', 'int32', 'int64', 'uint8', 'uint16', 'uint32', 'uint64')}
_F32_SAFE = 3.0e38
_INT64_MIN = -(1 << 63)
_INT64_MAX = (1 << 63) - 1
_INF = float('inf')

# Recorded calls kept per kernel object.
_MAX_PLANS = 256

# False: replays go through Function.launch_packed like first calls do (for
# code that watches launches there, e.g. to list the kernels of an operation)
use_quick = True

_SLOT_MARK = 0x5ca7c4a5c4a7c4a5       # stands in for a pointer while its byte offset is looked up


def scalar_value(v, descr):
    """``v`` as the Python object ``struct.pack`` takes for a kernel parameter
    of dtype ``descr``; same result (and same errors) as
    ``CScalar(v).apply_dtype(descr)._struct_value()``."""
    t = type(v)
    if t is float:
        if descr is _float64 or descr == _float64:
            return v
        if descr == _float32 and (-_F32_SAFE < v < _F32_SAFE or v != v
                                  or v == _INF or v == -_INF):
            return v        # struct rounds to nearest even exactly like NumPy
    elif t is int:
        lim = _INT_LIMITS.get(descr)
        if lim is not None:
            if lim[0] <= v <= lim[1]:
                return v
        elif descr == _float64 and -(1 << 53) <= v <= (1 << 53):
            return float(v)
        elif descr == _float32 and -(1 << 24) <= v <= (1 << 24):
            return float(v)     # (exact in 24 bits of mantissa)
    elif t is bool:
        if descr == _bool:
            return v
    s = CScalar(v)
    s.apply_dtype(descr)
    return s._struct_value()


class ArgBlock:
    """Values of one kernel's argument block, in order, with a note of which
    slots hold the data pointer of which argument and the value of which
    scalar.  ``ref`` numbers identify the call's arguments: user arguments
    first, then outputs the call allocates, then temporaries."""
    __slots__ = ('vals', 'ptrs', 'scalars')

    def __init__(self):
        self.vals = []
        self.ptrs = []
        self.scalars = []

    def ptr(self, ref, address):
        self.ptrs.append((len(self.vals), ref))
        self.vals.append(address)

    def scalar(self, ref, cscalar):
        self.scalars.append((len(self.vals), ref, cscalar.descr))
        self.vals.append(cscalar._struct_value())

    def const(self, *values):
        self.vals.extend(values)


class Recorder:
    """Collects the launches and temporaries of one call."""
    __slots__ = ('n_refs', 'launches', 'temps', 'stream', 'device')

    def __init__(self, n_refs):
        self.n_refs = n_refs      # user arguments + allocated outputs
        self.launches = []
        self.temps = []
        self.stream = None        # the one stream the launches may be replayed on
        self.device = None        # ... and the device that stream belongs to

    def bind_stream(self, stream_ptr, dev_id):
        """The recorded launches finish a split reduction inside one launch
        through memory that belongs to ``stream_ptr`` of device ``dev_id``: a
        replay on another stream takes the full path, and so does every replay
        once a kernel of that kind gave up a wait on the device."""
        self.stream = stream_ptr
        self.device = dev_id

    def temp(self, nbytes):
        """Registers a temporary of ``nbytes``; returns its ref number."""
        self.temps.append(nbytes)
        return self.n_refs + len(self.temps) - 1

    def launch(self, fn, grid, block, packer, argblock, shared_mem=0):
        self.launches.append((fn, grid, block, packer, list(argblock.vals),
                              tuple(argblock.ptrs), tuple(argblock.scalars),
                              shared_mem))


def launch(rec, fn, grid, block, packer, argblock, stream_ptr, shared_mem=0):
    """Launches now and, if a recorder is given, notes the launch for replay."""
    fn.launch_packed(grid, block, packer.pack(*argblock.vals), shared_mem, stream_ptr)
    if rec is not None:
        rec.launch(fn, grid, block, packer, argblock, shared_mem)


def call_signature(args, dev_id):
    """Hashable description of everything about ``args`` (a tuple) that launch
    decisions may depend on, or None if the call must take the full path:
    per array ``(dtype, shape, strides, address & 15)``, per scalar its type
    (Python ints beyond 64 bits, arrays of other devices and objects of other
    kinds take the full path).  Computed by the extension module."""
    return _signature(args, dev_id, _tuning.version())


_signature = _rt.hot.signature


def ranges_overlap(a, b):
    """True if the memory spans of two arrays intersect."""
    return _carray.may_share_bounds(a, b)


class FastCall:
    """Recorded call: allocates outputs and temporaries, patches pointers and
    scalar values, launches."""
    __slots__ = ('n_user', 'out_specs', 'temps', 'launches', 'ret', 'overlap', 'quick',
                 'stream', 'device', 'int_scalars')

    def __init__(self, n_user, out_specs, rec, ret, overlap=()):
        self.n_user = n_user
        self.out_specs = tuple(out_specs)     # (shape, dtype) of allocated outputs
        self.temps = tuple(rec.temps)
        self.launches = tuple(rec.launches)
        self.ret = ret                        # ref, tuple of refs, or None
        self.overlap = tuple(overlap)         # (input ref, output ref) pairs to check
        self.quick = _quick_launches(self.launches)
        # scalar arguments that are packed as integers: a Python integer outside
        # the type takes the full path, which raises or chooses another loop
        # as NumPy does
        self.int_scalars = tuple(sorted({
            (ref, descr) for launch in self.launches for _, ref, descr in launch[6]
            if descr in _INT_LIMITS}, key=lambda rd: rd[0]))
        self.stream = rec.stream
        self.device = rec.device

    def stale(self):
        """True for a record that must not be replayed any more, on any
        stream: it finishes a reduction inside one launch and a kernel of that
        kind has given up a wait on its device.  The full path then reports
        that (once) and records the two-launch form in this record's place."""
        return self.stream is not None and not _giveup.usable(self.device, _giveup.REDUCTION)

    def run(self, args, stream_ptr=None):
        from cupy_amd._core.core import ndarray
        if self.stream is not None:
            if stream_ptr is None:
                stream_ptr = _stream.get_current_stream_ptr()
            if stream_ptr != self.stream:
                return NotImplemented
            # (a wrong result must not be handed out twice: the reference's
            # reduction is a plain launch, cupy/_core/_reduction.pyx:481-508)
            if not _giveup.usable(self.device, _giveup.REDUCTION):
                return NotImplemented
        for ref, descr in self.int_scalars:
            v = args[ref]
            if type(v) is int:
                lo, hi = _INT_LIMITS[descr]
                if not lo <= v <= hi:
                    return NotImplemented
        for i, o in self.overlap:
            a, b = args[i], args[o]
            # (arrays of different allocations cannot overlap)
            if (a is not b and a.data.mem.ptr == b.data.mem.ptr
                    and _carray.may_share_bounds(a, b)):
                return NotImplemented
        if _memory._static_scratch_open and _memory.static_scratch_active():
            return self._run_static(args, stream_ptr)
        refs = list(args)
        for shape, dtype in self.out_specs:
            refs.append(ndarray._new_contiguous(shape, dtype))
        n_arr = len(refs)
        for nbytes in self.temps:
            refs.append(_memory.alloc(nbytes))
        if stream_ptr is None:
            stream_ptr = _stream.get_current_stream_ptr()
        quick = self.quick
        if quick is not None and use_quick:
            # pointer-only argument blocks: the extension splices the
            # addresses into the recorded bytes and launches
            status = _replay(quick[0], refs, n_arr, stream_ptr)
            if status != 0:
                _rt.check(status)
        else:
            for fn, grid, block, packer, template, ptrs, scalars, shmem in self.launches:
                vals = template[:]
                for slot, ref in ptrs:
                    if ref < n_arr:
                        vals[slot] = refs[ref].data.ptr
                    else:
                        vals[slot] = refs[ref].ptr
                for slot, ref, descr in scalars:
                    vals[slot] = scalar_value(refs[ref], descr)
                fn.launch_packed(grid, block, packer.pack(*vals), shmem, stream_ptr)
        ret = self.ret
        if ret is None:
            return None
        if type(ret) is tuple:
            return tuple(refs[r] for r in ret)
        return refs[ret]


def _quick_launches(launches):
    """The launches of a recorded call whose argument blocks change only in
    their pointers, as the record ``_rt.hot.replay`` takes: per launch the
    function handle, grid and block, shared memory, the byte offsets of the
    pointer slots with the ref each receives, and the argument block as
    recorded.  Returns ``(record, Functions kept alive)``, or None if any
    launch takes a scalar that changes from call to call."""
    out = [struct.pack('<II', len(launches), 0)]
    recorded_only = _dryrun.enabled()
    for fn, grid, block, packer, template, ptrs, scalars, shmem in launches:
        if scalars or not ptrs:
            return None
        gx, gy, gz = grid
        bx, by, bz = block
        if gx * bx > 0xffffffff or gy * by > 0xffffffff or gz * bz > 0xffffffff:
            return None
        vals = list(template)
        marks = {}
        for i, (slot, ref) in enumerate(ptrs):
            vals[slot] = _SLOT_MARK + i
            marks[(_SLOT_MARK + i).to_bytes(8, 'little')] = ref
        blob = packer.pack(*vals)
        if len(blob) > fn._arg_size or len(blob) < fn._arg_min:
            return None
        blob += b'\0' * (fn._arg_size - len(blob))
        found = []
        for mark, ref in marks.items():
            off = blob.find(mark)
            if off < 0 or off % 8 or blob.find(mark, off + 1) >= 0:
                return None
            found.append((off, ref))
        found.sort()
        handle = fn.ptr
        if recorded_only:
            # no function handles exist: a stand-in that names the kernel
            handle = id(fn)
            _function_names[handle] = fn.name
        out.append(struct.pack('<Q3I3IIIQ', handle, gx, gy, gz, bx, by, bz, shmem,
                               len(found), len(blob)))
        out.append(b''.join(struct.pack('<II', off, ref) for off, ref in found))
        out.append(blob + b'\0' * (-len(blob) % 8))
    return b''.join(out), tuple(launch[0] for launch in launches)


def _replay_recorded_only(record, refs, n_arr, stream_ptr):
    """Stand-in for ``_rt.hot.replay`` where launches are only recorded: the
    extension patches the argument blocks as it would for a launch and hands
    them back."""
    for handle, grid, block, shmem, blob in _rt.hot.splice(record, refs, n_arr):
        _dryrun.record_launch(_function_names[handle], grid, block, shmem, blob)
    return 0


_function_names = {}
_replay = _replay_recorded_only if _dryrun.enabled() else _rt.hot.replay


def _run_static(self, args, stream_ptr):
    """``FastCall.run`` without any allocation (``cuda.memory.static_scratch``):
    the one temporary the call may use is the runtime library's static device
    array, handed to the kernels by ``rt_launch_packed_scratch``."""
    refuse_allocation = _memory.refuse_allocation
    if self.out_specs:
        refuse_allocation('an output array')
    if len(self.temps) > 1:
        refuse_allocation('a second temporary')
    if self.temps and self.temps[0] > _rt.RT_SCRATCH_MAX_BYTES:
        raise RuntimeError(
            'static_scratch: the call needs %d bytes of scratch memory, the runtime '
            'library holds %d' % (self.temps[0], _rt.RT_SCRATCH_MAX_BYTES))
    refs = args
    n_arr = len(refs)
    if stream_ptr is None:
        stream_ptr = _stream.get_current_stream_ptr()
    for fn, grid, block, packer, template, ptrs, scalars, shmem in self.launches:
        vals = template[:]
        scratch_slot = None
        for slot, ref in ptrs:
            if ref < n_arr:
                vals[slot] = refs[ref].data.ptr
            else:
                if scratch_slot is not None:
                    refuse_allocation('a kernel with two scratch pointers')
                scratch_slot = slot
                vals[slot] = _SLOT_MARK
        for slot, ref, descr in scalars:
            vals[slot] = scalar_value(refs[ref], descr)
        block_bytes = packer.pack(*vals)
        if scratch_slot is None:
            fn.launch_packed(grid, block, block_bytes, shmem, stream_ptr)
            continue
        mark = _SLOT_MARK.to_bytes(8, 'little')
        offset = block_bytes.find(mark)
        if offset < 0 or offset % 8 or block_bytes.find(mark, offset + 1) >= 0:
            raise RuntimeError('static_scratch: cannot locate the scratch pointer of %s' % fn.name)
        fn.launch_packed_scratch(grid, block, block_bytes, offset, self.temps[0],
                                 shmem, stream_ptr)
    ret = self.ret
    if ret is None:
        return None
    if type(ret) is tuple:
        return tuple(refs[r] for r in ret)
    return refs[ret]


FastCall._run_static = _run_static


def remember(table, key, fast):
    """Stores a recorded call; the table is emptied when it grows too large
    (signatures include shapes, so a loop over many shapes must not pin an
    unbounded number of entries)."""
    if len(table) >= _MAX_PLANS:
        table.clear()
    table[key] = fast
