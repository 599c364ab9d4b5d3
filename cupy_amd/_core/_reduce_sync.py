"""Memory through which the workgroups of a split reduction hand their partial
results to the workgroup that finishes the reduction inside the same launch
(``_codegen_reduction._SYNC_HELPERS`` describes what the kernels do with it).

One block of memory per (device, stream): 64 words of header -- word 0 is the
number of the last launch that used the block, kept by the kernels themselves,
so that a recorded launch can be replayed without any change -- followed by
slots of 64 bits.  Launches on one stream run one after the other, and every
launch marks what it writes with its own number, so nothing is cleared between
launches.  A block is cleared once, when it is created; a block that has become
too small is retired (see ``_retired``) and a larger one takes its place.
"""
import threading

import numpy

from cupy_amd._core import _tuning
from cupy_amd.cuda import _giveup
from cupy_amd.cuda import memory as _memory
from cupy_amd.cuda import stream as _stream

HEADER_WORDS = 64
MAX_STREAMS = 64    # (device, stream) pairs that hold a block at a time

_lock = threading.Lock()
_blocks = {}        # (device id, stream) -> (array of uint32, slots it holds)
# Blocks that were replaced or evicted.  Recorded calls name a block by its
# address, so whenever blocks are retired the tuning version moves on (no
# earlier record is replayed again) and the blocks stay allocated until the
# retirement after the next: a thread that had picked up a record just before
# still finds the memory in place.
_retired = [[], []]


def _fault_word(dev_id):
    """Address of the word a workgroup that gives up waiting writes to."""
    return _giveup.word(dev_id, _giveup.REDUCTION)


def _retire(blocks):
    _retired[1] = _retired[0]       # (drops the generation before: freed)
    _retired[0] = list(blocks)
    _tuning.invalidate_records()


def acquire(dev_id, stream_ptr, current_stream_ptr, n_slots):
    """``(address of the block, address of the fault word)`` for a launch on
    ``stream_ptr`` that needs ``n_slots`` slots, or None where the reduction
    has to take two launches: switched off, a stream other than the current
    one (the block is cleared on the current stream), more slots than a block
    may hold, the per-thread default stream, no allocation allowed, or an
    earlier failure on this device."""
    if not _tuning.get('reduce_finish') or dev_id in _giveup.disabled[_giveup.REDUCTION]:
        return None
    if stream_ptr != current_stream_ptr or n_slots > _tuning.get('reduce_finish_max_slots'):
        return None
    if stream_ptr == _stream.STREAM_PER_THREAD:
        # one handle, a different stream in every thread: launches that share
        # a block could overlap
        return None
    if _memory._static_scratch_open and _memory.static_scratch_active():
        return None
    fault = _fault_word(dev_id)
    # Not expected to happen: say so, and stay away from the kernels.
    _giveup.poll(dev_id)
    key = (dev_id, stream_ptr)
    with _lock:
        block = _blocks.get(key)
        if block is None or block[1] < n_slots:
            from cupy_amd._core.core import ndarray
            slots = max(n_slots, 1 << 16)
            if block is not None:
                slots = max(slots, 2 * block[1])
                del _blocks[key]
                _retire([block])
            elif len(_blocks) >= MAX_STREAMS:
                evicted = list(_blocks.values())
                _blocks.clear()
                _retire(evicted)
            array = ndarray._new_contiguous((HEADER_WORDS + 2 * slots,), numpy.dtype('uint32'))
            # (a kernel on the current stream, not a memset: the caller may be
            # capturing the stream)
            array.fill(0)
            block = _blocks[key] = (array, slots)
    return block[0].data.ptr, fault
