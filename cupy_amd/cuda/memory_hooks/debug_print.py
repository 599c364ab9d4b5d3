"""A memory hook that logs every allocation event as one line of JSON
(reference: cupy/cuda/memory_hooks/debug_print.py; same keys, same order, so
that logs of both read alike)."""
import json
import sys

from cupy_amd.cuda import memory_hook

# the keys each hook point reports, in output order
_FIELDS = {
    'alloc': ('device_id', 'mem_size', 'mem_ptr'),
    'malloc': ('device_id', 'size', 'mem_size', 'mem_ptr', 'pmem_id'),
    'free': ('device_id', 'mem_size', 'mem_ptr', 'pmem_id'),
}


class DebugPrintHook(memory_hook.MemoryHook):
    """Prints what the pool did, right after it did it: ``alloc`` (memory taken
    from the device), ``malloc`` (a request served from the pool) and ``free``
    (a block handed back), e.g. ::

        {"hook":"alloc","device_id":0,"mem_size":512,"mem_ptr":140187860992000}
        {"hook":"malloc","device_id":0,"size":24,"mem_size":512,"mem_ptr":140187860992000,"pmem_id":"0x7f39200c5278"}
        {"hook":"free","device_id":0,"mem_size":512,"mem_ptr":140187860992000,"pmem_id":"0x7f39200c5278"}

    ``size`` is what was asked for, ``mem_size`` the rounded size of the
    block, ``pmem_id`` identifies the pooled-memory object.

    Args:
        file: text stream to write to (default ``sys.stdout``).
        flush (bool): flush the stream after every line (default True).
    """

    name = 'DebugPrintHook'

    def __init__(self, file=sys.stdout, flush=True):
        self.file = file
        self.flush = flush

    def _report(self, point, event):
        record = {'hook': point}
        for key in _FIELDS[point]:
            value = event[key]
            record[key] = hex(value) if key == 'pmem_id' else int(value)
        self.file.write(json.dumps(record, separators=(',', ':')) + '\n')
        if self.flush:
            self.file.flush()

    def alloc_postprocess(self, **kwargs):
        self._report('alloc', kwargs)

    def malloc_postprocess(self, **kwargs):
        self._report('malloc', kwargs)

    def free_postprocess(self, **kwargs):
        self._report('free', kwargs)
