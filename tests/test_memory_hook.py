"""Memory hooks: which callbacks fire, in what order, with which keyword
arguments (the reference's tests/cupy_tests/cuda_tests/test_memory_hook.py:
13-120, same scenario and the same expected dictionaries)."""
import gc
import threading

import pytest

import cupy_amd as cp
from cupy_amd.cuda import memory, memory_hook


class Recording(memory_hook.MemoryHook):
    name = 'Recording'

    def __init__(self):
        self.events = []

    def alloc_preprocess(self, **kw):
        self.events.append(('alloc_pre', kw))

    def alloc_postprocess(self, **kw):
        self.events.append(('alloc_post', kw))

    def malloc_preprocess(self, **kw):
        self.events.append(('malloc_pre', kw))

    def malloc_postprocess(self, **kw):
        self.events.append(('malloc_post', kw))

    def free_preprocess(self, **kw):
        self.events.append(('free_pre', kw))

    def free_postprocess(self, **kw):
        self.events.append(('free_post', kw))


def test_hook_sequence_and_arguments():
    gc.collect()
    pool = memory.MemoryPool()
    unit = 512
    hook = Recording()
    with hook:
        mem = pool.malloc(1)
        ptr1, pmem1 = mem.ptr, id(mem.mem)
        del mem
        mem = pool.malloc(1)
        ptr2, pmem2 = mem.ptr, id(mem.mem)
        del mem
    assert ptr1 == ptr2                       # the second request is a pool hit
    names = [e[0] for e in hook.events]
    assert names == ['malloc_pre', 'alloc_pre', 'alloc_post', 'malloc_post',
                     'free_pre', 'free_post',
                     'malloc_pre', 'malloc_post', 'free_pre', 'free_post']
    ev = dict(enumerate(e[1] for e in hook.events))
    assert ev[0] == {'device_id': 0, 'size': 1, 'mem_size': unit}
    assert ev[1] == {'device_id': 0, 'mem_size': unit}
    assert ev[2] == {'device_id': 0, 'mem_size': unit, 'mem_ptr': ptr1}
    assert ev[3] == {'device_id': 0, 'size': 1, 'mem_size': unit, 'mem_ptr': ptr1,
                     'pmem_id': pmem1}
    assert ev[4] == ev[5] == {'device_id': 0, 'mem_size': unit, 'mem_ptr': ptr1,
                              'pmem_id': pmem1}
    assert ev[7] == {'device_id': 0, 'size': 1, 'mem_size': unit, 'mem_ptr': ptr2,
                     'pmem_id': pmem2}
    assert ev[8] == ev[9] == {'device_id': 0, 'mem_size': unit, 'mem_ptr': ptr2,
                              'pmem_id': pmem2}
    # outside the `with` nothing is recorded
    n = len(hook.events)
    pool.malloc(1)
    assert len(hook.events) == n


def test_hooks_are_per_thread_and_names_are_unique():
    hook = Recording()
    seen = []

    def other():
        seen.append(dict(memory_hook.get_memory_hooks()))
        cp.ndarray((16,), 'f')

    with hook:
        assert memory_hook.get_memory_hooks() == {'Recording': hook}
        with pytest.raises(KeyError):
            with Recording():
                pass
        n = len(hook.events)
        t = threading.Thread(target=other)
        t.start()
        t.join()
        assert seen == [{}]
        assert len(hook.events) == n          # the other thread's allocation is not ours
    assert memory_hook.get_memory_hooks() == {}
    assert not memory_hook._has_memory_hooks()


def test_array_allocation_goes_through_the_hooks():
    hook = Recording()
    with hook:
        a = cp.ndarray((1000,), 'f')
        del a
    kinds = [e[0] for e in hook.events]
    assert kinds.count('malloc_pre') == 1 and kinds.count('free_post') == 1
    assert hook.events[0][1]['size'] == 4000 and hook.events[0][1]['mem_size'] == 4096


# ---- the ready-made hooks (reference: tests/cupy_tests/cuda_tests/memory_hooks_tests/) ----

def _fake_pool(monkeypatch):
    monkeypatch.setattr(memory._device, 'get_device_id', lambda: 0)

    class Fake(memory.BaseMemory):
        cur = [1 << 30]

        def __init__(self, size):
            self.ptr = Fake.cur[0]
            Fake.cur[0] += size + 4096
            self.size = size
            self.device_id = 0
    return memory.MemoryPool(lambda size: memory.MemoryPointer(Fake(size), 0))


def test_debug_print_hook_writes_one_json_line_per_event(monkeypatch):
    import io
    import json
    from cupy_amd.cuda import memory_hooks
    pool = _fake_pool(monkeypatch)
    out = io.StringIO()
    with memory_hooks.DebugPrintHook(file=out):
        mem = pool.malloc(1)
        ptr1, pmem1 = mem.ptr, id(mem.mem)
        del mem
        mem = pool.malloc(1)
        ptr2, pmem2 = mem.ptr, id(mem.mem)
        del mem
    lines = out.getvalue().splitlines()
    assert [json.loads(l) for l in lines] == [
        {'hook': 'alloc', 'device_id': 0, 'mem_size': 512, 'mem_ptr': ptr1},
        {'hook': 'malloc', 'device_id': 0, 'size': 1, 'mem_size': 512, 'mem_ptr': ptr1,
         'pmem_id': hex(pmem1)},
        {'hook': 'free', 'device_id': 0, 'mem_size': 512, 'mem_ptr': ptr1, 'pmem_id': hex(pmem1)},
        {'hook': 'malloc', 'device_id': 0, 'size': 1, 'mem_size': 512, 'mem_ptr': ptr2,
         'pmem_id': hex(pmem2)},
        {'hook': 'free', 'device_id': 0, 'mem_size': 512, 'mem_ptr': ptr2, 'pmem_id': hex(pmem2)}]
    # the reference's layout: no spaces, keys in its order
    assert lines[0].startswith('{"hook":"alloc","device_id":0,"mem_size":512,"mem_ptr":')
    assert memory_hooks.debug_print.DebugPrintHook is memory_hooks.DebugPrintHook


def test_line_profile_hook_reports_the_call_tree(monkeypatch):
    import io
    import re
    from cupy_amd.cuda import memory_hooks
    pool = _fake_pool(monkeypatch)
    p = pool.malloc(1000)
    del p
    hook = memory_hooks.LineProfileHook()
    with hook:
        p1 = pool.malloc(1000)      # served from the block freed above
        p2 = pool.malloc(2000)      # needs memory from the device
    del p1, p2
    f = io.StringIO()
    hook.print_report(file=f)
    text = f.getvalue()
    assert re.search(r'\A_root \(3\.00KB, 2\.00KB\)', text)
    assert re.search(r'.*\.py:[0-9]+:test_line_profile_hook_reports_the_call_tree '
                     r'\(1\.00KB, 0\.00B\)', text)
    assert re.search(r'.*\.py:[0-9]+:test_line_profile_hook_reports_the_call_tree '
                     r'\(2\.00KB, 2\.00KB\)', text)
    for depth in (1, 2):
        hook = memory_hooks.LineProfileHook(max_depth=depth)
        with hook:
            p = pool.malloc(1000)
        del p
        f = io.StringIO()
        hook.print_report(file=f)
        assert len(f.getvalue().split('\n')) == depth + 1
