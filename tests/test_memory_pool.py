"""Pool behaviour with a fake allocator that hands out made-up addresses (the
way the reference tests its pool, tests/cupy_tests/cuda_tests/test_memory.py:
20-36,291-648): rounding, best fit, split, merge, per-stream arenas,
free_all_blocks, limits and the byte counters.  No device memory is touched."""
import threading

import pytest

from cupy_amd.cuda import memory
from cupy_amd.cuda import stream as stream_module


class MockMemory(memory.BaseMemory):
    cur_ptr = 1 << 20

    def __init__(self, size):
        self.ptr = MockMemory.cur_ptr
        MockMemory.cur_ptr += size + (1 << 16)
        self.size = size
        self.device_id = 0


def mock_alloc(size):
    return memory.MemoryPointer(MockMemory(size), 0)


class FakeStream:
    def __init__(self, ptr):
        self.ptr = ptr

    def __enter__(self):
        self._prev = (getattr(stream_module._tls, 'stream', None),
                      getattr(stream_module._tls, 'ptr', 0))
        stream_module._tls.stream = self
        stream_module._tls.ptr = self.ptr
        return self

    def __exit__(self, *exc):
        stream_module._tls.stream, stream_module._tls.ptr = self._prev


@pytest.fixture
def pool(monkeypatch):
    monkeypatch.setattr(memory._device, 'get_device_id', lambda: 0)
    return memory.SingleDeviceMemoryPool(allocator=mock_alloc)


unit = memory._allocation_unit_size
stream = FakeStream(0x1234)
null_stream = FakeStream(0)


def test_round_size():
    assert memory._round_size(unit - 1) == unit
    assert memory._round_size(unit) == unit
    assert memory._round_size(unit + 1) == unit * 2


def test_alloc_distinct(pool):
    p1 = pool.malloc(unit * 4)
    p2 = pool.malloc(unit * 4)
    p3 = pool.malloc(unit * 8)
    assert len({p1.ptr, p2.ptr, p3.ptr}) == 3


def test_alloc_split(pool):
    p = pool.malloc(unit * 4)
    ptr = p.ptr
    del p
    head = pool.malloc(unit * 2)
    tail = pool.malloc(unit * 2)
    assert ptr == head.ptr
    assert ptr + unit * 2 == tail.ptr


def test_alloc_limit(pool):
    pool.set_limit(size=unit * 6)
    p1 = pool.malloc(unit * 5)
    p2 = pool.malloc(unit * 1)
    with pytest.raises(memory.OutOfMemoryError):
        pool.malloc(unit)
    pool.set_limit(size=unit * 7)
    p3 = pool.malloc(unit)
    del p1, p2, p3


def test_alloc_limit_fragmented(pool):
    pool.set_limit(size=unit * 6)
    p1 = pool.malloc(unit * 5)
    del p1
    p2 = pool.malloc(unit * 6)    # the cached 5-unit block is released first
    del p2


def test_free_reuses_block(pool):
    p1 = pool.malloc(unit * 4)
    ptr1 = p1.ptr
    del p1
    p2 = pool.malloc(unit * 4)
    assert ptr1 == p2.ptr


def test_free_is_per_stream(pool):
    p1 = pool.malloc(unit * 4)
    ptr1 = p1.ptr
    del p1
    with stream:
        p2 = pool.malloc(unit * 4)
    assert ptr1 != p2.ptr


def test_free_merge_both_orders(pool):
    p = pool.malloc(unit * 4)
    ptr = p.ptr
    del p
    head = pool.malloc(unit * 2)
    tail = pool.malloc(unit * 2)
    assert ptr == head.ptr
    del tail
    del head
    p = pool.malloc(unit * 4)
    assert ptr == p.ptr
    del p
    head = pool.malloc(unit * 2)
    tail = pool.malloc(unit * 2)
    assert ptr == head.ptr
    del head
    del tail
    p = pool.malloc(unit * 4)
    assert ptr == p.ptr


def test_free_different_size(pool):
    p1 = pool.malloc(unit * 4)
    ptr1 = p1.ptr
    del p1
    p2 = pool.malloc(unit * 8)
    assert ptr1 != p2.ptr


def test_best_fit_takes_smallest_block_that_fits(pool):
    big = pool.malloc(unit * 8)
    small = pool.malloc(unit * 3)
    big_ptr, small_ptr = big.ptr, small.ptr
    del big, small
    p = pool.malloc(unit * 2)
    assert p.ptr == small_ptr
    q = pool.malloc(unit * 5)
    assert q.ptr == big_ptr


def test_free_all_blocks(pool):
    p1 = pool.malloc(unit * 4)
    ptr1 = p1.ptr
    del p1
    pool.free_all_blocks()
    p2 = pool.malloc(unit * 4)
    assert ptr1 != p2.ptr


def test_free_all_blocks_keeps_split_blocks(pool):
    p = pool.malloc(unit * 4)
    del p
    head = pool.malloc(unit * 2)
    tail = pool.malloc(unit * 2)
    tailptr = tail.ptr
    del tail
    pool.free_all_blocks()
    p = pool.malloc(unit * 2)
    assert tailptr == p.ptr
    del head


def test_free_all_blocks_of_one_stream(pool):
    p1 = pool.malloc(unit * 4)
    ptr1 = p1.ptr
    del p1
    with stream:
        p2 = pool.malloc(unit * 4)
        ptr2 = p2.ptr
        del p2
    pool.free_all_blocks(stream=null_stream)
    p3 = pool.malloc(unit * 4)
    assert ptr1 != p3.ptr and ptr2 != p3.ptr
    with stream:
        p4 = pool.malloc(unit * 4)
        assert ptr1 != p4.ptr and ptr2 == p4.ptr


def test_free_all_blocks_all_streams(pool):
    p1 = pool.malloc(unit * 4)
    ptr1 = p1.ptr
    del p1
    with stream:
        p2 = pool.malloc(unit * 4)
        ptr2 = p2.ptr
        del p2
    pool.free_all_blocks()
    p3 = pool.malloc(unit * 4)
    assert ptr1 != p3.ptr and ptr2 != p3.ptr
    with stream:
        p4 = pool.malloc(unit * 4)
        assert ptr1 != p4.ptr and ptr2 != p4.ptr


def test_free_all_free_is_deprecated(pool):
    p1 = pool.malloc(unit * 4)
    del p1
    with pytest.warns(DeprecationWarning):
        pool.free_all_free()
    assert pool.n_free_blocks() == 0


def test_byte_counters(pool):
    p1 = pool.malloc(unit * 2)
    assert (pool.used_bytes(), pool.free_bytes(), pool.total_bytes()) == (unit * 2, 0, unit * 2)
    p2 = pool.malloc(unit * 4)
    assert (pool.used_bytes(), pool.free_bytes(), pool.total_bytes()) == (unit * 6, 0, unit * 6)
    del p2
    assert (pool.used_bytes(), pool.free_bytes(), pool.total_bytes()) == (unit * 2, unit * 4, unit * 6)
    del p1
    assert (pool.used_bytes(), pool.free_bytes(), pool.total_bytes()) == (0, unit * 6, unit * 6)
    p3 = pool.malloc(unit * 1)
    assert (pool.used_bytes(), pool.free_bytes(), pool.total_bytes()) == (unit, unit * 5, unit * 6)
    assert pool.used_bytes() + pool.free_bytes() == pool.total_bytes()
    del p3
    pool.free_all_blocks()
    assert pool.total_bytes() == 0


def test_counters_across_streams(pool):
    p1 = pool.malloc(unit * 4)
    del p1
    with stream:
        p2 = pool.malloc(unit * 2)
    assert pool.used_bytes() == unit * 2
    assert pool.free_bytes() == unit * 4
    assert pool.total_bytes() == unit * 6
    del p2


def test_limit_api(pool, monkeypatch):
    assert pool.get_limit() == 0
    pool.set_limit(size=1024)
    assert pool.get_limit() == 1024
    pool.set_limit(size=2 ** 33)
    assert pool.get_limit() == 2 ** 33
    pool.set_limit(size=0)
    assert pool.get_limit() == 0
    with pytest.raises(ValueError):
        pool.set_limit(size=-1)
    with pytest.raises(ValueError):
        pool.set_limit(size=1, fraction=0.5)
    total = 288 << 30
    monkeypatch.setattr(memory._device.Device, 'mem_info', property(lambda self: (total, total)))
    pool.set_limit(fraction=0)
    assert pool.get_limit() == 0
    pool.set_limit(fraction=0.5)
    assert pool.get_limit() == total * 0.5
    pool.set_limit(fraction=1.0)
    assert pool.get_limit() == total
    for bad in (-1, 1.1):
        with pytest.raises(ValueError):
            pool.set_limit(fraction=bad)


def test_parse_limit_string(golden):
    for text, size, fraction in golden['limit_strings']:
        got = memory._parse_limit_string(text)
        assert got['size'] == size and got['fraction'] == fraction


def test_zero_size_and_double_free(pool):
    mem = pool.malloc(0).mem
    assert isinstance(mem, memory.Memory) and not isinstance(mem, memory.PooledMemory)
    mem = pool.malloc(1).mem
    assert isinstance(mem, memory.PooledMemory)
    assert pool.n_free_blocks() == 0
    mem.free()
    mem.free()
    assert pool.n_free_blocks() == 1
    pool.free_all_blocks()
    assert pool.n_free_blocks() == 0


def test_out_of_memory_error_message():
    e = memory.OutOfMemoryError(1024, 4096, 8192)
    assert '1,024' in str(e) and '8,192' in str(e)
    import pickle
    assert str(pickle.loads(pickle.dumps(e))) == str(e)


def test_allocator_registry():
    calls = []

    def my_alloc(size):
        calls.append(size)
        return mock_alloc(size)

    old = memory.get_allocator()
    try:
        memory.set_allocator(my_alloc)
        memory.alloc(100)
        assert calls == [100]
        with memory.using_allocator(mock_alloc):
            memory.alloc(50)
            assert calls == [100]
            with pytest.raises(ValueError):
                memory.set_allocator(my_alloc)
            with memory.using_allocator(my_alloc):
                memory.alloc(7)
            assert calls == [100, 7]
            assert memory.get_allocator() is mock_alloc
        assert memory.get_allocator() is my_alloc
    finally:
        memory.set_allocator(old)


def test_using_allocator_is_thread_local():
    seen = {}

    def worker():
        seen['other'] = memory.get_allocator()

    with memory.using_allocator(mock_alloc):
        t = threading.Thread(target=worker)
        t.start()
        t.join()
        seen['this'] = memory.get_allocator()
    assert seen['this'] is mock_alloc
    assert seen['other'] is not mock_alloc


def test_threads_hammering_one_pool(pool):
    errors = []

    def worker(seed):
        import random
        rnd = random.Random(seed)
        held = []
        try:
            for _ in range(300):
                if held and rnd.random() < 0.5:
                    held.pop(rnd.randrange(len(held)))
                else:
                    held.append(pool.malloc(unit * rnd.randint(1, 8)))
        except Exception as e:       # pragma: no cover
            errors.append(e)

    threads = [threading.Thread(target=worker, args=(i,)) for i in range(8)]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    assert not errors
    assert pool.used_bytes() == 0
    assert pool.used_bytes() + pool.free_bytes() == pool.total_bytes()


def _run_with_deadline(fn, seconds=20):
    """Runs ``fn`` in a thread of its own: a pool that locks itself up fails
    the test instead of wedging the whole run."""
    result = {}

    def body():
        try:
            result['value'] = fn()
        except BaseException as e:      # pragma: no cover
            result['error'] = e

    t = threading.Thread(target=body, daemon=True)
    t.start()
    t.join(seconds)
    assert not t.is_alive(), 'the pool did not return (self-deadlock)'
    if 'error' in result:
        raise result['error']
    return result.get('value')


def test_allocator_may_free_into_the_same_pool(monkeypatch):
    # The allocator callback runs arbitrary code; here it drops the last
    # reference to another block of the very pool that is calling it.
    monkeypatch.setattr(memory._device, 'get_device_id', lambda: 0)
    held = []

    def alloc(size):
        if held:
            held.pop()          # PooledMemory.__del__ -> rt_pool_free
        return mock_alloc(size)

    pool = memory.SingleDeviceMemoryPool(allocator=alloc)

    def scenario():
        held.append(pool.malloc(unit * 2))
        big = pool.malloc(unit * 64)     # cache miss -> callback -> free
        return big.ptr, pool.used_bytes(), pool.n_free_blocks()

    ptr, used, nfree = _run_with_deadline(scenario)
    assert ptr
    assert not held
    assert used == unit * 64
    assert nfree == 1


def test_gc_inside_the_allocator_callback(monkeypatch):
    # A collector pass that starts inside the callback and finalises a
    # PooledMemory owned by a garbage cycle re-enters the pool on the same
    # thread.
    import gc
    monkeypatch.setattr(memory._device, 'get_device_id', lambda: 0)

    def alloc(size):
        gc.collect()
        return mock_alloc(size)

    pool = memory.SingleDeviceMemoryPool(allocator=alloc)

    class Node:
        pass

    def scenario():
        for k in range(4):
            a, b = Node(), Node()
            a.other, b.other = b, a
            a.block = pool.malloc(unit * (k + 1))
            del a, b                         # a cycle that owns a pool block
            pool.malloc(unit * (100 + k))    # miss -> callback -> gc -> free
        gc.collect()
        return pool.used_bytes()

    gc.disable()
    try:
        used = _run_with_deadline(scenario)
    finally:
        gc.enable()
    assert used == 0
    assert pool.used_bytes() + pool.free_bytes() == pool.total_bytes()


def test_hook_may_query_the_pool_from_the_callback(monkeypatch):
    from cupy_amd.cuda import memory_hook
    monkeypatch.setattr(memory._device, 'get_device_id', lambda: 0)
    pool = memory.SingleDeviceMemoryPool(allocator=mock_alloc)
    seen = []

    class Hook(memory_hook.MemoryHook):
        name = 'QueryHook'

        def alloc_preprocess(self, **kwargs):
            seen.append(pool.used_bytes())

        def alloc_postprocess(self, **kwargs):
            seen.append(pool.total_bytes())

    def scenario():
        with Hook():
            p = pool.malloc(unit * 3)
        return p.ptr

    assert _run_with_deadline(scenario)
    assert seen == [0, 0]


def test_slow_allocator_calls_overlap(monkeypatch):
    # Eight threads miss the cache at the same time; the allocator takes
    # 0.2 s.  With the pool's lock held across the callback this would take
    # 8 x 0.2 s and never show two calls in flight.
    import time
    monkeypatch.setattr(memory._device, 'get_device_id', lambda: 0)
    state = {'now': 0, 'peak': 0}
    guard = threading.Lock()

    def alloc(size):
        with guard:
            state['now'] += 1
            state['peak'] = max(state['peak'], state['now'])
        time.sleep(0.2)
        with guard:
            state['now'] -= 1
        return mock_alloc(size)

    pool = memory.SingleDeviceMemoryPool(allocator=alloc)
    start = threading.Barrier(8)
    blocks = []

    def worker(k):
        start.wait()
        blocks.append(pool.malloc(unit * (k + 1)))

    def scenario():
        threads = [threading.Thread(target=worker, args=(k,)) for k in range(8)]
        t0 = time.perf_counter()
        for t in threads:
            t.start()
        for t in threads:
            t.join()
        return time.perf_counter() - t0

    elapsed = _run_with_deadline(scenario)
    assert len({b.ptr for b in blocks}) == 8
    assert state['peak'] >= 2
    assert elapsed < 1.2
    assert pool.used_bytes() == sum(unit * (k + 1) for k in range(8))


def test_limit_holds_for_requests_side_by_side(monkeypatch):
    import time
    monkeypatch.setattr(memory._device, 'get_device_id', lambda: 0)

    def alloc(size):
        time.sleep(0.05)
        return mock_alloc(size)

    pool = memory.SingleDeviceMemoryPool(allocator=alloc)
    pool.set_limit(size=unit * 10)
    start = threading.Barrier(4)
    got, refused = [], []

    def worker():
        start.wait()
        try:
            got.append(pool.malloc(unit * 4))
        except memory.OutOfMemoryError:
            refused.append(1)

    def scenario():
        threads = [threading.Thread(target=worker) for _ in range(4)]
        for t in threads:
            t.start()
        for t in threads:
            t.join()

    _run_with_deadline(scenario)
    assert len(got) == 2 and len(refused) == 2
    assert pool.total_bytes() <= unit * 10


# ---- per-thread default stream (reference: cupy/cuda/memory.pyx:877-889 and
# tests/cupy_tests/cuda_tests/test_memory.py:866-926) ---------------------------

def _reuse_between_threads(pool, stream_main, stream_sub):
    """A block allocated and freed under ``stream_main`` in this thread, then
    one of the same size under ``stream_sub`` in another thread: both
    addresses."""
    seen = {}

    def job(key, s):
        with s:
            p = pool.malloc(unit * 4)
            seen[key] = p.ptr
            del p

    job('main', stream_main)
    t = threading.Thread(target=job, args=('sub', stream_sub), daemon=True)
    t.start()
    t.join()
    return seen['main'], seen['sub']


def test_reuse_between_threads_on_the_null_stream(pool):
    main_ptr, sub_ptr = _reuse_between_threads(pool, FakeStream(0), FakeStream(0))
    assert main_ptr == sub_ptr


def test_reuse_between_threads_on_the_same_stream(pool):
    main_ptr, sub_ptr = _reuse_between_threads(pool, FakeStream(0x77), FakeStream(0x77))
    assert main_ptr == sub_ptr


def test_no_reuse_between_threads_on_different_streams(pool):
    main_ptr, sub_ptr = _reuse_between_threads(pool, FakeStream(0x77), FakeStream(0x78))
    assert main_ptr != sub_ptr


def test_no_reuse_between_threads_on_the_per_thread_default_stream(pool):
    """One handle, another stream in every thread: the arenas are kept apart
    by thread."""
    ptds = stream_module.Stream.ptds
    assert ptds.ptr == stream_module.STREAM_PER_THREAD
    main_ptr, sub_ptr = _reuse_between_threads(pool, ptds, ptds)
    assert main_ptr != sub_ptr
    # ... and the same thread does get its block back
    with ptds:
        p = pool.malloc(unit * 4)
        assert p.ptr == main_ptr
        del p
        # free_all_blocks(stream=Stream.ptds) means this thread's arena
        assert pool.n_free_blocks() == 2
        pool.free_all_blocks(stream=ptds)
        assert pool.n_free_blocks() == 1


def test_thread_identifiers_of_the_per_thread_stream():
    ident = stream_module.stream_identifier
    assert ident(0) == 0 and ident(0x1234) == 0x1234
    mine = ident(stream_module.STREAM_PER_THREAD)
    assert mine == ident(stream_module.STREAM_PER_THREAD) and mine >> 63 == 1
    other = []
    t = threading.Thread(target=lambda: other.append(ident(stream_module.STREAM_PER_THREAD)))
    t.start()
    t.join()
    assert other[0] != mine and other[0] >> 63 == 1


def test_default_stream_follows_the_environment_switch(monkeypatch):
    """CUPY_CUDA_PER_THREAD_DEFAULT_STREAM=1 makes the per-thread stream the
    one a thread works on until it chooses another (reference:
    cupy_backends/cuda/stream.pyx:33-44,84-94; cupy/cuda/stream.pyx:74-75)."""
    S = stream_module.Stream
    assert stream_module.get_current_stream() is S.null
    assert stream_module.get_default_stream_ptr() == stream_module.STREAM_LEGACY
    monkeypatch.setattr(stream_module, '_ptds', True)
    assert stream_module.is_ptds_enabled()
    assert stream_module.get_current_stream_ptr() == stream_module.STREAM_PER_THREAD
    assert stream_module.get_current_stream() is S.ptds
    assert stream_module.get_default_stream_ptr() == stream_module.STREAM_PER_THREAD
    with FakeStream(0x99):
        assert stream_module.get_current_stream_ptr() == 0x99
    assert stream_module.get_current_stream_ptr() == stream_module.STREAM_PER_THREAD


def test_stream_singletons_compare_like_the_reference():
    """(tests/cupy_tests/cuda_tests/test_stream.py:32-51)"""
    S = stream_module.Stream
    assert S(null=True) == S.null and S(ptds=True) == S.ptds
    assert S(ptds=True) == S(ptds=True) and S(ptds=True) != S(null=True)
    assert hash(S(ptds=True)) == hash(S.ptds)
    s = S(ptds=True)
    s.__del__()                      # never destroyed
    assert s.ptr == stream_module.STREAM_PER_THREAD
    with S.ptds:
        assert stream_module.get_current_stream() is S.ptds
        assert stream_module.get_current_stream_ptr() == stream_module.STREAM_PER_THREAD
    assert stream_module.get_current_stream() is S.null
