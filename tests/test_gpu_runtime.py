"""The C-ABI shim on a real device, called through ctypes only: memory, copies,
streams, events, compile -> load -> launch, and the pool on hipMalloc."""
import ctypes

import numpy as np
import pytest

from cupy_amd import _rt
import cupy_amd as cp
from cupy_amd.cuda import memory

pytestmark = pytest.mark.gpu
lib = _rt.lib


def test_device_queries():
    n = ctypes.c_int(0)
    assert lib.rt_init() == 0
    assert lib.rt_device_count(ctypes.byref(n)) == 0 and n.value >= 1
    props = _rt.rt_device_props()
    assert lib.rt_device_get_props(0, ctypes.byref(props)) == 0
    assert props.arch.decode().startswith('gfx950')
    assert props.warp_size == 64 and props.compute_units > 0
    free = ctypes.c_size_t(0)
    total = ctypes.c_size_t(0)
    assert lib.rt_mem_info(ctypes.byref(free), ctypes.byref(total)) == 0
    assert 0 < free.value <= total.value


def test_raw_compile_load_launch_round_trip():
    src = (b'extern "C" __global__ void scale(const float* x, float* y, float a, int n) {'
           b' int i = blockIdx.x * blockDim.x + threadIdx.x; if (i < n) y[i] = a * x[i]; }')
    opts = [b'--offload-arch=gfx950', b'-O3']
    c_opts = (ctypes.c_char_p * len(opts))(*opts)
    code = ctypes.c_void_p()
    size = ctypes.c_size_t(0)
    log = ctypes.c_void_p()
    assert lib.rt_compile(src, b'scale.hip', len(opts), c_opts, 0, None, None,
                          ctypes.byref(code), ctypes.byref(size), ctypes.byref(log)) == 0
    mod = ctypes.c_void_p()
    assert lib.rt_module_load(code, ctypes.byref(mod)) == 0
    fn = ctypes.c_void_p()
    assert lib.rt_module_get_function(mod, b'scale', ctypes.byref(fn)) == 0
    missing = ctypes.c_void_p()
    assert lib.rt_module_get_function(mod, b'nope', ctypes.byref(missing)) != 0
    n = 1000
    host = np.arange(n, dtype=np.float32)
    dx = ctypes.c_void_p()
    dy = ctypes.c_void_p()
    assert lib.rt_malloc(ctypes.byref(dx), n * 4) == 0
    assert lib.rt_malloc(ctypes.byref(dy), n * 4) == 0
    assert lib.rt_memcpy(dx, host.ctypes.data, n * 4, _rt.MEMCPY_H2D) == 0
    stream = ctypes.c_void_p()
    assert lib.rt_stream_create(ctypes.byref(stream), 1) == 0
    e0, e1 = ctypes.c_void_p(), ctypes.c_void_p()
    assert lib.rt_event_create(ctypes.byref(e0), 0) == 0
    assert lib.rt_event_create(ctypes.byref(e1), 0) == 0
    # (a) pointer-array launch
    a = ctypes.c_float(3.0)
    cn = ctypes.c_int(n)
    params = (ctypes.c_void_p * 4)(
        ctypes.addressof(dx), ctypes.addressof(dy), ctypes.addressof(a), ctypes.addressof(cn))
    assert lib.rt_event_record(e0, stream) == 0
    assert lib.rt_launch(fn, 4, 1, 1, 256, 1, 1, 0, stream, params) == 0
    assert lib.rt_event_record(e1, stream) == 0
    assert lib.rt_stream_synchronize(stream) == 0
    ms = ctypes.c_float(-1)
    assert lib.rt_event_elapsed_ms(ctypes.byref(ms), e0, e1) == 0 and ms.value >= 0
    out = np.empty(n, np.float32)
    assert lib.rt_memcpy(out.ctypes.data, dy, n * 4, _rt.MEMCPY_D2H) == 0
    assert np.array_equal(out, host * 3)
    # (b) packed argument block
    import struct
    blob = struct.pack('@PPfi', dx.value, dy.value, 0.5, n)
    assert lib.rt_memset_async(dy, 0, n * 4, stream) == 0
    assert lib.rt_launch_packed(fn, 4, 1, 1, 256, 1, 1, 0, stream, blob, len(blob)) == 0
    assert lib.rt_memcpy_async(out.ctypes.data, dy, n * 4, _rt.MEMCPY_D2H, stream) == 0
    assert lib.rt_stream_synchronize(stream) == 0
    assert np.array_equal(out, host * 0.5)
    done = ctypes.c_int(0)
    assert lib.rt_stream_query(stream, ctypes.byref(done)) == 0 and done.value == 1
    occ = ctypes.c_int(0)
    assert lib.rt_occupancy_max_active_blocks(fn, 256, 0, ctypes.byref(occ)) == 0 and occ.value > 0
    regs = ctypes.c_int(0)
    assert lib.rt_func_get_attribute(4, fn, ctypes.byref(regs)) == 0 and regs.value > 0
    for e in (e0, e1):
        assert lib.rt_event_destroy(e) == 0
    assert lib.rt_stream_destroy(stream) == 0
    assert lib.rt_free(dx) == 0 and lib.rt_free(dy) == 0
    assert lib.rt_module_unload(mod) == 0
    lib.rt_free_buffer(code)
    lib.rt_free_buffer(log)


def test_pinned_host_memory_and_async_copy():
    n = 1 << 16
    h = ctypes.c_void_p()
    assert lib.rt_host_alloc(ctypes.byref(h), n) == 0
    buf = (ctypes.c_ubyte * n).from_address(h.value)
    for i in range(0, n, 4096):
        buf[i] = i // 4096
    d = ctypes.c_void_p()
    assert lib.rt_malloc(ctypes.byref(d), n) == 0
    assert lib.rt_memcpy_async(d, h, n, _rt.MEMCPY_H2D, None) == 0
    back = np.zeros(n, np.uint8)
    assert lib.rt_memcpy(back.ctypes.data, d, n, _rt.MEMCPY_D2H) == 0
    assert back[4096 * 3] == 3 and back[1] == 0
    assert lib.rt_free(d) == 0
    assert lib.rt_host_free(h) == 0


def test_pool_on_device_memory():
    pool = memory.SingleDeviceMemoryPool()
    p = pool.malloc(1000)
    assert p.ptr % 512 == 0
    assert pool.used_bytes() == 1024 and pool.total_bytes() == 1024
    ptr = p.ptr
    del p
    assert pool.free_bytes() == 1024
    q = pool.malloc(600)
    assert q.ptr == ptr
    s = cp.cuda.Stream()
    with s:
        r = pool.malloc(600)
        assert r.ptr != ptr
    del q, r
    assert pool.n_free_blocks() == 2
    pool.free_all_blocks()
    assert pool.total_bytes() == 0
    pool.set_limit(size=1 << 20)
    with pytest.raises(memory.OutOfMemoryError):
        pool.malloc(2 << 20)
    pool.set_limit(size=0)


def test_default_pool_backs_arrays_and_reuses_blocks():
    pool = cp.get_default_memory_pool()
    a = cp.zeros((1000,), np.float32)
    ptr = a.data.ptr
    used = pool.used_bytes()
    assert used >= 4096 - 512
    del a
    b = cp.empty((1000,), np.float32)
    assert b.data.ptr == ptr
    assert isinstance(b.data.mem, memory.PooledMemory)
    with cp.cuda.using_allocator(memory._malloc):
        c = cp.empty((10,), np.float32)
        assert not isinstance(c.data.mem, memory.PooledMemory)


def test_streams_events_and_stream_argument():
    x = np.arange(100000, dtype=np.float32)
    s = cp.cuda.Stream(non_blocking=True)
    k = cp.ElementwiseKernel('T x', 'T y', 'y = x + 1', 'plus_one')
    with s:
        d = cp.asarray(x)
        start = cp.cuda.Event()
        stop = cp.cuda.Event()
        start.record()
        y = k(d)
        stop.record()
        stop.synchronize()
        assert cp.cuda.get_elapsed_time(start, stop) >= 0
        assert cp.cuda.get_current_stream() is s
        assert np.array_equal(y.get(), x + 1)
    assert cp.cuda.get_current_stream().ptr == 0
    d = cp.asarray(x)
    y = k(d, stream=s)
    s.synchronize()
    assert s.done
    assert np.array_equal(y.get(), x + 1)


def test_compile_error_surfaces_as_exception():
    k = cp.ElementwiseKernel('T x', 'T y', 'y = undefined_function(x)', 'bad_kernel')
    with pytest.raises(cp.cuda.CompileException) as info:
        k(cp.zeros((4,), np.float32))
    assert 'undefined_function' in str(info.value)


def test_threads_with_their_own_streams():
    """Eight threads, each on its own stream, compile the same cold kernels at
    the same moment, then run elementwise, reduction, fused and scan calls on
    private data while allocating from the shared pool (the scenario of the
    reference's tests/cupy_tests/core_tests/test_multithreading.py:56-155)."""
    import threading
    n_threads = 8
    barrier = threading.Barrier(n_threads)
    kernel = cp.ElementwiseKernel('T x, T y, T a', 'T z', 'z = a * x + y + 7', 'threads_cold_axpy')
    fused = cp.fuse(lambda x, y: cp.sum((x - y) * (x - y), axis=1))
    errors = []
    results = [None] * n_threads

    def worker(k):
        try:
            rng = np.random.default_rng(100 + k)
            stream = cp.cuda.Stream()
            with stream:
                barrier.wait()
                for it in range(12):
                    rows = 50 + 7 * k + it
                    x = rng.standard_normal((rows, 257)).astype(np.float32)
                    y = rng.standard_normal((rows, 257)).astype(np.float32)
                    dx, dy = cp.asarray(x), cp.asarray(y)
                    z = kernel(dx, dy, np.float32(k + 1))
                    s = (dx * dy).sum(axis=0)
                    f = fused(dx, dy)
                    c = cp.cumsum(dx, axis=1)
                    idx = dx.argmax(axis=1)
                    stream.synchronize()
                    assert np.array_equal(z.get(), np.float32(k + 1) * x + y + np.float32(7))
                    np.testing.assert_allclose(s.get(), (x * y).sum(axis=0), rtol=1e-4, atol=1e-4)
                    np.testing.assert_allclose(f.get(), ((x - y) ** 2).sum(axis=1), rtol=1e-4)
                    np.testing.assert_allclose(c.get(), np.cumsum(x, axis=1), rtol=1e-4, atol=1e-4)
                    assert np.array_equal(idx.get(), x.argmax(axis=1))
            results[k] = True
        except Exception as e:          # noqa: BLE001 - reported by the main thread
            errors.append((k, repr(e)))

    threads = [threading.Thread(target=worker, args=(k,)) for k in range(n_threads)]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    assert not errors, errors
    assert all(results)
    # one compiled kernel per input type tuple, however many threads raced for it
    assert len(kernel._cached_codes) == 1


def test_work_on_the_per_thread_default_stream():
    """Kernels, split reductions and scans on ``Stream.ptds`` from two threads
    (reference: cupy/cuda/stream.pyx:494-505; the pool keeps the threads'
    blocks apart, cupy/cuda/memory.pyx:877-889)."""
    import threading
    from cupy_amd.cuda import stream as stream_module
    rng = np.random.default_rng(31)
    h = rng.integers(-50, 50, 1 << 21).astype(np.int32)
    results = {}

    def job(key):
        with cp.cuda.Device(0):
            with cp.cuda.Stream.ptds as s:
                assert cp.cuda.get_current_stream().ptr == stream_module.STREAM_PER_THREAD
                a = cp.asarray(h)
                total = a.sum()
                running = (a * 2).cumsum()
                ptr = a.data.ptr
                s.synchronize()
                results[key] = (int(total), running.get(), ptr)

    job('main')
    t = threading.Thread(target=job, args=('sub',))
    t.start()
    t.join()
    for key in ('main', 'sub'):
        total, running, _ = results[key]
        assert total == int(h.sum())
        assert np.array_equal(running, (h * 2).cumsum())


def test_show_config_on_the_device(capsys):
    cp.show_config()
    text = capsys.readouterr().out
    assert 'Device 0 Name' in text and 'gfx950' in text and 'hipRTC Version' in text
