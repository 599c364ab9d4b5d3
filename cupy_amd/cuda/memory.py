"""Device memory: allocations, pointers and the caching pool.

Python face of the native pool in ``csrc/pool.cpp``.  API and behaviour follow
the reference's ``cupy/cuda/memory.pyx`` (Memory :105-124, MemoryPointer
:458-765, PooledMemory :943-1038, SingleDeviceMemoryPool :1217-1563,
MemoryPool :1566-1737, allocator registry :892-940).
"""
import contextlib
import ctypes
import gc
import threading
import warnings

from cupy_amd import _dryrun
from cupy_amd import _rt
from cupy_amd.cuda import _giveup
from cupy_amd.cuda import device as _device
from cupy_amd.cuda import stream as _stream
from cupy_amd.cuda import memory_hook as _memory_hook

_STREAM_PER_THREAD = _stream.STREAM_PER_THREAD

_allocation_unit_size = 512


class OutOfMemoryError(MemoryError):
    """Raised when the pool (or its limit) cannot satisfy a request
    (reference: memory.pyx:55-81)."""

    def __init__(self, size, total, limit=0):
        self._size, self._total, self._limit = size, total, limit
        if limit == 0:
            msg = ('Out of memory allocating {:,} bytes '
                   '(allocated so far: {:,} bytes).'.format(size, total))
        else:
            msg = ('Out of memory allocating {:,} bytes '
                   '(allocated so far: {:,} bytes, '
                   'limit set to: {:,} bytes).'.format(size, total, limit))
        super().__init__(msg)

    def __reduce__(self):
        return (type(self), (self._size, self._total, self._limit))


class BaseMemory:
    """A piece of device memory: ``ptr``, ``size``, ``device_id``."""
    ptr = 0
    size = 0
    device_id = 0

    def __int__(self):
        return self.ptr

    @property
    def device(self):
        return _device.Device(self.device_id)


class Memory(BaseMemory):
    """An allocation straight from the driver, freed when collected."""

    def __init__(self, size):
        self.size = size
        self.device_id = _device.get_device_id()
        self.ptr = 0
        if size > 0:
            if _dryrun.enabled():
                self.ptr = _dryrun.fake_alloc(size)
            else:
                p = ctypes.c_void_p()
                _rt.check(_rt.lib.rt_malloc(ctypes.byref(p), size))
                self.ptr = p.value or 0

    def __del__(self):
        ptr, self.ptr = getattr(self, 'ptr', 0), 0
        if not ptr or _dryrun is None or _rt is None:     # interpreter shutdown
            return
        if type(self) is Memory and not _dryrun.enabled():
            try:
                _rt.lib.rt_free(ptr)
            except Exception:
                pass


class UnownedMemory(BaseMemory):
    """Memory owned by somebody else (``owner`` is kept alive)."""

    def __init__(self, ptr, size, owner, device_id=-1):
        if device_id < 0:
            device_id = _device.get_device_id()
        self.ptr = ptr
        self.size = size
        self.device_id = device_id
        self._owner = owner


class PooledMemory(BaseMemory):
    """A block handed out by a pool; returns to the pool when collected or on
    ``free()`` (a second ``free()`` does nothing)."""

    def __init__(self, ptr, size, device_id, pool):
        self.ptr = ptr
        self.size = size
        self.device_id = device_id
        # A strong reference to the native pool's holder, not a weak one to
        # the Python pool: the collector clears weak references that are part
        # of a garbage cycle BEFORE it runs the cycle's finalisers, so a block
        # owned by such a cycle would find its pool gone and never return.
        self._pool = pool._native

    def free(self):
        ptr, self.ptr = self.ptr, 0
        if not ptr:
            return
        pool = self._pool
        hooks = _memory_hook.get_memory_hooks() if _memory_hook._has_memory_hooks() else None
        if hooks:
            kw = dict(device_id=self.device_id, mem_size=self.size, mem_ptr=ptr,
                      pmem_id=id(self))
            for hook in list(hooks.values()):
                hook.free_preprocess(**kw)
            try:
                if pool is not None:
                    pool._free(ptr, self.size)
            finally:
                for hook in list(hooks.values()):
                    hook.free_postprocess(**kw)
            return
        if pool is not None:
            pool._free(ptr, self.size)

    def __del__(self):
        try:
            self.free()
        except Exception:
            pass


def _as_host_address(obj):
    if isinstance(obj, int):
        return obj
    if isinstance(obj, ctypes.c_void_p):
        return obj.value or 0
    if hasattr(obj, 'ctypes'):          # numpy array
        return obj.ctypes.data
    return ctypes.cast(obj, ctypes.c_void_p).value or 0


class MemoryPointer:
    """Address inside a ``BaseMemory``: ``ptr == mem.ptr + offset``."""
    __slots__ = ('mem', 'ptr', 'device_id')

    def __init__(self, mem, offset):
        self.mem = mem
        self.ptr = mem.ptr + offset
        self.device_id = mem.device_id

    def __int__(self):
        return self.ptr

    def __repr__(self):
        return '<MemoryPointer 0x%x device=%d mem=%r>' % (
            self.ptr, self.device_id, self.mem)

    @property
    def device(self):
        return _device.Device(self.device_id)

    def __add__(self, offset):
        return MemoryPointer(self.mem, self.ptr - self.mem.ptr + int(offset))

    __radd__ = __add__

    def __iadd__(self, offset):
        self.ptr += int(offset)
        return self

    def __sub__(self, offset):
        return self + (-int(offset))

    def __isub__(self, offset):
        self.ptr -= int(offset)
        return self

    # -- copies ---------------------------------------------------------------
    def copy_from_device(self, src, size):
        if size > 0 and not _dryrun.enabled():
            _rt.check(_rt.lib.rt_memcpy(self.ptr, src.ptr, size, _rt.MEMCPY_D2D))

    def copy_from_device_async(self, src, size, stream=None):
        if size > 0 and not _dryrun.enabled():
            sptr = _stream.get_current_stream_ptr() if stream is None else stream.ptr
            _rt.check(_rt.lib.rt_memcpy_async(
                self.ptr, src.ptr, size, _rt.MEMCPY_D2D, sptr))

    def copy_from_host(self, mem, size):
        if size > 0 and not _dryrun.enabled():
            _rt.check(_rt.lib.rt_memcpy(
                self.ptr, _as_host_address(mem), size, _rt.MEMCPY_H2D))

    def copy_from_host_async(self, mem, size, stream=None):
        if size > 0 and not _dryrun.enabled():
            sptr = _stream.get_current_stream_ptr() if stream is None else stream.ptr
            _rt.check(_rt.lib.rt_memcpy_async(
                self.ptr, _as_host_address(mem), size, _rt.MEMCPY_H2D, sptr))

    def copy_from(self, mem, size):
        if isinstance(mem, MemoryPointer):
            self.copy_from_device(mem, size)
        else:
            self.copy_from_host(mem, size)

    def copy_from_async(self, mem, size, stream=None):
        if isinstance(mem, MemoryPointer):
            self.copy_from_device_async(mem, size, stream)
        else:
            self.copy_from_host_async(mem, size, stream)

    def copy_to_host(self, mem, size):
        if _dryrun.enabled():
            _dryrun.forbid('copying device memory to the host')
        if size > 0:
            _rt.check(_rt.lib.rt_memcpy(
                _as_host_address(mem), self.ptr, size, _rt.MEMCPY_D2H))
            # the copy waited for the kernels before it: a value one of them
            # reported as wrong must not reach the caller
            if _giveup.armed:
                _giveup.poll()

    def copy_to_host_async(self, mem, size, stream=None):
        if _dryrun.enabled():
            _dryrun.forbid('copying device memory to the host')
        if size > 0:
            sptr = _stream.get_current_stream_ptr() if stream is None else stream.ptr
            _rt.check(_rt.lib.rt_memcpy_async(
                _as_host_address(mem), self.ptr, size, _rt.MEMCPY_D2H, sptr))

    def memset(self, value, size):
        if size > 0 and not _dryrun.enabled():
            _rt.check(_rt.lib.rt_memset(self.ptr, value, size))

    def memset_async(self, value, size, stream=None):
        if size > 0 and not _dryrun.enabled():
            sptr = _stream.get_current_stream_ptr() if stream is None else stream.ptr
            _rt.check(_rt.lib.rt_memset_async(self.ptr, value, size, sptr))


def _malloc(size):
    """Plain driver allocation wrapped as a pointer (no pooling)."""
    return MemoryPointer(Memory(size), 0)


def _round_size(size):
    """Rounds up to the pool's 512-byte allocation unit."""
    return (size + _allocation_unit_size - 1) // _allocation_unit_size \
        * _allocation_unit_size


def _parse_limit_string(limit=None):
    """``'1073741824'`` -> size, ``'70.5%'`` -> fraction (value of
    ``CUPY_GPU_MEMORY_LIMIT``)."""
    import os
    if limit is None:
        limit = os.environ.get('CUPY_GPU_MEMORY_LIMIT')
    size = None
    fraction = None
    if limit is not None:
        if limit.endswith('%'):
            fraction = float(limit[:-1]) / 100.0
        else:
            size = int(limit)
    return {'size': size, 'fraction': fraction}


class _NativePool:
    """Owner of one native pool handle and of the callbacks it calls.  Shared by
    the Python pool and every block it handed out, so the native bookkeeping
    lives until the last block has come back."""

    __slots__ = ('handle', 'value', 'callbacks', 'live')

    def __init__(self, alloc_cb, free_cb, live):
        self.live = live
        self.callbacks = (_rt.POOL_ALLOC_FN(alloc_cb), _rt.POOL_FREE_FN(free_cb))
        self.handle = ctypes.c_void_p()
        self.value = 0
        _rt.check(_rt.lib.rt_pool_create_with_allocator(
            ctypes.byref(self.handle), self.callbacks[0], self.callbacks[1], None))
        self.value = self.handle.value or 0      # the handle as the integer the extension takes

    def _free(self, ptr, size):
        value = self.value
        if value:
            _rt.hot.pool_free(value, ptr)

    def __del__(self):
        handle, self.handle = getattr(self, 'handle', None), None
        self.value = 0
        if handle:
            try:
                _rt.lib.rt_pool_destroy(handle)
            except Exception:
                pass


class SingleDeviceMemoryPool:
    """Caching pool of one device.

    ``allocator`` is a callable ``size -> MemoryPointer`` used to obtain fresh
    memory; by default the native core calls ``hipMalloc`` itself.
    """

    def __init__(self, allocator=None):
        self._device_id = _device.get_device_id()
        self._live = {}      # address -> MemoryPointer from a Python allocator
        # Fresh memory always comes through this Python callback (a pool hit
        # never gets here, and a device allocation costs far more than the
        # call): that is where a custom allocator plugs in and where the
        # alloc_* memory hooks are run.
        if allocator is None:
            allocator = _malloc
        live = self._live
        device_id = self._device_id

        def alloc_cb(ctx, size, out):
            hooks = (_memory_hook.get_memory_hooks()
                     if _memory_hook._has_memory_hooks() else None)
            memptr = None
            try:
                if hooks:
                    for hook in list(hooks.values()):
                        hook.alloc_preprocess(device_id=device_id, mem_size=size)
                try:
                    memptr = allocator(size)
                finally:
                    if hooks:
                        for hook in list(hooks.values()):
                            hook.alloc_postprocess(
                                device_id=device_id, mem_size=size,
                                mem_ptr=memptr.ptr if memptr is not None else 0)
            except Exception:
                return 1
            live[memptr.ptr] = memptr
            out[0] = memptr.ptr
            return 0

        def free_cb(ctx, address, size):
            live.pop(address, None)

        self._native = _NativePool(alloc_cb, free_cb, live)
        self._handle = self._native.handle
        self._handle_value = self._native.value
        limit = _parse_limit_string()
        if limit['size'] is not None or limit['fraction'] is not None:
            self.set_limit(**limit)

    # -- allocation -------------------------------------------------------------
    def malloc(self, size):
        if _memory_hook._has_memory_hooks():
            hooks = _memory_hook.get_memory_hooks()
            if hooks:
                rounded = _round_size(size)
                memptr = None
                for hook in list(hooks.values()):
                    hook.malloc_preprocess(device_id=self._device_id, size=size,
                                           mem_size=rounded)
                try:
                    memptr = self._malloc(size)
                finally:
                    for hook in list(hooks.values()):
                        hook.malloc_postprocess(
                            device_id=self._device_id, size=size, mem_size=rounded,
                            mem_ptr=memptr.ptr if memptr is not None else 0,
                            pmem_id=id(memptr.mem) if memptr is not None else 0)
                return memptr
        return self._malloc(size)

    def _malloc(self, size):
        if size == 0:
            return MemoryPointer(Memory(0), 0)
        rounded = _round_size(size)
        stream_ident = _stream.get_current_stream_ptr()
        if stream_ident == _STREAM_PER_THREAD:
            stream_ident = _stream.stream_identifier(stream_ident)
        handle = self._handle_value
        pool_malloc = _rt.hot.pool_malloc
        addr = pool_malloc(handle, rounded, stream_ident)
        if addr < 0:
            if -addr == _rt.RT_ERR_POOL_OOM:
                # Last resort before giving up: collect garbage cycles that may
                # be keeping arrays (and so pool blocks) alive.
                gc.collect()
                addr = pool_malloc(handle, rounded, stream_ident)
                if -addr == _rt.RT_ERR_POOL_OOM:
                    raise OutOfMemoryError(rounded, self.total_bytes(), self.get_limit())
            if addr < 0:
                _rt.check(-addr)
        mem = PooledMemory(addr, rounded, self._device_id, self)
        return MemoryPointer(mem, 0)

    def _free(self, ptr, size):
        self._native._free(ptr, size)

    def free_all_blocks(self, stream=None):
        if stream is None:
            _rt.check(_rt.lib.rt_pool_free_all_blocks(self._handle, 1, 0))
        else:
            _rt.check(_rt.lib.rt_pool_free_all_blocks(
                self._handle, 0, _stream.stream_identifier(stream.ptr)))

    def free_all_free(self):
        warnings.warn('free_all_free is deprecated. Use free_all_blocks instead.',
                      DeprecationWarning)
        self.free_all_blocks()

    # -- statistics ---------------------------------------------------------------
    def _stats(self):
        vals = [ctypes.c_size_t(0) for _ in range(4)]
        _rt.check(_rt.lib.rt_pool_stats(self._handle, *[ctypes.byref(v) for v in vals]))
        return tuple(v.value for v in vals)

    def used_bytes(self):
        return self._stats()[0]

    def free_bytes(self):
        return self._stats()[1]

    def total_bytes(self):
        return self._stats()[2]

    def n_free_blocks(self):
        return self._stats()[3]

    # -- limit -----------------------------------------------------------------------
    def set_limit(self, size=None, fraction=None):
        if size is None:
            if fraction is None:
                size = 0
            else:
                if not 0 <= fraction <= 1:
                    raise ValueError('memory limit fraction out of range: %r' % fraction)
                _, total = _device.Device(self._device_id).mem_info
                size = int(fraction * total)
        else:
            if fraction is not None:
                raise ValueError('size and fraction cannot be specified at one time')
            if size < 0:
                raise ValueError('memory limit size out of range: %r' % size)
        _rt.check(_rt.lib.rt_pool_set_limit(self._handle, int(size)))

    def get_limit(self):
        v = ctypes.c_size_t(0)
        _rt.check(_rt.lib.rt_pool_get_limit(self._handle, ctypes.byref(v)))
        return v.value


class MemoryPool:
    """Pool for every device of the process; one ``SingleDeviceMemoryPool`` per
    device, created on first use."""

    def __init__(self, allocator=None):
        self._allocator = allocator
        self._pools = {}
        self._lock = threading.Lock()

    def _pool(self):
        dev = _device.get_device_id()
        pool = self._pools.get(dev)
        if pool is None:
            with self._lock:
                pool = self._pools.get(dev)
                if pool is None:
                    pool = SingleDeviceMemoryPool(self._allocator)
                    self._pools[dev] = pool
        return pool

    def malloc(self, size):
        pool = self._pools.get(_device.get_device_id())
        if pool is None:
            pool = self._pool()
        if _memory_hook._n_registered > 0:
            return pool.malloc(size)
        return pool._malloc(size)

    def free_all_blocks(self, stream=None):
        self._pool().free_all_blocks(stream)

    def free_all_free(self):
        self._pool().free_all_free()

    def n_free_blocks(self):
        return self._pool().n_free_blocks()

    def used_bytes(self):
        return self._pool().used_bytes()

    def free_bytes(self):
        return self._pool().free_bytes()

    def total_bytes(self):
        return self._pool().total_bytes()

    def set_limit(self, size=None, fraction=None):
        self._pool().set_limit(size, fraction)

    def get_limit(self):
        return self._pool().get_limit()


# -- allocator registry ------------------------------------------------------------
_current_allocator = _malloc
_thread_local = threading.local()


# number of ``static_scratch`` contexts open in any thread: the per-call checks
# look at the thread's own flag only while this is non-zero
_static_scratch_open = 0
_static_scratch_lock = threading.Lock()
_allocator_overrides = 0        # ``using_allocator`` contexts open in any thread


def alloc(size):
    """Allocates through the current allocator (thread-local override first)."""
    if _static_scratch_open and getattr(_thread_local, 'static_scratch', False):
        refuse_allocation('a request for %d bytes' % size)
    if _allocator_overrides:
        return get_allocator()(size)
    return _current_allocator(size)


class static_scratch:
    """Context manager: calls made inside allocate NO device memory.

    For callers that cannot allocate: code under HIP graph capture, tight
    serving loops.  Outputs must be passed in (``out=``), and the one temporary
    a call may use -- the partial results of a reduction split over workgroups
    -- lives in the runtime library's static device array
    (``rt_launch_packed_scratch``, ``RT_SCRATCH_MAX_BYTES``) instead of coming
    from the pool.  The call must have run once before with arguments of the
    same signature (outside the context), so that its kernels are compiled and
    its launches recorded; whatever would allocate raises ``RuntimeError``
    instead.  All calls on one GPU share the one array: calls that overlap in
    time on one GPU (other streams, other threads) race on it."""

    def __enter__(self):
        global _static_scratch_open
        self._prev = getattr(_thread_local, 'static_scratch', False)
        with _static_scratch_lock:
            _static_scratch_open += 1
        _thread_local.static_scratch = True
        return self

    def __exit__(self, *exc):
        global _static_scratch_open
        _thread_local.static_scratch = self._prev
        with _static_scratch_lock:
            _static_scratch_open -= 1


def static_scratch_active():
    return bool(_static_scratch_open) and getattr(_thread_local, 'static_scratch', False)


def refuse_allocation(what):
    raise RuntimeError(
        'static_scratch: %s would allocate device memory; run the call once outside the '
        'context and pass every output with out=' % what)


def set_allocator(allocator=None):
    """Sets the process-wide allocator; ``None`` means plain driver allocation."""
    global _current_allocator
    if getattr(_thread_local, 'allocator', None) is not None:
        raise ValueError('Can\'t change the global allocator inside '
                         '`using_allocator` context manager')
    _current_allocator = _malloc if allocator is None else allocator


def get_allocator():
    override = getattr(_thread_local, 'allocator', None)
    return _current_allocator if override is None else override


@contextlib.contextmanager
def using_allocator(allocator=None):
    """Thread-local, nestable allocator override."""
    if allocator is None:
        allocator = _malloc
    global _allocator_overrides
    previous = getattr(_thread_local, 'allocator', None)
    with _static_scratch_lock:
        _allocator_overrides += 1
    _thread_local.allocator = allocator
    try:
        yield
    finally:
        _thread_local.allocator = previous
        with _static_scratch_lock:
            _allocator_overrides -= 1
