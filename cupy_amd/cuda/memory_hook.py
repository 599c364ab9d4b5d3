"""Hooks around device-memory allocation.

Counterpart of the reference's cupy/cuda/memory_hook.pyx (``MemoryHook`` :35-180,
thread-local registry :4-32).  A hook registered with ``with hook:`` is called

* ``alloc_preprocess / alloc_postprocess`` around every allocation the pool
  makes on the device (cupy/cuda/memory.pyx:1303-1321),
* ``malloc_preprocess / malloc_postprocess`` around every request served by
  the pool (:1323-1352),
* ``free_preprocess / free_postprocess`` around every block handed back to the
  pool (:1012-1036),

each with keyword arguments only.  Hooks are per thread.
"""
import threading

_thread_local = threading.local()
# number of hooks registered in any thread: lets the allocation path skip the
# thread-local lookup when nobody listens
_n_registered = 0
_count_lock = threading.Lock()


def _has_memory_hooks():
    return _n_registered > 0


def get_memory_hooks():
    """The calling thread's registered hooks (name -> hook), in registration
    order."""
    hooks = getattr(_thread_local, 'memory_hooks', None)
    if hooks is None:
        hooks = _thread_local.memory_hooks = {}
    return hooks


class MemoryHook:
    """Base class of memory hooks; override the callbacks of interest."""

    name = 'MemoryHook'

    def __enter__(self):
        global _n_registered
        hooks = get_memory_hooks()
        if self.name in hooks:
            raise KeyError('memory hook %s already exists' % self.name)
        hooks[self.name] = self
        with _count_lock:
            _n_registered += 1
        return self

    def __exit__(self, *_):
        global _n_registered
        del get_memory_hooks()[self.name]
        with _count_lock:
            _n_registered -= 1

    def alloc_preprocess(self, **kwargs):
        """Before the pool allocates on the device.
        Keyword args: device_id, mem_size (rounded size)."""

    def alloc_postprocess(self, **kwargs):
        """After the pool allocated on the device.
        Keyword args: device_id, mem_size, mem_ptr (0 if it failed)."""

    def malloc_preprocess(self, **kwargs):
        """Before a request is served by the pool.
        Keyword args: device_id, size (requested), mem_size (rounded)."""

    def malloc_postprocess(self, **kwargs):
        """After a request was served by the pool.
        Keyword args: device_id, size, mem_size, mem_ptr (0 if it failed),
        pmem_id (identity of the block object)."""

    def free_preprocess(self, **kwargs):
        """Before a block goes back to the pool.
        Keyword args: device_id, mem_size, mem_ptr, pmem_id."""

    def free_postprocess(self, **kwargs):
        """After a block went back to the pool.  Same keyword args."""
