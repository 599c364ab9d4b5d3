"""Device resources of the hot path: devices, streams, events, memory, the
run-time compiler and kernel launch.  The sub-package keeps the reference's
``cupy.cuda`` name so existing call sites keep working."""
from cupy_amd.cuda import device  # noqa
from cupy_amd.cuda import stream  # noqa
from cupy_amd.cuda import memory  # noqa
from cupy_amd.cuda import memory_hook  # noqa
from cupy_amd.cuda import function  # noqa
from cupy_amd.cuda import compiler  # noqa
from cupy_amd.cuda import runtime  # noqa
from cupy_amd.cuda.device import Device, get_device_id, is_available  # noqa
from cupy_amd.cuda.stream import (  # noqa
    Stream, Event, get_current_stream, get_elapsed_time)
from cupy_amd.cuda.memory import (  # noqa
    alloc, BaseMemory, Memory, UnownedMemory, PooledMemory, MemoryPointer,
    MemoryPool, SingleDeviceMemoryPool, OutOfMemoryError,
    set_allocator, get_allocator, using_allocator)
from cupy_amd.cuda.function import Module, Function  # noqa
from cupy_amd.cuda.compiler import CompileException, compile_with_cache  # noqa
