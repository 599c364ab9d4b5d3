"""Function-style access to the runtime with the reference's names
(cupy_backends/cuda/api/runtime.pyx): thin forwards onto the C-ABI shim."""
import ctypes

from cupy_amd import _rt
from cupy_amd.cuda import _giveup
from cupy_amd.cuda import device as _device

is_hip = True
HIPError = _rt.HIPError
CUDARuntimeError = _rt.HIPError

memcpyHostToHost = _rt.MEMCPY_H2H
memcpyHostToDevice = _rt.MEMCPY_H2D
memcpyDeviceToHost = _rt.MEMCPY_D2H
memcpyDeviceToDevice = _rt.MEMCPY_D2D
memcpyDefault = _rt.MEMCPY_DEFAULT


def getDeviceCount():
    return _device.get_device_count()


def getDevice():
    return _device.get_device_id()


def setDevice(device):
    _rt.check(_rt.lib.rt_set_device(int(device)))


def getDeviceProperties(device):
    props = dict(_device.get_device_properties(device))
    props['multiProcessorCount'] = props['compute_units']
    props['warpSize'] = props['warp_size']
    props['gcnArchName'] = props['arch']
    props['totalGlobalMem'] = props['total_global_mem']
    return props


def deviceSynchronize():
    _rt.check(_rt.lib.rt_device_synchronize())
    if _giveup.armed:
        _giveup.poll()


def driverGetVersion():
    v = ctypes.c_int(0)
    _rt.check(_rt.lib.rt_driver_version(ctypes.byref(v)))
    return v.value


def runtimeGetVersion():
    v = ctypes.c_int(0)
    _rt.check(_rt.lib.rt_runtime_version(ctypes.byref(v)))
    return v.value


def memGetInfo():
    free = ctypes.c_size_t(0)
    total = ctypes.c_size_t(0)
    _rt.check(_rt.lib.rt_mem_info(ctypes.byref(free), ctypes.byref(total)))
    return free.value, total.value


def malloc(size):
    p = ctypes.c_void_p()
    _rt.check(_rt.lib.rt_malloc(ctypes.byref(p), size))
    return p.value or 0


def free(ptr):
    _rt.check(_rt.lib.rt_free(ptr))


def hostAlloc(size, flags=0):
    p = ctypes.c_void_p()
    _rt.check(_rt.lib.rt_host_alloc(ctypes.byref(p), size))
    return p.value or 0


def freeHost(ptr):
    _rt.check(_rt.lib.rt_host_free(ptr))


def memcpy(dst, src, size, kind):
    _rt.check(_rt.lib.rt_memcpy(dst, src, size, kind))


def memcpyAsync(dst, src, size, kind, stream):
    _rt.check(_rt.lib.rt_memcpy_async(dst, src, size, kind, stream))


def memset(ptr, value, size):
    _rt.check(_rt.lib.rt_memset(ptr, value, size))


def memsetAsync(ptr, value, size, stream):
    _rt.check(_rt.lib.rt_memset_async(ptr, value, size, stream))


def streamSynchronize(stream):
    _rt.check(_rt.lib.rt_stream_synchronize(stream))
    if _giveup.armed:
        _giveup.poll()
