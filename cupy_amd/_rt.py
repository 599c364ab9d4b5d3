"""ctypes binding of the C-ABI shim (``include/mi355rt.h``).

This is the only module that touches the shared library.  It plays the role of
the reference's Cython FFI layer (``cupy_backends/cuda/api/driver.pyx``,
``cupy_backends/cuda/api/runtime.pyx``, ``cupy_backends/cuda/libs/nvrtc.pyx``):
a status code comes back from every call and is turned into an exception that
carries ``.status``.

The library is mandatory: there is no fallback path.  If it cannot be loaded
the import fails with an explanation of how to build it.
"""
import ctypes
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, '_lib', 'libmi355rt.so')

RT_ERR_RTC_BASE = 10000
RT_ERR_POOL_OOM = 20001
RT_ERR_INVALID = 20002
RT_SCRATCH_MAX_BYTES = 8 << 20      # size of the library's static scratch array per GPU

MEMCPY_H2H, MEMCPY_H2D, MEMCPY_D2H, MEMCPY_D2D, MEMCPY_DEFAULT = range(5)

hipErrorOutOfMemory = 2
hipErrorNoDevice = 100


class HIPError(RuntimeError):
    """A failed HIP runtime/driver call (reference: ``CUDARuntimeError`` /
    ``CUDADriverError``, cupy_backends/cuda/api/runtime.pyx:104-126,
    driver.pyx:48-64)."""

    def __init__(self, status, detail=None):
        self.status = status
        name = lib.rt_error_name(status).decode()
        msg = lib.rt_error_string(status).decode()
        text = '%s: %s' % (name, msg)
        if detail:
            text += ' [%s]' % detail
        super().__init__(text)

    def __reduce__(self):
        return (type(self), (self.status,))


class HIPRTCError(RuntimeError):
    """A failed hiprtc call (reference: ``NVRTCError``,
    cupy_backends/cuda/libs/nvrtc.pyx:37-49)."""

    def __init__(self, status, detail=None):
        self.status = status
        msg = lib.rt_error_string(status).decode()
        text = '%s (%d)' % (msg, status - RT_ERR_RTC_BASE)
        if detail:
            text += ' [%s]' % detail
        super().__init__(text)

    def __reduce__(self):
        return (type(self), (self.status,))


class rt_device_props(ctypes.Structure):
    _fields_ = [
        ('name', ctypes.c_char * 256),
        ('arch', ctypes.c_char * 64),
        ('compute_units', ctypes.c_int32),
        ('warp_size', ctypes.c_int32),
        ('max_threads_per_block', ctypes.c_int32),
        ('max_threads_per_cu', ctypes.c_int32),
        ('clock_khz', ctypes.c_int32),
        ('memory_clock_khz', ctypes.c_int32),
        ('memory_bus_width', ctypes.c_int32),
        ('l2_cache_bytes', ctypes.c_int32),
        ('shared_mem_per_block', ctypes.c_int64),
        ('total_global_mem', ctypes.c_int64),
    ]


POOL_ALLOC_FN = ctypes.CFUNCTYPE(
    ctypes.c_int, ctypes.c_void_p, ctypes.c_size_t,
    ctypes.POINTER(ctypes.c_uint64))
POOL_FREE_FN = ctypes.CFUNCTYPE(
    None, ctypes.c_void_p, ctypes.c_uint64, ctypes.c_size_t)

_c = ctypes
_vp = _c.c_void_p
_PROTOTYPES = {
    # name: (restype, argtypes)
    'rt_error_string': (_c.c_char_p, [_c.c_int]),
    'rt_error_name': (_c.c_char_p, [_c.c_int]),
    'rt_last_error_string': (_c.c_char_p, []),
    'rt_init': (_c.c_int, []),
    'rt_device_count': (_c.c_int, [_c.POINTER(_c.c_int)]),
    'rt_get_device': (_c.c_int, [_c.POINTER(_c.c_int)]),
    'rt_set_device': (_c.c_int, [_c.c_int]),
    'rt_device_get_props': (_c.c_int, [_c.c_int, _c.POINTER(rt_device_props)]),
    'rt_device_synchronize': (_c.c_int, []),
    'rt_driver_version': (_c.c_int, [_c.POINTER(_c.c_int)]),
    'rt_runtime_version': (_c.c_int, [_c.POINTER(_c.c_int)]),
    'rt_mem_info': (_c.c_int, [_c.POINTER(_c.c_size_t), _c.POINTER(_c.c_size_t)]),
    'rt_rtc_version': (_c.c_int, [_c.POINTER(_c.c_int), _c.POINTER(_c.c_int)]),
    'rt_compile': (_c.c_int, [
        _c.c_char_p, _c.c_char_p, _c.c_int, _c.POINTER(_c.c_char_p),
        _c.c_int, _c.POINTER(_c.c_char_p), _c.POINTER(_c.c_char_p),
        _c.POINTER(_vp), _c.POINTER(_c.c_size_t), _c.POINTER(_vp)]),
    'rt_compile_named': (_c.c_int, [
        _c.c_char_p, _c.c_char_p, _c.c_int, _c.POINTER(_c.c_char_p),
        _c.c_int, _c.POINTER(_c.c_char_p), _c.POINTER(_c.c_char_p),
        _c.c_int, _c.POINTER(_c.c_char_p), _c.POINTER(_vp),
        _c.POINTER(_vp), _c.POINTER(_c.c_size_t), _c.POINTER(_vp)]),
    'rt_free_buffer': (None, [_vp]),
    'rt_module_load': (_c.c_int, [_vp, _c.POINTER(_vp)]),
    'rt_module_unload': (_c.c_int, [_vp]),
    'rt_module_get_function': (_c.c_int, [_vp, _c.c_char_p, _c.POINTER(_vp)]),
    'rt_module_get_global': (_c.c_int, [
        _vp, _c.c_char_p, _c.POINTER(_vp), _c.POINTER(_c.c_size_t)]),
    'rt_func_get_attribute': (_c.c_int, [_c.c_int, _vp, _c.POINTER(_c.c_int)]),
    'rt_occupancy_max_active_blocks': (_c.c_int, [
        _vp, _c.c_int, _c.c_size_t, _c.POINTER(_c.c_int)]),
    'rt_func_set_attribute': (_c.c_int, [_vp, _c.c_int, _c.c_int]),
    'rt_launch': (_c.c_int, [_vp] + [_c.c_uint] * 7 + [_vp, _c.POINTER(_vp)]),
    'rt_launch_cooperative': (_c.c_int, [_vp] + [_c.c_uint] * 7 + [_vp, _c.POINTER(_vp)]),
    'rt_launch_packed': (_c.c_int, [_vp] + [_c.c_uint] * 7 + [_vp, _vp, _c.c_size_t]),
    'rt_launch_packed_timed': (_c.c_int, [_vp] + [_c.c_uint] * 7 + [
        _vp, _vp, _c.c_size_t, _vp, _vp]),
    'rt_launch_packed_scratch': (_c.c_int, [_vp] + [_c.c_uint] * 7 + [
        _vp, _vp, _c.c_size_t, _c.c_size_t, _c.c_size_t]),
    'rt_malloc': (_c.c_int, [_c.POINTER(_vp), _c.c_size_t]),
    'rt_free': (_c.c_int, [_vp]),
    'rt_host_alloc': (_c.c_int, [_c.POINTER(_vp), _c.c_size_t]),
    'rt_host_free': (_c.c_int, [_vp]),
    'rt_memcpy': (_c.c_int, [_vp, _vp, _c.c_size_t, _c.c_int]),
    'rt_memcpy_async': (_c.c_int, [_vp, _vp, _c.c_size_t, _c.c_int, _vp]),
    'rt_memset': (_c.c_int, [_vp, _c.c_int, _c.c_size_t]),
    'rt_memset_async': (_c.c_int, [_vp, _c.c_int, _c.c_size_t, _vp]),
    'rt_stream_create': (_c.c_int, [_c.POINTER(_vp), _c.c_int]),
    'rt_stream_destroy': (_c.c_int, [_vp]),
    'rt_stream_synchronize': (_c.c_int, [_vp]),
    'rt_stream_query': (_c.c_int, [_vp, _c.POINTER(_c.c_int)]),
    'rt_stream_wait_event': (_c.c_int, [_vp, _vp]),
    'rt_event_create': (_c.c_int, [_c.POINTER(_vp), _c.c_int]),
    'rt_event_destroy': (_c.c_int, [_vp]),
    'rt_event_record': (_c.c_int, [_vp, _vp]),
    'rt_event_synchronize': (_c.c_int, [_vp]),
    'rt_event_query': (_c.c_int, [_vp, _c.POINTER(_c.c_int)]),
    'rt_event_elapsed_ms': (_c.c_int, [_c.POINTER(_c.c_float), _vp, _vp]),
    'rt_pool_create': (_c.c_int, [_c.POINTER(_vp)]),
    'rt_pool_create_with_allocator': (_c.c_int, [
        _c.POINTER(_vp), POOL_ALLOC_FN, POOL_FREE_FN, _vp]),
    'rt_pool_destroy': (_c.c_int, [_vp]),
    'rt_pool_malloc': (_c.c_int, [
        _vp, _c.c_size_t, _c.c_uint64, _c.POINTER(_c.c_uint64)]),
    'rt_pool_free': (_c.c_int, [_vp, _c.c_uint64]),
    'rt_pool_free_all_blocks': (_c.c_int, [_vp, _c.c_int, _c.c_uint64]),
    'rt_pool_stats': (_c.c_int, [_vp] + [_c.POINTER(_c.c_size_t)] * 4),
    'rt_pool_set_limit': (_c.c_int, [_vp, _c.c_size_t]),
    'rt_pool_get_limit': (_c.c_int, [_vp, _c.POINTER(_c.c_size_t)]),
    'rt_pool_round_size': (_c.c_size_t, [_c.c_size_t]),
}

EXPORTED_SYMBOLS = tuple(sorted(_PROTOTYPES))


def _load():
    if not os.path.exists(LIB_PATH):
        raise ImportError(
            'cupy_amd: the native runtime shim %s is missing. Build it with '
            '`python -c "import __graft_entry__ as g; g.build()"` from the '
            'repository root (or `python cupy_amd/csrc/build.py`). There is '
            'no fallback path without it.' % LIB_PATH)
    try:
        handle = ctypes.CDLL(LIB_PATH, mode=ctypes.RTLD_GLOBAL)
    except OSError as e:
        raise ImportError(
            'cupy_amd: cannot load %s (%s). ROCm 7 libamdhip64/libhiprtc must '
            'be on the loader path.' % (LIB_PATH, e)) from e
    for name, (restype, argtypes) in _PROTOTYPES.items():
        fn = getattr(handle, name)
        fn.restype = restype
        fn.argtypes = argtypes
    return handle


lib = _load()

HOTPATH_PATH = os.path.join(_HERE, '_lib', '_hotpath.so')


def _load_hotpath():
    """The extension module with the per-launch calls (``launch``, ``replay``,
    ``pool_malloc``, ``pool_free``): callers of ``rt_launch_packed``,
    ``rt_pool_malloc`` and ``rt_pool_free`` that skip ctypes' conversion of
    every argument.  Mandatory like the library it links against."""
    import importlib.machinery
    import importlib.util
    if not os.path.exists(HOTPATH_PATH):
        raise ImportError(
            'cupy_amd: the extension module %s is missing. Build it with '
            '`python -c "import __graft_entry__ as g; g.build()"` from the '
            'repository root (or `python cupy_amd/csrc/build.py`).' % HOTPATH_PATH)
    loader = importlib.machinery.ExtensionFileLoader('_hotpath', HOTPATH_PATH)
    spec = importlib.util.spec_from_loader('_hotpath', loader)
    module = importlib.util.module_from_spec(spec)
    loader.exec_module(module)
    return module


hot = _load_hotpath()


def check(status):
    """Raises the exception matching a non-zero status."""
    if status == 0:
        return
    detail = lib.rt_last_error_string().decode(errors='replace')
    if RT_ERR_RTC_BASE <= status < RT_ERR_POOL_OOM:
        raise HIPRTCError(status, detail)
    raise HIPError(status, detail)
