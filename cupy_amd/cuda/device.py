"""Device handle and properties (reference: cupy/cuda/device.pyx:39,111,125-199)."""
import ctypes
import threading

from cupy_amd import _dryrun
from cupy_amd import _rt
from cupy_amd.cuda import _giveup

_props_cache = {}
_props_lock = threading.Lock()

# What a MI355X reports; used only by the compile-check mode, where no device
# can be queried.
_DRYRUN_PROPS = {
    'name': 'AMD Instinct MI355X (dry run)', 'arch': 'gfx950:sramecc+:xnack-',
    'compute_units': 256, 'warp_size': 64, 'max_threads_per_block': 1024,
    'max_threads_per_cu': 2048, 'clock_khz': 2400000,
    'memory_clock_khz': 2000000, 'memory_bus_width': 8192,
    'l2_cache_bytes': 4 << 20, 'shared_mem_per_block': 65536,
    'total_global_mem': 288 << 30,
}


def get_device_id():
    """Index of the calling thread's current device."""
    if _dryrun.enabled():
        return 0
    dev = _hot_get_device()
    if dev < 0:
        _rt.check(-dev)
    return dev


_hot_get_device = _rt.hot.get_device


def get_device_count():
    if _dryrun.enabled():
        return 1
    n = ctypes.c_int(0)
    _rt.check(_rt.lib.rt_device_count(ctypes.byref(n)))
    return n.value


def is_available():
    if _dryrun.enabled():
        return False
    n = ctypes.c_int(0)
    status = _rt.lib.rt_device_count(ctypes.byref(n))
    return status == 0 and n.value > 0


def get_device_properties(device_id=None):
    """dict of the fields of ``rt_device_props`` for a device (memoised)."""
    if device_id is None:
        device_id = get_device_id()
    props = _props_cache.get(device_id)
    if props is not None:
        return props
    if _dryrun.enabled():
        props = dict(_DRYRUN_PROPS)
    else:
        raw = _rt.rt_device_props()
        _rt.check(_rt.lib.rt_device_get_props(device_id, ctypes.byref(raw)))
        props = {name: getattr(raw, name) for name, _ in raw._fields_}
        props['name'] = props['name'].decode(errors='replace')
        props['arch'] = props['arch'].decode(errors='replace')
    with _props_lock:
        _props_cache[device_id] = props
    return props


def get_compute_units(device_id=None):
    return get_device_properties(device_id)['compute_units']


class Device:
    """A GPU; ``with Device(i):`` makes it current for the block."""

    def __init__(self, device=None):
        if device is None:
            device = get_device_id()
        elif isinstance(device, Device):
            device = device.id
        self.id = int(device)
        self._prev = []

    def __int__(self):
        return self.id

    def __repr__(self):
        return '<CUDA Device %d>' % self.id

    def __eq__(self, other):
        return isinstance(other, Device) and other.id == self.id

    def __hash__(self):
        return hash(('Device', self.id))

    def use(self):
        if not _dryrun.enabled():
            _rt.check(_rt.lib.rt_set_device(self.id))
        return self

    def __enter__(self):
        self._prev.append(get_device_id())
        self.use()
        return self

    def __exit__(self, *exc):
        prev = self._prev.pop()
        if not _dryrun.enabled():
            _rt.check(_rt.lib.rt_set_device(prev))

    def synchronize(self):
        if _dryrun.enabled():
            return
        with self:
            _rt.check(_rt.lib.rt_device_synchronize())
        # results become visible to the host here: none may be a wrong one
        if _giveup.armed:
            _giveup.poll(self.id)

    @property
    def attributes(self):
        return dict(get_device_properties(self.id))

    @property
    def compute_capability(self):
        return get_device_properties(self.id)['arch'].split(':')[0]

    @property
    def mem_info(self):
        if _dryrun.enabled():
            total = _DRYRUN_PROPS['total_global_mem']
            return total, total
        free = ctypes.c_size_t(0)
        total = ctypes.c_size_t(0)
        with self:
            _rt.check(_rt.lib.rt_mem_info(ctypes.byref(free), ctypes.byref(total)))
        return free.value, total.value
