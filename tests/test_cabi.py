"""The C-ABI library loads and exports every symbol ``include/mi355rt.h``
declares (no compute calls here)."""
import ctypes
import os
import re

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared_symbols():
    text = open(os.path.join(ROOT, 'include', 'mi355rt.h')).read()
    text = re.sub(r'/\*.*?\*/', '', text, flags=re.S)
    names = re.findall(r'\b(rt_[a-z0-9_]+)\s*\(', text)
    # typedef'd callback types are not exports
    return sorted(set(n for n in names if not n.endswith('_fn')))


def test_header_symbols_are_exported():
    from cupy_amd import _rt
    lib = ctypes.CDLL(_rt.LIB_PATH)
    declared = _declared_symbols()
    assert len(declared) >= 45
    for name in declared:
        assert hasattr(lib, name), 'missing export ' + name


def test_binding_covers_header():
    from cupy_amd import _rt
    assert sorted(_rt.EXPORTED_SYMBOLS) == _declared_symbols()


def test_status_strings():
    from cupy_amd import _rt
    assert _rt.lib.rt_error_string(0) == b'success'
    assert b'memory' in _rt.lib.rt_error_string(_rt.RT_ERR_POOL_OOM)
    assert _rt.lib.rt_error_name(2) == b'hipErrorOutOfMemory'
    assert _rt.lib.rt_pool_round_size(1) == 512
    assert _rt.lib.rt_pool_round_size(512) == 512
    assert _rt.lib.rt_pool_round_size(513) == 1024


def test_invalid_arguments_are_reported_not_crashed():
    from cupy_amd import _rt
    assert _rt.lib.rt_launch(None, 1, 1, 1, 1, 1, 1, 0, None, None) == _rt.RT_ERR_INVALID
    assert _rt.lib.rt_pool_malloc(None, 16, 0, None) == _rt.RT_ERR_INVALID
    assert b'null' in _rt.lib.rt_last_error_string()
    assert _rt.lib.rt_launch_cooperative(None, 1, 1, 1, 1, 1, 1, 0, None, None) == _rt.RT_ERR_INVALID
    assert _rt.lib.rt_func_set_attribute(None, 8, 1024) == _rt.RT_ERR_INVALID
    fake = ctypes.addressof((ctypes.c_ubyte * 8)())
    assert _rt.lib.rt_launch_cooperative(fake, 0, 1, 1, 1, 1, 1, 0, None, None) == _rt.RT_ERR_INVALID
    # only the two attributes the reference can set (cupy/_core/raw.pyx:226-287)
    assert _rt.lib.rt_func_set_attribute(fake, 4, 1) == _rt.RT_ERR_INVALID
    assert b'cannot be set' in _rt.lib.rt_last_error_string()
    major = ctypes.c_int(0)
    minor = ctypes.c_int(0)
    assert _rt.lib.rt_rtc_version(ctypes.byref(major), ctypes.byref(minor)) == 0
    assert major.value >= 7 or major.value == 9 or major.value > 0


def test_scratch_launch_refuses_a_pointer_slot_outside_the_argument_block():
    """Every check of ``rt_launch_packed_scratch`` comes before anything
    touches a device, so the refusals can be seen without one.  An offset near
    the top of ``size_t`` must not wrap the bounds check around."""
    from cupy_amd import _rt
    args = (ctypes.c_ubyte * 64)()
    fn = ctypes.addressof(args)         # never called: the checks refuse first
    launch = _rt.lib.rt_launch_packed_scratch
    for offset in (2 ** 64 - 8, 2 ** 64 - 16, 64, 60, 57, 2 ** 63):
        assert launch(fn, 1, 1, 1, 64, 1, 1, 0, None, args, 64, offset, 16) == _rt.RT_ERR_INVALID
        assert b'pointer slot' in _rt.lib.rt_last_error_string()
    assert launch(fn, 1, 1, 1, 64, 1, 1, 0, None, args, 4, 0, 16) == _rt.RT_ERR_INVALID
    assert launch(fn, 1, 1, 1, 64, 1, 1, 0, None, args, 64, 0,
                  _rt.RT_SCRATCH_MAX_BYTES + 1) == _rt.RT_ERR_INVALID
    assert launch(fn, 1, 1, 1, 64, 1, 1, 0, None, args, 8192, 0, 16) == _rt.RT_ERR_INVALID
