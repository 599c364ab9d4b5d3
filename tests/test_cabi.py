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
    major = ctypes.c_int(0)
    minor = ctypes.c_int(0)
    assert _rt.lib.rt_rtc_version(ctypes.byref(major), ctypes.byref(minor)) == 0
    assert major.value >= 7 or major.value == 9 or major.value > 0
