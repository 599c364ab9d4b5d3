"""Compile-check mode for machines without a GPU.

With ``CUPY_AMD_DRYRUN=1`` in the environment the host layer runs end to end
-- argument handling, broadcasting, type resolution, code generation and the
hiprtc compile for gfx950 -- but nothing is executed: device memory is a range
of fake addresses, copies are skipped and every launch is only recorded in
``launches``.  No result is ever produced in this mode (reading an array back
raises), so it cannot stand in for the GPU; it exists to catch code-generation
and compile errors, and to warm the on-disk kernel cache, before a GPU run.
"""
import os
import threading

_enabled = os.environ.get('CUPY_AMD_DRYRUN', '0') not in ('', '0')
_lock = threading.Lock()
_next_address = 0x7f0000000000

# (kernel name, grid, block, shared_mem, packed argument bytes)
launches = []


def enabled():
    return _enabled


def fake_alloc(size):
    global _next_address
    with _lock:
        addr = _next_address
        _next_address += (size + 4095) // 4096 * 4096 + 4096
    return addr


def record_launch(name, grid, block, shared_mem, arg_bytes):
    launches.append((name, tuple(grid), tuple(block), shared_mem, arg_bytes))
    if len(launches) > 4096:
        del launches[:2048]


class DryRunError(RuntimeError):
    pass


def forbid(what):
    raise DryRunError(
        '%s is not available with CUPY_AMD_DRYRUN=1: no kernel has run, '
        'there is no data to return' % what)
