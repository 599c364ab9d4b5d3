"""Words in pinned host memory through which kernels report that a wait ran out.

Two kernel families wait, inside one launch, for other workgroups of the same
launch: split reductions that finish in their one launch
(``_core/_codegen_reduction._SYNC_HELPERS``) and the one-pass scans
(``_core/_scan._emit_chain*``).  Every such wait is bounded.  A workgroup whose
wait runs out stores 1 into its family's word, runs to its end and leaves a
WRONG result behind.  The reference's reductions and scans are plain launches
that cannot do that (cupy/_core/_reduction.pyx:481-508,
cupy/_core/_routines_math.pyx:160-751), so a set word must never go unnoticed:

* every host call that makes device results visible to the host
  (``ndarray.get``, ``Stream.synchronize``, ``Event.synchronize``,
  ``Device.synchronize``) calls :func:`poll` after the device has finished and
  raises there, before the caller can look at the value;
* the launch paths of both families call :func:`poll` before they use the
  kernels again, and replays of recorded one-launch reductions ask
  :func:`usable` first (``_launch_plan.FastCall.run``);
* once a word was found set the family stays switched off on that device
  (reductions take two launches, scans three passes).

One allocation of 64 bytes per device: word 0 belongs to the reductions, word 1
to the scans.
"""
import ctypes
import threading

from cupy_amd import _dryrun

REDUCTION = 0
SCAN = 1

_MESSAGES = (
    'a reduction on device %d gave up waiting for the partial results of its '
    'workgroups: its result is wrong.  Reductions take two launches from now on.',
    'a one-pass scan on device %d gave up waiting for its neighbouring tiles: its '
    'result is wrong.  Scans use the three-pass kernels from now on.',
)

_lock = threading.Lock()
_base = {}                  # device id -> address of the device's words (0: none)
disabled = (set(), set())   # per family: devices on which a wait ran out
armed = False               # True once any device has its words (guards poll())


def word(dev_id, family):
    """Address of the word kernels of ``family`` on ``dev_id`` report into, or
    0 where launches are only recorded."""
    global armed
    base = _base.get(dev_id)
    if base is None:
        base = 0
        if not _dryrun.enabled():
            from cupy_amd.cuda import runtime
            base = runtime.hostAlloc(64, 0)
            ctypes.memset(base, 0, 64)
        with _lock:
            base = _base.setdefault(dev_id, base)
            if base:
                armed = True
    return base + 4 * family if base else 0


def usable(dev_id, family):
    """False once a kernel of ``family`` gave up on ``dev_id`` -- reported
    already or not.  Reads, raises nothing: for the replay of a recorded call,
    which then leaves the call to the full path (that one raises)."""
    if dev_id in disabled[family]:
        return False
    base = _base.get(dev_id)
    if base and ctypes.c_uint32.from_address(base + 4 * family).value:
        return False
    return True


def poll(dev_id=None):
    """Raises RuntimeError if a kernel on ``dev_id`` (None: any device)
    reported that it gave up; the family is switched off on that device and
    the word cleared, so the report is made once."""
    if not armed:
        return
    for dev, base in list(_base.items()):
        if not base or (dev_id is not None and dev != dev_id):
            continue
        if not ctypes.c_uint64.from_address(base).value:
            continue
        messages = []
        for family in (REDUCTION, SCAN):
            w = ctypes.c_uint32.from_address(base + 4 * family)
            if w.value:
                w.value = 0
                disabled[family].add(dev)
                messages.append(_MESSAGES[family] % dev)
        if messages:
            raise RuntimeError('  '.join(messages))
