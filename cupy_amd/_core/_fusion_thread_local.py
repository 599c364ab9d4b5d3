"""Thread-local switch telling ufuncs and reductions that a ``cupy.fuse``
trace is in progress (reference: cupy/_core/_fusion_thread_local.pyx:1-46)."""
import threading

thread_local = threading.local()
# recordings in progress in any thread: callers on the launch path test this
# before they look at their own thread's state
recording = 0
_recording_lock = threading.Lock()


def begin_recording():
    global recording
    with _recording_lock:
        recording += 1


def end_recording():
    global recording
    with _recording_lock:
        recording -= 1


def is_fusing():
    return recording != 0 and getattr(thread_local, 'history', None) is not None


def is_old_fusing():
    return recording != 0 and getattr(thread_local, 'is_old_fusing', False)


def call_ufunc(fusion_op, *args, **kwargs):
    return thread_local.history.call_ufunc(fusion_op, *args, **kwargs)


def records_keepdims():
    """True while a function is recorded for a kernel sequence: reductions
    may then keep the reduced axes (the single-kernel tracer cannot)."""
    return getattr(getattr(thread_local, 'history', None), 'split', False)


def call_reduction(fusion_op, *args, **kwargs):
    history = thread_local.history
    if getattr(history, 'split', False):
        return history.call_reduction(fusion_op, *args, **kwargs)
    from cupy_amd._core import fusion
    return fusion._call_reduction(fusion_op, *args, **kwargs)
