"""Streams and events (reference: cupy/cuda/stream.pyx:101-186,459-598 and
cupy_backends/cuda/stream.pyx:14-100 for the thread-local current stream)."""
import ctypes
import itertools
import os
import threading

from cupy_amd import _dryrun
from cupy_amd import _rt
from cupy_amd.cuda import _giveup

_tls = threading.local()

# hipStreamLegacy / hipStreamPerThread: handles the runtime itself knows
STREAM_LEGACY = 1
STREAM_PER_THREAD = 2

# CUPY_CUDA_PER_THREAD_DEFAULT_STREAM=1: a thread that has made no stream
# current works on its own default stream instead of the one all threads share
# (reference: cupy_backends/cuda/stream.pyx:10-11,33-44)
_ptds = int(os.environ.get('CUPY_CUDA_PER_THREAD_DEFAULT_STREAM', '0') or '0') != 0
_thread_numbers = itertools.count(1)


def is_ptds_enabled():
    return _ptds


def get_default_stream_ptr():
    """Handle of the default stream (cupy_backends/cuda/stream.pyx:84-94)."""
    return STREAM_PER_THREAD if _ptds else STREAM_LEGACY


def get_current_stream_ptr():
    """Raw handle of the calling thread's current stream (0 = null stream;
    with per-thread default streams switched on, the per-thread stream where
    the thread has made no other stream current)."""
    ptr = getattr(_tls, 'ptr', 0)
    if _ptds and ptr == 0:
        return STREAM_PER_THREAD
    return ptr


def get_current_stream():
    cur = getattr(_tls, 'stream', None)
    if cur is None:
        return Stream.ptds if _ptds else Stream.null
    return cur


def stream_identifier(stream_ptr):
    """What tells the memory of one stream from another's: the handle, except
    for the per-thread default stream, whose one handle stands for a different
    stream in every thread (reference: cupy/cuda/memory.pyx:877-889).  Thread
    numbers are never reused and have the top bit set, which no handle has."""
    if stream_ptr != STREAM_PER_THREAD:
        return stream_ptr
    ident = getattr(_tls, 'ident', None)
    if ident is None:
        ident = _tls.ident = (1 << 63) | next(_thread_numbers)
    return ident


def _set_current(stream):
    _tls.stream = stream
    _tls.ptr = 0 if stream is None else stream.ptr


class Event:
    """hipEvent wrapper; ``disable_timing=True`` makes it a pure marker."""

    def __init__(self, block=False, disable_timing=False, interprocess=False):
        if interprocess:
            raise NotImplementedError('interprocess events are not supported')
        self.ptr = 0
        if _dryrun.enabled():
            return
        p = ctypes.c_void_p()
        _rt.check(_rt.lib.rt_event_create(ctypes.byref(p), int(disable_timing)))
        self.ptr = p.value or 0

    def __del__(self):
        ptr, self.ptr = getattr(self, 'ptr', 0), 0
        if ptr:
            try:
                _rt.lib.rt_event_destroy(ptr)
            except Exception:
                pass

    @property
    def done(self):
        if _dryrun.enabled():
            return True
        d = ctypes.c_int(0)
        _rt.check(_rt.lib.rt_event_query(self.ptr, ctypes.byref(d)))
        return bool(d.value)

    def record(self, stream=None):
        if _dryrun.enabled():
            return
        sptr = get_current_stream_ptr() if stream is None else stream.ptr
        _rt.check(_rt.lib.rt_event_record(self.ptr, sptr))

    def synchronize(self):
        if _dryrun.enabled():
            return
        _rt.check(_rt.lib.rt_event_synchronize(self.ptr))
        # results become visible to the host here: none may be a wrong one
        if _giveup.armed:
            _giveup.poll()


def get_elapsed_time(start_event, end_event):
    """Milliseconds between two recorded events."""
    if _dryrun.enabled():
        return 0.0
    ms = ctypes.c_float(0)
    _rt.check(_rt.lib.rt_event_elapsed_ms(
        ctypes.byref(ms), start_event.ptr, end_event.ptr))
    return ms.value


class Stream:
    """hipStream wrapper.  ``Stream.null`` is the default stream all threads
    share, ``Stream.ptds`` the calling thread's own default stream
    (``hipStreamPerThread``).  Streams are created at the default priority."""

    null = None
    ptds = None

    def __init__(self, null=False, non_blocking=False, ptds=False):
        self._owned = False
        self._prev = []
        self.ptr = 0
        if null:
            return
        if ptds:
            self.ptr = STREAM_PER_THREAD
            return
        if _dryrun.enabled():
            return
        p = ctypes.c_void_p()
        _rt.check(_rt.lib.rt_stream_create(ctypes.byref(p), int(non_blocking)))
        self.ptr = p.value or 0
        self._owned = True

    def __del__(self):
        if getattr(self, '_owned', False) and self.ptr:
            ptr, self.ptr = self.ptr, 0
            try:
                _rt.lib.rt_stream_destroy(ptr)
            except Exception:
                pass

    def __repr__(self):
        return '<Stream %d>' % self.ptr

    def __eq__(self, other):
        return isinstance(other, Stream) and other.ptr == self.ptr

    def __hash__(self):
        return hash(('Stream', self.ptr))

    def use(self):
        _set_current(self)
        return self

    def __enter__(self):
        self._prev.append(getattr(_tls, 'stream', None))
        _set_current(self)
        return self

    def __exit__(self, *exc):
        _set_current(self._prev.pop())

    @property
    def done(self):
        if _dryrun.enabled():
            return True
        d = ctypes.c_int(0)
        _rt.check(_rt.lib.rt_stream_query(self.ptr, ctypes.byref(d)))
        return bool(d.value)

    def synchronize(self):
        if _dryrun.enabled():
            return
        _rt.check(_rt.lib.rt_stream_synchronize(self.ptr))
        # results become visible to the host here: none may be a wrong one
        if _giveup.armed:
            _giveup.poll()

    def record(self, event=None):
        if event is None:
            event = Event(disable_timing=True)
        event.record(self)
        return event

    def wait_event(self, event):
        if _dryrun.enabled():
            return
        _rt.check(_rt.lib.rt_stream_wait_event(self.ptr, event.ptr))


Stream.null = Stream(null=True)
Stream.ptds = Stream(ptds=True)
