"""Timing helper with the protocol of the reference's
``cupyx.profiler.benchmark`` (cupyx/profiler/_time.py:164-234): warm-up calls,
then per repeat an event is recorded before the call, the host time around the
call is taken with ``perf_counter``, and a second event is recorded and
waited for after it."""
import time

import numpy

from cupy_amd.cuda import stream as _stream


class PerfCaseResult:
    """``cpu_times`` / ``gpu_times``: seconds per repeat."""

    def __init__(self, name, cpu_times, gpu_times):
        self.name = name
        self.cpu_times = numpy.asarray(cpu_times, dtype=numpy.float64)
        self.gpu_times = numpy.asarray(gpu_times, dtype=numpy.float64)

    @staticmethod
    def _fmt(t):
        us = t * 1e6
        return '%9.3f us   +/- %6.3f (min: %9.3f / max: %9.3f) us' % (
            us.mean(), us.std(), us.min(), us.max())

    def __str__(self):
        return '%-20s:    CPU: %s     GPU-0: %s' % (
            self.name, self._fmt(self.cpu_times), self._fmt(self.gpu_times))

    __repr__ = __str__


def benchmark(func, args=(), kwargs={}, n_repeat=10000, *, name=None,
              n_warmup=10, max_duration=float('inf')):
    """Times ``func(*args, **kwargs)`` on the host and on the current stream."""
    if name is None:
        name = getattr(func, '__name__', 'func')
    if not callable(func):
        raise ValueError('`func` should be a callable object.')
    if not isinstance(args, tuple):
        raise ValueError('`args` should be of tuple type.')
    if not isinstance(kwargs, dict):
        raise ValueError('`kwargs` should be of dict type.')
    ev1 = _stream.Event()
    ev2 = _stream.Event()
    for _ in range(n_warmup):
        func(*args, **kwargs)
    ev1.record()
    ev1.synchronize()
    cpu_times = []
    gpu_times = []
    duration = 0.0
    for _ in range(n_repeat):
        ev1.record()
        t1 = time.perf_counter()
        func(*args, **kwargs)
        t2 = time.perf_counter()
        ev2.record()
        ev2.synchronize()
        cpu_times.append(t2 - t1)
        gpu_times.append(_stream.get_elapsed_time(ev1, ev2) * 1e-3)
        duration += time.perf_counter() - t1
        if duration > max_duration:
            break
    return PerfCaseResult(name, cpu_times, gpu_times)


class KernelTimer:
    """Times every kernel launched inside the ``with`` block by the device's
    own clock: each launch carries two events that receive the start and the
    end of that kernel's execution (``rt_launch_packed_timed``), which is the
    duration a profiler's kernel trace shows for the dispatch.  Unlike events
    recorded between calls, this adds no marker to the stream between the
    kernels, so back-to-back launches run as they do untimed.

    While a timer is active every launch takes the full Python launch path
    (recorded calls are replayed launch by launch instead of in one go), so
    host time per call is higher; device time is what is measured.

    ``durations()`` waits for the device and returns ``[(kernel name,
    seconds), ...]`` in launch order.  Not thread-safe: one timer at a time.
    """

    def __init__(self):
        self._launches = []     # (name, start event, stop event)
        self._spare = []

    def _next(self, name):
        pair = self._spare.pop() if self._spare else (_stream.Event(), _stream.Event())
        self._launches.append((name,) + pair)
        return pair

    def __enter__(self):
        from cupy_amd._core import _launch_plan
        from cupy_amd.cuda import function
        if function._kernel_timer is not None:
            raise RuntimeError('another KernelTimer is active')
        self._quick = _launch_plan.use_quick
        _launch_plan.use_quick = False
        function._kernel_timer = self
        return self

    def __exit__(self, *exc):
        from cupy_amd._core import _launch_plan
        from cupy_amd.cuda import function
        function._kernel_timer = None
        _launch_plan.use_quick = self._quick

    def mark(self):
        """Number of launches seen so far (to tell one call's kernels from the
        next call's)."""
        return len(self._launches)

    def durations(self):
        from cupy_amd.cuda import device
        device.Device().synchronize()
        out = []
        for name, start, stop in self._launches:
            out.append((name, _stream.get_elapsed_time(start, stop) * 1e-3))
        self._spare.extend((a, b) for _, a, b in self._launches)
        self._launches = []
        return out
