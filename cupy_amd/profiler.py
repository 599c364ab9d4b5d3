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
