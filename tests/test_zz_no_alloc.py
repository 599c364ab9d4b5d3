"""``rt_launch_packed_scratch``: the launch entry point that allocates nothing.

A reduction split over workgroups keeps its partial results in a scratch
buffer.  Through ``rt_launch_packed`` that buffer is an allocation (the Python
layer takes it from the pool); through ``rt_launch_packed_scratch`` it is the
runtime library's static device array.  The same kernels with the same launch
geometry run either way, so the results must agree bit for bit -- on two calls
in a row, the second with a smaller input, whose kernels then find the first
call's partials still lying in the array.
"""
import ctypes
import struct

import numpy as np
import pytest

import cupy_amd as cp
from cupy_amd import _rt
from cupy_amd._core import _launch_plan
from cupy_amd.cuda import function as _function
from cupy_amd.cuda import memory as _memory

pytestmark = pytest.mark.gpu


def _record_launches(fn):
    """Runs ``fn`` and returns what it launched:
    [(function handle, grid, block, shared memory, argument block bytes)]."""
    seen = []
    real = _function.Function.launch_packed

    def spy(self, grid, block, arg_block, shared_mem=0, stream_ptr=None):
        seen.append((self.ptr, tuple(grid), tuple(block), shared_mem, bytes(arg_block)))
        return real(self, grid, block, arg_block, shared_mem, stream_ptr)
    _function.Function.launch_packed = spy
    _launch_plan.use_quick = False       # replays through Function.launch_packed too
    try:
        fn()
    finally:
        _function.Function.launch_packed = real
        _launch_plan.use_quick = True
    return seen


def _recorded_call(fn):
    """The launch record (``FastCall``) behind ``fn()``: made by the first call
    with a signature, replayed by the second."""
    found = []
    real_remember, real_run = _launch_plan.remember, _launch_plan.FastCall.run

    def remember(table, key, fast):
        found.append(fast)
        return real_remember(table, key, fast)

    def run(self, args, stream_ptr=None):
        found.append(self)
        return real_run(self, args, stream_ptr)
    _launch_plan.remember, _launch_plan.FastCall.run = remember, run
    try:
        fn()
        fn()
    finally:
        _launch_plan.remember, _launch_plan.FastCall.run = real_remember, real_run
    assert found
    return found[-1]


@pytest.fixture(autouse=True)
def _reductions_with_scratch_memory():
    """The calls here are reductions that keep partial results in scratch
    memory for a second launch; reductions of this size would otherwise finish
    inside their one launch and use none."""
    from cupy_amd._core import _tuning
    _tuning.set(reduce_finish=False)
    try:
        yield
    finally:
        _tuning.set(reduce_finish=True)


_MARK = 0x1badc0de1badc0de


def _argument_blocks(fast, addresses, temp_address):
    """Packs the argument block of every recorded launch with the given array
    addresses; the temporary's slot gets ``temp_address``.  Returns
    [(function handle, grid, block, shared memory, bytes, byte offset of the
    temporary's pointer or None)]."""
    out = []
    for fn, grid, block, packer, template, ptrs, scalars, shmem in fast.launches:
        assert not scalars
        vals = list(template)
        marked = list(template)
        has_temp = False
        for slot, ref in ptrs:
            if ref < len(addresses):
                vals[slot] = marked[slot] = addresses[ref]
            else:
                vals[slot], marked[slot], has_temp = temp_address, _MARK, True
        offset = None
        if has_temp:
            blob = packer.pack(*marked)
            offset = blob.find(struct.pack('<Q', _MARK))
            assert offset >= 0 and offset % 8 == 0
        out.append((fn.ptr, tuple(grid), tuple(block), shmem, packer.pack(*vals), offset))
    return out


CASES = [
    # (shape, dtype, reduction, second (smaller) shape, the same in NumPy)
    ((1 << 22,), np.float32, lambda a, out: a.sum(out=out), ((1 << 20) + 3,),
     lambda h: h.sum(dtype=np.float64)),
    ((4096, 512), np.float64, lambda a, out: a.sum(axis=0, out=out), (1024, 512),
     lambda h: h.sum(axis=0)),
    ((1 << 21,), np.int32, lambda a, out: a.sum(out=out), (300001,),
     lambda h: h.sum()),
    ((1 << 22,), np.float32, lambda a, out: a.argmax(out=out), ((1 << 20) + 3,),
     lambda h: h.argmax()),
]


@pytest.mark.parametrize('shape,dtype,op,small,numpy_op', CASES)
def test_two_calls_in_a_row_match_the_allocating_entry_point(shape, dtype, op, small, numpy_op):
    rng = np.random.default_rng(41)
    lib = _rt.lib
    stream = cp.cuda.get_current_stream().ptr
    for shp in (shape, small):            # the second call is the smaller one
        h = (rng.standard_normal(shp) * 100).astype(dtype)
        d = cp.asarray(h)
        probe = op(d, None)
        out_ref = cp.empty(probe.shape, probe.dtype)
        out_new = cp.empty(probe.shape, probe.dtype)
        out_py = cp.empty(probe.shape, probe.dtype)
        fast = _recorded_call(lambda: op(d, out_ref))
        assert len(fast.launches) == 2 and len(fast.temps) == 1, \
            'expected a split reduction: partial results, then a combine kernel'
        assert fast.temps[0] <= _rt.RT_SCRATCH_MAX_BYTES
        cp.cuda.Device().synchronize()
        expect = out_ref.get()

        # (a) the existing entry point, straight through ctypes, scratch = rt_malloc
        buf = ctypes.c_void_p()
        _rt.check(lib.rt_malloc(ctypes.byref(buf), fast.temps[0]))
        try:
            out_a = cp.full(probe.shape, 0, probe.dtype)
            for fptr, grid, block, shmem, args, _ in _argument_blocks(
                    fast, [d.data.ptr, out_a.data.ptr], buf.value):
                _rt.check(lib.rt_launch_packed(fptr, *grid, *block, shmem, stream,
                                               args, len(args)))
            cp.cuda.Device().synchronize()
            got_a = out_a.get()
        finally:
            _rt.check(lib.rt_free(buf))

        # (b) the new entry point, straight through ctypes; what stands in the
        # pointer slot must not matter, the library overwrites it
        for fptr, grid, block, shmem, args, offset in _argument_blocks(
                fast, [d.data.ptr, out_new.data.ptr], 0xeeeeeeeeeeeeeeee):
            assert offset is not None
            _rt.check(lib.rt_launch_packed_scratch(
                fptr, *grid, *block, shmem, stream, args, len(args), offset, fast.temps[0]))
        cp.cuda.Device().synchronize()
        got_b = out_new.get()

        # (c) the same through the package: nothing may be allocated inside
        pool = cp.get_default_memory_pool()
        before = (pool.used_bytes(), pool.total_bytes())
        with _memory.static_scratch():
            assert op(d, out_py) is out_py
            after = (pool.used_bytes(), pool.total_bytes())
        cp.cuda.Device().synchronize()
        got_c = out_py.get()
        assert after == before

        assert got_a.tobytes() == expect.tobytes()
        assert got_b.tobytes() == expect.tobytes()
        assert got_c.tobytes() == expect.tobytes()
        # and the result is right in the first place
        want = numpy_op(h)
        if expect.dtype.kind == 'f':
            rtol = 1e-5 if expect.dtype == np.float32 else 1e-12
            scale = np.abs(h).sum(axis=0 if h.ndim == 2 else None, dtype=np.float64)
            assert np.all(np.abs(expect.astype(np.float64) - want) <= rtol * scale)
        else:
            assert np.array_equal(expect, want)


def test_package_path_uses_the_entry_point_and_refuses_to_allocate():
    h = np.arange(1 << 21, dtype=np.float32)
    d = cp.asarray(h)
    out = cp.empty((), np.float32)
    d.sum(out=out)                        # plans and records outside the context
    calls = []
    real = _function.Function.launch_packed_scratch

    def spy(self, *a, **k):
        calls.append(self.name)
        return real(self, *a, **k)
    _function.Function.launch_packed_scratch = spy
    try:
        with _memory.static_scratch():
            d.sum(out=out)
            with pytest.raises(RuntimeError, match='static_scratch'):
                d.sum()                               # would allocate the output
            with pytest.raises(RuntimeError, match='static_scratch'):
                cp.empty((4,), np.float32)
            other = d[: (1 << 20) + 5]
            with pytest.raises(RuntimeError, match='static_scratch'):
                other.sum(out=out)                    # no recorded call for this signature
    finally:
        _function.Function.launch_packed_scratch = real
    assert calls == ['cupy_sum', 'cupy_sum_combine']
    assert float(out.get()) == pytest.approx(float(h.sum(dtype=np.float64)), rel=1e-5)
    # outside the context everything allocates again
    assert d.sum().shape == ()


def test_limits_are_refused_with_a_clear_error():
    lib = _rt.lib
    d = cp.asarray(np.ones(1 << 21, np.float32))
    out = cp.empty((), np.float32)
    launches = _record_launches(lambda: d.sum(out=out))
    fptr, grid, block, shmem, args = launches[0]
    stream = cp.cuda.get_current_stream().ptr

    def call(args, offset, nbytes):
        return lib.rt_launch_packed_scratch(fptr, *grid, *block, shmem, stream,
                                            args, len(args), offset, nbytes)
    assert call(args, 0, _rt.RT_SCRATCH_MAX_BYTES + 1) == _rt.RT_ERR_INVALID
    assert b'bytes of scratch requested' in lib.rt_last_error_string()
    assert call(args, 4, 1024) == _rt.RT_ERR_INVALID            # misaligned slot
    assert call(args, len(args), 1024) == _rt.RT_ERR_INVALID    # slot past the end
    big = args + b'\0' * 8192
    assert call(big, 0, 1024) == _rt.RT_ERR_INVALID             # argument block too large
    assert lib.rt_launch_packed_scratch(None, 1, 1, 1, 1, 1, 1, 0, stream, args, len(args),
                                        0, 16) == _rt.RT_ERR_INVALID
    cp.cuda.Device().synchronize()
