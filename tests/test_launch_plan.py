"""A call that repeats an earlier call's argument signature replays the recorded
launch.  These tests compare, launch for launch and byte for byte, what the
replay puts into the kernel's argument block with what the full path puts there
for the same arguments.  They inspect recorded launches, so they need the
compile-check mode (no GPU); the GPU suite checks the replayed results
numerically (tests/test_gpu_runtime.py)."""
import struct

import numpy as np
import pytest

import cupy_amd as cp
from cupy_amd import _dryrun
from cupy_amd._core import _launch_plan

pytestmark = pytest.mark.skipif(not _dryrun.enabled(),
                                reason='inspects recorded launches')


def launches_of(fn):
    n0 = len(_dryrun.launches)
    ret = fn()
    return ret, _dryrun.launches[n0:]


def words(blob, known):
    """Argument block as a list of 8-byte words; words that look like device
    addresses are replaced by the name of the array they point into, or by
    'tmp' for memory the call allocated itself."""
    out = []
    pad = (-len(blob)) % 8
    data = blob + b'\0' * pad
    for (w,) in struct.iter_unpack('<Q', data):
        if 0x7f0000000000 <= w < 0x7f8000000000:
            out.append(known.get(w, 'tmp'))
        else:
            out.append(w)
    return out


def describe(launches, known):
    return [(name, grid, block, shmem, words(blob, known))
            for name, grid, block, shmem, blob in launches]


def check_replay(kernel_tables, call, make_args, known_of):
    """``call(*args)`` three times: the recording call, a replay with the
    same arguments, then -- with other arrays of the same signature -- a replay
    and, after the recorded calls have been dropped, the full path again."""
    args1 = make_args()
    _, first = launches_of(lambda: call(*args1))
    assert first
    _, again = launches_of(lambda: call(*args1))
    k1 = known_of(args1)
    assert describe(again, k1) == describe(first, k1)

    args2 = make_args()
    k2 = known_of(args2)
    n_recorded = sum(len(t) for t in kernel_tables())
    assert n_recorded >= 1
    _, replay = launches_of(lambda: call(*args2))
    assert sum(len(t) for t in kernel_tables()) == n_recorded      # nothing new recorded
    for t in kernel_tables():
        t.clear()
    _, full = launches_of(lambda: call(*args2))
    assert describe(replay, k2) == describe(full, k2)
    # same structure as the first call, other addresses
    assert [l[:4] for l in replay] == [l[:4] for l in first]


def names(args):
    known = {}
    for i, a in enumerate(args):
        if isinstance(a, cp.ndarray):
            known[a.data.ptr] = 'arg%d' % i
    return known


def test_elementwise_kernel_replay_patches_pointers_and_scalars():
    saxpy = cp.ElementwiseKernel('float32 x, float32 y, float32 a', 'float32 z',
                                 'z = a * x + y', 'saxpy_replay')

    def make():
        n = 1 << 16
        return (cp.ndarray((n,), np.float32), cp.ndarray((n,), np.float32), 2.5,
                cp.ndarray((n,), np.float32))
    check_replay(lambda: [saxpy._fast_calls], saxpy, make, names)
    # another scalar value goes into the same slot
    x, y, _, z = make()
    _, a = launches_of(lambda: saxpy(x, y, 2.5, z))
    _, b = launches_of(lambda: saxpy(x, y, -7.25, z))
    wa, wb = words(a[0][4], names((x, y, 0, z))), words(b[0][4], names((x, y, 0, z)))
    diff = [i for i, (p, q) in enumerate(zip(wa, wb)) if p != q]
    assert len(diff) == 1
    assert struct.pack('<Q', wb[diff[0]])[:4] == struct.pack('<f', -7.25)


def test_elementwise_kernel_allocates_a_new_output_on_every_replay():
    sq = cp.ElementwiseKernel('T x', 'T y', 'y = x * x', 'square_replay')
    x = cp.ndarray((1000,), np.float64)
    r1 = sq(x)
    r2 = sq(x)
    r3 = sq(x)
    assert r1 is not r2 and r2 is not r3
    assert r2.data.ptr != r3.data.ptr
    assert r3.shape == (1000,) and r3.dtype == np.float64
    assert len(sq._fast_calls) == 1


def test_ufunc_replay_tiled_flat_and_generic():
    def tiled():
        base = cp.ndarray((512, 256), np.float32)
        return (base.T, cp.ndarray((1, 512), np.float16), cp.ndarray((256, 512), np.float32))

    def flat():
        return (cp.ndarray((300, 7), np.int32), 3, cp.ndarray((300, 7), np.int32))

    def generic():
        big = cp.ndarray((6, 10, 14), np.float64)
        return (big[::2, 1:9:3, ::-1], cp.ndarray((3, 3, 14), np.float64),
                cp.ndarray((3, 3, 14), np.float64))

    def known(args):
        k = names(args)
        for i, a in enumerate(args):
            if isinstance(a, cp.ndarray) and a.base is not None:
                k[a.data.ptr] = 'arg%d' % i
        return k
    for make, fn in ((tiled, cp.multiply), (flat, cp.add), (generic, cp.subtract)):
        check_replay(lambda: [fn._fast_calls], fn, make, known)


def test_ufunc_keyword_out_and_fresh_output_share_nothing():
    a = cp.ndarray((64, 64), np.float32)
    b = cp.ndarray((64, 64), np.float32)
    o = cp.ndarray((64, 64), np.float32)
    cp.maximum._fast_calls.clear()
    assert cp.maximum(a, b, out=o) is o
    assert cp.maximum(a, b, out=o) is o           # replay returns the given array
    assert cp.maximum(a, b, o) is o
    assert len(cp.maximum._fast_calls) == 1       # keyword and positional: one entry
    r = cp.maximum(a, b)
    r2 = cp.maximum(a, b)
    assert r is not o and r2 is not r
    assert len(cp.maximum._fast_calls) == 2


def test_ufunc_replay_still_copies_overlapping_inputs():
    buf = cp.ndarray((1025,), np.float32)
    a, b = buf[:-1], buf[1:]
    other = cp.ndarray((1024,), np.float32)
    cp.add._fast_calls.clear()
    # record with disjoint arrays of this signature ...
    x = cp.ndarray((1025,), np.float32)[:-1]
    y = cp.ndarray((1025,), np.float32)[1:]
    launches_of(lambda: cp.add(x, other, y))
    _, rep = launches_of(lambda: cp.add(x, other, y))
    assert len(rep) == 1
    # ... then call with an input that overlaps the output: the input must be
    # copied first (an extra launch), exactly as on the full path
    assert a.data.ptr % 16 == x.data.ptr % 16 and b.data.ptr % 16 == y.data.ptr % 16
    _, ls = launches_of(lambda: cp.add(a, other, b))
    w = words(ls[0][4], {a.data.ptr: 'a', other.data.ptr: 'other', b.data.ptr: 'b'})
    assert w[:3] == ['tmp', 'other', 'b']          # reads a copy of `a`
    _, ls = launches_of(lambda: cp.add(x, other, y))
    w = words(ls[0][4], {x.data.ptr: 'x', other.data.ptr: 'other', y.data.ptr: 'y'})
    assert w[:3] == ['x', 'other', 'y']
    # in == out (the very same array) needs no copy
    _, ls = launches_of(lambda: cp.add(y, other, y))
    _, ls = launches_of(lambda: cp.add(y, other, y))
    assert len(ls) == 1


def test_scalar_conversion_matches_the_full_path():
    from cupy_amd._core._scalar import CScalar

    def full(v, dt):
        s = CScalar(v)
        s.apply_dtype(np.dtype(dt))
        return s._struct_value()
    cases = [(2.5, 'float32'), (1e39, 'float32'), (-1e39, 'float32'), (float('nan'), 'float32'),
             (float('inf'), 'float32'), (3.0e38, 'float32'), (0.1, 'float64'), (0.1, 'float16'),
             (7, 'int32'), (-1, 'int8'), (255, 'uint8'), (2 ** 40, 'int64'), (3, 'float64'),
             (3, 'float32'), (True, 'bool'), (True, 'int32'), (2.75, 'int32'),
             (np.float32(1.5), 'float64'), (np.int8(-3), 'int64')]
    for v, dt in cases:
        got = _launch_plan.scalar_value(v, np.dtype(dt))
        want = full(v, dt)
        code = {'float32': 'f', 'float64': 'd', 'float16': 'e', 'bool': '?', 'int8': 'b',
                'uint8': 'B', 'int32': 'i', 'int64': 'q'}[dt]
        assert struct.pack(code, got) == struct.pack(code, want), (v, dt, got, want)
    for v, dt in ((300, 'uint8'), (-1, 'uint8'), (2 ** 31, 'int32')):
        with pytest.raises(OverflowError):
            full(v, dt)
        with pytest.raises(OverflowError):
            _launch_plan.scalar_value(v, np.dtype(dt))


def test_python_int_out_of_range_still_raises_after_recording():
    a = cp.ndarray((16,), np.uint8)
    o = cp.ndarray((16,), np.uint8)
    cp.add(a, 3, o)
    cp.add(a, 4, o)
    with pytest.raises(OverflowError):
        cp.add(a, 300, o)


def test_reduction_replay_with_and_without_partials():
    def known(args):
        return names(args)

    def rows():
        return (cp.ndarray((2048, 1024), np.float32), cp.ndarray((2048,), np.float32))

    def cols_split():
        return (cp.ndarray((4096, 512), np.float64), cp.ndarray((512,), np.float64))

    def full():
        return (cp.ndarray((1 << 22,), np.float32), cp.ndarray((), np.float32))

    from cupy_amd._core import _routines_math as rm
    from cupy_amd._core import _tuning
    sumk = rm._sum_auto_dtype
    check_replay(lambda: [sumk._fast_calls], lambda a, o: sumk(a, 1, None, o, False), rows, known)
    _tuning.set(reduce_finish=False)
    try:
        _split_reductions_in_two_launches(sumk, cols_split, full, known)
    finally:
        _tuning.set(reduce_finish=True)
    # split reductions that finish in their one launch: the first call on a
    # stream also clears the memory the workgroups hand their results over in;
    # replays launch the one kernel with the same arguments
    def cols_short():
        return (cp.ndarray((512, 512), np.float64), cp.ndarray((512,), np.float64))

    for make, axis in ((cols_short, 0), (full, None)):
        a, o = make()
        _, first = launches_of(lambda: sumk(a, axis, None, o, False))
        assert [l[0] for l in first if not l[0].startswith('cupy_copy')] == ['cupy_sum']
        _, again = launches_of(lambda: sumk(a, axis, None, o, False))
        assert [l[0] for l in again] == ['cupy_sum']
        k = known((a, o))
        assert describe(again, k) == describe(first[-1:], k)
        b, p = make()
        _, other = launches_of(lambda: sumk(b, axis, None, p, False))
        assert describe(other, known((b, p))) == describe(again, k)
        # on another stream the recorded call is not used: that stream gets
        # memory of its own
        side = cp.cuda.Stream()
        with side:
            _, elsewhere = launches_of(lambda: sumk(a, axis, None, o, False))
        assert [l[0] for l in elsewhere if not l[0].startswith('cupy_copy')] == ['cupy_sum']
        if side.ptr != cp.cuda.get_current_stream().ptr:
            assert (words(elsewhere[-1][4], names((a, o)))
                    != words(again[-1][4], names((a, o))))


def _split_reductions_in_two_launches(sumk, cols_split, full, known):
    check_replay(lambda: [sumk._fast_calls], lambda a, o: sumk(a, 0, None, o, False), cols_split, known)
    check_replay(lambda: [sumk._fast_calls], lambda a, o: sumk(a, None, None, o, False), full, known)
    # the split reductions launch two kernels sharing one temporary
    a, o = full()
    _, ls = launches_of(lambda: sumk(a, None, None, o, False))
    assert [l[0] for l in ls] == ['cupy_sum', 'cupy_sum_combine']
    w0, w1 = words(ls[0][4], names((a, o))), words(ls[1][4], names((a, o)))
    assert w0.count('tmp') == 1 and w1.count('tmp') == 1
    raw0 = [w for (w,) in struct.iter_unpack('<Q', ls[0][4] + b'\0' * ((-len(ls[0][4])) % 8))
            if 0x7f0000000000 <= w < 0x7f8000000000]
    raw1 = [w for (w,) in struct.iter_unpack('<Q', ls[1][4] + b'\0' * ((-len(ls[1][4])) % 8))
            if 0x7f0000000000 <= w < 0x7f8000000000]
    tmp0 = [w for w in raw0 if w not in (a.data.ptr, o.data.ptr)]
    tmp1 = [w for w in raw1 if w not in (a.data.ptr, o.data.ptr)]
    assert tmp0 == tmp1            # both passes address the same temporary


def test_reduction_axis_and_dtype_are_part_of_the_signature():
    a = cp.ndarray((64, 32), np.float32)
    r1 = a.sum(axis=0)
    r2 = a.sum(axis=1)
    r3 = a.sum(axis=0, keepdims=True)
    r4 = a.sum(axis=0, dtype=np.float64)
    r5 = a.sum(axis=0)
    assert r1.shape == (32,) and r2.shape == (64,) and r3.shape == (1, 32)
    assert r4.dtype == np.float64 and r5.dtype == np.float32 and r5.shape == (32,)
    r6 = a.argmax(axis=1)
    r7 = a.argmax(axis=1)
    assert r6.dtype == np.int64 and r7.shape == (64,) and r6 is not r7


def test_reduction_kernel_and_fuse_replay():
    l2 = cp.ReductionKernel('T x, T y', 'T z', '(x - y) * (x - y)', 'a + b', 'z = sqrt(a)',
                            '0', 'l2_replay')

    def make():
        return (cp.ndarray((256, 512), np.float32), cp.ndarray((256, 512), np.float32))
    check_replay(lambda: [l2._fast_calls], lambda x, y: l2(x, y, axis=1), make,
                 lambda args: names(args))

    f = cp.fuse(lambda x, y, w: cp.sum((x - y) ** 2 * w, axis=-1))

    def make3():
        return (cp.ndarray((1024, 256), np.float16), cp.ndarray((1024, 256), np.float16),
                cp.ndarray((256,), np.float32))
    r = f(*make3())
    args = make3()
    r1, first = launches_of(lambda: f(*args))
    r2, again = launches_of(lambda: f(*args))
    assert r1 is not r2 and r1.shape == r2.shape == r.shape == (1024,)
    k = names(args)
    assert describe(first, k) == describe(again, k)
    f.clear_cache()
    r3, fresh = launches_of(lambda: f(*args))
    assert describe(fresh, k) == describe(first, k)


def test_tuning_change_invalidates_recorded_calls():
    from cupy_amd._core import _tuning
    k = cp.ElementwiseKernel('T x, T w', 'T y', 'y = x + w', 'add_replay')
    x = cp.ndarray((1 << 16,), np.float32)
    w = cp.ndarray((1 << 16,), np.float32)
    y = cp.ndarray((1 << 16,), np.float32)
    k(x, w, y)
    _, a = launches_of(lambda: k(x, w, y))
    old = _tuning.get('flat_block')
    try:
        _tuning.set(flat_block=256)
        _, b = launches_of(lambda: k(x, w, y))
        assert b[0][2] == (256, 1, 1) and a[0][2] == (old, 1, 1)
    finally:
        _tuning.set(flat_block=old)
    _, c = launches_of(lambda: k(x, w, y))
    assert c[0][2] == (old, 1, 1)


def test_other_calls_take_the_full_path():
    k = cp.ElementwiseKernel('T x', 'T y', 'y = x', 'copy_replay')
    x = cp.ndarray((128,), np.float32)
    y = cp.ndarray((128,), np.float32)
    k(x, y, block_size=64)
    k(x, y, stream=cp.cuda.Stream.null)
    assert len(k._fast_calls) == 0
    k(x, y)
    assert len(k._fast_calls) == 1
    # zero-size calls launch nothing and record nothing
    e = cp.ndarray((0,), np.float32)
    k(e, cp.ndarray((0,), np.float32))
    assert len(k._fast_calls) == 1
    with pytest.raises(TypeError):
        k(x, y, x)


def test_casting_rule_joins_the_signature():
    """``astype``, copies and fills pass ``casting='unsafe'``: such calls are
    recorded and replayed too, under a key of their own; a cast that warns is
    never recorded, so it warns on every call."""
    import warnings
    from cupy_amd._core._ufuncs import elementwise_copy
    a = cp.ndarray((1 << 16,), np.float32)
    n0 = len(elementwise_copy._fast_calls)
    r1, first = launches_of(lambda: a.astype(np.float64))
    assert len(elementwise_copy._fast_calls) == n0 + 1
    assert any(key[-1] == 'unsafe' for key in elementwise_copy._fast_calls)
    r2, again = launches_of(lambda: a.astype(np.float64))
    assert r1.dtype == r2.dtype == np.float64 and r1.data.ptr != r2.data.ptr
    k = names((a,))
    assert [(l[0], l[1], l[2]) for l in again] == [(l[0], l[1], l[2]) for l in first]
    assert words(again[0][4], k)[0] == 'arg0'
    # stricter rules refuse what 'unsafe' allows, recorded or not
    b = cp.ndarray((1 << 16,), np.int32)
    elementwise_copy(a, b, casting='unsafe')
    elementwise_copy(a, b, casting='unsafe')
    with pytest.raises(TypeError):
        elementwise_copy(a, b, casting='same_kind')
    with pytest.raises(TypeError):
        elementwise_copy(a, b, casting='safe')
    # complex to real warns every time
    c = cp.ndarray((100,), np.complex64)
    with warnings.catch_warnings(record=True) as seen:
        warnings.simplefilter('always')
        for _ in range(3):
            c.astype(np.float32)
    assert len(seen) == 3


@pytest.fixture
def giveup_words():
    """Stands in for the pinned words of device 0 (none exist where launches
    are only recorded): 16 words of host memory the test may write."""
    import ctypes
    from cupy_amd.cuda import _giveup
    words = (ctypes.c_uint32 * 16)()
    saved = dict(_giveup._base), _giveup.armed
    _giveup._base[0] = ctypes.addressof(words)
    _giveup.armed = True
    try:
        yield words
    finally:
        _giveup._base.clear()
        _giveup._base.update(saved[0])
        _giveup.armed = saved[1]
        for family in _giveup.disabled:
            family.clear()


def test_a_one_launch_reduction_is_not_replayed_after_a_give_up(giveup_words):
    """A recorded call whose kernel waits for other workgroups is left to the
    full path as soon as the device's word is set; that path raises once and
    records the two-launch form in its place."""
    from cupy_amd._core import _routines_math as rm
    from cupy_amd.cuda import _giveup
    sumk = rm._sum_auto_dtype
    a, o = cp.ndarray((1 << 22,), np.float32), cp.ndarray((), np.float32)
    b, p = cp.ndarray((512, 512), np.float64), cp.ndarray((512,), np.float64)

    def kernels(ls):
        return [l[0] for l in ls if not l[0].startswith('cupy_copy')]
    for x, out, axis in ((a, o, None), (b, p, 0)):
        sumk(x, axis, None, out, False)
        _, again = launches_of(lambda: sumk(x, axis, None, out, False))
        assert kernels(again) == ['cupy_sum']
    giveup_words[_giveup.REDUCTION] = 1
    assert not _giveup.usable(0, _giveup.REDUCTION)
    with pytest.raises(RuntimeError, match='gave up waiting'):
        sumk(a, None, None, o, False)
    assert giveup_words[_giveup.REDUCTION] == 0 and 0 in _giveup.disabled[_giveup.REDUCTION]
    for x, out, axis in ((a, o, None), (b, p, 0), (a, o, None), (b, p, 0)):
        _, ls = launches_of(lambda: sumk(x, axis, None, out, False))
        assert kernels(ls) == ['cupy_sum', 'cupy_sum_combine']
    # the scans' word is a different one
    assert _giveup.usable(0, _giveup.SCAN)


def test_poll_reports_each_family_once(giveup_words):
    from cupy_amd.cuda import _giveup
    _giveup.poll()
    giveup_words[_giveup.SCAN] = 1
    with pytest.raises(RuntimeError, match='one-pass scan on device 0 gave up waiting'):
        _giveup.poll()
    _giveup.poll()
    assert 0 in _giveup.disabled[_giveup.SCAN] and 0 not in _giveup.disabled[_giveup.REDUCTION]
    giveup_words[_giveup.REDUCTION] = 1
    _giveup.poll(5)             # another device: nothing to say
    with pytest.raises(RuntimeError, match='a reduction on device 0 gave up waiting'):
        _giveup.poll(0)


def test_a_second_stream_replays_a_record_of_its_own():
    """One-launch reductions are recorded per stream: the third call on a
    second stream is a replay, not the full path."""
    from cupy_amd._core import _routines_math as rm
    sumk = rm._sum_auto_dtype
    a, o = cp.ndarray((1 << 21,), np.float32), cp.ndarray((), np.float32)
    sumk(a, None, None, o, False)
    side = cp.cuda.Stream()
    side.ptr = 0x5151            # (streams have no handles here: any other number)
    calls = []
    orig = sumk._call
    sumk._call = lambda *x, **k: (calls.append(1), orig(*x, **k))[1]
    try:
        with side:
            _, first = launches_of(lambda: sumk(a, None, None, o, False))
            assert len(calls) == 1
            n = len(sumk._fast_calls)
            _, second = launches_of(lambda: sumk(a, None, None, o, False))
            _, third = launches_of(lambda: sumk(a, None, None, o, False))
        assert len(calls) == 1 and len(sumk._fast_calls) == n
        _, home = launches_of(lambda: sumk(a, None, None, o, False))
        assert len(calls) == 1
    finally:
        del sumk._call
        side.ptr = 0
    k = names((a, o))
    assert describe(second, k) == describe(third, k) == describe(first[-1:], k)
    # each stream hands its partial results over in memory of its own
    assert home[-1][4] != third[-1][4]


def test_retired_blocks_are_freed_two_retirements_later():
    """Streams come and go: the blocks of evicted streams do not pile up."""
    from cupy_amd._core import _reduce_sync, _tuning
    saved = dict(_reduce_sync._blocks)
    try:
        _reduce_sync._blocks.clear()
        v0 = _tuning.version()
        for s in range(3 * _reduce_sync.MAX_STREAMS + 5):
            assert _reduce_sync.acquire(0, 1000 + s, 1000 + s, 100) is not None
            held = (len(_reduce_sync._blocks) + len(_reduce_sync._retired[0])
                    + len(_reduce_sync._retired[1]))
            assert held <= 3 * _reduce_sync.MAX_STREAMS
        # records that name retired blocks are never replayed again
        assert _tuning.version() == v0 + 3
    finally:
        _reduce_sync._blocks.clear()
        _reduce_sync._blocks.update(saved)


def test_a_python_integer_outside_the_recorded_type_is_not_replayed():
    """A record made with a Python integer that fitted the arrays' type must
    not pack one that does not: the call goes the full way, which chooses
    another loop (comparisons) or raises (arithmetic) as NumPy does."""
    import numpy as np
    import cupy_amd as cp
    a = cp.ndarray((5,), np.int8)
    for value in (-1, -1, -1, 300, 300, -1, 1 << 40):
        assert (a == value).dtype == np.bool_
        assert cp.true_divide(a, value).dtype == np.float64
    for value in (1, 1, 1):
        assert cp.add(a, value).dtype == np.int8
    with pytest.raises(OverflowError):
        cp.add(a, 300)
    assert cp.add(a, 2).dtype == np.int8
