"""Split reductions that finish inside the launch that makes the partial
results: results against numpy and against the two-launch route, replays,
other streams, and what a call launches."""
import contextlib
import ctypes

import numpy as np
import pytest

import cupy_amd as cp
from cupy_amd._core import _tuning

pytestmark = pytest.mark.gpu


@contextlib.contextmanager
def tuned(**kw):
    old = {k: _tuning.get(k) for k in kw}
    _tuning.set(**kw)
    try:
        yield
    finally:
        _tuning.set(**old)


def _launched(call):
    """(result, names of the kernels ``call`` launches)."""
    from cupy_amd.cuda import function
    names = []
    orig = function.Function.launch_packed

    def spy(self, *a, **k):
        names.append(self.name)
        return orig(self, *a, **k)
    # (a new version of the settings: no recorded call is replayed, every
    # launch goes through Function.launch_packed)
    _tuning.set()
    function.Function.launch_packed = spy
    try:
        out = call()
    finally:
        function.Function.launch_packed = orig
    # (the first such launch on a stream also clears the memory the workgroups
    # hand their partial results over in)
    return out, [n for n in names if not n.startswith('cupy_copy')]


@pytest.mark.parametrize('shape,axis,one', [
    ((1 << 21,), None, True), ((3, 1 << 19), 1, True), ((1 << 9, 1 << 10), 0, True),
    ((500, 1030), 0, True), ((5, 7, 1 << 15), 2, True), (((1 << 20) + 12345,), 0, True),
    # many partial results per column, much input: a second launch combines them
    ((1 << 16, 8), 0, False), ((1 << 12, 1030), 0, False), ((1 << 23,), None, False)])
@pytest.mark.parametrize('dtype', ['int32', 'float64', 'int8', 'complex64'])
def test_one_launch_gives_what_two_give(shape, axis, one, dtype):
    rng = np.random.default_rng(hash((shape, dtype)) % 2 ** 31)
    if dtype == 'complex64':
        h = (rng.integers(-8, 9, shape) + 1j * rng.integers(-8, 9, shape)).astype(dtype)
    else:
        h = rng.integers(-8, 9, shape).astype(dtype)
    a = cp.asarray(h)
    (got, names) = _launched(lambda: a.sum(axis=axis))
    if one:
        assert len(names) == 1, names
    elif a.nbytes > 16 << 20:
        assert len(names) == 2, names
    with tuned(reduce_finish=False):
        two, names2 = _launched(lambda: a.sum(axis=axis))
    # (rows of 32 KiB are not split at all)
    assert len(names2) == 2 or (dtype == 'int8' and axis == 2), names2
    # (small integers: every order of summation gives the same)
    np.testing.assert_array_equal(got.get(), h.sum(axis=axis))
    np.testing.assert_array_equal(got.get(), two.get())


@pytest.mark.parametrize('op', ['max', 'min', 'argmax', 'argmin', 'mean', 'var', 'prod', 'any'])
@pytest.mark.parametrize('shape,axis', [((1 << 21,), None), ((400, 600), 0), ((120, 600), 0),
                                        ((2, 1 << 20), 1), ((1 << 13, 600), 0)])
def test_other_reductions_in_one_launch(op, shape, axis):
    rng = np.random.default_rng(7)
    h = rng.standard_normal(shape)
    if op == 'prod':
        h = np.where(rng.random(shape) < 0.5, 1.0, -1.0)
    if op == 'any':
        h = np.zeros(shape)
        h.reshape(-1)[h.size // 3] = 1.0
    a = cp.asarray(h)
    if op in ('argmax', 'argmin') and axis is None:
        got = getattr(a, op)()
        want = getattr(h, op)()
    else:
        got = getattr(a, op)(axis=axis)
        want = getattr(h, op)(axis=axis)
    if op in ('mean', 'var'):
        np.testing.assert_allclose(got.get(), want, rtol=1e-12, atol=1e-14)
        with tuned(reduce_finish=False):
            two = getattr(a, op)(axis=axis)
        # the same partial results, combined in another order
        np.testing.assert_allclose(got.get(), two.get(), rtol=1e-12, atol=1e-14)
        # and in the same order call after call
        for _ in range(3):
            np.testing.assert_array_equal(getattr(a, op)(axis=axis).get(), got.get())
    else:
        np.testing.assert_array_equal(got.get(), want)


def test_replays_and_results_stay_right_call_after_call():
    rng = np.random.default_rng(3)
    hs = [rng.integers(-100, 100, 1 << 21).astype('int64') for _ in range(3)]
    arrays = [cp.asarray(h) for h in hs]
    for rep in range(50):
        for a, h in zip(arrays, hs):
            assert int(a.sum()) == int(h.sum())
            assert int(a.max()) == int(h.max())
    # a smaller and a larger problem on the same memory in between
    small = cp.asarray(hs[0][:300000])
    assert int(small.sum()) == int(hs[0][:300000].sum())
    big = cp.asarray(np.ones((1 << 13, 1 << 10), 'int32'))
    np.testing.assert_array_equal(big.sum(axis=0).get(), np.full(1 << 10, 1 << 13))
    assert int(arrays[1].sum()) == int(hs[1].sum())


def test_another_stream_gets_memory_of_its_own():
    rng = np.random.default_rng(5)
    h = rng.integers(-100, 100, 1 << 22).astype('int32')
    a = cp.asarray(h)
    want = int(h.sum())
    assert int(a.sum()) == want
    s = cp.cuda.Stream()
    with s:
        for _ in range(5):
            r = a.sum()
        s.synchronize()
        assert int(r) == want
    assert int(a.sum()) == want


def test_large_inputs_take_two_launches():
    a = cp.ones(1 << 25, 'float32')       # 128 MiB: the tail of a launch that also finishes costs more
    got, names = _launched(lambda: a.sum())
    assert len(names) == 2, names
    assert float(got) == float(1 << 25)


@contextlib.contextmanager
def _reported_give_up(family):
    """Writes what a workgroup that gave up would have written into the
    device's word (every kernel still exits normally) and restores the state
    of the device afterwards."""
    from cupy_amd.cuda import _giveup
    dev = cp.cuda.Device().id
    fault = _giveup.word(dev, family)
    ctypes.c_uint32.from_address(fault).value = 1
    try:
        yield
    finally:
        _giveup.disabled[family].discard(dev)
        ctypes.c_uint32.from_address(fault).value = 0


def test_a_workgroup_that_gives_up_is_reported():
    """The recorded one-launch call is NOT replayed once the word is set: the
    call raises, and later calls take two launches (and are replayed as such)."""
    from cupy_amd.cuda import _giveup
    a = cp.ones(1 << 22, 'int32')
    out = cp.zeros((), 'int64')
    assert int(a.sum()) == 1 << 22
    assert int(a.sum()) == 1 << 22          # (a replay)
    a.sum(out=out)
    a.sum(out=out)
    with _reported_give_up(_giveup.REDUCTION):
        with pytest.raises(RuntimeError, match='gave up waiting'):
            a.sum()
        # two launches from here on, for the other recorded call as well
        from cupy_amd.cuda import function
        names = []
        orig = function.Function.launch_packed
        from cupy_amd._core import _launch_plan
        _launch_plan.use_quick = False
        function.Function.launch_packed = lambda self, *x, **k: (names.append(self.name),
                                                                orig(self, *x, **k))[1]
        try:
            got = a.sum()
            a.sum(out=out)
            again = a.sum()
        finally:
            function.Function.launch_packed = orig
            _launch_plan.use_quick = True
        assert names == ['cupy_sum', 'cupy_sum_combine'] * 3, names
        assert int(got) == int(out) == int(again) == 1 << 22


def test_a_give_up_cannot_reach_the_host_unnoticed():
    """Whatever makes device results visible to the host raises when a kernel
    has reported a wait that ran out."""
    from cupy_amd.cuda import _giveup
    a = cp.ones(1 << 20, 'int32')
    r = a.sum()
    for family in (_giveup.REDUCTION, _giveup.SCAN):
        for look in (lambda: r.get(), lambda: int(r), lambda: cp.cuda.Device().synchronize(),
                     lambda: cp.cuda.Stream.null.synchronize(),
                     lambda: cp.cuda.get_current_stream().record().synchronize()):
            with _reported_give_up(family):
                with pytest.raises(RuntimeError, match='gave up waiting'):
                    look()
                look()      # reported once
        s = cp.cuda.Stream()
        with s:
            with _reported_give_up(family):
                with pytest.raises(RuntimeError, match='gave up waiting'):
                    r.get()
    assert int(r) == 1 << 20


def test_a_wait_that_runs_out_never_delivers_its_value():
    """With no patience at all (one poll per wait) a finishing workgroup may
    find partial results missing: then the value must not come back."""
    from cupy_amd.cuda import _giveup
    dev = cp.cuda.Device().id
    a = cp.ones((1 << 22) + 17, 'int32')
    try:
        with tuned(reduce_finish_spin_limit=0):
            for _ in range(4):
                r = a.sum()
                try:
                    value = int(r)
                except RuntimeError as e:
                    assert 'gave up waiting' in str(e)
                    break
                assert value == (1 << 22) + 17
    finally:
        _giveup.disabled[_giveup.REDUCTION].discard(dev)
    assert int(a.sum()) == (1 << 22) + 17


def test_a_second_stream_records_a_replay_of_its_own():
    rng = np.random.default_rng(9)
    h = rng.integers(-100, 100, 1 << 21).astype('int32')
    a = cp.asarray(h)
    out = cp.zeros((), 'int64')
    from cupy_amd._core import _routines_math as rm
    a.sum(out=out)
    s = cp.cuda.Stream()
    with s:
        a.sum(out=out)
        n = len(rm._sum_auto_dtype._fast_calls)
        calls = []
        orig = rm._sum_auto_dtype._call
        rm._sum_auto_dtype._call = lambda *x, **k: (calls.append(1), orig(*x, **k))[1]
        try:
            for _ in range(3):
                a.sum(out=out)
        finally:
            del rm._sum_auto_dtype._call
        s.synchronize()
        assert not calls                    # replays, not the full path
        assert len(rm._sum_auto_dtype._fast_calls) == n
        assert int(out) == int(h.sum())
    a.sum(out=out)
    assert int(out) == int(h.sum())


@pytest.mark.parametrize('dtype', ['complex64', 'complex128'])
def test_any_and_all_of_complex_values(dtype):
    # (reference: cupy/_core/_routines_logic.pyx:43-56 lists 'F->?' and 'D->?')
    rng = np.random.default_rng(11)
    h = np.zeros((300, 70), dtype)
    h[rng.integers(0, 300, 40), rng.integers(0, 70, 40)] = 1j
    h[5, :] = 2.0
    a = cp.asarray(h)
    for axis in (None, 0, 1):
        np.testing.assert_array_equal(a.any(axis=axis).get(), h.any(axis=axis))
        np.testing.assert_array_equal(a.all(axis=axis).get(), h.all(axis=axis))
    big = np.zeros(1 << 21, dtype)
    assert not bool(cp.asarray(big).any())
    big[-3] = 1j
    assert bool(cp.asarray(big).any())
    assert not bool(cp.asarray(big).all())
