"""The one-pass scan of long rows (tiles chained through published totals)
against NumPy and against the three-pass kernels on the same seeded inputs."""
import numpy as np
import pytest

import cupy_amd as cp
from cupy_amd._core import _scan, _tuning
from cupy_amd.cuda import _giveup
from helpers import assert_exact

pytestmark = pytest.mark.gpu


@pytest.fixture(autouse=True)
def _restore():
    yield
    _tuning.set(scan_chain=True, scan_chain_spin_limit=1 << 18, scan_chain_parts=0,
                scan_chain_cols=True, scan_chain_cols_waves=16, scan_chain_cols_trips=0,
                scan_chain_cols_vec_bytes=0, scan_chain_cols_xcd='auto',
                scan_chain_cols_unaligned=True, scan_chain_cols_short=True,
                scan_chain_xcd='auto')
    _giveup.disabled[_giveup.SCAN].clear()


def three_pass(fn):
    _tuning.set(scan_chain=False)
    try:
        return fn()
    finally:
        _tuning.set(scan_chain=True)


def launched(fn):
    """Names of the kernels ``fn`` launches."""
    from cupy_amd.cuda import function
    names = []
    orig = function.Function.launch_packed

    def spy(self, *a, **k):
        names.append(self.name)
        return orig(self, *a, **k)
    function.Function.launch_packed = spy
    try:
        fn()
    finally:
        function.Function.launch_packed = orig
    return names


@pytest.mark.parametrize('n', [(1 << 22) + 12345, 1 << 22, (1 << 20) + 1, 3 * 4096 * 32 + 7])
def test_integer_scans_are_exact(n):
    rng = np.random.default_rng(n & 0xffff)
    h = rng.integers(-5, 6, n).astype(np.int32)
    d = cp.asarray(h)
    assert 'cupy_scan_chain' in launched(lambda: d.cumsum())
    assert_exact(d.cumsum().get(), h.cumsum())
    out = cp.empty(n, np.int32)
    cp.cumsum(d, out=out)
    assert_exact(out.get(), h.cumsum(dtype=np.int32))


@pytest.mark.parametrize('dtype,rtol', [('float32', 1e-5), ('float64', 1e-13), ('float16', 2e-3),
                                        ('complex64', 1e-5), ('complex128', 1e-13)])
def test_floating_scans(dtype, rtol):
    rng = np.random.default_rng(17)
    n = (1 << 21) + 4321
    h = rng.uniform(0, 1, n)
    if np.dtype(dtype).kind == 'c':
        h = h + 1j * rng.uniform(-1, 1, n)
    if dtype == 'float16':
        h = h * 1e-3                      # the running sum stays representable
    h = h.astype(dtype)
    d = cp.asarray(h)
    # (long sums of complex128 run over the real and imaginary parts as two columns)
    assert ('cupy_scan_chain_tile' if dtype == 'complex128' else 'cupy_scan_chain') in launched(
        lambda: d.cumsum())
    got = d.cumsum().get()
    wide = np.complex128 if np.dtype(dtype).kind == 'c' else np.float64
    want = np.cumsum(h.astype(wide))
    scale = np.cumsum(np.abs(h).astype(np.float64))
    assert (np.abs(got - want) <= rtol * scale + 1e-30).all()
    # same bits on every run, and close to the three-pass result
    assert_exact(d.cumsum().get(), got)
    other = three_pass(lambda: d.cumsum().get())
    assert (np.abs(got - other) <= 2 * rtol * scale + 1e-30).all()


@pytest.mark.parametrize('parts', [1, 2, 3, 8])
def test_every_tile_size_and_many_launches_on_one_stream(parts):
    """The slots of the published totals are reused from call to call without
    being cleared: totals of an earlier call (other data, other tile size) must
    never be taken for this call's."""
    _tuning.set(scan_chain_parts=parts)
    rng = np.random.default_rng(parts)
    for n in ((1 << 21) + 77, 1 << 20, (1 << 21) + 77, 3 << 19):
        h = rng.integers(-50, 51, n).astype(np.int32)
        d = cp.asarray(h)
        assert_exact(d.cumsum().get(), h.cumsum())
    stream = cp.cuda.Stream()
    with stream:
        h = rng.integers(-50, 51, 1 << 21).astype(np.int64)
        d = cp.asarray(h)
        for _ in range(3):
            got = d.cumsum()
        stream.synchronize()
        assert_exact(got.get(), h.cumsum())


@pytest.mark.parametrize('mode', ['auto', True, False])
@pytest.mark.parametrize('shape', [(300, 8191), (67, 8190), (1000, 6001)])
def test_rows_dealt_out_die_by_die(shape, mode):
    """Rows of two tiles that do not start on cache lines: every compute die
    takes whole rows (row counts that are no multiple of eight leave some
    workgroups without a row)."""
    _tuning.set(scan_chain_xcd=mode)
    rng = np.random.default_rng(shape[1])
    h = rng.integers(-5, 6, shape).astype(np.int32)
    d = cp.asarray(h)
    assert 'cupy_scan_chain' in launched(lambda: d.cumsum(axis=1))
    assert_exact(d.cumsum(axis=1).get(), h.cumsum(axis=1))
    e = d.copy()
    cp.cumsum(e, axis=1, out=e)
    assert_exact(e.get(), h.cumsum(axis=1, dtype=np.int32))


def test_few_long_rows_products_and_nans():
    rng = np.random.default_rng(5)
    h = rng.integers(-5, 6, (3, 300001)).astype(np.int64)
    d = cp.asarray(h)
    assert 'cupy_scan_chain' in launched(lambda: d.cumsum(axis=1))
    assert_exact(d.cumsum(axis=1).get(), h.cumsum(axis=1))
    # int8 in, int64 out; int8 all the way (wraps as NumPy wraps)
    h8 = rng.integers(-100, 100, 1 << 21).astype(np.int8)
    assert_exact(cp.asarray(h8).cumsum().get(), h8.cumsum())
    assert_exact(cp.cumsum(cp.asarray(h8), dtype=np.int8).get(), h8.cumsum(dtype=np.int8))
    # products of +-1 and a few 2s
    hp = np.ones(1 << 21, np.int64)
    hp[rng.choice(hp.size, 40, replace=False)] = rng.choice([-1, 2], 40)
    assert_exact(cp.cumprod(cp.asarray(hp)).get(), np.cumprod(hp))
    # NaNs count as zero
    hf = rng.uniform(0, 1, (2, 700001)).astype(np.float32)
    hf[0, ::1000] = np.nan
    got = cp.nancumsum(cp.asarray(hf), axis=1).get()
    want = np.nancumsum(hf.astype(np.float64), axis=1)
    assert (np.abs(got - want) <= 1e-5 * want + 1e-6).all()
    # a row whose length is no multiple of the vector, rows not aligned to it
    ho = rng.integers(-5, 6, (5, 99991)).astype(np.int32)
    assert_exact(cp.asarray(ho).cumsum(axis=1).get(), ho.cumsum(axis=1))
    hv = rng.integers(-5, 6, (1 << 21) + 3).astype(np.int32)
    assert_exact(cp.asarray(hv)[1:].cumsum().get(), hv[1:].cumsum())


def test_a_tile_that_gives_up_is_reported_and_the_kernel_retired():
    """With no patience at all (one poll per wait) some tile finds its
    neighbours unfinished, gives up and says so: every workgroup still runs to
    its end, the next chained scan raises, and scans go on through the
    three-pass kernels."""
    rng = np.random.default_rng(6)
    h = rng.integers(-5, 6, 1 << 23).astype(np.int32)
    d = cp.asarray(h)
    _tuning.set(scan_chain_spin_limit=0)
    wrong = d.cumsum()
    # the result cannot be looked at without the report
    with pytest.raises(RuntimeError, match='gave up waiting'):
        wrong.get()
    _tuning.set(scan_chain_spin_limit=1 << 18)
    names = launched(lambda: d.cumsum())
    assert 'cupy_scan_chain' not in names and 'cupy_scan_rows_seeded' in names
    assert_exact(d.cumsum().get(), h.cumsum())


@pytest.mark.parametrize('shape,axis', [((700001, 3), 0), ((2, 300000, 5), 1), ((1 << 20, 2), 0),
                                        ((150000, 32), 0), ((3, 99999, 7), 1), ((400000, 12), 0)])
def test_columns_of_narrow_arrays_in_one_pass(shape, axis):
    """Long columns of arrays with a narrow tail: tiles of whole rows, one
    published total per column."""
    rng = np.random.default_rng(shape[-1])
    h = rng.integers(-5, 6, shape).astype(np.int32)
    d = cp.asarray(h)
    assert 'cupy_scan_chain_tile' in launched(lambda: d.cumsum(axis=axis))
    assert_exact(d.cumsum(axis=axis).get(), h.cumsum(axis=axis))
    hf = rng.uniform(0, 1, shape).astype(np.float32)
    df = cp.asarray(hf)
    got = df.cumsum(axis=axis).get()
    want = np.cumsum(hf.astype(np.float64), axis=axis)
    assert (np.abs(got - want) <= 1e-5 * want + 1e-6).all()
    assert_exact(df.cumsum(axis=axis).get(), got)                 # same bits on every run
    other = three_pass(lambda: df.cumsum(axis=axis).get())
    assert (np.abs(got - other) <= 2e-5 * want + 1e-6).all()


@pytest.mark.parametrize('parts', [1, 2, 4])
def test_narrow_arrays_other_types_and_tile_sizes(parts):
    _tuning.set(scan_chain_parts=parts)
    rng = np.random.default_rng(40 + parts)
    h8 = rng.integers(-100, 100, (500001, 3)).astype(np.int8)
    assert_exact(cp.cumsum(cp.asarray(h8), axis=0).get(), np.cumsum(h8, axis=0))
    hd = rng.standard_normal((300000, 5))
    got = cp.cumsum(cp.asarray(hd), axis=0).get()
    scale = np.cumsum(np.abs(hd), axis=0)
    assert (np.abs(got - np.cumsum(hd, axis=0)) <= 1e-13 * scale).all()
    hc = (rng.standard_normal((200001, 6)) + 1j * rng.standard_normal((200001, 6))).astype(np.complex64)
    got = cp.cumsum(cp.asarray(hc), axis=0).get()
    want = np.cumsum(hc.astype(np.complex128), axis=0)
    scale = np.cumsum(np.abs(hc).astype(np.float64), axis=0)
    assert (np.abs(got - want) <= 1e-5 * scale + 1e-5).all()
    hp = np.ones((400000, 4), np.int64)
    hp[rng.choice(400000, 30, replace=False), rng.integers(0, 4, 30)] = rng.choice([-1, 2], 30)
    assert_exact(cp.cumprod(cp.asarray(hp), axis=0).get(), np.cumprod(hp, axis=0))
    hn = rng.uniform(0, 1, (500000, 3)).astype(np.float32)
    hn[::777, 1] = np.nan
    got = cp.nancumsum(cp.asarray(hn), axis=0).get()
    want = np.nancumsum(hn.astype(np.float64), axis=0)
    assert (np.abs(got - want) <= 1e-5 * want + 1e-6).all()


def test_scans_on_two_streams_at_once():
    """Two one-pass scans in flight together share the CUs: tiles of either
    wait only for tiles of their own launch that started earlier, so both
    finish, and each stream has its own slots."""
    rng = np.random.default_rng(77)
    ha = rng.integers(-5, 6, (1 << 23) + 17).astype(np.int32)
    hb = rng.integers(-5, 6, (3, 1 << 22)).astype(np.int64)
    da, db = cp.asarray(ha), cp.asarray(hb)
    s1, s2 = cp.cuda.Stream(), cp.cuda.Stream()
    outs = []
    for _ in range(4):
        with s1:
            ra = da.cumsum()
        with s2:
            rb = db.cumsum(axis=1)
        outs.append((ra, rb))
    s1.synchronize()
    s2.synchronize()
    for ra, rb in outs:
        assert_exact(ra.get(), ha.cumsum())
        assert_exact(rb.get(), hb.cumsum(axis=1))
    # nothing gave up on the way
    d = cp.asarray(ha)
    assert 'cupy_scan_chain' in launched(lambda: d.cumsum())


# ---- many long columns: tiles of rows x columns, totals published per column

def within(got, want, bound):
    off = np.abs(got - want) > bound
    if off.any():
        where = np.argwhere(off)
        first = tuple(where[0])
        raise AssertionError('%d values out of bound, first at %s: got %r, expected %r; rows %s, '
                             'columns %s' % (len(where), first, got[first], want[first],
                                             sorted(set(where[:, -2].tolist()))[:8],
                                             sorted(set(where[:, -1].tolist()))[:8]))


@pytest.mark.parametrize('shape,axis', [
    ((8192, 2048), 0),            # whole blocks of columns, whole tiles of rows
    ((5000, 1000), 0),            # ragged on both sides
    ((3, 3001, 516), 1),          # several slices
    ((70001, 100), 0),            # many tiles down a column, the last block of columns part empty
    ((1029, 4098), 0),            # the last tile holds few rows
    ((40000, 37), 0),             # odd row length: the last vector of a row overlaps its neighbour
    ((9001, 2113), 0),            # ... with enough blocks of columns for a band per compute die
    ((2, 5003, 2051), 1),
    ((20001, 65), 0),             # ... a block of columns with a single column
    ((130, 511, 509), 1),         # slices of a few hundred odd rows: tiles of 256 rows
])
def test_many_long_columns_in_one_pass(shape, axis):
    rng = np.random.default_rng(shape[-1])
    h = rng.integers(-5, 6, shape).astype(np.int32)
    d = cp.asarray(h)
    assert launched(lambda: d.cumsum(axis=axis))[-1] == 'cupy_scan_chain_cols'
    assert_exact(d.cumsum(axis=axis).get(), h.cumsum(axis=axis))
    # in place (no overlapping vectors then), and with the bands and the
    # overlapping vectors switched off
    e = d.copy()
    cp.cumsum(e, axis=axis, out=e)
    assert_exact(e.get(), h.cumsum(axis=axis, dtype=np.int32))
    _tuning.set(scan_chain_cols_xcd=False, scan_chain_cols_unaligned=False)
    assert_exact(d.cumsum(axis=axis).get(), h.cumsum(axis=axis))
    _tuning.set(scan_chain_cols_xcd=True, scan_chain_cols_unaligned=True)
    assert_exact(d.cumsum(axis=axis).get(), h.cumsum(axis=axis))
    _tuning.set(scan_chain_cols_xcd='auto')
    hf = rng.uniform(0, 1, shape).astype(np.float32)
    df = cp.asarray(hf)
    got = df.cumsum(axis=axis).get()
    want = np.cumsum(hf.astype(np.float64), axis=axis)
    assert (np.abs(got - want) <= 1e-5 * want + 1e-6).all()
    assert_exact(df.cumsum(axis=axis).get(), got)                 # same bits on every run
    other = three_pass(lambda: df.cumsum(axis=axis).get())
    assert (np.abs(got - other) <= 2e-5 * want + 1e-6).all()


@pytest.mark.parametrize('waves,trips,vec_bytes', [(16, 0, 0), (8, 8, 16), (2, 64, 4), (16, 4, 8),
                                                   (4, 16, 8)])
def test_long_columns_other_types_and_tile_shapes(waves, trips, vec_bytes):
    _tuning.set(scan_chain_cols_waves=waves, scan_chain_cols_trips=trips,
                scan_chain_cols_vec_bytes=vec_bytes)
    rng = np.random.default_rng(waves * 100 + trips)
    h8 = rng.integers(-100, 100, (30001, 200)).astype(np.int8)
    d8 = cp.asarray(h8)
    assert launched(lambda: cp.cumsum(d8, axis=0))[-1] == 'cupy_scan_chain_cols'
    assert_exact(cp.cumsum(d8, axis=0).get(), np.cumsum(h8, axis=0))
    hd = rng.standard_normal((9000, 300))
    got = cp.cumsum(cp.asarray(hd), axis=0).get()
    within(got, np.cumsum(hd, axis=0), 1e-13 * np.cumsum(np.abs(hd), axis=0))
    hc = (rng.standard_normal((2, 7001, 130)) + 1j * rng.standard_normal((2, 7001, 130)))
    got = cp.cumsum(cp.asarray(hc), axis=1).get()
    within(got, np.cumsum(hc, axis=1), 1e-13 * np.cumsum(np.abs(hc), axis=1))
    hh = rng.uniform(0, 1, (6000, 256)).astype(np.float16)
    got = cp.cumsum(cp.asarray(hh), axis=0).get().astype(np.float64)
    want = np.cumsum(hh.astype(np.float64), axis=0)
    assert (np.abs(got - want) <= 2e-3 * want + 1e-3).all()
    hp = np.ones((20000, 96), np.int64)
    hp[rng.choice(20000, 30, replace=False), rng.integers(0, 96, 30)] = rng.choice([-1, 2], 30)
    assert_exact(cp.cumprod(cp.asarray(hp), axis=0).get(), np.cumprod(hp, axis=0))
    hn = rng.uniform(0, 1, (25000, 160)).astype(np.float32)
    hn[::777, 1::7] = np.nan
    got = cp.nancumsum(cp.asarray(hn), axis=0).get()
    want = np.nancumsum(hn.astype(np.float64), axis=0)
    assert (np.abs(got - want) <= 1e-5 * want + 1e-6).all()
    # negative zeros survive: nothing is added to the first row
    hz = np.full((5000, 128), -0.0, np.float32)
    assert_exact(cp.cumsum(cp.asarray(hz), axis=0).get(), np.cumsum(hz, axis=0))
    # a view that starts off the 16-byte grid
    hv = rng.integers(-5, 6, 4000 * 256 + 1).astype(np.int32)
    assert_exact(cp.asarray(hv)[1:].reshape(4000, 256).cumsum(axis=0).get(),
                 hv[1:].reshape(4000, 256).cumsum(axis=0))


def test_a_reported_scan_raises_on_the_next_scan_and_retires_the_kernel():
    """The twin of the reduction's test: the host writes what a tile that gave
    up would have written (every kernel exits normally); the next scan raises,
    later ones take three passes."""
    import ctypes
    rng = np.random.default_rng(12)
    h = rng.integers(-5, 6, 1 << 22).astype(np.int32)
    d = cp.asarray(h)
    assert 'cupy_scan_chain' in launched(lambda: d.cumsum())
    fault = _giveup.word(cp.cuda.Device().id, _giveup.SCAN)
    ctypes.c_uint32.from_address(fault).value = 1
    try:
        with pytest.raises(RuntimeError, match='gave up waiting'):
            d.cumsum()
    finally:
        ctypes.c_uint32.from_address(fault).value = 0
    names = launched(lambda: d.cumsum())
    assert 'cupy_scan_chain' not in names and 'cupy_scan_rows_seeded' in names
    assert_exact(d.cumsum().get(), h.cumsum())


def test_a_column_tile_that_gives_up_is_reported():
    rng = np.random.default_rng(8)
    h = rng.integers(-5, 6, (1 << 15, 512)).astype(np.int32)
    d = cp.asarray(h)
    _tuning.set(scan_chain_spin_limit=0)
    d.cumsum(axis=0)
    with pytest.raises(RuntimeError, match='gave up waiting'):
        cp.cuda.Device().synchronize()
    _tuning.set(scan_chain_spin_limit=1 << 18)
    names = launched(lambda: d.cumsum(axis=0))
    assert 'cupy_scan_chain_cols' not in names
    assert_exact(d.cumsum(axis=0).get(), h.cumsum(axis=0))


def test_slots_of_a_new_stream_start_cleared_whatever_the_memory_held():
    """The first launch on a stream gets fresh memory for its published
    totals, which must be cleared whole: here the pool hands back a block
    filled with what looks like totals marked with the number of that very
    launch."""
    rng = np.random.default_rng(21)
    h = rng.integers(-5, 6, (20000, 512)).astype(np.int32)
    d = cp.asarray(h)
    _scan._chain_arenas.clear()
    assert launched(lambda: d.cumsum(axis=0))[-1] == 'cupy_scan_chain_cols'
    (arena,) = _scan._chain_arenas.values()
    words = arena[0].size
    del arena
    cp.cuda.Device().synchronize()
    _scan._chain_arenas.clear()
    junk = cp.empty(words // 2, np.uint64)
    junk[...] = (1 << 32) | 0x12345678
    cp.cuda.Device().synchronize()
    del junk
    assert_exact(d.cumsum(axis=0).get(), h.cumsum(axis=0))
    (arena,) = _scan._chain_arenas.values()
    assert arena[1] == 1 and arena[0].size == words
