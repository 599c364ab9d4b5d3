"""Joining, splitting, tiling and rolling against NumPy on the same inputs
(reference tests: tests/cupy_tests/manipulation_tests/test_join.py,
test_split.py, test_tiling.py, test_rearrange.py restated over NumPy)."""
import itertools

import numpy as np
import pytest

import cupy_amd as cp

pytestmark = pytest.mark.gpu


def pair(shape, dtype='float32', seed=0):
    rng = np.random.default_rng(seed)
    h = rng.integers(-5, 6, size=shape).astype(dtype)
    return h, cp.asarray(h)


def same(got, want):
    assert isinstance(got, cp.ndarray)
    assert got.shape == want.shape and got.dtype == want.dtype
    assert np.array_equal(got.get(), want)


@pytest.mark.parametrize('axis', [0, 1, 2, -1, None])
def test_concatenate_axes_and_views(axis):
    ha, da = pair((4, 5, 6), seed=1)
    hb, db = pair((4, 5, 6), seed=2)
    same(cp.concatenate([da, db], axis=axis), np.concatenate([ha, hb], axis=axis))
    # transposed, stepped and broadcast pieces
    hs = [ha.transpose(2, 1, 0), hb.transpose(2, 1, 0)[::-1], np.broadcast_to(hb[0, 0][:, None, None], (6, 5, 4))]
    ds = [da.transpose(2, 1, 0), db.transpose(2, 1, 0)[::-1], cp.broadcast_to(db[0, 0][:, None, None], (6, 5, 4))]
    same(cp.concatenate(ds, axis=axis), np.concatenate(hs, axis=axis))


def test_concatenate_ragged_mixed_types_out_and_empty():
    hs = [pair((n, 7), dt, seed=n)[0] for n, dt in ((3, 'int8'), (0, 'float32'), (5, 'float64'), (1, 'uint16'))]
    ds = [cp.asarray(h) for h in hs]
    same(cp.concatenate(ds), np.concatenate(hs))
    same(cp.concatenate(ds, dtype=np.float32), np.concatenate(hs, dtype=np.float32))
    out = cp.empty((9, 7), np.float64)
    assert cp.concatenate(ds, out=out) is out
    same(out, np.concatenate(hs).astype(np.float64))
    # into a window of a larger array
    big = cp.zeros((11, 9), np.float64)
    cp.concatenate(ds, out=big[1:-1, 1:-1])
    want = np.zeros((11, 9))
    want[1:-1, 1:-1] = np.concatenate(hs)
    same(big, want)
    with pytest.raises(TypeError):
        cp.concatenate(ds, dtype=np.int8)
    same(cp.concatenate(ds, dtype=np.int8, casting='unsafe'), np.concatenate(hs, dtype=np.int8, casting='unsafe'))
    with pytest.raises(TypeError):
        cp.concatenate(ds, out=out, dtype=np.float64)
    with pytest.raises(ValueError):
        cp.concatenate(ds, out=cp.empty((9, 8), np.float64))
    with pytest.raises(ValueError):
        cp.concatenate([])
    with pytest.raises(TypeError):
        cp.concatenate([ds[0], hs[1]])
    with pytest.raises(np.exceptions.AxisError):
        cp.concatenate(ds, axis=2)


def test_concatenate_many_large_pieces():
    rng = np.random.default_rng(5)
    hs = [rng.standard_normal((rng.integers(1, 3000), 513), dtype=np.float32) for _ in range(40)]
    ds = [cp.asarray(h) for h in hs]
    same(cp.concatenate(ds), np.concatenate(hs))
    hs = [h[:1, :].T for h in hs]
    ds = [d[:1, :].T for d in ds]
    same(cp.concatenate(ds, axis=1), np.concatenate(hs, axis=1))


def test_stack_family():
    ha, da = pair((3, 4), seed=1)
    hb, db = pair((3, 4), 'int16', seed=2)
    for axis in (0, 1, 2, -1, -3):
        same(cp.stack([da, db], axis=axis), np.stack([ha, hb], axis=axis))
    same(cp.stack([da, db], dtype=np.float64), np.stack([ha, hb], dtype=np.float64))
    out = cp.empty((3, 2, 4), np.float32)
    assert cp.stack([da, db], axis=1, out=out) is out
    same(out, np.stack([ha, hb], axis=1).astype(np.float32))
    with pytest.raises(ValueError):
        cp.stack([da, db[:2]])
    with pytest.raises(np.exceptions.AxisError):
        cp.stack([da, db], axis=3)
    same(cp.hstack([da, db]), np.hstack([ha, hb]))
    same(cp.vstack([da, db]), np.vstack([ha, hb]))
    same(cp.row_stack([da, db[0]]), np.vstack([ha, hb[0]]))
    same(cp.dstack([da, db]), np.dstack([ha, hb]))
    same(cp.hstack([da[0], db[1]]), np.hstack([ha[0], hb[1]]))
    same(cp.vstack([da[0], db[1]]), np.vstack([ha[0], hb[1]]))
    same(cp.dstack([da[0], db[1]]), np.dstack([ha[0], hb[1]]))
    same(cp.column_stack([da[:, 0], db, da[:, 1]]), np.column_stack([ha[:, 0], hb, ha[:, 1]]))
    with pytest.raises(ValueError):
        cp.column_stack([da.reshape(3, 2, 2)])
    same(cp.hstack([da, db], dtype=np.float64), np.hstack([ha, hb], dtype=np.float64))


@pytest.mark.parametrize('sections', [1, 2, 3, 5, 7, [2, 4], [4, 2], [-2], [0, 3, 3, 20], []])
@pytest.mark.parametrize('axis', [0, 1, -1])
def test_array_split_gives_numpy_pieces_as_views(sections, axis):
    h, d = pair((6, 6, 6))
    got = cp.array_split(d, sections, axis)
    want = np.array_split(h, sections, axis)
    assert len(got) == len(want)
    for g, w in zip(got, want):
        same(g, w)
    if got and got[0].size:
        got[0][...] = 99           # a view: the base sees it
        h2 = h.copy()
        np.array_split(h2, sections, axis)[0][...] = 99
        same(d, h2)


def test_split_variants_and_errors():
    h, d = pair((4, 6, 8))
    for fn, arg in (('split', 2), ('hsplit', 3), ('vsplit', 2), ('dsplit', [1, 5]), ('hsplit', [2])):
        for g, w in zip(getattr(cp, fn)(d, arg), getattr(np, fn)(h, arg)):
            same(g, w)
    for g, w in zip(cp.hsplit(d[0, 0], 4), np.hsplit(h[0, 0], 4)):
        same(g, w)
    with pytest.raises(ValueError):
        cp.split(d, 3)
    with pytest.raises(IndexError):
        cp.split(d, 2, axis=3)
    with pytest.raises(ValueError):
        cp.vsplit(d[0, 0], 2)
    with pytest.raises(ValueError):
        cp.dsplit(d[0], 2)
    with pytest.raises(ValueError):
        cp.array_split(d, 0)


@pytest.mark.parametrize('reps', [2, (2, 3), (2, 1, 2), (1, 1), (0, 2), (3, 1, 1, 2)])
def test_tile(reps):
    h, d = pair((3, 5), 'int32')
    same(cp.tile(d, reps), np.tile(h, reps))
    same(cp.tile(d.T, reps), np.tile(h.T, reps))
    same(cp.tile(d[0, 0], reps), np.tile(h[0, 0], reps))


@pytest.mark.parametrize('axis', [None, 0, 1, -1])
def test_repeat(axis):
    h, d = pair((4, 5), 'float64')
    same(cp.repeat(d, 3, axis), np.repeat(h, 3, axis))
    same(cp.repeat(d.T, 2, axis), np.repeat(h.T, 2, axis))
    same(cp.repeat(d, 0, axis), np.repeat(h, 0, axis))
    same(cp.repeat(d, [2], axis), np.repeat(h, [2], axis))
    n = h.size if axis is None else h.shape[axis]
    counts = [(3 * i) % 4 for i in range(n)]
    same(cp.repeat(d, counts, axis), np.repeat(h, counts, axis))
    with pytest.raises(ValueError):
        cp.repeat(d, [1, 2], axis)
    with pytest.raises(ValueError):
        cp.repeat(d, -1, axis)


def test_roll_and_quarter_turns():
    h, d = pair((5, 6, 7))
    from cupy_amd._core import _tuning
    hw, dw = pair((40, 3, 129), 'float64', seed=3)      # rows that end in partial vectors
    try:
        for on in (True, False):
            _tuning.set(concatenate_one_launch=on)
            for shift, axis in [(1, None), (-3, None), (0, None), (212, None), (2, 0), (-1, 2), (9, 1),
                                ((1, 2), (0, 1)), ((1, -2, 3), (0, 1, 2)), (3, (0, 2)), ((1, 1), (1, 1))]:
                same(cp.roll(d, shift, axis), np.roll(h, shift, axis))
                same(cp.roll(dw, shift, axis), np.roll(hw, shift, axis))
    finally:
        _tuning.set(concatenate_one_launch=True)
    same(cp.roll(d.transpose(2, 0, 1), 3, 1), np.roll(h.transpose(2, 0, 1), 3, 1))
    with pytest.raises(np.exceptions.AxisError):
        cp.roll(d, 1, 3)
    for k, axes in itertools.product(range(-1, 5), [(0, 1), (1, 0), (0, 2), (-1, 0)]):
        same(cp.ascontiguousarray(cp.rot90(d, k, axes)), np.ascontiguousarray(np.rot90(h, k, axes)))
    with pytest.raises(ValueError):
        cp.rot90(d, 1, (0, 0))
    with pytest.raises(ValueError):
        cp.rot90(d[0, 0])


@pytest.mark.parametrize('dtype', ['int8', 'float16', 'float32', 'float64', 'complex128'])
def test_one_launch_and_piecewise_concatenation_agree(dtype):
    """Layouts the one-launch kernel takes (windows with contiguous rows, whole
    arrays, many ragged pieces), with the kernel on and off."""
    from cupy_amd._core import _tuning
    rng = np.random.default_rng(11)
    hbase = rng.integers(-9, 10, size=(37, 21, 130)).astype(dtype)
    dbase = cp.asarray(hbase)
    cases = [
        ([np.s_[:], np.s_[3:9], np.s_[30:]], 0),
        ([np.s_[:, 1:], np.s_[:, :3], np.s_[:, 5:6]], 1),
        ([np.s_[:, :, :64], np.s_[:, :, 65:], np.s_[:, :, 1:128]], 2),
        ([np.s_[::2, :, 2:], np.s_[1:19, :, :128]], 0),
        ([np.s_[i:i + 1 + i % 3] for i in range(0, 36, 2)], 0),
        ([np.s_[:, :, 3:]] * 9, -1),
    ]
    try:
        for slices, axis in cases:
            want = np.concatenate([hbase[s] for s in slices], axis=axis)
            for on in (True, False):
                _tuning.set(concatenate_one_launch=on)
                same(cp.concatenate([dbase[s] for s in slices], axis=axis), want)
            big = cp.zeros(tuple(e + 2 for e in want.shape), dtype)
            inner = tuple(slice(1, -1) for _ in want.shape)
            _tuning.set(concatenate_one_launch=True)
            cp.concatenate([dbase[s] for s in slices], axis=axis, out=big[inner])
            hbig = np.zeros(big.shape, dtype)
            hbig[inner] = want
            same(big, hbig)
    finally:
        _tuning.set(concatenate_one_launch=True)


@pytest.mark.parametrize('dtype', ['int8', 'float32', 'complex128'])
def test_tile_and_repeat_through_the_pieces_kernel(dtype):
    """Rows of 64 bytes and more: the tiles and the repeated rows are stored
    from the registers that hold the source (kernel on), or by a broadcast
    copy (kernel off); both must give NumPy's result."""
    from cupy_amd._core import _tuning
    rng = np.random.default_rng(4)
    h = rng.integers(-9, 10, size=(6, 5, 64)).astype(dtype)
    d = cp.asarray(h)
    try:
        for on in (True, False):
            _tuning.set(concatenate_one_launch=on)
            for reps in (2, (2, 3), (3, 1, 2), (1, 4, 1), (2, 2, 2), (5, 1, 1, 1), (70, 1, 1)):
                same(cp.tile(d, reps), np.tile(h, reps))
            same(cp.tile(d[:, 1:3, 8:], (2, 2, 2)), np.tile(h[:, 1:3, 8:], (2, 2, 2)))
            same(cp.tile(d[0, 0], 7), np.tile(h[0, 0], 7))
            for axis in (0, 1):
                same(cp.repeat(d, 3, axis), np.repeat(h, 3, axis))
                same(cp.repeat(d[1:, :, 16:], 2, axis), np.repeat(h[1:, :, 16:], 2, axis))
            same(cp.repeat(d, 1, 0), np.repeat(h, 1, 0))
    finally:
        _tuning.set(concatenate_one_launch=True)
