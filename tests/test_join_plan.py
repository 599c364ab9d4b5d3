"""The one-launch concatenation kernel on the host: its argument tables are
replayed in NumPy the way the kernel walks them (workgroup -> piece by the
table of first workgroups, thread -> vector, vector -> row and column), every
access is checked against the bounds of the buffers first, and the result must
be NumPy's concatenation."""
import numpy as np
import pytest

from cupy_amd import _join

# struct Piece of the kernel source
PIECE = np.dtype([('src', np.uint64), ('dst', np.uint64), ('src_pitch', np.int64),
                  ('dst_pitch', np.int64), ('vecs_per_row', np.uint32), ('n_vecs', np.uint32),
                  ('first_block', np.uint32), ('n_rep', np.uint32), ('rep_step', np.int64),
                  ('row_len', np.uint32), ('pad', np.uint32)])


def describe(pairs):
    return [(s.shape, s.strides, s.ctypes.data, d.strides, d.ctypes.data) for s, d in pairs]


def replay(pairs, sbase, dbase, copies=1, copy_step=0):
    """Runs the kernel's arithmetic over host buffers.  Returns False if the
    planner declines the pairs."""
    plan = _join._plan_pieces(describe(pairs), pairs[0][1].dtype, copies, copy_step)
    if plan is None:
        return False
    word, nv, forms = plan
    s0, d0 = sbase.ctypes.data, dbase.ctypes.data
    sw, dw = sbase.reshape(-1).view(np.uint8), dbase.reshape(-1).view(np.uint8)
    block, unroll = _join._geometry()
    per_block = block * unroll
    for table, n_pieces, blocks in _join._piece_tables(nv, forms):
        assert len(table) == 64 * _join._MAX_PIECES and n_pieces <= _join._MAX_PIECES
        table = np.frombuffer(table, PIECE)
        firsts = [int(table[k]['first_block']) for k in range(n_pieces)]
        assert firsts == sorted(firsts) and firsts[0] == 0
        for block in range(blocks):
            k = max(j for j in range(n_pieces) if block >= firsts[j])
            pc = table[k]
            local = np.arange(per_block, dtype=np.int64) + (block - firsts[k]) * per_block
            local = local[local < int(pc['n_vecs'])]
            assert local.size, 'a workgroup without work'
            r = local // int(pc['vecs_per_row'])
            c = (local - r * int(pc['vecs_per_row'])) * nv
            assert int(pc['vecs_per_row']) == -(-int(pc['row_len']) // nv)
            have = np.minimum(int(pc['row_len']) - c, nv)     # the last vector of a row may be partial
            assert have.min() >= 1
            src = int(pc['src']) - s0 + (r * int(pc['src_pitch']) + c) * word
            dst = int(pc['dst']) - d0 + (r * int(pc['dst_pitch']) + c) * word
            assert src.min() >= 0 and (src + have * word).max() <= sw.size
            for j in range(int(pc['n_rep'])):
                at = dst + j * int(pc['rep_step']) * word
                assert at.min() >= 0 and (at + have * word).max() <= dw.size
                for b in range(nv * word):
                    inside = b < have * word
                    dw[at[inside] + b] = sw[src[inside] + b]
        # every vector of every piece has a workgroup
        assert blocks == sum(-(-int(table[k]['n_vecs']) // per_block) for k in range(n_pieces))
    return True


CASES = [
    # (shape of the base, slices of the pieces, axis, dtype)
    ((64, 96), [np.s_[:, :48], np.s_[:, 48:]], 0, 'float32'),
    ((64, 96), [np.s_[:32], np.s_[32:]], 1, 'float32'),
    ((64, 96), [np.s_[:40], np.s_[3:5], np.s_[40:]], 0, 'int8'),
    ((5, 6, 40), [np.s_[:, 1:], np.s_[:, :3]], 1, 'float64'),
    ((6, 6, 40), [np.s_[::2], np.s_[1::2]], 1, 'int16'),
    ((7, 3, 33), [np.s_[:], np.s_[2:4], np.s_[:1]], 0, 'complex128'),
    ((4, 5, 96), [np.s_[:, :, :32], np.s_[:, :, 33:80], np.s_[:, :, 64:]], 2, 'float16'),
    ((2050, 3), [np.s_[:1000], np.s_[1000:]], 0, 'uint8'),
    ((300, 17), [np.s_[i * 10:(i + 1) * 10 + (i % 3)] for i in range(19)], 0, 'float32'),
    ((33, 67), [np.s_[:, 1:], np.s_[:, :66]], 0, 'float32'),          # rows of 66: partial last vectors
    ((9, 70), [np.s_[:, :33], np.s_[:, 33:36], np.s_[:, 69:]], 1, 'int8'),   # rows of 33, 3 and 1 bytes
    ((50, 3), [np.s_[:, :2], np.s_[:, 2:]], 1, 'float64'),             # a small piece of narrow rows
]


@pytest.mark.parametrize('base_shape,slices,axis,dtype', CASES)
def test_tables_copy_what_numpy_concatenates(base_shape, slices, axis, dtype):
    rng = np.random.default_rng(0)
    sbase = rng.integers(0, 100, size=base_shape).astype(dtype)
    pieces = [sbase[s] for s in slices]
    want = np.concatenate(pieces, axis=axis)
    # the result sits inside a larger buffer so that an access past it is seen
    dbase = np.zeros((want.shape[0] + 2,) + want.shape[1:], dtype)
    out = dbase[1:-1]
    pairs, at = [], 0
    for p in pieces:
        ext = p.shape[axis]
        pairs.append((p, _join._window(out, axis, at, at + ext)))
        at += ext
    assert replay(pairs, sbase, dbase)
    assert np.array_equal(out, want)
    assert not dbase[0].any() and not dbase[-1].any()


def test_layouts_the_kernel_declines():
    def plan(pairs):
        return _join._plan_pieces(describe(pairs), pairs[0][1].dtype)

    base = np.zeros((40, 50), np.float32)
    out = np.zeros((80, 50), np.float32)
    assert plan([(base, out[:40]), (base, out[40:])]) is not None
    # transposed pieces, rows of a few elements, a single piece, reversed rows
    t = np.zeros((50, 80), np.float32)
    assert plan([(base.T, t[:, :40]), (base.T, t[:, 40:])]) is None
    narrow = np.zeros((100000, 3), np.float32)            # many rows of a few elements
    wide = np.zeros((100000, 6), np.float32)
    assert plan([(narrow, wide[:, :3]), (narrow, wide[:, 3:])]) is None
    assert plan([(base, out[:40])]) is None
    rev = base[::-1]
    assert plan([(rev, out[:40]), (rev, out[40:])]) is None
    rec = np.zeros((4, 50), np.dtype([('a', np.int32), ('b', np.float32)]))
    assert plan([(rec, rec), (rec, rec)]) is None


def test_row_decomposition():
    def rows(arr, lead):
        return _join._as_rows(arr.shape, arr.strides, arr.itemsize, lead)

    a = np.zeros((6, 8, 10), np.float32)
    assert rows(a, 0) == (1, 480, 480)
    assert rows(a, 1) == (6, 80, 80)
    assert rows(a[:, :4], 1) == (6, 40, 80)
    assert rows(a[:, :4], 0) is None
    assert rows(a[:, :, :5], 2) == (48, 5, 10)
    assert rows(a[::2], 1) == (3, 80, 160)
    assert rows(a[:, ::2], 1) is None
    assert rows(a[:, ::2], 2) == (24, 10, 20)
    assert rows(a[:, :3], 2) is None           # leading axes do not step evenly
    assert rows(a[:, :1], 1) == (6, 10, 80)
    assert rows(a.transpose(1, 0, 2), 2) is None
    assert rows(np.broadcast_to(a[:1], (3, 8, 10)), 1) is None


@pytest.mark.parametrize('shape,reps,dtype', [
    ((6, 32), (2, 3), 'float32'), ((6, 64), (3, 2), 'int8'), ((5, 4, 16), (2, 1, 4), 'float64'),
    ((40,), (7,), 'complex128'), ((3, 64), (1, 5), 'int16'),
])
def test_tiles_as_pieces_with_copies(shape, reps, dtype):
    rng = np.random.default_rng(1)
    sbase = rng.integers(0, 100, size=shape).astype(dtype)
    want = np.tile(sbase, reps)
    dbase = np.zeros((want.shape[0] + 2,) + want.shape[1:], dtype)
    out = dbase[1:-1]
    pair_shape = tuple(x for rs in zip(reps, shape) for x in rs)
    paired = out.reshape(pair_shape)
    assert np.shares_memory(paired, out)
    most = max(range(len(reps)), key=lambda k: reps[k])
    rep_strides, own = paired.strides[0::2], paired.strides[1::2]
    pairs = []
    for combo in np.ndindex(*[r if k != most else 1 for k, r in enumerate(reps)]):
        index = tuple(x for ci in combo for x in (ci, slice(None)))
        pairs.append((sbase, paired[index]))
        assert paired[index].strides == own
    assert replay(pairs, sbase, dbase, reps[most], rep_strides[most])
    assert np.array_equal(out, want)
    assert not dbase[0].any() and not dbase[-1].any()
