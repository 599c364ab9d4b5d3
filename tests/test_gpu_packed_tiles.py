"""Elementwise kernels whose tiles span several axes (``emit_packed``): arrays
of three and four axes permuted differently, small trailing axes, broadcast
operands, mixed types, views.  Every result is compared with NumPy's."""
import itertools

import numpy as np
import pytest

import cupy_amd as cp
from cupy_amd._core import _tuning

pytestmark = pytest.mark.gpu


@pytest.fixture(autouse=True)
def _restore_settings():
    yield
    _tuning.set(packed_tiles='auto', packed_xcd='auto', packed_tiles_below=2048,
                order_by_outputs=True, packed_short_rows_bytes=64)


def _values(shape, dtype, seed=0):
    rng = np.random.default_rng(seed)
    dtype = np.dtype(dtype)
    if dtype.kind == 'c':
        return (rng.integers(-99, 100, size=shape) + 1j * rng.integers(-99, 100, size=shape)).astype(dtype)
    if dtype.kind == 'b':
        return rng.integers(0, 2, size=shape).astype(dtype)
    return rng.integers(0 if dtype.kind == 'u' else -99, 100, size=shape).astype(dtype)


SHAPES_3D = [(1000, 4, 3), (777, 3, 4), (333, 2, 2), (70, 8, 8), (41, 16, 16), (9, 33, 31),
             (5, 130, 7), (64, 5, 129), (3, 257, 65), (129, 1, 66), (2, 3, 4099)]
SHAPES_4D = [(5, 12, 44, 4), (17, 36, 12, 2), (3, 17, 100, 2), (9, 7, 5, 3), (2, 24, 45, 15),
             (42, 6, 4, 29), (31, 67, 2, 4), (10, 4, 43, 10), (2, 2, 2, 513), (33, 1, 2, 65)]


@pytest.mark.parametrize('mode', [True, 'auto'])
@pytest.mark.parametrize('dtype', ['float32', 'float16', 'int64', 'uint8', 'complex128'])
def test_permuted_copies_of_three_axes(dtype, mode):
    _tuning.set(packed_tiles=mode)
    for shape in SHAPES_3D:
        h = _values(shape, dtype)
        d = cp.asarray(h)
        for perm in itertools.permutations(range(3)):
            got = cp.ascontiguousarray(d.transpose(perm))
            np.testing.assert_array_equal(got.get(), np.ascontiguousarray(h.transpose(perm)),
                                          err_msg='%s %s %s' % (dtype, shape, perm))


@pytest.mark.parametrize('mode', [True, 'auto'])
@pytest.mark.parametrize('dtype', ['float32', 'float64', 'int8', 'complex64'])
def test_permuted_copies_of_four_axes(dtype, mode):
    _tuning.set(packed_tiles=mode)
    for shape in SHAPES_4D:
        h = _values(shape, dtype)
        d = cp.asarray(h)
        for perm in itertools.permutations(range(4)):
            got = cp.ascontiguousarray(d.transpose(perm))
            np.testing.assert_array_equal(got.get(), np.ascontiguousarray(h.transpose(perm)),
                                          err_msg='%s %s %s' % (dtype, shape, perm))


def test_permuted_copies_of_five_and_six_axes():
    rng = np.random.default_rng(11)
    for shape in [(3, 4, 5, 6, 7), (2, 3, 2, 65, 4), (5, 1, 7, 3, 33), (2, 3, 4, 5, 3, 4), (3, 2, 2, 17, 2, 9)]:
        nd = len(shape)
        for dtype in ('float32', 'int16', 'complex128'):
            h = _values(shape, dtype)
            d = cp.asarray(h)
            for trial in range(12):
                perm = tuple(int(p) for p in rng.permutation(nd))
                got = cp.ascontiguousarray(d.transpose(perm))
                np.testing.assert_array_equal(got.get(), np.ascontiguousarray(h.transpose(perm)),
                                              err_msg='%s %s %s' % (dtype, shape, perm))
                hb = _values(shape, dtype, 7).transpose(perm)
                got = d.transpose(perm) - cp.asarray(np.ascontiguousarray(hb))
                np.testing.assert_array_equal(got.get(), h.transpose(perm) - hb)


@pytest.mark.parametrize('mode', [True, 'auto'])
def test_binary_operations_on_differently_permuted_operands(mode):
    _tuning.set(packed_tiles=mode)
    rng = np.random.default_rng(5)
    for shape in SHAPES_3D[:8] + SHAPES_4D[:8]:
        nd = len(shape)
        for trial in range(6):
            pa = tuple(int(p) for p in rng.permutation(nd))
            pb = tuple(int(p) for p in rng.permutation(nd))
            ta, tb = ('float32', 'float64', 'int32', 'float16')[trial % 4], ('float32', 'int8')[trial % 2]
            # arrays stored in other orders, seen in the common shape
            ha = _values(tuple(shape[p] for p in np.argsort(pa)), ta, 1).transpose(pa)
            hb = _values(tuple(shape[p] for p in np.argsort(pb)), tb, 2).transpose(pb)
            assert ha.shape == shape and hb.shape == shape
            da = cp.asarray(np.ascontiguousarray(ha.transpose(np.argsort(pa)))).transpose(pa)
            db = cp.asarray(np.ascontiguousarray(hb.transpose(np.argsort(pb)))).transpose(pb)
            assert da.strides == ha.strides and db.strides == hb.strides
            got = da * 2 + db
            want = ha * 2 + hb
            assert got.dtype == want.dtype
            np.testing.assert_array_equal(got.get(), want, err_msg='%s %s %s' % (shape, pa, pb))
            got = cp.subtract(da, db)
            np.testing.assert_array_equal(got.get(), np.subtract(ha, hb))


@pytest.mark.parametrize('mode', [True, 'auto'])
def test_broadcast_operands_and_views(mode):
    _tuning.set(packed_tiles=mode)
    h = _values((60, 9, 14, 6), 'float32')
    d = cp.asarray(h)
    for perm in [(0, 2, 1, 3), (3, 1, 0, 2), (1, 3, 2, 0)]:
        ht, dt = h.transpose(perm), d.transpose(perm)
        for axis in range(4):
            shape = list(ht.shape)
            shape[axis] = 1
            hb = _values(tuple(shape), 'float32', 3)
            np.testing.assert_array_equal((dt + cp.asarray(hb)).get(), ht + hb)
        # views: offsets, steps, a reversed axis
        hv, dv = ht[1:, ::2, :, 1:-1], dt[1:, ::2, :, 1:-1]
        np.testing.assert_array_equal((dv * 3).get(), hv * 3)
        hv, dv = ht[::-1, :, ::-1], dt[::-1, :, ::-1]
        np.testing.assert_array_equal(cp.ascontiguousarray(dv).get(), np.ascontiguousarray(hv))
        # into a given output, itself a view
        out = cp.zeros((ht.shape[0] + 2,) + ht.shape[1:], 'float64')
        cp.add(dt, 1, out=out[1:-1])
        want = np.zeros(out.shape)
        want[1:-1] = ht + 1
        np.testing.assert_array_equal(out.get(), want)


def test_tiles_numbered_die_by_die_or_not():
    h = _values((37, 61, 67), 'float32')
    d = cp.asarray(h)
    for xcd in (True, False):
        _tuning.set(packed_tiles=True, packed_xcd=xcd)
        for perm in [(0, 2, 1), (2, 1, 0), (1, 2, 0)]:
            np.testing.assert_array_equal(cp.ascontiguousarray(d.transpose(perm)).get(),
                                          np.ascontiguousarray(h.transpose(perm)))


def test_large_batches_of_small_matrices_transposed():
    # what tiles of two axes would take one tile per matrix for
    for shape, dtype in [((300001, 4, 3), 'float16'), ((100003, 8, 8), 'float32'),
                         ((200001, 2, 2), 'float64'), ((3, 200001, 4), 'float32')]:
        h = _values(shape, dtype)
        d = cp.asarray(h)
        perm = (0, 2, 1) if shape[0] > 3 else (2, 1, 0)
        np.testing.assert_array_equal(cp.ascontiguousarray(d.transpose(perm)).get(),
                                      np.ascontiguousarray(h.transpose(perm)))
        np.testing.assert_array_equal((d.transpose(perm) + d.transpose(perm)).get(),
                                      h.transpose(perm) * 2)


@pytest.mark.parametrize('by_outputs', [True, False])
def test_permuted_destinations(by_outputs):
    _tuning.set(order_by_outputs=by_outputs)
    rng = np.random.default_rng(3)
    for shape in [(37, 9, 14, 4), (120, 5, 33), (6, 7, 8, 9, 3), (2, 300, 4, 3)]:
        nd = len(shape)
        h = _values(shape, 'float32')
        d = cp.asarray(h)
        for trial in range(8):
            perm = tuple(int(p) for p in rng.permutation(nd))
            base = cp.zeros(tuple(shape[p] for p in np.argsort(perm)), 'float64')
            dst = base.transpose(perm)
            assert dst.shape == shape
            cp.copyto(dst, d)
            np.testing.assert_array_equal(base.get(), np.ascontiguousarray(h.transpose(np.argsort(perm))),
                                          err_msg='%s %s' % (shape, perm))
            # two inputs stored in other orders again, written into the permuted destination
            other = tuple(int(p) for p in rng.permutation(nd))
            hb = _values(tuple(shape[p] for p in np.argsort(other)), 'float32', 9).transpose(other)
            db = cp.asarray(np.ascontiguousarray(hb.transpose(np.argsort(other)))).transpose(other)
            cp.multiply(d, db, out=dst)
            np.testing.assert_array_equal(dst.get(), h * hb)


def test_a_value_per_row_under_pieces_of_several_rows():
    for shape, dtype in [((3, 15983, 7), 'float32'), ((4001, 5, 3), 'float64'), ((2, 9, 1001, 6), 'float16')]:
        h = _values(shape, dtype)
        d = cp.asarray(h)
        for axis in range(len(shape) - 1):
            mshape = [1] * len(shape)
            mshape[axis] = shape[axis]
            hm = _values(tuple(mshape), dtype, 4)
            dm = cp.asarray(hm)
            np.testing.assert_array_equal((d - dm).get(), h - hm)
            fused = cp.fuse(lambda a, b, c: (a - b) * c)
            np.testing.assert_array_equal(fused(d, dm, dm).get(), (h - hm) * hm)
            # one value per row of the two last axes together
            mshape[-1] = shape[-1]
            hm = _values(tuple(mshape), dtype, 5)
            np.testing.assert_array_equal((d + cp.asarray(hm)).get(), h + hm)


def test_windows_of_narrow_matrices_of_small_elements():
    for dtype in ('uint8', 'float16', 'int16', 'bool'):
        for shape in [(100003, 6), (50001, 13), (33333, 31), (70001, 2)]:
            h = _values(shape, dtype)
            d = cp.asarray(h)
            if dtype == 'bool':
                np.testing.assert_array_equal((d[:-1, :-1] ^ d[1:, 1:]).get(), h[:-1, :-1] ^ h[1:, 1:])
            else:
                np.testing.assert_array_equal((d[:-1, :-1] - d[1:, 1:]).get(), h[:-1, :-1] - h[1:, 1:])
            np.testing.assert_array_equal((d[:, 1:] + d[:, :-1]).get(), h[:, 1:] + h[:, :-1])
            out = cp.zeros((shape[0], shape[1] + 2), dtype)
            cp.copyto(out[:, 1:-1], d)
            want = np.zeros((shape[0], shape[1] + 2), dtype)
            want[:, 1:-1] = h
            np.testing.assert_array_equal(out.get(), want)
