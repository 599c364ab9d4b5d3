"""Host helpers against the known-answer tables the reference's tests hold."""
import numpy as np
import pytest

from cupy_amd._core import internal
from cupy_amd._core.core import _reshape_strides, _basic_index
from oracle import numpy_oracle as o


def test_prod():
    assert internal.prod([]) == 1
    assert internal.prod([2]) == 2
    assert internal.prod((2, 3)) == 6


def test_get_size():
    assert internal.get_size([1, 2, 3]) == (1, 2, 3)
    assert internal.get_size((1, 2, 3)) == (1, 2, 3)
    assert internal.get_size(1) == (1,)
    assert internal.get_size(np.int32(1)) == (1,)
    assert internal.get_size(np.array(1)) == (1,)
    assert internal.get_size((np.int32(1), np.array(1))) == (1, 1)
    assert internal.get_size(1.0) == (1.0,)
    for value in (True, np.bool_(True), np.array(True, dtype='?')):
        with pytest.raises(TypeError):
            internal.get_size(value)
        with pytest.raises(TypeError):
            internal.get_size((value, value))


def test_vector_equal():
    assert internal.vector_equal([], []) is True
    assert internal.vector_equal([1, 2, 3], [1, 2, 0]) is False
    assert internal.vector_equal([-1, 0, 1], [-1, 0, 1]) is True
    assert internal.vector_equal([1, 2, 3], [1, 2]) is False


def test_clp2_table(golden):
    for x, expect in golden['clp2']:
        assert internal.clp2(x) == expect


def test_complete_slice_table(golden):
    for given, expect in golden['complete_slice_dim10']:
        assert internal.complete_slice(slice(*given), 10) == slice(*expect), given


def test_complete_slice_agrees_with_python_indexing():
    seq = list(range(10))
    for start in (None, -12, -10, -3, 0, 4, 9, 10, 13):
        for stop in (None, -12, -10, -3, 0, 4, 9, 10, 13):
            for step in (None, 1, 2, 3, -1, -2, -7):
                s = internal.complete_slice(slice(start, stop, step), 10)
                picked = []
                i = s.start
                while (i < s.stop) if s.step > 0 else (i > s.stop):
                    picked.append(seq[i])
                    i += s.step
                assert picked == seq[slice(start, stop, step)]


def test_complete_slice_errors():
    with pytest.raises(ValueError):
        internal.complete_slice(slice(1, 1, 0), 1)
    with pytest.raises(TypeError):
        internal.complete_slice(slice(1, 1, (1, 2)), 1)
    with pytest.raises(TypeError):
        internal.complete_slice(slice((1, 2), 1, 1), 1)
    with pytest.raises(TypeError):
        internal.complete_slice(slice(1, (1, 2), -1), 1)


def test_get_c_contiguity_table(golden):
    for shape, strides, itemsize, expect in golden['get_c_contiguity']:
        assert internal.get_c_contiguity(tuple(shape), tuple(strides), itemsize) is expect


def test_contiguity_matches_numpy_flags():
    base = np.zeros((4, 1, 6, 5), dtype=np.float32)
    views = [base, base.T, base[:, :, ::2], base[::2], base[:, :, :, ::-1],
             base.transpose(0, 2, 1, 3), base[1:2], base[:, :, 2:3, :]]
    for v in views:
        assert internal.get_c_contiguity(v.shape, v.strides, 4) == v.flags.c_contiguous
        assert internal.get_f_contiguity(v.shape, v.strides, 4) == v.flags.f_contiguous


def test_infer_unknown_dimension(golden):
    for shape, size, expect in golden['infer_unknown_dimension']:
        assert internal.infer_unknown_dimension(shape, size) == expect
    with pytest.raises(ValueError):
        internal.infer_unknown_dimension((-1, 1, -1), 10)


def test_reduced_dims_visit_same_addresses():
    base = np.zeros((3, 4, 5, 6), dtype=np.int16)
    views = [base, base[:, ::2], base.transpose(1, 0, 2, 3), base[:, :, ::-1],
             base[1:], base[:, :, :, 1:5], base.reshape(12, 30)[:, ::3],
             np.broadcast_to(base[:, :1], (3, 4, 5, 6))]
    for v in views:
        shape, strides = internal.get_reduced_dims(v.shape, v.strides, 2)
        assert len(shape) <= v.ndim
        assert np.array_equal(o.element_offsets(shape, strides),
                              o.element_offsets(v.shape, v.strides))


def test_normalize_axis():
    assert internal._normalize_axis_index(-1, 3) == 2
    with pytest.raises(np.exceptions.AxisError):
        internal._normalize_axis_index(3, 3)
    assert internal._normalize_axis_indices((2, -3), 3) == (0, 2)
    with pytest.raises(ValueError):
        internal._normalize_axis_indices((0, -3), 3)


def test_broadcast_shapes_match_numpy():
    cases = [((10,), (1,)), ((3, 1), (1, 4)), ((2, 1, 4), (3, 1)), ((0,), (1,)),
             ((256, 256), (256, 1)), ((), (3,)), ((5, 0, 1), (1, 7))]
    for shapes in cases:
        assert internal._broadcast_shapes(list(shapes)) == np.broadcast_shapes(*shapes)
    for bad in [((3,), (4,)), ((2, 3), (3, 2))]:
        with pytest.raises(ValueError):
            internal._broadcast_shapes(list(bad))


def test_nocopy_reshape_strides_match_numpy():
    base = np.arange(2 * 3 * 4 * 5, dtype=np.int32).reshape(2, 3, 4, 5)
    views = [base, base.transpose(1, 0, 2, 3), base[:, :, ::2], base[:, 1:],
             base.transpose(0, 1, 3, 2)]
    targets = [(6, 20), (2, 12, 5), (24, 5), (2, 3, 20), (120,), (2, 3, 2, 2, 5),
               (1, 6, 1, 20), (6, 4, 5)]
    for v in views:
        for t in targets:
            if int(np.prod(t)) != v.size:
                continue
            st = _reshape_strides(v.shape, v.strides, t, 4)
            try:
                w = v.view()
                w.shape = t             # raises if a copy would be needed
                expect = w.strides
            except AttributeError:
                expect = None
            if expect is None:
                assert st is None, (v.shape, v.strides, t)
            else:
                assert st is not None
                assert np.array_equal(o.element_offsets(t, st),
                                      o.element_offsets(t, expect))


def test_basic_index_matches_numpy():
    base = np.arange(4 * 5 * 6, dtype=np.int64).reshape(4, 5, 6)
    keys = [1, -1, slice(None), slice(1, 3), (slice(None), 2), (Ellipsis, 0),
            (None, 1), (slice(None, None, -1),), (slice(3, 0, -2), slice(None), 4),
            (1, Ellipsis, None), (slice(0, 0),), Ellipsis, (2, 3, 4)]
    for k in keys:
        shape, strides, off = _basic_index(base.shape, base.strides, k)
        v = base[k]
        if not isinstance(v, np.ndarray):       # full integer index: keep a view
            v = base[k + (Ellipsis,)]
        assert shape == v.shape
        got = off + o.element_offsets(shape, strides)
        expect = (v.__array_interface__['data'][0] - base.__array_interface__['data'][0]
                  + o.element_offsets(v.shape, v.strides)) if v.size else got
        assert np.array_equal(got, expect), k
    with pytest.raises(IndexError):
        _basic_index(base.shape, base.strides, 4)
    with pytest.raises(IndexError):
        _basic_index(base.shape, base.strides, (0, 0, 0, 0))
