"""Operator and container protocol of ndarray against NumPy: augmented
assignments update the array they are applied to (so a view writes through to
its base), reflected shifts, divmod, iteration, copies, pickles, conversions
(reference: cupy/_core/core.pyx:1500-1830, 2040-2062, 708-731)."""
import copy
import io
import operator
import pickle

import numpy as np
import pytest

import cupy_amd as cp

pytestmark = pytest.mark.gpu


INPLACE = [
    (operator.iadd, 'int32'), (operator.isub, 'int32'), (operator.imul, 'int32'),
    (operator.ifloordiv, 'int32'), (operator.imod, 'int32'),
    (operator.iand, 'int32'), (operator.ior, 'int32'), (operator.ixor, 'int32'),
    (operator.ilshift, 'int32'), (operator.irshift, 'int32'),
    (operator.ipow, 'int64'), (operator.itruediv, 'float32'),
    (operator.iand, 'bool'), (operator.ior, 'bool'), (operator.ixor, 'bool'),
    (operator.ifloordiv, 'float64'), (operator.imod, 'float32'),
]


@pytest.mark.parametrize('op,dtype', INPLACE, ids=lambda v: getattr(v, '__name__', v))
def test_augmented_assignment_writes_through_a_view(op, dtype):
    rng = np.random.default_rng(7)
    if dtype == 'bool':
        base = rng.integers(0, 2, size=(6, 50)).astype(dtype)
        other = rng.integers(0, 2, size=(3, 49)).astype(dtype)
    else:
        base = rng.integers(1, 9, size=(6, 50)).astype(dtype)
        other = rng.integers(1, 5, size=(3, 49)).astype(dtype)
    dbase, dother = cp.asarray(base), cp.asarray(other)
    hview, dview = base[::2, 1:], dbase[::2, 1:]
    before = dview
    hview = op(hview, other)
    dview = op(dview, dother)
    assert dview is before           # the same object, not a new array
    got = dbase.get()
    assert got.dtype == base.dtype
    if base.dtype.kind == 'f':
        np.testing.assert_allclose(got, base, rtol=1e-6)
    else:
        assert np.array_equal(got, base)


def test_augmented_assignment_with_a_scalar():
    h = np.arange(40, dtype=np.uint8)
    d = cp.asarray(h)
    d &= 0x0f
    h &= 0x0f
    d |= 0x40
    h |= 0x40
    d ^= 3
    h ^= 3
    d <<= 1
    h <<= 1
    d >>= 2
    h >>= 2
    d %= 7
    h %= 7
    d //= 2
    h //= 2
    assert d.dtype == h.dtype and np.array_equal(d.get(), h)


def test_augmented_assignment_refuses_an_unsafe_cast_like_numpy():
    d = cp.asarray(np.arange(5, dtype=np.int32))
    with pytest.raises(TypeError):
        d &= cp.asarray(np.ones(5, np.float32))
    with pytest.raises(TypeError):
        d //= 1.5


def test_reflected_shifts_and_divmod():
    h = np.array([0, 1, 2, 5, 7], np.int64)
    d = cp.asarray(h)
    assert np.array_equal((1 << d).get(), 1 << h)
    assert np.array_equal((4096 >> d).get(), 4096 >> h)
    hv = np.array([-7, -1, 0, 3, 9], np.int32)
    dv = cp.asarray(hv)
    q, r = divmod(dv, 4)
    hq, hr = divmod(hv, 4)
    assert q.dtype == hq.dtype and r.dtype == hr.dtype
    assert np.array_equal(q.get(), hq) and np.array_equal(r.get(), hr)
    q, r = divmod(17, cp.asarray(np.array([1, 2, 3, 5], np.int32)))
    hq, hr = divmod(17, np.array([1, 2, 3, 5], np.int32))
    assert np.array_equal(q.get(), hq) and np.array_equal(r.get(), hr)
    fq, fr = divmod(cp.asarray(np.array([-7.5, 2.25, 9.0], np.float32)), cp.asarray(np.array([2.0, -0.5, 4.0], np.float32)))
    hq, hr = divmod(np.array([-7.5, 2.25, 9.0], np.float32), np.array([2.0, -0.5, 4.0], np.float32))
    assert np.array_equal(fq.get(), hq) and np.array_equal(fr.get(), hr)


def test_iteration_goes_over_the_first_axis():
    h = np.arange(24, dtype=np.float32).reshape(4, 3, 2)
    d = cp.asarray(h)
    rows = list(d)
    assert len(rows) == 4
    for got, want in zip(rows, h):
        assert isinstance(got, cp.ndarray) and np.array_equal(got.get(), want)
    a, b, c = cp.asarray(np.array([3, 4, 5], np.int16))
    assert (int(a), int(b), int(c)) == (3, 4, 5)
    with pytest.raises(TypeError):
        iter(cp.asarray(np.float32(1.0)))


def test_copy_module_and_pickle_round_trip():
    h = np.arange(30, dtype=np.float64).reshape(5, 6)[:, ::2]
    d = cp.asarray(np.arange(30, dtype=np.float64).reshape(5, 6))[:, ::2]
    for clone in (copy.copy(d), copy.deepcopy(d)):
        assert clone is not d and clone.data.ptr != d.data.ptr
        assert np.array_equal(clone.get(), h)
    back = pickle.loads(pickle.dumps(d))
    assert isinstance(back, cp.ndarray) and back.dtype == h.dtype and np.array_equal(back.get(), h)
    back = pickle.loads(d.dumps())
    assert np.array_equal(back.get(), h)
    f = io.BytesIO()
    d.dump(f)
    f.seek(0)
    assert np.array_equal(pickle.load(f).get(), h)
    # a Fortran-ordered array comes back in its order
    df = cp.asarray(np.arange(12, dtype=np.int32).reshape(3, 4)).T
    back = pickle.loads(pickle.dumps(df))
    assert back.flags.f_contiguous and np.array_equal(back.get(), df.get())


def test_conversions_to_python_objects(tmp_path):
    assert complex(cp.asarray(np.complex64(1.5 - 2j))) == 1.5 - 2j
    assert complex(cp.asarray(np.array([[2.0]], np.float32))) == 2.0
    h = np.arange(12, dtype=np.int16).reshape(3, 4)
    d = cp.asarray(h)
    assert d.tobytes() == h.tobytes()
    assert d.T.tobytes() == h.T.tobytes()
    assert d.tobytes('F') == h.tobytes('F')
    path = tmp_path / 'a.bin'
    d.tofile(str(path))
    assert np.array_equal(np.fromfile(str(path), dtype=np.int16), h.ravel())
    d.tofile(str(path), sep=',')
    assert path.read_text() == ','.join(str(v) for v in h.ravel())
