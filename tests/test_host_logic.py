"""Host-side logic of the kernel generators, checked against NumPy itself:
loop selection (promotion), parameter parsing, placeholder binding, stride
canonicalisation and reduction axis handling."""
import numpy as np
import pytest

import cupy_amd as cp
from cupy_amd._core import _kernel
from cupy_amd._core import _reduction
from cupy_amd._core._scalar import CScalar, get_scalar_literal
from oracle import numpy_oracle as o

_CHARS = '?bBhHiIlLefdFD'

# ufuncs whose loop table is exactly NumPy's without the long double, datetime
# and object loops ('GgMmO') ...
_SAME_TYPES = (
    'abs absolute acos acosh add arccos arccosh arcsin arcsinh arctan arctan2 arctanh asin '
    'asinh atan atan2 atanh bitwise_and bitwise_count bitwise_invert bitwise_left_shift '
    'bitwise_not bitwise_or bitwise_right_shift bitwise_xor cbrt ceil conj conjugate copysign '
    'cos cosh deg2rad degrees divmod equal exp exp2 expm1 fabs float_power floor floor_divide fmax '
    'fmin fmod frexp greater greater_equal heaviside hypot invert isfinite isinf isnan ldexp '
    'left_shift less less_equal log log10 log1p log2 logaddexp logaddexp2 logical_and '
    'logical_not logical_or logical_xor maximum minimum mod modf multiply nextafter not_equal '
    'rad2deg radians reciprocal remainder right_shift rint sign signbit sin sinh sqrt square '
    'tan tanh trunc').split()
# ... and those with extra entries: a boolean loop that raises the reference's
# error text (cupy/_core/_routines_math.pyx:952-973,1047-1050) or returns int8
# (power), integer loops of true division that NumPy reaches by promotion
_EXTRA_TYPES = {
    'subtract': ['??->?'], 'negative': ['?->?'], 'positive': ['?->?'], 'power': ['??->b'],
    'gcd': ['??->?'], 'lcm': ['??->?'],
    'true_divide': ['%s%s->d' % (c, c) for c in 'bBhHiIlLqQ'],
    'divide': ['%s%s->d' % (c, c) for c in 'bBhHiIlLqQ'],
}


def _numpy_types(uf):
    out = []
    for t in uf.types:
        if not any(c in 'GgMmO' for c in t) and t not in out:
            out.append(t)
    return out


@pytest.mark.parametrize('name', _SAME_TYPES)
def test_ufunc_types_are_numpys(name):
    assert list(getattr(cp, name).types) == _numpy_types(getattr(np, name))


@pytest.mark.parametrize('name', sorted(_EXTRA_TYPES))
def test_ufunc_types_are_numpys_plus_documented_entries(name):
    ours = list(getattr(cp, name).types)
    extra = _EXTRA_TYPES[name]
    assert [t for t in ours if t not in extra] == _numpy_types(getattr(np, name))
    assert all(t in ours for t in extra)


@pytest.mark.parametrize('ufn', ['add', 'multiply', 'subtract'])
def test_loop_selection_reproduces_numpy_promotion(ufn):
    uf = getattr(cp, ufn)
    for a in _CHARS:
        for b in _CHARS:
            if ufn == 'subtract' and a == b == '?':
                continue
            da, db = np.dtype(a), np.dtype(b)
            op = uf._ops._guess_routine_from_in_types((da, db))
            expect = np.result_type(da, db)
            assert op is not None, (a, b)
            assert np.dtype(op.out_types[0]) == expect, (a, b, op, expect)


def test_weak_python_scalars_keep_array_dtype():
    cases = [('B', 1, 'B'), ('b', 2, 'b'), ('f', 3, 'f'), ('f', 3.5, 'f'), ('e', 1.5, 'e'),
             ('i', 2.5, 'd'), ('B', 2.5, 'd'), ('?', 1, 'l'), ('h', True, 'h')]
    for arr_char, scalar, expect in cases:
        s = CScalar(scalar)
        in_types = (np.dtype(arr_char), s.descr)
        weaks = (False, s.weak_t)
        if not _kernel._check_should_use_weak_scalar(in_types, weaks if s.weak_t else None):
            weaks = (False, False)
        op = cp.add._ops._guess_routine_from_in_types(in_types, weaks)
        assert np.dtype(op.out_types[0]) == np.result_type(np.dtype(arr_char), scalar) \
            == np.dtype(expect), (arr_char, scalar)


def test_scalar_packing_rules():
    s = CScalar(300)
    s.apply_dtype(np.uint8)
    with pytest.raises(OverflowError):
        s._struct_value()
    s = CScalar(3e100)
    s.apply_dtype(np.float32)
    assert s._struct_value() == float('inf')
    for v, dt, expect in [(np.int64(-1), np.uint8, 255), (np.int64(2 ** 32), np.int32, 0),
                          (np.int64(2 ** 63 - 1), np.int32, -1),
                          (np.int64(-2 ** 63), np.int16, 0), (np.float64(2.75), np.int8, 2)]:
        s = CScalar(v)
        s.apply_dtype(dt)
        assert s._struct_value() == expect == np.asarray(v).astype(dt).item()
    assert CScalar(True).weak_t is False
    assert CScalar(2 ** 63).descr == np.uint64
    with pytest.raises(TypeError):
        CScalar('text')


def test_scalar_literals_round_trip():
    for v in (0.1, 1e-8, 3.0, 65504.0, 1e-45, 2.5):
        lit = get_scalar_literal(v, np.float32)
        assert lit.endswith('f')
        assert np.float32(float(lit[:-1])) == np.float32(v)
    assert get_scalar_literal(float('nan'), np.float64) == 'CUDART_NAN'
    assert get_scalar_literal(-float('inf'), np.float32) == '-CUDART_INF_F'
    assert get_scalar_literal(1e39, np.float32) == 'CUDART_INF_F'
    assert get_scalar_literal(5, np.int64) == '5ll'
    assert get_scalar_literal(5, np.uint16) == '5u'
    assert get_scalar_literal(True, np.bool_) == 'true'


def test_parameter_parsing():
    ps = _kernel._get_param_info('float32 x, raw T y, _non_const int64 z', True)
    assert [p.name for p in ps] == ['x', 'y', 'z']
    assert ps[0].dtype == np.float32 and ps[0].ctype == 'float' and not ps[0].raw
    assert ps[1].raw and ps[1].ctype == 'T' and ps[1].dtype is None
    assert ps[2].is_const is False and ps[2].ctype == 'long long'
    assert _kernel._get_param_info('', True) == ()
    with pytest.raises(Exception):
        _kernel.ParameterInfo('x', True)
    with pytest.raises(Exception):
        _kernel.ParameterInfo('static float32 x', True)


def test_placeholder_binding():
    ins = _kernel._get_param_info('T x, T y, float32 w', True)
    outs = _kernel._get_param_info('U z', False)
    it, ot, tm = _kernel._decide_params_type_core(
        ins, outs, (np.dtype('int16'), None, np.dtype('float32')), (np.dtype('float64'),))
    assert it == (np.dtype('int16'), np.dtype('int16'), np.dtype('float32'))
    assert ot == (np.dtype('float64'),)
    assert 'typedef short T;' in tm.get_typedef_code()
    assert 'typedef double U;' in tm.get_typedef_code()
    with pytest.raises(TypeError, match='Type is mismatched'):
        _kernel._decide_params_type_core(
            ins, outs, (np.dtype('int16'), np.dtype('int32'), np.dtype('float32')), ())
    with pytest.raises(TypeError, match='Type is mismatched'):
        _kernel._decide_params_type_core(
            ins, outs, (np.dtype('int16'), None, np.dtype('float64')), ())


class _FakeArray:
    def __init__(self, a):
        self._shape = a.shape
        self._strides = a.strides
        self.dtype = a.dtype


def test_canonical_dims_preserve_addresses():
    base = np.zeros((4, 3, 5, 2), dtype=np.float32)
    groups = [
        [base, base],
        [base, base[:, :, :, ::-1]],
        [base, np.broadcast_to(base[:, :1], base.shape)],
        [base.transpose(1, 0, 2, 3), base.transpose(1, 0, 2, 3)],
        [base[:, :, 0:4:2], base[:, :, 1:5:2]],
        [base[1:3], np.broadcast_to(np.zeros((5, 2), np.float16), (2, 3, 5, 2))],
    ]
    for views in groups:
        shape = views[0].shape
        cshape, cstrides = _kernel._canonical_dims([_FakeArray(v) for v in views], shape)
        assert int(np.prod(cshape)) == int(np.prod(shape))
        assert len(cshape) <= len(shape)
        for v, cs in zip(views, cstrides):
            assert np.array_equal(o.element_offsets(cshape, cs),
                                  o.element_offsets(v.shape, v.strides))
    cshape, _ = _kernel._canonical_dims([_FakeArray(base), _FakeArray(base)], base.shape)
    assert cshape == (120,)


def test_vector_width_choice():
    assert _kernel._max_vector_width([4]) == 4
    assert _kernel._max_vector_width([4, 2]) == 8
    assert _kernel._max_vector_width([8]) == 2
    assert _kernel._max_vector_width([1]) == 16
    assert _kernel._max_vector_width([1, 8]) == 8
    assert _kernel._max_vector_width([2, 2, 4]) == 8


def test_reduction_axis_partition():
    assert _reduction._get_axis(None, 3) == ((0, 1, 2), ())
    assert _reduction._get_axis(1, 3) == ((1,), (0, 2))
    assert _reduction._get_axis((-1, 0), 3) == ((0, 2), (1,))
    with pytest.raises(ValueError, match='duplicate'):
        _reduction._get_axis((0, -3), 3)
    with pytest.raises(np.exceptions.AxisError):
        _reduction._get_axis(3, 3)
    assert _reduction._get_out_shape((2, 3, 4), (1,), (0, 2), False) == (2, 4)
    assert _reduction._get_out_shape((2, 3, 4), (1,), (0, 2), True) == (2, 1, 4)
    assert _reduction._get_out_shape((2, 3, 4), (0, 1, 2), (), True) == (1, 1, 1)


def test_merge_dims_of_reduction_axes():
    a = np.zeros((6, 5, 4, 3), dtype=np.float64)
    shape, strides = _reduction._merge_dims((6, 5), [a.strides[:2]])
    assert shape == [30] and strides == [[a.strides[1]]]
    t = a.transpose(1, 0, 2, 3)
    shape, strides = _reduction._merge_dims(t.shape[:2], [t.strides[:2]])
    assert shape == [5, 6]


def test_squaring_short_cut_follows_numpy_result_types():
    """``x ** 2`` with a Python exponent squares (bool gives int8, integers
    keep their type); a float exponent on integers does not."""
    import cupy_amd as cp
    for dt in ('bool', 'int8', 'uint16', 'int64', 'float16', 'float32', 'complex64'):
        a = cp.ndarray((3,), dt)
        h = np.ones(3, dt)
        for e in (2, 3, 0.5) + ((2.0,) if dt != 'bool' else ()):
            assert (a ** e).dtype == (h ** e).dtype, (dt, e)
            assert cp.fuse(lambda x: x ** e)(a).dtype == (h ** e).dtype, (dt, e)
