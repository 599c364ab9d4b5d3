"""complex64 / complex128 on the GPU against NumPy on the same seeded inputs.

Bars: add, subtract, negative, conjugate, comparisons and casts are bit-exact.
Multiply, square, divide and reciprocal are within 4 eps * (1 + |result|) in the
complex plane: NumPy's own result for them depends on the host (its vectorised
loops fuse one product into the sum where the CPU can, its scalar tails and
strided loops are left to the C compiler), so there is no single bit pattern to
match.  Absolute value within 2 ulp.  The elementary functions: within
4 eps * (1 + |result|) of the g++ build of the same header run on the host
(observed: at most 2.01), which tests/test_complex_functions_host.py in turn
holds to 4 eps of extended-precision NumPy; and within 8 eps of NumPy's own
result in the same precision, whose C library routines are a few eps off
themselves (observed GPU against double-precision NumPy: at most 2.14).  Sums
within the reduction tolerance of the real types."""
import numpy as np
import pytest

import cupy_amd as cp
from helpers import assert_exact, assert_ulp

pytestmark = pytest.mark.gpu

CTYPES = ['complex64', 'complex128']


def crandom(shape, dtype, seed, scale=1.0):
    rng = np.random.default_rng(seed)
    z = rng.standard_normal(shape) + 1j * rng.standard_normal(shape)
    return (z * scale).astype(dtype)


def assert_cclose(got, want, eps_factor=8):
    got, want = np.asarray(got), np.asarray(want)
    assert got.dtype == want.dtype and got.shape == want.shape, (got.dtype, want.dtype)
    eps = np.finfo(want.real.dtype).eps
    err = np.abs(got.astype(np.complex128) - want.astype(np.complex128))
    bound = eps_factor * eps * (1 + np.abs(want.astype(np.complex128)))
    bad = ~(err <= bound)
    assert not bad.any(), (got[bad][:4], want[bad][:4])


@pytest.mark.parametrize('dtype', CTYPES)
def test_arithmetic_is_bit_exact(dtype):
    a = crandom((97, 53), dtype, 1)
    b = crandom((97, 53), dtype, 2)
    da, db = cp.asarray(a), cp.asarray(b)
    assert_exact((da + db).get(), a + b)
    assert_exact((da - db).get(), a - b)
    assert_cclose((da * db).get(), a * b, 4)
    assert_cclose((da / db).get(), a / b, 4)
    assert_exact((-da).get(), -a)
    assert_cclose(cp.square(da).get(), np.square(a), 4)
    assert_exact(cp.conjugate(da).get(), np.conjugate(a))
    assert_exact(da.conj().get(), a.conj())
    assert_cclose(cp.reciprocal(da).get(), np.reciprocal(a), 4)
    assert_ulp(abs(da).get(), abs(a), 2)
    # broadcasting and non-contiguous operands
    assert_cclose((da[::2, 1::3] * db.T[1::3, ::2].T).get(), a[::2, 1::3] * b.T[1::3, ::2].T, 4)
    assert_exact((da + db[0]).get(), a + b[0])
    assert_exact((da - db[:, :1]).get(), a - b[:, :1])
    assert_exact(cp.ascontiguousarray(da.T).get(), np.ascontiguousarray(a.T))


@pytest.mark.parametrize('dtype', CTYPES)
def test_scalars_and_mixed_types(dtype):
    a = crandom((1000,), dtype, 3)
    f = np.random.default_rng(4).standard_normal(1000).astype(np.float32)
    h = f.astype(np.float16)
    i = np.arange(1000, dtype=np.int32) - 500
    da = cp.asarray(a)
    for s in (2, 2.5, 1 - 2j, np.float32(3), np.complex64(1 + 1j), np.complex128(2 - 1j)):
        assert_cclose((da * s).get(), a * s, 4)
        assert_exact((s + da).get(), s + a)
        assert_exact((da - s).get(), a - s)          # replayed launch, other operator
        assert_exact((s + da).get(), s + a)          # replayed launch
    for other in (f, h, i):
        assert_cclose((da * cp.asarray(other)).get(), a * other, 4)
        assert_exact((cp.asarray(other) - da).get(), other - a)
    assert_cclose((cp.asarray(f) * 1j).get(), f * 1j, 4)
    assert_exact((cp.asarray(i) + 1j).get(), i + 1j)


@pytest.mark.parametrize('dtype', CTYPES)
def test_division_special_cases(dtype):
    t = np.dtype(dtype).type
    num = np.array([1 + 1j, 1 + 1j, 0j, 1e30 + 1e30j, 1e-30 + 1e-30j, 3 - 4j, np.inf + 1j], dtype)
    den = np.array([0j, 1e-30 + 1e30j, 0j, 1e30 + 1e-30j, 1e30 - 1e30j, 0 + 2j, 2 + 0j], dtype)
    with np.errstate(all='ignore'):
        want = num / den
    got = (cp.asarray(num) / cp.asarray(den)).get()
    finite = np.isfinite(want)
    assert np.array_equal(np.isnan(got.real), np.isnan(want.real))
    assert np.array_equal(np.isnan(got.imag), np.isnan(want.imag))
    assert np.array_equal(np.isinf(got), np.isinf(want))
    assert_cclose(got[finite], want[finite], 4)
    assert t is not None


@pytest.mark.parametrize('dtype', CTYPES)
@pytest.mark.parametrize('name', [
    'sqrt', 'exp', 'log', 'log2', 'log10', 'sin', 'cos', 'tan', 'sinh', 'cosh', 'tanh',
    'arcsin', 'arccos', 'arctan', 'arcsinh', 'arccosh', 'arctanh', 'log1p', 'expm1', 'exp2',
    'rint'])
def test_elementary_functions(name, dtype):
    a = crandom((4000,), dtype, 5, scale=1.5)
    with np.errstate(all='ignore'):
        want = getattr(np, name)(a)
    assert_cclose(getattr(cp, name)(cp.asarray(a)).get(), want)


@pytest.mark.parametrize('dtype', CTYPES)
def test_power_sign_and_angle(dtype):
    a = crandom((3000,), dtype, 6)
    b = crandom((3000,), dtype, 7)
    da, db = cp.asarray(a), cp.asarray(b)
    assert_cclose(cp.power(da, db).get(), np.power(a, b), 64)
    assert_cclose((da ** 2).get(), a ** 2)
    assert_cclose((da ** 0.5).get(), a ** 0.5)
    got = cp.float_power(da, db)
    assert got.dtype == np.complex128
    assert_cclose(got.get(), np.float_power(a, b), 64)
    assert_cclose(cp.sign(da).get(), np.sign(a), 4)
    z = np.array([0j, np.nan + 1j, np.inf + 1j, 1 - np.inf * 1j], dtype)
    with np.errstate(all='ignore'):
        assert_exact(cp.sign(cp.asarray(z)).get(), np.sign(z))
    real_t = a.real.dtype
    eps = np.finfo(real_t).eps
    np.testing.assert_allclose(cp.angle(da).get(), np.angle(a), rtol=4 * eps, atol=4 * eps)
    np.testing.assert_allclose(cp.angle(da, deg=True).get(), np.angle(a, deg=True),
                               rtol=4 * eps, atol=400 * eps)
    assert cp.angle(da).dtype == real_t
    r = np.array([-2.0, 0.0, 3.0, np.nan], np.float32)
    assert_exact(cp.angle(cp.asarray(r)).get(), np.angle(r))
    k = np.array([-2, 0, 3], np.int32)
    assert_exact(cp.angle(cp.asarray(k)).get(), np.angle(k))


@pytest.mark.parametrize('dtype', CTYPES)
def test_comparisons_and_predicates(dtype):
    rng = np.random.default_rng(8)
    a = (rng.integers(-2, 3, 500) + 1j * rng.integers(-2, 3, 500)).astype(dtype)
    b = (rng.integers(-2, 3, 500) + 1j * rng.integers(-2, 3, 500)).astype(dtype)
    a[::7] = np.nan + 1j
    b[::11] = complex(1, np.nan)
    a[3] = np.inf
    da, db = cp.asarray(a), cp.asarray(b)
    for name in ('equal', 'not_equal', 'less', 'less_equal', 'greater', 'greater_equal',
                 'logical_and', 'logical_or', 'logical_xor', 'maximum', 'minimum',
                 'fmax', 'fmin'):
        assert_exact(getattr(cp, name)(da, db).get(), getattr(np, name)(a, b))
    for name in ('isnan', 'isinf', 'isfinite', 'logical_not'):
        assert_exact(getattr(cp, name)(da).get(), getattr(np, name)(a))
    c = rng.integers(0, 2, 500).astype(bool)
    assert_exact(cp.where(cp.asarray(c), da, db).get(), np.where(c, a, b))


def test_casts_follow_numpy():
    a = crandom((300,), 'complex128', 9, scale=50)
    a[::5] = 0
    d = cp.asarray(a)
    assert_exact(d.astype(np.complex64).get(), a.astype(np.complex64))
    with pytest.warns(np.exceptions.ComplexWarning):
        got = d.astype(np.float32).get()
    with pytest.warns(np.exceptions.ComplexWarning):
        assert_exact(got, a.astype(np.float32))
    assert_exact(d.astype(bool).get(), a.astype(bool))
    f = np.random.default_rng(10).standard_normal(300).astype(np.float16)
    assert_exact(cp.asarray(f).astype(np.complex64).get(), f.astype(np.complex64))
    i = np.arange(-150, 150, dtype=np.int64)
    assert_exact(cp.asarray(i).astype(np.complex128).get(), i.astype(np.complex128))
    b = np.array([True, False, True])
    assert_exact(cp.asarray(b).astype(np.complex64).get(), b.astype(np.complex64))
    with pytest.raises(TypeError):
        cp.add(d, d, out=cp.zeros(300, np.float64))


@pytest.mark.parametrize('dtype', CTYPES)
def test_real_and_imag_are_views(dtype):
    a = crandom((40, 30), dtype, 11)
    d = cp.asarray(a)
    assert_exact(d.real.get(), a.real)
    assert_exact(d.imag.get(), a.imag)
    assert_exact(d.T[::2].imag.get(), a.T[::2].imag)
    assert_exact((d.real * d.imag).get(), a.real * a.imag)          # real arithmetic
    assert_exact(cp.real(d).get(), np.real(a))
    assert_exact(cp.imag(d).get(), np.imag(a))
    new = np.random.default_rng(12).standard_normal((40, 30)).astype(a.real.dtype)
    d.real = cp.asarray(new)
    d.imag = 2.5
    a = a.copy()
    a.real = new
    a.imag = 2.5
    assert_exact(d.get(), a)
    assert_exact(cp.iscomplex(d).get(), np.iscomplex(a))
    assert cp.iscomplexobj(d) and not cp.isrealobj(d)
    r = cp.asarray(new)
    assert_exact(r.imag.get(), new.imag)
    assert not cp.iscomplexobj(r)


@pytest.mark.parametrize('dtype', CTYPES)
def test_reductions_and_scans(dtype):
    a = crandom((301, 203), dtype, 13)
    d = cp.asarray(a)
    rtol = 1e-5 if dtype == 'complex64' else 1e-12
    for axis in (None, 0, 1):
        bound = rtol * np.abs(a).sum(axis=axis)
        assert (np.abs(d.sum(axis=axis).get() - a.sum(axis=axis)) <= bound).all()
        assert (np.abs(d.mean(axis=axis).get() - a.mean(axis=axis)) <= bound).all()
        assert d.sum(axis=axis).dtype == a.dtype
        want = np.cumsum(a, axis=axis)
        got = cp.cumsum(d, axis=axis).get()
        assert got.shape == want.shape and got.dtype == want.dtype
        assert (np.abs(got - want) <= rtol * np.cumsum(np.abs(a), axis=axis)).all()
    small = crandom((6, 5), dtype, 14)
    np.testing.assert_allclose(cp.asarray(small).prod(axis=1).get(), small.prod(axis=1),
                               rtol=100 * rtol)
    np.testing.assert_allclose(cp.cumprod(cp.asarray(small), axis=0).get(),
                               np.cumprod(small, axis=0), rtol=100 * rtol)
    z = a.copy()
    z[::3, ::2] = complex(np.nan, 1)
    z[1::3, 1::2] = 0
    dz = cp.asarray(z)
    np.testing.assert_allclose(cp.nansum(dz, axis=0).get(), np.nansum(z, axis=0),
                               rtol=1000 * rtol, atol=1000 * rtol)
    assert_exact(cp.count_nonzero(dz, axis=1).get(), np.count_nonzero(z, axis=1))
    # big enough for the multi-block paths
    big = crandom((3, 200000), dtype, 15)
    db = cp.asarray(big)
    for axis in (None, 0, 1):
        bound = rtol * np.abs(big).sum(axis=axis)
        assert (np.abs(db.sum(axis=axis).get() - big.sum(axis=axis)) <= bound).all()
    got = cp.cumsum(db, axis=1).get()
    assert (np.abs(got - np.cumsum(big, axis=1)) <= rtol * np.cumsum(np.abs(big), axis=1)).all()


@pytest.mark.parametrize('dtype', CTYPES)
def test_user_kernels_with_complex_parameters(dtype):
    a = crandom((513,), dtype, 16)
    d = cp.asarray(a)
    k = cp.ElementwiseKernel('T x, T s, float32 t', 'T y', 'y = x * s + conj(x) * (T)t',
                             'cplx_axpy')
    s = 2 - 3j
    want = a * a.dtype.type(s) + np.conj(a) * a.dtype.type(0.5)
    assert_cclose(k(d, s, 0.5).get(), want, 8)
    assert_cclose(k(d, 1j, 0.25).get(),
                  a * a.dtype.type(1j) + np.conj(a) * a.dtype.type(0.25), 8)
    r = cp.ReductionKernel('T x', 'T y', 'x * conj(x)', 'a + b', 'y = a', '0', 'cplx_norm2')
    m = crandom((37, 41), dtype, 17)
    got = r(cp.asarray(m), axis=1).get()
    rtol = 1e-5 if dtype == 'complex64' else 1e-12
    np.testing.assert_allclose(got, (m * m.conj()).sum(axis=1), rtol=rtol, atol=rtol)

    scaled = cp.ReductionKernel('T x, T s, float32 t', 'T y', 'x * s + (T)t', 'a + b', 'y = a',
                                '0', 'cplx_scaled_sum')
    for axis in (0, 1, None):
        for s, t in ((2 - 3j, 0.5), (1j, 0.25)):          # second pair: replayed launch
            want = (m * m.dtype.type(s) + m.dtype.type(t)).sum(axis=axis)
            np.testing.assert_allclose(scaled(cp.asarray(m), s, t, axis=axis).get(), want,
                                       rtol=20 * rtol, atol=20 * rtol)

    @cp.fuse()
    def f(x, y):
        return x * y + cp.conj(x)
    assert_cclose(f(d, d).get(), a * a + np.conj(a), 8)


@pytest.mark.parametrize('dtype', CTYPES)
def test_variance_of_complex_is_real(dtype):
    a = crandom((61, 47), dtype, 21)
    d = cp.asarray(a)
    rtol = 1e-5 if dtype == 'complex64' else 1e-12
    for axis in (None, 0, 1):
        for ddof in (0, 1):
            got = d.var(axis=axis, ddof=ddof)
            want = a.var(axis=axis, ddof=ddof)
            assert got.dtype == want.dtype and got.shape == want.shape
            np.testing.assert_allclose(got.get(), want, rtol=20 * rtol)
            np.testing.assert_allclose(d.std(axis=axis, ddof=ddof).get(),
                                       a.std(axis=axis, ddof=ddof), rtol=20 * rtol)


@pytest.mark.parametrize('dtype', ['complex64', 'complex128'])
def test_extrema_order_by_real_then_imaginary_part(dtype):
    rng = np.random.default_rng(51)
    # few distinct real parts, so that the imaginary parts decide often
    x = (rng.integers(-3, 4, (300, 71)) + 1j * rng.integers(-50, 50, (300, 71))).astype(dtype)
    dx = cp.asarray(x)
    for axis in (None, 0, 1):
        assert_exact(dx.max(axis=axis).get(), x.max(axis=axis))
        assert_exact(dx.min(axis=axis).get(), x.min(axis=axis))
        assert_exact(dx.argmax(axis=axis).get(), x.argmax(axis=axis))
        assert_exact(dx.argmin(axis=axis).get(), x.argmin(axis=axis))
    flat = x.reshape(-1)[:70001 // 4]
    assert_exact(cp.asarray(flat).argmax().get(), flat.argmax())
    y = x.copy()
    y[5, 7] = complex(np.nan, 1)
    y[9, 3] = complex(2, np.nan)
    y[200, 70] = complex(np.nan, np.nan)
    dy = cp.asarray(y)
    for axis in (None, 0, 1):
        got, want = dy.max(axis=axis).get(), y.max(axis=axis)
        assert np.array_equal(np.isnan(got), np.isnan(want))
        assert np.array_equal(got[~np.isnan(got)], want[~np.isnan(want)])
        assert_exact(dy.argmax(axis=axis).get(), y.argmax(axis=axis))
        assert_exact(dy.argmin(axis=axis).get(), y.argmin(axis=axis))
        with np.errstate(all='ignore'):
            assert_exact(cp.nanmax(dy, axis=axis).get(), np.nanmax(y, axis=axis))
            assert_exact(cp.nanmin(dy, axis=axis).get(), np.nanmin(y, axis=axis))
            assert_exact(cp.nanargmax(dy, axis=axis).get(), np.nanargmax(y, axis=axis))
            assert_exact(cp.nanargmin(dy, axis=axis).get(), np.nanargmin(y, axis=axis))


# ---- the GPU against the host build of the same header ---------------------------------------
# tests/test_complex_functions_host.py holds the formulas of cupy/complex.cuh,
# compiled with g++, to 4 eps * (1 + |result|) of NumPy.  Here the GPU runs the
# same header: what can differ is only how the device's sin / cos / exp / log /
# atan2 / hypot round, so the two must agree far more closely than either is
# asked to agree with NumPy.

_HOST_UNARY = ('sqrt exp log log2 log10 sin cos tan sinh cosh tanh arcsin arccos arctan '
               'arcsinh arccosh arctanh log1p expm1 exp2').split()
# Bound on the distance GPU <-> host build over the inputs below, in units of
# eps * (1 + |result|).  Observed (printed by the test): 0.5 (arctan, arctanh)
# to 2.01 (tanh, complex128); exp, sin, cos, sinh, cosh, tan, expm1, exp2 1.7
# to 2.0; sqrt, the logarithms, arcsin, arccos, arcsinh, arccosh 0.8 to 1.8.
_GPU_VS_HOST_EPS = {name: 4 for name in _HOST_UNARY}


@pytest.fixture(scope='module')
def host_lib(tmp_path_factory):
    import ctypes
    import os
    import subprocess
    here = os.path.dirname(os.path.abspath(__file__))
    out = str(tmp_path_factory.mktemp('complex_host') / 'libcomplex_host.so')
    subprocess.check_call([
        'g++', '-O2', '-ffp-contract=off', '-shared', '-fPIC',
        '-I', os.path.join(os.path.dirname(here), 'cupy_amd', 'include'),
        '-o', out, os.path.join(here, 'complex_host_shim.cpp')])
    return ctypes.CDLL(out)


def _host_call(lib, name, z):
    import ctypes
    prefix = 'c64_' if z.dtype == np.complex64 else 'c128_'
    out = np.empty_like(z)
    getattr(lib, prefix + name)(z.ctypes.data_as(ctypes.c_void_p),
                                out.ctypes.data_as(ctypes.c_void_p), ctypes.c_int(z.size))
    return out


def _distance_in_eps(got, want, real_dtype):
    eps = np.finfo(real_dtype).eps
    both = np.isfinite(got) & np.isfinite(want)
    assert np.array_equal(np.isfinite(got), np.isfinite(want))
    err = np.abs(got.astype(np.complex128)[both] - want.astype(np.complex128)[both])
    scale = eps * (1 + np.abs(want.astype(np.complex128)[both]))
    return float((err / scale).max()) if err.size else 0.0


@pytest.mark.parametrize('dtype', CTYPES)
@pytest.mark.parametrize('name', _HOST_UNARY)
def test_gpu_agrees_with_the_host_build_of_the_header(host_lib, name, dtype):
    real_dtype = np.float32 if dtype == 'complex64' else np.float64
    worst_host = worst_numpy = 0.0
    for scale in (1.5, 0.01, 1e-5, 30.0):
        z = crandom((50000,), dtype, 5, scale=scale)
        with np.errstate(all='ignore'):
            want_np = getattr(np, name)(z.astype(np.clongdouble)).astype(np.complex128)
        got = getattr(cp, name)(cp.asarray(z)).get()
        host = _host_call(host_lib, name, z)
        worst_host = max(worst_host, _distance_in_eps(got, host, real_dtype))
        with np.errstate(all='ignore'):
            finite = np.isfinite(want_np.astype(dtype))
        worst_numpy = max(worst_numpy, _distance_in_eps(
            got[finite], want_np[finite].astype(np.complex128), real_dtype))
    print('%-8s %-10s GPU vs host build %.2f eps, GPU vs NumPy %.2f eps' % (
        name, dtype, worst_host, worst_numpy))
    assert worst_host <= _GPU_VS_HOST_EPS[name], (name, dtype, worst_host)
    # ... and the GPU itself within 4 eps of extended-precision NumPy
    assert worst_numpy <= 4, (name, dtype, worst_numpy)
