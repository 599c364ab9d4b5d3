"""The formulas of cupy/complex.cuh, compiled for the host and compared with
NumPy (whose complex functions come from the C library): a check of the
algorithms -- branch cuts, cancellation near |z| = 1 and near the poles of
tanh, small and large arguments -- that needs no GPU.  complex64 results are
compared with NumPy's complex128 results for the same inputs; complex128
results with NumPy's own.  Bound: 4 eps * (1 + |result|) in the complex plane
(the GPU tests allow 32: the device math library rounds differently)."""
import ctypes
import os
import subprocess

import numpy as np
import pytest

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)

UNARY = ('sqrt exp log log2 log10 sin cos tan sinh cosh tanh arcsin arccos arctan '
         'arcsinh arccosh arctanh log1p expm1 exp2').split()


@pytest.fixture(scope='module')
def lib(tmp_path_factory):
    out = str(tmp_path_factory.mktemp('complex_host') / 'libcomplex_host.so')
    subprocess.check_call([
        'g++', '-O2', '-ffp-contract=off', '-shared', '-fPIC',
        '-I', os.path.join(ROOT, 'cupy_amd', 'include'),
        '-o', out, os.path.join(HERE, 'complex_host_shim.cpp')])
    return ctypes.CDLL(out)


def call(lib, name, dtype, *arrays):
    prefix = 'c64_' if np.dtype(dtype) == np.complex64 else 'c128_'
    out = np.empty_like(arrays[0])
    ptrs = [a.ctypes.data_as(ctypes.c_void_p) for a in arrays]
    getattr(lib, prefix + name)(*ptrs, out.ctypes.data_as(ctypes.c_void_p),
                                ctypes.c_int(arrays[0].size))
    return out


def check(got, want, dtype, factor):
    eps = np.finfo(np.float32 if np.dtype(dtype) == np.complex64 else np.float64).eps
    with np.errstate(all='ignore'):
        want_cast = want.astype(dtype)
    finite = np.isfinite(want_cast)
    assert np.array_equal(np.isfinite(got), finite)
    got = got.astype(np.complex128)[finite]
    want = want[finite]
    err = np.abs(got - want)
    bound = factor * eps * (1 + np.abs(want)) + np.finfo(np.float32).tiny
    assert (err <= bound).all(), (got[err > bound][:4], want[err > bound][:4])


@pytest.mark.parametrize('dtype', [np.complex64, np.complex128])
@pytest.mark.parametrize('scale', [1.5, 0.01, 1e-5, 30.0])
@pytest.mark.parametrize('name', UNARY)
def test_unary_function(lib, name, scale, dtype):
    rng = np.random.default_rng(5)
    z = ((rng.standard_normal(50000) + 1j * rng.standard_normal(50000)) * scale).astype(dtype)
    # (in extended precision: NumPy's own double-precision exp2 is
    # exp(z log 2) with the product rounded, |z| eps off at large |z|)
    with np.errstate(all='ignore'):
        want = getattr(np, name)(z.astype(np.clongdouble)).astype(np.complex128)
    check(call(lib, name, dtype, z), want, dtype, 4)


@pytest.mark.parametrize('dtype', [np.complex64, np.complex128])
def test_branch_cuts_and_special_points(lib, dtype):
    # both sides of every cut (the sign of a zero part selects the side), the
    # branch points themselves, the axes
    pts = []
    for re in (-3.0, -1.0, -0.5, -0.0, 0.0, 0.5, 1.0, 3.0):
        for im in (-2.0, -1.0, -0.0, 0.0, 1.0, 2.0):
            pts.append(complex(re, im))
    z = np.array(pts, dtype)
    for name in UNARY:
        with np.errstate(all='ignore'):
            want = getattr(np, name)(z.astype(np.complex128))
        got = call(lib, name, dtype, z)
        check(got, want, dtype, 8)
        # the side of the cut shows in the signs of the parts
        finite = np.isfinite(want) & (np.abs(want.imag) > 1e-3)
        assert np.array_equal(np.sign(got.imag[finite]), np.sign(want.imag[finite])), name


@pytest.mark.parametrize('dtype', [np.complex64, np.complex128])
def test_multiply_divide_power(lib, dtype):
    rng = np.random.default_rng(6)
    a = (rng.standard_normal(50000) + 1j * rng.standard_normal(50000)).astype(dtype)
    b = (rng.standard_normal(50000) + 1j * rng.standard_normal(50000)).astype(dtype)
    wide_a, wide_b = a.astype(np.complex128), b.astype(np.complex128)
    check(call(lib, 'multiply', dtype, a, b), wide_a * wide_b, dtype, 2)
    check(call(lib, 'divide', dtype, a, b), wide_a / wide_b, dtype, 4)
    check(call(lib, 'power', dtype, a, b), wide_a ** wide_b, dtype, 32)
    # Smith's division does not overflow where the textbook formula would
    big = np.array([1e30 + 1e30j, 1e-30 + 1e-30j], dtype)
    den = np.array([1e30 + 1e-30j, 1e30 - 1e30j], dtype)
    with np.errstate(all='ignore'):
        want = big.astype(np.complex128) / den.astype(np.complex128)
    check(call(lib, 'divide', dtype, big, den), want, dtype, 4)
