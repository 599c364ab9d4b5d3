"""Complex scalars in argument blocks and complex loops in the type tables (no
GPU: the kernels are compiled for gfx950 and the recorded launches inspected).
A ``complex<T>`` kernel parameter sits at twice the alignment of its parts; the
code object's metadata says where, and the host must put the two parts there."""
import struct

import numpy as np
import pytest

import cupy_amd as cp
from cupy_amd import _dryrun
from cupy_amd._core._kernel import _make_packer

pytestmark = pytest.mark.skipif(not _dryrun.enabled(),
                                reason='inspects recorded launches')


def test_packer_aligns_complex_scalars_like_the_compiler():
    p = _make_packer('@PfDiF?D')
    blob = p.pack(7, 1.5, 2 + 3j, 9, 4 - 5j, True, -1j)
    # P@0, f@8, complex128@16 (16-aligned), i@32, complex64@40 (8-aligned), ?@48, complex128@64
    assert struct.unpack_from('<Q', blob, 0) == (7,)
    assert struct.unpack_from('<f', blob, 8) == (1.5,)
    assert struct.unpack_from('<dd', blob, 16) == (2.0, 3.0)
    assert struct.unpack_from('<i', blob, 32) == (9,)
    assert struct.unpack_from('<ff', blob, 40) == (4.0, -5.0)
    assert struct.unpack_from('<?', blob, 48) == (True,)
    assert struct.unpack_from('<dd', blob, 64) == (0.0, -1.0)
    assert len(blob) == 80 and p.size == 80
    # without complex members it is the plain struct packer
    assert isinstance(_make_packer('@Pqi'), struct.Struct)


def test_complex_scalars_land_at_the_offsets_in_the_code_object():
    k = cp.ElementwiseKernel(
        'float32 x, float32 t, complex128 s, int8 b, complex64 u', 'complex128 y',
        'y = complex<double>(x * t) * s + complex<double>(u) + (double)b', 'cplx_args')
    x = cp.asarray(np.arange(6, dtype=np.float32))
    n0 = len(_dryrun.launches)
    k(x, 0.5, 2 + 3j, 7, 4 - 5j)
    (name, grid, block, shmem, blob), = _dryrun.launches[n0:]
    # the launch went through Function.launch_packed, which checks the block's
    # size against the code object; here the values' places are checked too
    (fn, _, _), = k._planner._memo.values()
    assert fn.name == name
    args = fn.meta['args']
    sizes = [size for _, size, _ in args]
    i_s = sizes.index(16)
    assert struct.unpack_from('<dd', blob, args[i_s][0]) == (2.0, 3.0)
    assert args[i_s][0] % 16 == 0
    i_u = [i for i, (_, size, _) in enumerate(args) if size == 8 and i > i_s][0]
    assert struct.unpack_from('<ff', blob, args[i_u][0]) == (4.0, -5.0)
    # replay of the recorded call patches both parts of a new value
    k(x, 0.5, 1 - 1j, 7, 8j)
    (_, _, _, _, blob2), = _dryrun.launches[n0 + 1:]
    assert struct.unpack_from('<dd', blob2, args[i_s][0]) == (1.0, -1.0)
    assert struct.unpack_from('<ff', blob2, args[i_u][0]) == (0.0, 8.0)


@pytest.mark.parametrize('name', [
    'add', 'subtract', 'multiply', 'true_divide', 'power', 'negative', 'square',
    'absolute', 'reciprocal', 'sign', 'sqrt', 'exp', 'log', 'log2', 'log10', 'sin', 'cos',
    'tan', 'arcsin', 'arccos', 'arctan', 'sinh', 'cosh', 'tanh', 'arcsinh', 'arccosh',
    'arctanh', 'conjugate', 'equal', 'not_equal', 'less', 'less_equal', 'greater',
    'greater_equal', 'logical_and', 'logical_or', 'logical_xor', 'logical_not', 'isnan',
    'isinf', 'isfinite', 'maximum', 'minimum', 'fmax', 'fmin'])
def test_loop_tables_resolve_complex_types_like_numpy(name):
    ours, theirs = getattr(cp, name), getattr(np, name)
    for c in 'FD':
        host = np.ones(3, np.dtype(c))
        dev = cp.asarray(host)
        args_h = (host,) * theirs.nin
        args_d = (dev,) * theirs.nin
        assert ours(*args_d).dtype == theirs(*args_h).dtype
    if theirs.nin == 2:
        f = np.ones(3, np.float32)
        z = np.ones(3, np.complex64)
        assert ours(cp.asarray(f), cp.asarray(z)).dtype == theirs(f, z).dtype
        assert ours(cp.asarray(z), 2).dtype == theirs(z, 2).dtype
        assert ours(cp.asarray(z), 2.5).dtype == theirs(z, 2.5).dtype
        assert ours(cp.asarray(f), 1j).dtype == theirs(f, 1j).dtype
        i = np.ones(3, np.int32)
        assert ours(cp.asarray(i), cp.asarray(z)).dtype == theirs(i, z).dtype


def test_reductions_scans_and_views_keep_numpy_types():
    for c in 'FD':
        h = (np.arange(12) + 1j).astype(c).reshape(3, 4)
        d = cp.asarray(h)
        for axis in (None, 0, 1):
            assert d.sum(axis=axis).dtype == h.sum(axis=axis).dtype
            assert d.prod(axis=axis).dtype == h.prod(axis=axis).dtype
            assert d.mean(axis=axis).dtype == h.mean(axis=axis).dtype
            assert cp.cumsum(d, axis=axis).dtype == np.cumsum(h, axis=axis).dtype
        assert d.real.dtype == h.real.dtype and d.imag.dtype == h.imag.dtype
        assert d.real.strides == h.real.strides and d.imag.shape == h.imag.shape
        assert d.imag.data.ptr - d.data.ptr == h.real.dtype.itemsize
        assert d.conj().dtype == h.dtype
        assert cp.angle(d).dtype == np.angle(h).dtype
    r = cp.asarray(np.ones(3, np.float32))
    assert r.real is r and r.conj() is r and r.imag.dtype == np.float32
    with pytest.raises(TypeError):
        r.imag = 1.0


def test_literals_of_complex_constants():
    from cupy_amd._core._scalar import get_scalar_literal
    assert get_scalar_literal(1 + 2j, np.complex64) == 'complex<float>(1.0f, 2.0f)'
    assert get_scalar_literal(complex(0, -0.5), np.complex128) == 'complex<double>(0.0, -0.5)'
    assert get_scalar_literal(complex('nan'), np.complex128) == 'complex<double>(CUDART_NAN, 0.0)'
