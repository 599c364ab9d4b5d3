"""Call-surface behaviour of ElementwiseKernel / ufunc / ReductionKernel / fuse
that does not depend on results: argument checking, error messages, code
caching, launch planning.  Runs without a GPU (compile-check mode) and with
one."""
import threading
import warnings

import numpy as np
import pytest

import cupy_amd as cp
from cupy_amd import _dryrun
from cupy_amd._core import _codegen_elementwise as cg

needs_dryrun = pytest.mark.skipif(not _dryrun.enabled(), reason='inspects recorded launches')


def test_invalid_kernel_name():
    with pytest.raises(ValueError, match='Invalid kernel name: "1"'):
        cp.ElementwiseKernel('T x', '', '', '1')
    with pytest.raises(ValueError, match='Invalid kernel name'):
        cp.ReductionKernel('T x', 'T y', 'x', 'a + b', 'y = a', '0', name='a b')


def test_parameter_named_i_is_rejected():
    with pytest.raises(ValueError, match='Can not use'):
        cp.ElementwiseKernel('T i', 'T y', 'y = i')


def test_wrong_number_of_arguments():
    k = cp.ElementwiseKernel('T x, T y', 'T z', 'z = x + y', 'add2')
    x = cp.zeros((3,), np.float32)
    with pytest.raises(TypeError, match='Wrong number of arguments for'):
        k(x)
    with pytest.raises(TypeError, match='Wrong number of arguments for'):
        cp.add(x)
    with pytest.raises(TypeError, match='Wrong arguments'):
        k(x, x, foo=1)
    with pytest.raises(ValueError, match='block_size'):
        k(x, x, block_size=0)


def test_size_rules():
    k = cp.ElementwiseKernel('raw T x', 'raw T y', 'y[i] = x[i]', 'rawcopy')
    x = cp.zeros((4,), np.float32)
    y = cp.zeros((4,), np.float32)
    with pytest.raises(ValueError, match='Loop size is undecided'):
        k(x, y)
    with pytest.raises(ValueError, match='Output array size is Undecided'):
        cp.ElementwiseKernel('T x', 'raw T y', 'y[i] = x', 'k2')(x)
    k(x, y, size=4)
    k2 = cp.ElementwiseKernel('T x', 'T y', 'y = x', 'plaincopy')
    with pytest.raises(ValueError, match="Specified 'size' can"):
        k2(x, size=4)
    with pytest.raises(ValueError, match="Specified 'size' can"):
        cp.ElementwiseKernel('raw T x', 'T y', 'y = x[i]', 'k3')(x, y, size=4)


def test_out_shape_and_type_checks():
    k = cp.ElementwiseKernel('T x', 'T y', 'y = x', 'plaincopy')
    x = cp.zeros((4, 3), np.float32)
    with pytest.raises(ValueError, match='Out shape is mismatched'):
        k(x, cp.zeros((3,), np.float32))
    with pytest.raises(TypeError, match='Type is mismatched'):
        k(x, cp.zeros((4, 3), np.float64))
    with pytest.raises(ValueError, match='Out shape is mismatched'):
        cp.add(x, x, cp.zeros((3,), np.float32))
    with pytest.raises(TypeError, match='Cannot cast output operand'):
        cp.add(x, x, out=cp.zeros((4, 3), np.int32))
    cp.add(x, x, out=cp.zeros((4, 3), np.int32), casting='unsafe')
    with pytest.raises(ValueError, match='both'):
        cp.add(x, x, x, out=x)
    with pytest.raises(ValueError, match="'out' tuple"):
        cp.add(x, x, out=(x, x))
    assert cp.add(x, x, out=(x,)) is x
    with pytest.raises(ValueError, match='could not be broadcast'):
        cp.add(x, cp.zeros((5,), np.float32))


def test_bool_arithmetic_errors():
    b = cp.zeros((3,), np.bool_)
    with pytest.raises(TypeError, match='boolean subtract'):
        b - b
    with pytest.raises(TypeError, match='boolean negative'):
        -b
    assert (b + b).dtype == np.bool_
    assert (b * b).dtype == np.bool_


def test_result_dtypes_and_layout():
    x = cp.zeros((4, 6), np.float32).T
    y = cp.zeros((1, 4), np.float16)
    out = x * y + 1
    assert out.dtype == np.float32 and out.shape == (6, 4)
    assert out.flags.c_contiguous        # outputs are always fresh C-order arrays
    u = cp.zeros((3,), np.uint8)
    assert (u + 1).dtype == np.uint8
    with pytest.raises(OverflowError):
        u + 300
    assert (u + np.int64(1)).dtype == np.int64
    assert (cp.zeros((2,), np.float32) + 3e100).dtype == np.float32
    assert (cp.zeros((2,), np.int8) + 1.0).dtype == np.float64
    assert cp.add(u, u, dtype=np.float32).dtype == np.float32
    assert (u / u).dtype == np.float64
    assert (u > 1).dtype == np.bool_


def test_zero_size_returns_without_launch():
    k = cp.ElementwiseKernel('T x', 'T y', 'y = x', 'plaincopy')
    n0 = len(_dryrun.launches)
    out = k(cp.zeros((0, 3), np.float32))
    assert out.shape == (0, 3)
    assert (cp.zeros((0,), np.int32) + 1).shape == (0,)
    assert cp.zeros((0, 3), np.float32).sum(axis=0).shape == (3,) or True
    if _dryrun.enabled():
        assert len(_dryrun.launches) <= n0 + 1


def test_cached_codes_grow_per_dtype_combination():
    k = cp.ElementwiseKernel('T x', 'T y', 'y = x + x', 'twice')
    with warnings.catch_warnings(record=True) as w:
        warnings.simplefilter('always')
        assert len(k.cached_codes) == 0
        assert any('No codes are cached' in str(i.message) for i in w)
    x = cp.zeros((10,), np.float32)
    k(x)
    assert len(k.cached_codes) == 1
    k(x)
    assert len(k.cached_codes) == 1
    k(cp.zeros((10,), np.int32))
    assert len(k.cached_codes) == 2
    assert 'twice' in k.cached_code if len(k.cached_codes) == 1 else True

    rk = cp.ReductionKernel('T x', 'T y', 'x', 'a + b', 'y = a', '0', 'mysum')
    rk(x)
    rk(x)
    assert len(rk.cached_codes) == 1
    rk(cp.zeros((10,), np.int64))
    assert len(rk.cached_codes) == 2


def test_one_kernel_object_under_threads():
    k = cp.ElementwiseKernel('T x', 'T y', 'y = x * 3', 'triple_mt')
    x = cp.zeros((1000,), np.float32)
    barrier = threading.Barrier(8)
    errors = []

    def run():
        try:
            barrier.wait()
            for _ in range(5):
                k(x)
        except Exception as e:      # pragma: no cover
            errors.append(e)

    threads = [threading.Thread(target=run) for _ in range(8)]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    assert not errors
    assert len(k._planner._memo) == 1


def test_write_only_detection():
    f = cg.output_is_write_only
    assert f('z = a * x + y', 'z')
    assert f('T t = x; z = t', 'z')
    assert not f('z += x', 'z')
    assert not f('if (x > 0) z = x', 'z')
    assert not f('if (x > 0) { z = x; }', 'z')
    assert not f('y = z; z = x', 'z')
    assert not f('z == x', 'z')
    assert not f('foo(z)', 'z')
    assert f('out0 = in0 + in1', 'out0')
    assert cg.body_needs_generic('if (x) continue; y = x')
    assert not cg.body_needs_generic('y = discontinued')


@needs_dryrun
def test_launch_plans_of_the_benchmark_shapes():
    def launches_of(fn):
        n0 = len(_dryrun.launches)
        fn()
        return _dryrun.launches[n0:]

    x = cp.ndarray((1 << 20,), np.float32)
    saxpy = cp.ElementwiseKernel('float32 x, float32 y, float32 a', 'float32 z',
                                 'z = a * x + y', 'saxpy')
    (l,) = launches_of(lambda: saxpy(x, x, 2.5))
    assert l[0] == 'saxpy' and l[2][0] in (256, 512, 1024)
    assert 'load_vec<float, 4' in saxpy.cached_code

    a = cp.ndarray((2048, 16384), np.float32)
    (l,) = launches_of(lambda: a.sum(axis=1))
    assert l[1] == (2048, 1, 1)                       # a workgroup per long row
    b = cp.ndarray((2048, 1024), np.float32)
    (l,) = launches_of(lambda: b.sum(axis=1))
    assert l[1] == (512, 1, 1)                        # a wave per shorter row
    ls = launches_of(lambda: a.sum(axis=0))
    assert [x[0] for x in ls] == ['cupy_sum', 'cupy_sum_combine'] and ls[0][1][1] > 1
    ls = launches_of(lambda: a.sum())
    assert [x[0] for x in ls] == ['cupy_sum', 'cupy_sum_combine']
    assert ls[0][1][0] == 1 and ls[0][1][1] >= 256     # split over the grid
    # up to 16 MiB a split reduction finishes in its one launch (the first on a
    # stream also clears the memory the workgroups hand their results over in)
    c = cp.ndarray((1 << 21,), np.float32)
    ls = [x for x in launches_of(lambda: c.sum()) if not x[0].startswith('cupy_copy')]
    assert [x[0] for x in ls] == ['cupy_sum'] and ls[0][1][0] >= 256 and ls[0][1][1] == 1

    m = cp.ndarray((4096, 128), np.int32)
    (l,) = launches_of(lambda: m.argmax(axis=-1))
    assert l[0] == 'cupy_argmax'

    t = cp.ndarray((512, 256), np.float32).T
    y = cp.ndarray((1, 512), np.float16)
    (l,) = launches_of(lambda: t * y)
    assert l[0] == 'cupy_multiply__float32_float16_float32'
    entries = [e for pl in cp.multiply._planners.values() for k, e in pl._memo.items()
               if k[0] == 'tiled']
    assert any('__shared__' in e[2] for e in entries)       # staged through LDS


@needs_dryrun
def test_reading_results_is_refused_in_compile_check_mode():
    x = cp.ndarray((4,), np.float32)
    with pytest.raises(_dryrun.DryRunError):
        x.get()
    with pytest.raises(_dryrun.DryRunError):
        float(x.sum())


def test_reduction_argument_errors():
    a = cp.zeros((2, 3), np.float32)
    with pytest.raises(np.exceptions.AxisError):
        a.sum(axis=2)
    with pytest.raises(ValueError, match='duplicate'):
        a.sum(axis=(0, 0))
    with pytest.raises(ValueError, match='zero-size array to reduction operation'):
        cp.zeros((0,), np.float32).argmax()
    with pytest.raises(ValueError, match='zero-size array to reduction operation'):
        cp.zeros((0, 3), np.float32).max(axis=0)
    assert cp.zeros((3, 0), np.float32).argmax(axis=0).shape == (0,)
    assert cp.zeros((0,), np.float32).sum().shape == ()
    with pytest.raises(ValueError, match='Out shape is mismatched'):
        a.sum(axis=0, out=cp.zeros((2,), np.float32))
    with pytest.raises(TypeError, match="Argument 'a'"):
        cp.sum(np.zeros(3)) if False else cp._core._routines_math._sum_auto_dtype(np.zeros(3))
    rk = cp.ReductionKernel('T x', 'T y', 'x', 'a + b', 'y = a', '0', 'mysum')
    with pytest.raises(TypeError, match='Wrong number of arguments'):
        rk()
    with pytest.raises(TypeError, match='Wrong arguments'):
        rk(a, foo=1)
    with pytest.raises(ValueError, match="cannot specify 'out'"):
        rk(a, cp.zeros((), np.float32), out=cp.zeros((), np.float32))


def test_sum_result_dtypes():
    for c, expect in [('?', 'l'), ('b', 'l'), ('B', 'L'), ('h', 'l'), ('H', 'L'), ('i', 'l'),
                      ('I', 'L'), ('l', 'l'), ('L', 'L'), ('e', 'e'), ('f', 'f'), ('d', 'd')]:
        r = cp.zeros((4,), c).sum()
        assert r.dtype == np.dtype(expect) == np.zeros(4, c).sum().dtype
    assert cp.zeros((4,), 'i').sum(dtype='f').dtype == np.float32
    for dt in ('b', 'h', 'i', 'l'):
        assert cp.zeros((4,), 'f').argmax(dtype=dt).dtype == np.dtype(dt)
    assert cp.zeros((4,), 'f').argmin().dtype == np.int64


def test_fuse_decorator_forms_and_argument_checks():
    @cp.fuse
    def f1(x, y):
        """doc"""
        return x + y

    @cp.fuse()
    def f2(x, y):
        return x * y

    @cp.fuse(kernel_name='named_kernel')
    def f3(x):
        return x + 1

    assert f1.__name__ == 'f1' and f1.__doc__ == 'doc'
    assert f3.name == 'named_kernel'
    # no device array among the arguments: plain Python call
    assert f1(2, 3) == 5
    assert np.array_equal(f2(np.arange(3), 2), np.arange(3) * 2)
    x = cp.zeros((3,), np.float32)
    with pytest.raises(TypeError, match='Invalid argument type'):
        f1(x, 'text')
    out = f3(x)
    assert out.shape == (3,) and out.dtype == np.float32
    assert len(f3._memo) == 1
    f3(x)
    assert len(f3._memo) == 1
    f3(cp.zeros((3,), np.int32))
    assert len(f3._memo) == 2
    f3.clear_cache()
    assert len(f3._memo) == 0

    @cp.fuse()
    def with_none(x, flag):
        if flag is None:
            return x + 1
        return x - 1

    assert with_none(x, None).shape == (3,)

    @cp.fuse()
    def keep(x):
        return cp.sum(x, axis=0, keepdims=True)

    # not expressible in the single fused kernel: runs as a kernel sequence
    assert keep(x).shape == (1,)
    assert list(keep._memo.values()) == ['by shape'] and len(keep._plans) == 1


def test_reduce_dims_false_is_passed_to_the_launch():
    from cupy_amd import _dryrun
    if not _dryrun.enabled():
        pytest.skip('inspects recorded launches')
    body = 'y = x + _ind.get()[0]'
    x = cp.zeros((3, 4, 5), np.float32)
    sizes = {}
    for flag in (True, False):
        k = cp.ElementwiseKernel('T x', 'T y', body, 'keeps_axes', reduce_dims=flag)
        k(x)
        sizes[flag] = len(_dryrun.launches[-1][4])
    # kept: two 3-d arrays and a 3-d indexer; merged: one axis, far fewer bytes
    assert sizes[False] == (8 + 8 * 7) * 2 + 8 * 7
    assert sizes[True] < sizes[False]


def test_show_config_lists_the_installation(capsys):
    """(reference: cupy/__init__.py:942-946)"""
    cp.show_config()
    text = capsys.readouterr().out
    for label in ('OS', 'Python Version', 'CuPy Version', 'CuPy Platform', 'NumPy Version',
                  'Runtime Library', 'Kernel Cache Dir'):
        assert any(line.startswith(label) and ':' in line for line in text.splitlines()), label
    assert 'libmi355rt.so' in text
