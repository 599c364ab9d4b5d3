"""Host side of the elementwise tiles over several axes: which problems get
them, and that every plan keeps the promises the kernel relies on (compile-check
mode: kernels are built, launches recorded; tests/test_gpu_packed_tiles.py
checks the values on the GPU)."""
import numpy as np
import pytest

import cupy_amd as cp
from cupy_amd import _dryrun
from cupy_amd._core import _codegen_elementwise as _cg
from cupy_amd._core import _tuning

pytestmark = pytest.mark.skipif(not _dryrun.enabled(),
                                reason='inspects recorded launches and plans')


@pytest.fixture
def plans(monkeypatch):
    seen = []
    emit = _cg.emit_packed

    def spy(name, operands, operation, *args, **kw):
        seen.append(dict(kw, operands=operands))
        return emit(name, operands, operation, *args, **kw)
    monkeypatch.setattr(_cg, 'emit_packed', spy)
    yield seen
    _tuning.set(packed_tiles='auto', order_by_outputs=True)


def _check(plan, shape_hint=None):
    tile, in_order = plan['tile'], plan['in_order']
    nd = len(tile)
    assert sorted(in_order) == list(range(nd))
    arrays = [op for op in plan['operands'] if op.kind == 'array']
    sizes = {'bool': 1, 'signed char': 1, 'unsigned char': 1, 'short': 2, 'float16': 2, 'int': 4,
             'float': 4, 'double': 8, 'long long': 8, 'complex<float>': 8, 'complex<double>': 16}
    item = max(sizes[op.store_t] for op in arrays)
    volume = int(np.prod(tile))
    assert volume <= 32768 // item
    staged = [op for op in arrays if op.name in plan['staged']]
    # the LDS image of every staged input, padding included, fits a workgroup's share
    assert sum(sizes[op.store_t] for op in staged) * (volume + volume // 8 + 1) <= 64 * 1024
    piece_out = int(np.prod(tile[nd - plan['ogroup']:]))
    piece_in = int(np.prod([tile[a] for a in in_order[:plan['group']]]))
    for piece, width in ((piece_out, plan['vec']), (piece_in, plan['svec'])):
        assert width == 1 or piece % width == 0 or piece >= 4 * width
    assert plan['unit_first'] or (plan['svec'] == 1 and plan['group'] == 1)
    assert set(plan['zero_moving']) <= set(plan['zero_last'])
    assert not set(plan['staged']) & set(plan['zero_last'])


@pytest.mark.parametrize('dtype', ['float32', 'float16', 'int64', 'uint8', 'complex128'])
def test_small_trailing_axes_get_tiles_over_several_axes(plans, dtype):
    cases = [((5000, 4, 3), (0, 2, 1)), ((4, 9000, 4), (2, 1, 0)), ((9, 168, 1024, 2), (0, 2, 1, 3)),
             ((4000, 8, 8), (0, 2, 1)), ((5, 51, 144, 4), (1, 3, 2, 0)), ((3, 4, 5, 6, 70), (4, 1, 0, 3, 2)),
             ((2, 3, 4, 5, 6, 7), (5, 4, 3, 2, 1, 0))]
    for shape, perm in cases:
        n0 = len(plans)
        x = cp.asarray(np.ones(shape, dtype))
        out = cp.ascontiguousarray(x.transpose(perm))
        assert out.shape == tuple(shape[p] for p in perm)
        assert len(plans) == n0 + 1, (shape, perm)
        assert plans[-1]['staged'] == ('in0',)
        _check(plans[-1])


def test_large_tiles_of_two_axes_keep_the_tiled_kernel(plans):
    x = cp.asarray(np.ones((64, 256, 256), 'float32'))
    cp.ascontiguousarray(x.transpose(0, 2, 1))
    cp.ascontiguousarray(x.transpose(2, 1, 0))
    assert not plans
    _tuning.set(packed_tiles=True)
    cp.ascontiguousarray(x.transpose(0, 2, 1))
    assert len(plans) == 1
    _check(plans[-1])
    _tuning.set(packed_tiles=False)
    y = cp.asarray(np.ones((500, 4, 3), 'float32'))
    cp.ascontiguousarray(y.transpose(0, 2, 1))
    assert len(plans) == 1


def test_a_permuted_destination_becomes_the_array_that_is_walked_in_order(plans):
    x = cp.asarray(np.ones((369, 81, 14, 4), 'complex64'))
    base = cp.asarray(np.zeros((81, 4, 369, 14), 'complex64'))
    dst = base.transpose(2, 0, 3, 1)
    cp.copyto(dst, x)
    assert len(plans) == 1
    plan = plans[-1]
    _check(plan)
    # the axes come in the order of the destination's strides: its last axis has unit stride
    assert plan['staged'] == ('in0',) and plan['tile'][-1] > 1
    _tuning.set(order_by_outputs=False)
    cp.copyto(dst, x)
    assert len(plans) == 1


def test_a_value_per_row(plans):
    x = cp.asarray(np.ones((3, 15983, 7), 'float32'))
    m = cp.asarray(np.ones((1, 15983, 1), 'float32'))
    x - m
    plan = plans[-1]
    _check(plan)
    # rows of 28 bytes: pieces of several rows, the value looked up per element
    assert plan['zero_last'] == ('in1',) and plan['zero_moving'] == ('in1',) and plan['ogroup'] >= 2
    y = cp.asarray(np.ones((2685, 5, 78), 'float16'))
    s = cp.asarray(np.ones((1, 5, 1), 'float16'))
    y * s
    plan = plans[-1]
    _check(plan)
    # rows of 156 bytes: one row per piece, the value read once per access
    assert plan['zero_last'] == ('in1',) and plan['zero_moving'] == () and plan['ogroup'] == 1


def test_bodies_that_use_the_element_index_stay_out(plans):
    k = cp.ElementwiseKernel('T x', 'T y', 'y = x + i', 'plus_index')
    x = cp.asarray(np.ones((500, 4, 3), 'float32'))
    k(x.transpose(0, 2, 1))
    assert not plans
