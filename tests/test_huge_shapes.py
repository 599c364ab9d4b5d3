"""Launch geometry for arrays beyond 2**31 elements, without a GPU: in the
compile-check mode allocations are addresses only, so the host path can be
driven with shapes of any size.  A dispatch holds its size in work-items in 32
bits per dimension; launches beyond that are rejected by Function.launch_packed,
so every case below would raise if a grid were too large.  The same shapes run
on the device in tests/test_gpu_huge.py."""
import numpy as np
import pytest

import cupy_amd as cp
from cupy_amd import _dryrun

pytestmark = pytest.mark.skipif(not _dryrun.enabled(),
                                reason='drives the host path with fake allocations')


def launches_of(fn):
    n0 = len(_dryrun.launches)
    out = fn()
    return out, _dryrun.launches[n0:]


CASES = {
    'flat': lambda: cp.empty((2 ** 32 + 1,), np.int8) + cp.empty((2 ** 32 + 1,), np.int8),
    'full_sum': lambda: cp.empty((2 ** 32 + 1,), np.int8).sum(),
    'argmax': lambda: cp.empty((2 ** 32 + 1,), np.int8).argmax(),
    'rows_few': lambda: cp.empty((3, 2 ** 30 + 1), np.int8).sum(axis=1),
    'rows_many': lambda: cp.empty((2 ** 25, 64), np.int8).sum(axis=1),
    'rows_very_many': lambda: cp.empty((2 ** 29, 4), np.int8).sum(axis=1),
    'flat_row_vector': lambda: cp.empty((2 ** 30 + 1, 3), np.int8) + cp.empty((1, 3), np.int8),
    'rows_flat': lambda: cp.empty((2 ** 29, 5), np.int8).sum(axis=1),
    'windows': lambda: cp.empty((2 ** 29, 5), np.int8)[:, 1:4] + cp.empty((2 ** 29, 5), np.int8)[:, 0:3],
    'batched_transpose': lambda: cp.ascontiguousarray(
        cp.empty((3, 30000, 30000), np.int8).transpose(0, 2, 1)),
    'middle_axis': lambda: cp.empty((3, 30000, 30000), np.int8).sum(axis=1),
    'cols_wide': lambda: cp.empty((9, 2 ** 30 + 1), np.int8).sum(axis=0),
    'cols_wide_few_rows': lambda: cp.empty((3, 2 ** 30 + 1), np.int8).sum(axis=0),
    'cols_split': lambda: cp.empty((2 ** 16, 2 ** 16), np.int8).sum(axis=0),
    'tiled': lambda: cp.empty((2 ** 17, 2 ** 16), np.int8).T * np.int8(2),
    'generic': lambda: cp.empty((70, 2 ** 13, 2 ** 13), np.int8)[::2, :, ::2].sum(axis=1),
    'scan_rows': lambda: cp.cumsum(cp.empty((2 ** 32 + 1,), np.int8), dtype='b'),
    'scan_cols': lambda: cp.cumsum(cp.empty((3, 2 ** 30 + 1), np.int8), axis=0, dtype='b'),
}


@pytest.mark.parametrize('name', sorted(CASES))
def test_dispatch_fits_32_bit_work_item_counts(name):
    _, launches = launches_of(CASES[name])
    assert launches
    for kernel, grid, block, _, _ in launches:
        for g, b in zip(grid, block):
            assert 1 <= g * b <= 0xffffffff, (kernel, grid, block)
        assert grid[1] <= 65535 and grid[2] <= 65535, (kernel, grid)


def test_an_oversized_dispatch_is_rejected_not_truncated():
    k = cp.RawKernel('extern "C" __global__ void nop(int* p) {}', 'nop')
    x = cp.empty((4,), np.int32)
    with pytest.raises(ValueError, match='work-items'):
        k((2 ** 24,), (256,), (x,))


def test_column_blocks_beyond_grid_x_continue_along_grid_z():
    from cupy_amd._core import _tuning
    # a thread per column here, so that the column blocks outnumber grid.x
    _tuning.set(unaligned_vectors=False)
    try:
        out, launches = launches_of(CASES['cols_wide'])
    finally:
        _tuning.set(unaligned_vectors=True)
    (kernel, grid, block, _, _), = launches
    assert grid[2] == 2 and grid[0] * grid[2] * 64 >= 2 ** 30 + 1
    assert out.shape == (2 ** 30 + 1,)


def test_reduction_over_a_middle_axis_is_one_batched_column_kernel():
    out, launches = launches_of(lambda: cp.empty((33, 65, 31277), np.float32).sum(axis=1))
    (kernel, grid, block, _, _), = launches
    assert out.shape == (33, 31277)
    # column blocks of 64 lanes x 4 columns, none straddling two batch rows
    assert grid[0] == 33 * ((31277 + 255) // 256) and grid[1] == 1
    out, launches = launches_of(lambda: cp.empty((4, 100000, 64), np.float32).max(axis=1))
    assert len(launches) == 2 and launches[0][1][1] > 1       # reduce axis split, then combined
    assert out.shape == (4, 64)
