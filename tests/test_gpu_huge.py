"""Arrays beyond 2**31 elements or 2**31 bytes: the kernels then compute
offsets (and, for arg-reductions, indices) in 64 bits.  The reference holds
such cases as slow tests (tests/cupy_tests/sorting_tests/test_search.py:88-92,
168-173 index beyond 2**32; math_tests/test_sumprod.py:68-74 broadcast sum of
2**31 elements; :845-856 scan of 2**32 elements).

Inputs are generated on the device from the element index and results are
checked on the device against closed forms of the same index, so nothing large
crosses to the host."""
import numpy as np
import pytest

import cupy_amd as cp

pytestmark = pytest.mark.gpu

_fill_mod100_i8 = cp.ElementwiseKernel('', 'int8 y', 'y = i % 100', 'fill_mod100_i8')
_fill_mod50_i8 = cp.ElementwiseKernel('', 'int8 y', 'y = i % 50', 'fill_mod50_i8')
_fill_mod1000_f32 = cp.ElementwiseKernel('', 'float32 y', 'y = i % 1000', 'fill_mod1000_f32')
_fill_half_f64 = cp.ElementwiseKernel('', 'float64 y', 'y = i * 0.5', 'fill_half_f64')


@pytest.fixture(autouse=True)
def release_memory():
    yield
    cp.get_default_memory_pool().free_all_blocks()


def sum_mod(n, m):
    """sum(i % m for i in range(n))"""
    full, rest = divmod(n, m)
    return full * (m * (m - 1) // 2) + rest * (rest - 1) // 2


def sum_mod100(n):
    return sum_mod(n, 100)


def test_elementwise_and_full_reductions_beyond_2_to_32_elements():
    n = 2 ** 32 + 5
    a = _fill_mod50_i8(size=n)                        # loop index in 64 bits
    assert a.shape == (n,)
    for pos in (0, 49, 50, 2 ** 31 - 1, 2 ** 31, 2 ** 32 - 1, 2 ** 32, n - 1):
        assert int(a[pos].get()) == pos % 50, pos
    assert int(a.sum().get()) == sum_mod(n, 50)       # two-pass reduction, 64-bit offsets
    b = a + a                                         # flat vector kernel
    assert int(b.sum().get()) == 2 * sum_mod(n, 50)
    for pos in (2 ** 31 + 7, 2 ** 32 + 3, n - 1):
        assert int(b[pos].get()) == 2 * (pos % 50), pos
    del b
    # index beyond 2**32 out of an arg-reduction; ties resolve to the first
    assert int(a.argmax().get()) == 49
    assert int(a.argmin().get()) == 0
    a.fill(0)
    a[n - 1] = 1
    assert int(a.argmax().get()) == n - 1
    a[2 ** 32 + 1] = 1
    assert int(a.argmax().get()) == 2 ** 32 + 1
    a[n - 1] = -1
    assert int(a.argmin().get()) == n - 1


def test_scan_of_2_to_32_elements():
    n = 2 ** 32
    a = cp.ones(n, 'b')
    r = cp.cumprod(a, dtype='b')
    assert r.shape == (n,) and r.dtype == np.int8
    assert bool((r == 1).all().get())
    del r
    a[2 ** 31 + 11] = 0                               # everything after it becomes 0
    r = cp.cumprod(a, dtype='b')
    assert int(r.sum().get()) == 2 ** 31 + 11
    assert int(r[2 ** 31 + 10].get()) == 1 and int(r[2 ** 31 + 11].get()) == 0
    assert int(r[n - 1].get()) == 0


def test_more_than_2_to_31_bytes_with_fewer_elements():
    n = 2 ** 28 + 3
    x = _fill_half_f64(size=n)
    y = x * 2.0
    check = cp.ElementwiseKernel('float64 y', 'bool ok', 'ok = y == (double)i', 'is_index_f64')
    assert bool(check(y).all().get())
    assert float(y[n - 1].get()) == n - 1


def test_transposed_operand_beyond_2_to_31_bytes():
    rows, cols = 40000, 20000                         # 3.2 GB of float32
    x = _fill_mod1000_f32(size=rows * cols).reshape(rows, cols)
    t = x.T * 2.0                                     # tiled kernel, 64-bit offsets
    assert t.shape == (cols, rows) and t._c_contiguous
    check = cp.ElementwiseKernel(
        'float32 t', 'bool ok',
        'const long long c = i / 40000, r = i % 40000;'
        'ok = t == 2.0f * (float)((r * 20000 + c) % 1000)', 'is_transposed_mod1000')
    assert bool(check(t).all().get())
    host = t[cols - 3:, rows - 5:].get()
    r, c = np.meshgrid(np.arange(rows - 5, rows), np.arange(cols - 3, cols))
    assert np.array_equal(host, (2.0 * ((r * cols + c) % 1000)).astype(np.float32))


def test_scan_down_the_columns_of_a_narrow_array_beyond_2_to_31_elements():
    """(2**29 + 3, 5) int8 along axis 0: the one-pass kernel for narrow arrays
    with 64-bit offsets; the running count wraps as int8 wraps."""
    rows = 2 ** 29 + 3
    a = cp.ones((rows, 5), 'b')
    r = cp.cumsum(a, axis=0, dtype='b')
    assert r.shape == (rows, 5) and r.dtype == np.int8
    check = cp.ElementwiseKernel(
        'int8 s', 'bool ok', 'ok = s == (signed char)(((i / 5) + 1) & 255)', 'is_row_count_mod256')
    assert bool(check(r).all().get())


def test_axis_reductions_and_scans_with_rows_beyond_2_to_30():
    m = 2 ** 30 + 1
    a = _fill_mod100_i8(size=3 * m).reshape(3, m)
    rows = a.sum(axis=1).get()
    want = [sum_mod100((k + 1) * m) - sum_mod100(k * m) for k in range(3)]
    assert rows.tolist() == want
    colsum = a.sum(axis=0)
    assert colsum.shape == (m,) and colsum.dtype == np.int64
    check = cp.ElementwiseKernel(
        'int64 s', 'bool ok',
        'const long long m = 1073741825LL;'
        'ok = s == (i % 100) + ((m + i) % 100) + ((2 * m + i) % 100)', 'is_colsum_mod100')
    assert bool(check(colsum).all().get())
    del colsum
    running = cp.cumsum(a, axis=0, dtype=np.int16)
    check3 = cp.ElementwiseKernel(
        'int16 s', 'bool ok',
        'const long long m = 1073741825LL; const long long k = i / m, j = i % m;'
        'long long w = 0; for (long long q = 0; q <= k; ++q) w += (q * m + j) % 100;'
        'ok = s == w', 'is_running_colsum_mod100')
    assert bool(check3(running).all().get())
    del running
    # argmax over rows whose element offsets need 64 bits although the index
    # within a row does not
    b = a.reshape(-1)[:3000000 * 1027].reshape(3000000, 1027)
    idx = b.argmax(axis=1)
    check2 = cp.ElementwiseKernel(
        'int64 k', 'bool ok', 'ok = k == (99 - ((long long)i * 1027) % 100) % 100', 'is_first_99')
    assert bool(check2(idx).all().get())


def test_column_reduction_whose_blocks_continue_along_grid_z():
    m = 2 ** 30 + 1                                   # more column blocks than grid.x holds
    a = _fill_mod100_i8(size=9 * m).reshape(9, m)
    from cupy_amd._core import _tuning
    _tuning.set(unaligned_vectors=False)              # rows of odd length: a thread per column
    try:
        colsum = a.sum(axis=0)
    finally:
        _tuning.set(unaligned_vectors=True)
    check = cp.ElementwiseKernel(
        'int64 s', 'bool ok',
        'const long long m = 1073741825LL; long long w = 0;'
        'for (long long k = 0; k < 9; ++k) w += (k * m + i) % 100;'
        'ok = s == w', 'is_colsum9_mod100')
    assert bool(check(colsum).all().get())


def test_narrow_matrix_walked_as_one_piece_beyond_2_to_31_elements():
    """Column sums of a (2**24 + 3, 130) int8 matrix: the kernel that walks a
    narrow matrix as one contiguous piece computes its offsets in 64 bits."""
    rows, width = 2 ** 24 + 3, 130
    a = _fill_mod100_i8(size=rows * width).reshape(rows, width)
    from cupy_amd.cuda import function
    seen = []
    orig = function.Function.launch_packed
    function.Function.launch_packed = lambda self, grid, *args, **kw: (
        seen.append((self.name, grid)), orig(self, grid, *args, **kw))[1]
    try:
        colsum = a.sum(axis=0)
        colmax = a.max(axis=0)
    finally:
        function.Function.launch_packed = orig
    assert seen[0][0] == 'cupy_sum' and seen[0][1][1] == 1 and seen[0][1][2] == 1
    # element (r, c) holds (130 r + c) % 100 = (30 (r % 10) + c) % 100
    r10 = np.arange(10)
    counts = np.array([(rows - k + 9) // 10 for k in range(10)], dtype=np.int64)
    table = (30 * r10[:, None] + np.arange(width)[None, :]) % 100          # (10, width)
    np.testing.assert_array_equal(colsum.get(), (counts[:, None] * table).sum(axis=0))
    np.testing.assert_array_equal(colmax.get(), table.max(axis=0).astype(np.int8))


def test_broadcast_input_of_2_to_31_elements():
    base = _fill_mod100_i8(size=2048 * 1024).reshape(2048, 1, 1024)
    a = cp.broadcast_to(base, (2048, 1024, 1024))
    got = a.sum(axis=2)
    assert got.shape == (2048, 1024) and got.dtype == np.int64
    want = base.sum(axis=2)                           # (2048, 1), the same for every copy
    assert bool((got == want).all().get())
    assert np.array_equal(want.get()[:3, 0],
                          [sum_mod100((k + 1) * 1024) - sum_mod100(k * 1024) for k in range(3)])


def test_strided_view_into_more_than_2_to_31_bytes():
    n = 1300
    base = _fill_mod100_i8(size=n * n * n).reshape(n, n, n)
    other = _fill_mod100_i8(size=n * (n // 2) * n).reshape(n, n // 2, n)
    r = base[:, ::2, :] + other
    assert r.shape == (n, n // 2, n)
    for k in (0, n // 2, n - 1):
        i0, i1, i2 = np.meshgrid([k], np.arange(0, n, 2), np.arange(n), indexing='ij')
        lhs = (i0 * n * n + i1 * n + i2) % 100
        j0, j1, j2 = np.meshgrid([k], np.arange(n // 2), np.arange(n), indexing='ij')
        rhs = (j0 * (n // 2) * n + j1 * n + j2) % 100
        assert np.array_equal(r[k].get(), (lhs + rhs)[0].astype(np.int8)), k


def test_many_short_rows():
    n_rows, width = 2 ** 25, 64                      # 2 GiB of int8, 33.5 million results
    a = _fill_mod100_i8(size=n_rows * width).reshape(n_rows, width)
    rows = a.sum(axis=1)
    assert rows.shape == (n_rows,) and rows.dtype == np.int64
    assert int(rows.sum().get()) == sum_mod100(n_rows * width)
    for k in (0, 1, 2 ** 24 + 3, n_rows - 1):
        assert int(rows[k].get()) == sum_mod100((k + 1) * width) - sum_mod100(k * width), k
    first = a.argmax(axis=1)
    check = cp.ElementwiseKernel(
        'int64 k', 'bool ok',
        # the row starts at (64 i) % 100; the largest value is 99 if the row
        # reaches it, the last element of the row otherwise
        'const long long s = ((long long)i * 64) % 100;'
        'ok = k == (s + 63 >= 99 ? 99 - s : 63)', 'is_row_argmax_mod100')
    assert bool(check(first).all().get())


def test_very_many_tiny_rows():
    n_rows = 2 ** 29                                  # 2 GiB in, 4 GiB of int64 out
    a = _fill_mod100_i8(size=n_rows * 4).reshape(n_rows, 4)
    rows = a.sum(axis=1)
    check = cp.ElementwiseKernel(
        'int64 s', 'bool ok',
        'const long long b = (long long)i * 4;'
        'ok = s == b % 100 + (b + 1) % 100 + (b + 2) % 100 + (b + 3) % 100', 'is_rowsum4_mod100')
    assert bool(check(rows).all().get())


def test_three_dimensional_view_that_does_not_merge():
    na, nb, nc = 70, 8192, 8192                       # 4.7e9 elements underneath
    base = _fill_mod100_i8(size=na * nb * nc).reshape(na, nb, nc)
    view = base[::2, ::2, ::2]                        # no two axes merge
    assert view.shape == (35, 4096, 4096)
    value = '(2 * a * 8192LL * 8192 + 2 * b * 8192 + 2 * c) % 100'
    # elementwise through the indexer kernel, offsets in 64 bits
    r = view + np.int8(1)
    assert r._c_contiguous and r.shape == view.shape
    check = cp.ElementwiseKernel(
        'int8 v', 'bool ok',
        'const long long c = i % 4096, b = (i / 4096) % 4096, a = i / (4096LL * 4096);'
        'ok = v == VALUE + 1'.replace('VALUE', value), 'is_view_plus_one')
    assert bool(check(r).all().get())
    del r
    # reduction over the middle axis of the same view
    s = view.sum(axis=1)
    assert s.shape == (35, 4096) and s.dtype == np.int64
    check2 = cp.ElementwiseKernel(
        'int64 s', 'bool ok',
        'const long long c = i % 4096, a = i / 4096; long long w = 0;'
        'for (long long b = 0; b < 4096; ++b) w += VALUE;'
        'ok = s == w'.replace('VALUE', value), 'is_view_middle_sum')
    assert bool(check2(s).all().get())
    # and an arg-reduction over its leading axis
    k = view.argmax(axis=0)
    assert k.shape == (4096, 4096) and k.dtype == np.int64
    check3 = cp.ElementwiseKernel(
        'int64 k', 'bool ok',
        'const long long c = i % 4096, b = i / 4096; long long best = -1, at = -1;'
        'for (long long a = 0; a < 35; ++a) {'
        '  const long long v = VALUE;'
        '  if (v > best) { best = v; at = a; } }'
        'ok = k == at'.replace('VALUE', value), 'is_view_leading_argmax')
    assert bool(check3(k).all().get())


def test_matrix_plus_row_vector_beyond_2_to_31_elements():
    m = 2 ** 30 + 1
    a = _fill_mod100_i8(size=3 * m).reshape(m, 3)
    row = cp.asarray(np.array([[1, 2, 3]], np.int8))
    r = a + row                                       # flat kernel, row and column by division
    check = cp.ElementwiseKernel(
        'int8 v', 'bool ok', 'ok = v == (signed char)(i % 100 + i % 3 + 1)', 'is_plus_row')
    assert bool(check(r).all().get())
    del r
    col = _fill_mod50_i8(size=m).reshape(m, 1)
    r = a - col
    check2 = cp.ElementwiseKernel(
        'int8 v', 'bool ok', 'ok = v == (signed char)(i % 100 - (i / 3) % 50)', 'is_minus_col')
    assert bool(check2(r).all().get())


def test_short_odd_rows_and_windows_beyond_2_to_31_elements():
    n_rows = 2 ** 29
    a = _fill_mod100_i8(size=n_rows * 5).reshape(n_rows, 5)
    rows = a.sum(axis=1)                              # rows staged through the LDS
    check = cp.ElementwiseKernel(
        'int64 s', 'bool ok',
        'const long long b = (long long)i * 5; long long w = 0;'
        'for (int k = 0; k < 5; ++k) w += (b + k) % 100; ok = s == w', 'is_rowsum5_mod100')
    assert bool(check(rows).all().get())
    del rows
    w = a[:, 1:4] + a[:, 0:3]                         # windows: row by row in vectors
    check2 = cp.ElementwiseKernel(
        'int8 v', 'bool ok',
        'const long long r = i / 3, c = i % 3;'
        'ok = v == (signed char)((r * 5 + c + 1) % 100 + (r * 5 + c) % 100)', 'is_window_sum')
    assert bool(check2(w).all().get())


def test_permuted_axes_beyond_2_to_31_elements():
    nb, n = 3, 30000                                  # 2.7e9 elements
    a = _fill_mod100_i8(size=nb * n * n).reshape(nb, n, n)
    t = cp.ascontiguousarray(a.transpose(0, 2, 1))    # tiled kernel with a batch axis
    check = cp.ElementwiseKernel(
        'int8 v', 'bool ok',
        'const long long n = 30000, c = i % n, r = (i / n) % n, b = i / (n * n);'
        'ok = v == (signed char)((b * n * n + c * n + r) % 100)', 'is_batch_transposed')
    assert bool(check(t).all().get())
    del t
    s = a.sum(axis=1)                                 # reduction over the middle axis
    assert s.shape == (nb, n) and s.dtype == np.int64
    check2 = cp.ElementwiseKernel(
        'int64 s', 'bool ok',
        'const long long n = 30000, c = i % n, b = i / n; long long w = 0;'
        'for (long long r = 0; r < n; ++r) w += (b * n * n + r * n + c) % 100; ok = s == w',
        'is_middle_sum')
    assert bool(check2(s).all().get())


def test_tiles_over_several_axes_beyond_2_to_31_elements():
    from cupy_amd._core import _tuning
    nb = 180000001                                    # 2.16e9 elements
    a = _fill_mod100_i8(size=nb * 12).reshape(nb, 4, 3)
    t = cp.ascontiguousarray(a.transpose(0, 2, 1))    # every tile spans the two small axes
    check = cp.ElementwiseKernel(
        'int8 v', 'bool ok',
        'const long long c = i % 4, r = (i / 4) % 3, b = i / 12;'
        'ok = v == (signed char)((b * 12 + c * 3 + r) % 100)', 'is_small_transposed')
    assert bool(check(t).all().get())
    del t, a
    nb, n = 3, 30000                                  # 2.7e9 elements
    a = _fill_mod100_i8(size=nb * n * n).reshape(nb, n, n)
    _tuning.set(packed_tiles=True)
    try:
        t = cp.ascontiguousarray(a.transpose(0, 2, 1))
    finally:
        _tuning.set(packed_tiles='auto')
    check = cp.ElementwiseKernel(
        'int8 v', 'bool ok',
        'const long long n = 30000, c = i % n, r = (i / n) % n, b = i / (n * n);'
        'ok = v == (signed char)((b * n * n + c * n + r) % 100)', 'is_batch_transposed')
    assert bool(check(t).all().get())
