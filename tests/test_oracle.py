"""Pins the oracle: golden vectors held by the reference's tests, closed forms,
brute force and exactly-rounded arithmetic -- not re-typed formulas."""
import math

import numpy as np
import pytest

from oracle import c_oracle
from oracle import numpy_oracle as o


def test_saxpy_is_two_roundings():
    rng = np.random.default_rng(11)
    x = rng.uniform(-1, 1, 2000).astype(np.float32)
    y = rng.uniform(-1, 1, 2000).astype(np.float32)
    a = 2.5
    # each step in float64 is exact for float32 operands' product / nearly so for
    # the sum; rounding once per step must reproduce the oracle
    p = (np.float64(np.float32(a)) * x.astype(np.float64)).astype(np.float32)
    z = (p.astype(np.float64) + y.astype(np.float64)).astype(np.float32)
    assert np.array_equal(o.saxpy(a, x, y), z)
    # independent C statement of the same loop
    assert np.array_equal(c_oracle.saxpy_f32(a, x, y), z)
    # a fused multiply-add would differ somewhere on this many samples
    fused = (np.float64(a) * x.astype(np.float64) + y.astype(np.float64)).astype(np.float32)
    assert not np.array_equal(fused, z)


def test_saxpy_special_values():
    x = np.array([0.0, -0.0, np.inf, -np.inf, np.nan, 1e-45, 3e38], np.float32)
    y = np.array([-0.0, 0.0, -np.inf, 1.0, 1.0, -1e-45, 3e38], np.float32)
    with np.errstate(all='ignore'):
        z = o.saxpy(2.5, x, y)
    assert np.signbit(z[0]) == np.signbit(np.float32(0.0) + np.float32(-0.0))
    assert np.isnan(z[2]) and np.isnan(z[4])
    assert z[3] == -np.inf
    assert z[6] == np.inf          # overflow, not clamped
    # denormals are kept (2.5 * 1e-45 rounds to 3 ulp of the smallest denormal)
    assert z[5] == np.float32(2.5) * np.float32(1e-45) + np.float32(-1e-45)
    assert z[5] != 0


def test_promotion_follows_nep50(golden):
    scope = {'array': np.array, 'uint8': np.uint8, 'int64': np.int64,
             'float32': np.float32, 'float64': np.float64, 'int16': np.int16,
             'bool_': np.bool_, 'int32': np.int32, 'int8': np.int8}
    for ex in golden['nep50_examples']:
        if '==' in ex:
            continue
        lhs, rhs = ex.split(' + ')
        try:
            expect = eval(ex, dict(scope))
        except OverflowError:
            continue
        a = eval(lhs, dict(scope))
        b = eval(rhs, dict(scope))
        assert o.promote(a, b) == np.asarray(expect).dtype, ex


def test_broadcast_mul_add_types_and_values():
    rng = np.random.default_rng(2)
    x = rng.standard_normal((6, 5), dtype=np.float32).T
    y = rng.uniform(0, 2, (1, 6)).astype(np.float16)
    out = o.broadcast_mul_add(x, y, 1)
    assert out.dtype == np.float32 and out.shape == (5, 6)
    # float16 widens exactly, so float64 evaluation rounded per step must agree
    t = (x.astype(np.float64) * y.astype(np.float64)).astype(np.float32)
    assert np.array_equal(out, (t.astype(np.float64) + 1.0).astype(np.float32))


@pytest.mark.parametrize('dtype', ['int8', 'uint8', 'int32', 'int64', 'float16',
                                   'float32', 'float64'])
def test_arg_extreme_golden_cases(golden, dtype):
    dt = np.dtype(dtype)
    for case in golden['argmax_cases']:
        if case.get('float_only') and dt.kind != 'f':
            continue
        a = np.array([float(v) for v in case['values']]).astype(dt)
        assert o.argmax_first(a) == case['argmax'] == np.argmax(a)
    for case in golden['argmin_cases']:
        if case.get('float_only') and dt.kind != 'f':
            continue
        a = np.array([float(v) for v in case['values']]).astype(dt)
        assert o.argmin_first(a) == case['argmin'] == np.argmin(a)


def test_arg_extreme_brute_force_matches_numpy_and_c():
    rng = np.random.default_rng(5)
    m = rng.integers(0, 4, (40, 37)).astype(np.float64)
    m[3, 5] = np.nan
    m[3, 9] = np.nan
    m[7, 0] = np.nan
    for axis in (0, 1, None):
        assert np.array_equal(o.argmax_first(m, axis), np.argmax(m, axis))
        assert np.array_equal(o.argmin_first(m, axis), np.argmin(m, axis))
    clean = rng.integers(0, 4, (40, 300)).astype(np.float64)
    assert np.array_equal(c_oracle.block_reduce_arg(clean, True), np.argmax(clean, 1))
    assert np.array_equal(c_oracle.block_reduce_arg(clean, False), np.argmin(clean, 1))
    assert np.array_equal(o.argmax_fast(clean, 1), np.argmax(clean, 1))
    assert np.array_equal(o.argmin_fast(clean, 0), np.argmin(clean, 0))


def test_argmax_f_order_flattens_in_c_order():
    a = np.asfortranarray(np.array([[1, 9, 3], [9, 2, 9]], np.int32))
    assert o.argmax_first(a) == 1 == np.argmax(a)


def test_sum_against_exact_sum():
    rng = np.random.default_rng(3)
    a = rng.standard_normal(5000).astype(np.float32)
    exact = o.sum_exact(a)
    scale = math.fsum(abs(float(v)) for v in a)
    assert abs(float(o.sum_fp(a)) - exact) <= 1e-6 * scale
    rows = a.reshape(50, 100)
    for r, got in zip(rows, c_oracle.block_reduce_sum(rows, 1)):
        assert abs(float(got) - o.sum_exact(r)) <= 1e-5 * math.fsum(abs(float(v)) for v in r)
    cols = c_oracle.block_reduce_sum(rows, 0)
    for j in range(100):
        assert abs(float(cols[j]) - o.sum_exact(rows[:, j])) <= 1e-5 * 50


def test_integer_sums_are_exact_and_wrap(small_configs):
    i8 = small_configs['i8']
    assert np.array_equal(o.sum_int(i8, 0), small_configs['i8_ax0'])
    assert np.array_equal(c_oracle.block_reduce_sum(i8, 0), small_configs['i8_ax0'])
    assert np.array_equal(c_oracle.block_reduce_sum(i8, 1), small_configs['i8_ax1'])
    big = np.full(4, 2 ** 62, dtype=np.int64)
    assert o.sum_int(big) == np.int64(0)          # wraps modulo 2**64


def test_reference_block_geometry(golden):
    """A RESTATEMENT check, not a pin: the expected triples in the fixture were
    worked out by hand from the very formula the C function restates
    (cupy/_core/_reduction.pyx:239-253), so agreement only shows that the C
    text and the hand evaluation read the formula the same way.  What the
    formula itself guarantees is checked below for a range of sizes: the
    stride is the largest power of two not above max(contiguous capped at 32,
    256 / elements per output), it never exceeds the block, and the blocks
    cover every output exactly once."""
    for case in golden['block_specs']:
        got = c_oracle.get_block_specs(case['in_size'], case['out_size'], case['contiguous'])
        assert list(got) == case['expect']
    for out_size in (1, 2, 3, 31, 32, 33, 255, 256, 257, 4096, 16384, 1 << 20):
        for per_out in (1, 2, 7, 8, 100, 256, 257, 4096, 1 << 14):
            for contiguous in (1, 2, 5, 16, 32, 33, 1000, out_size):
                block, stride, blocks = c_oracle.get_block_specs(
                    out_size * per_out, out_size, contiguous)
                bound = max(min(contiguous, 32), 256 // per_out)
                assert block == 256
                assert stride & (stride - 1) == 0 and stride <= max(1, bound) < 2 * stride
                assert stride <= block
                assert (blocks - 1) * stride < out_size <= blocks * stride


def test_fused_pipeline_rounding():
    rng = np.random.default_rng(7)
    x = rng.standard_normal((9, 256)).astype(np.float16)
    y = rng.standard_normal((9, 256)).astype(np.float16)
    w = rng.uniform(0, 1, 256).astype(np.float32)
    got = o.fused_sqdiff_wsum(x, y, w)
    assert got.dtype == np.float32
    # NumPy evaluating the user's expression is the definition
    assert np.array_equal(got, np.sum((x - y) ** 2 * w, axis=-1))
    # identical operands: every term is exactly zero
    assert np.array_equal(o.fused_sqdiff_wsum(x, x, w), np.zeros(9, np.float32))
    # squares of float16 values are exact in float32, so x**2 == x*x bit for bit
    d = x - y
    assert np.array_equal(d ** 2, (d.astype(np.float32) * d.astype(np.float32)).astype(np.float16))
    # a pipeline without the float16 roundings gives different numbers
    unrounded = np.sum((x.astype(np.float32) - y.astype(np.float32)) ** 2 * w, axis=-1,
                       dtype=np.float32)
    assert not np.array_equal(unrounded, got)


def test_small_config_fixtures_are_what_numpy_computes(small_configs):
    c = small_configs
    assert np.array_equal(o.saxpy(2.5, c['c1_x'], c['c1_y']), c['c1_z'])
    assert np.array_equal(o.broadcast_mul_add(c['c2_base'].T, c['c2_y']), c['c2_out'])
    assert np.array_equal(o.argmax_first(c['c4_i32'], -1), c['c4_i32_argmax'])
    assert np.array_equal(o.argmin_first(c['c4_i32'], -1), c['c4_i32_argmin'])
    assert np.array_equal(o.argmax_first(c['c4_f32'], 1), c['c4_f32_argmax'])
    assert np.array_equal(o.fused_sqdiff_wsum(c['c5_x'], c['c5_y'], c['c5_w']), c['c5_out'])


def test_element_offsets_closed_form():
    shape, strides = (3, 4, 5), (400, 8, 80)
    offs = o.element_offsets(shape, strides)
    expect = [i * 400 + j * 8 + k * 80 for i in range(3) for j in range(4) for k in range(5)]
    assert offs.tolist() == expect
