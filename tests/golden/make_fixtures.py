"""Writes tests/golden/configs_small.npz: seeded inputs of the five benchmark
configurations at reduced shapes, and what NumPy computes from them.

Run from the repository root: ``python tests/golden/make_fixtures.py``.
Nothing from the reference is imported; NumPy is the parity target of this
path.  Seeds and distributions are the ones the benchmark uses at full size.
"""
import os

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))


def main():
    out = {}
    # C1: saxpy
    rng = np.random.default_rng(1)
    n = 4099
    x = rng.uniform(-1, 1, n).astype(np.float32)
    y = rng.uniform(-1, 1, n).astype(np.float32)
    out['c1_x'], out['c1_y'] = x, y
    out['c1_z'] = np.float32(2.5) * x + y
    # C2: transposed f32 * broadcast f16 + 1
    rng = np.random.default_rng(2)
    base = rng.standard_normal((96, 80), dtype=np.float32)
    yy = rng.uniform(0, 2, (1, 96)).astype(np.float16)
    out['c2_base'], out['c2_y'] = base, yy
    out['c2_out'] = base.T * yy + 1
    # C3: sums
    rng = np.random.default_rng(3)
    a32 = rng.standard_normal((130, 257), dtype=np.float32)
    out['c3_f32'] = a32
    out['c3_f32_ax0'] = a32.sum(axis=0)
    out['c3_f32_ax1'] = a32.sum(axis=1)
    out['c3_f32_all'] = np.asarray(a32.sum())
    rng = np.random.default_rng(4)
    a64 = rng.standard_normal((65, 129))
    out['c3_f64'] = a64
    out['c3_f64_ax0'] = a64.sum(axis=0)
    out['c3_f64_ax1'] = a64.sum(axis=1)
    out['c3_f64_all'] = np.asarray(a64.sum())
    # C4: argmax / argmin with heavy ties
    rng = np.random.default_rng(5)
    m = rng.integers(0, 16, (300, 128), dtype=np.int32)
    out['c4_i32'] = m
    out['c4_i32_argmax'] = m.argmax(axis=-1)
    out['c4_i32_argmin'] = m.argmin(axis=-1)
    rng = np.random.default_rng(6)
    f = rng.standard_normal((33, 4096), dtype=np.float32)
    out['c4_f32'] = f
    out['c4_f32_argmax'] = f.argmax(axis=1)
    # C5: fused map-reduce
    rng = np.random.default_rng(7)
    fx = rng.standard_normal((70, 256)).astype(np.float16)
    fy = rng.standard_normal((70, 256)).astype(np.float16)
    fw = rng.uniform(0, 1, 256).astype(np.float32)
    out['c5_x'], out['c5_y'], out['c5_w'] = fx, fy, fw
    out['c5_out'] = np.sum((fx - fy) ** 2 * fw, axis=-1)
    # int8 sums with wrap-around widths (pattern of the reference's
    # tests/cupy_tests/core_tests/test_reduction.py:59-88)
    rng = np.random.default_rng(8)
    i8 = rng.integers(-128, 128, (513, 65), dtype=np.int8)
    out['i8'] = i8
    out['i8_ax0'] = i8.sum(axis=0)
    out['i8_ax1'] = i8.sum(axis=1)
    np.savez_compressed(os.path.join(HERE, 'configs_small.npz'), **out)
    print('wrote', len(out), 'arrays')


if __name__ == '__main__':
    main()
