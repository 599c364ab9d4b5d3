"""The device-side bfloat16 type (include/cupy/bfloat16.cuh) against a bit-level
NumPy model: conversion from float32 rounds to nearest even, arithmetic is
float arithmetic rounded once.  NumPy has no bfloat16 here (no ml_dtypes), so
arrays hold the 16-bit patterns."""
import numpy as np
import pytest

import cupy_amd as cp

pytestmark = pytest.mark.gpu


def to_bf16_bits(x):
    u = np.asarray(x, np.float32).view(np.uint32).astype(np.uint64)
    nan = (u & 0x7fffffff) > 0x7f800000
    rounded = (u + 0x7fff + ((u >> 16) & 1)) >> 16
    return np.where(nan, (u >> 16) | 0x40, rounded).astype(np.uint16)


def from_bf16_bits(b):
    return (np.asarray(b, np.uint16).astype(np.uint32) << 16).view(np.float32)


SRC = r'''
#include <cupy/carray.cuh>
#include <cupy/bfloat16.cuh>
extern "C" __global__ void convert(const float* x, unsigned short* y, int n) {
  int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) y[i] = bfloat16(x[i]).to_bits();
}
extern "C" __global__ void arith(const unsigned short* a, const unsigned short* b,
                                 unsigned short* out, int n) {
  int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= n) return;
  bfloat16 x = bfloat16::from_bits(a[i]), y = bfloat16::from_bits(b[i]);
  out[i] = (x + y).to_bits();
  out[n + i] = (x * y).to_bits();
  out[2 * n + i] = (x - y).to_bits();
  out[3 * n + i] = max(x, y).to_bits();
  out[4 * n + i] = fmin(x, y).to_bits();
  out[5 * n + i] = (unsigned short)((x < y) | (isnan(x) << 1) | (isinf(y) << 2) | (signbit(x) << 3));
  out[6 * n + i] = nextafter(x, y).to_bits();
}
'''


def test_conversion_rounds_to_nearest_even():
    rng = np.random.default_rng(7)
    x = np.concatenate([
        rng.standard_normal(100000).astype(np.float32) * 1e3,
        rng.integers(0, 2 ** 32, 100000, dtype=np.uint64).astype(np.uint32).view(np.float32),
        np.array([0.0, -0.0, np.inf, -np.inf, np.nan, 1.0, 1.00390625, 1.01171875, 3.3895314e38,
                  1e-40, -1e-45], np.float32)])
    mod = cp.RawModule(code=SRC)
    dx = cp.asarray(x)
    dy = cp.empty(x.size, np.uint16)
    mod.get_function('convert')(((x.size + 255) // 256,), (256,), (dx, dy, np.int32(x.size)))
    got, want = dy.get(), to_bf16_bits(x)
    nan = np.isnan(x)
    assert np.array_equal(got[~nan], want[~nan])
    assert np.all(np.isnan(from_bf16_bits(got[nan])))


def test_arithmetic_is_float_arithmetic_rounded_once():
    rng = np.random.default_rng(8)
    n = 50000
    a = to_bf16_bits(rng.standard_normal(n).astype(np.float32) * 8)
    b = to_bf16_bits(rng.standard_normal(n).astype(np.float32) * 8)
    a[:4] = to_bf16_bits(np.array([np.nan, 1.0, np.inf, -0.0], np.float32))
    b[:4] = to_bf16_bits(np.array([1.0, np.nan, np.inf, 0.0], np.float32))
    mod = cp.RawModule(code=SRC)
    out = cp.zeros(7 * n, np.uint16)
    mod.get_function('arith')(((n + 255) // 256,), (256,),
                              (cp.asarray(a), cp.asarray(b), out, np.int32(n)))
    got = out.get().reshape(7, n)
    fa, fb = from_bf16_bits(a), from_bf16_bits(b)
    ok = ~(np.isnan(fa) | np.isnan(fb))
    with np.errstate(all='ignore'):
        for row, want in ((0, fa + fb), (1, fa * fb), (2, fa - fb)):
            w = to_bf16_bits(want)
            num = ok & ~np.isnan(want)
            assert np.array_equal(got[row][num], w[num]), row
            assert np.all(np.isnan(from_bf16_bits(got[row][~num])))
        assert np.array_equal(got[3][ok], to_bf16_bits(np.maximum(fa, fb))[ok])
        assert np.all(np.isnan(from_bf16_bits(got[3][~ok])))          # max propagates NaN
        fm = np.fmin(fa, fb)
        assert np.array_equal(got[4][~np.isnan(fm)], to_bf16_bits(fm)[~np.isnan(fm)])
    flags = (fa < fb).astype(np.uint16) | (np.isnan(fa).astype(np.uint16) << 1) \
        | (np.isinf(fb).astype(np.uint16) << 2) | (np.signbit(fa).astype(np.uint16) << 3)
    assert np.array_equal(got[5], flags)
    nxt = from_bf16_bits(got[6])
    step = ok & (fa != fb)
    up = fa < fb
    assert np.all(nxt[step & up] > fa[step & up]) and np.all(nxt[step & ~up] < fa[step & ~up])
    # one step: no other bfloat16 lies between x and its neighbour
    between = to_bf16_bits((fa.astype(np.float64) + nxt.astype(np.float64)) / 2)
    assert np.all((between[step] == a[step]) | (between[step] == got[6][step]))
    assert np.array_equal(got[6][ok & (fa == fb)], b[ok & (fa == fb)])
