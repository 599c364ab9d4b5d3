/*
 * TEST INFRASTRUCTURE ONLY -- never linked into or called by the product.
 *
 * Plain-C restatement of what the REFERENCE's generated kernels compute for
 * the operations of the benchmark configurations, in the reference's own
 * evaluation order, so that tests can compare three things: NumPy, this
 * restatement and the GPU result.
 *
 *  - ref_block_reduce_*: the generic reduction kernel of
 *    cupy/_core/_reduction.pyx:59-112.  A block of `block_size` threads owns
 *    `block_stride` adjacent outputs; thread tid accumulates the elements
 *    J = tid / block_stride, + block_size / block_stride, ... of output
 *    i = base + tid % block_stride serially (lines 86-93), then an LDS tree
 *    halves the active threads down to block_stride (lines 96-102).
 *    Geometry: cupy/_core/_reduction.pyx:239-253 (_get_block_specs) with
 *    block_size 256 on HIP (:232-236).
 *  - ref_argmax combine: cupy/_core/_routines_statistics.pyx:234-274
 *    (my_argmax / my_argmax_float: equal values -> smaller index, NaN wins).
 *  - ref_saxpy_f32: the elementwise template cupy/_core/_kernel.pyx:86-97 with
 *    the body `z = a * x + y`, evaluated without contraction.
 *
 * Pinning: integer results are exact by construction and compared bit for bit
 * with NumPy; floating-point sums are a permutation of the same addends and
 * are compared with math.fsum within rtol.  The summation order itself cannot
 * be validated against the reference here (it needs a GPU build of the
 * reference): parity unpinned for the order.
 *
 * Who uses this file: tests/test_oracle.py only (through oracle/c_oracle.py).
 * No GPU test, no benchmark and no product code consumes it: GPU results are
 * compared with NumPy (oracle/numpy_oracle.py), whose values this restatement
 * is itself compared with.  ref_get_block_specs exists for the summation
 * order of ref_block_reduce_*; its table of expected triples in
 * tests/golden/reference_kats.json was evaluated by hand from the same
 * formula, which pins nothing beyond a consistent reading of that formula.
 */
#include <math.h>
#include <stddef.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

static size_t clp2(size_t x) {
  size_t p = 1;
  if (x == 0) return 0;
  while (p < x) p <<= 1;
  return p;
}

/* _get_block_specs, cupy/_core/_reduction.pyx:239-253 */
void ref_get_block_specs(int64_t in_size, int64_t out_size, int64_t contiguous_size,
                         int64_t* block_size, int64_t* block_stride,
                         int64_t* out_block_num) {
  int64_t bs = 256;
  int64_t reduce_block_size = in_size / out_size;
  if (reduce_block_size < 1) reduce_block_size = 1;
  if (contiguous_size > 32) contiguous_size = 32;
  int64_t stride = bs / reduce_block_size;
  if (contiguous_size > stride) stride = contiguous_size;
  stride = (int64_t)clp2((size_t)(stride / 2 + 1));
  *block_size = bs;
  *block_stride = stride;
  *out_block_num = (out_size + stride - 1) / stride;
}

/*
 * Canonical problem: out[i] = reduce_j in[i * so + j * sr] (strides in
 * elements), i < n_out, j < n_red, evaluated in the reference kernel's order.
 */
#define DEFINE_BLOCK_REDUCE_SUM(NAME, IN_T, ACC_T, OUT_T)                         \
  void NAME(const IN_T* in, OUT_T* out, int64_t n_out, int64_t n_red, int64_t so, \
            int64_t sr, int64_t block_size, int64_t block_stride) {              \
    ACC_T* sdata = (ACC_T*)malloc(sizeof(ACC_T) * (size_t)block_size);           \
    int64_t j_stride = block_size / block_stride;                                 \
    for (int64_t base = 0; base < n_out; base += block_stride) {                  \
      for (int64_t tid = 0; tid < block_size; ++tid) {                            \
        int64_t i = base + (tid % block_stride);                                  \
        ACC_T s = 0;                                                              \
        if (i < n_out)                                                            \
          for (int64_t j = tid / block_stride; j < n_red; j += j_stride)          \
            s = s + (ACC_T)in[i * so + j * sr];                                   \
        sdata[tid] = s;                                                           \
      }                                                                           \
      for (int64_t blk = block_size / 2; blk >= block_stride; blk >>= 1)          \
        for (int64_t tid = 0; tid < blk; ++tid)                                   \
          sdata[tid] = sdata[tid] + sdata[tid + blk];                             \
      for (int64_t tid = 0; tid < block_stride; ++tid)                            \
        if (base + tid < n_out) out[base + tid] = (OUT_T)sdata[tid];              \
    }                                                                             \
    free(sdata);                                                                  \
  }

DEFINE_BLOCK_REDUCE_SUM(ref_block_reduce_sum_f32, float, float, float)
DEFINE_BLOCK_REDUCE_SUM(ref_block_reduce_sum_f64, double, double, double)
DEFINE_BLOCK_REDUCE_SUM(ref_block_reduce_sum_i32_i64, int32_t, int64_t, int64_t)
DEFINE_BLOCK_REDUCE_SUM(ref_block_reduce_sum_i8_i64, int8_t, int64_t, int64_t)

typedef struct {
  double value;
  int64_t index;
} mm_t;

/* my_argmax_float / my_argmin_float, _routines_statistics.pyx:234-274 */
static mm_t mm_pick(mm_t a, mm_t b, int want_max) {
  if (a.index == -1) return b;
  if (b.index == -1) return a;
  if (a.value == b.value) {
    mm_t r = a;
    r.index = a.index < b.index ? a.index : b.index;
    return r;
  }
  if (isnan(a.value)) return a;
  if (isnan(b.value)) return b;
  if (want_max) return (a.value >= b.value) ? a : b;
  return (a.value <= b.value) ? a : b;
}

/* argmax/argmin of rows of a C-contiguous (n_out, n_red) matrix of doubles,
 * combined in the reference kernel's order (block_stride as chosen by
 * ref_get_block_specs for contiguous_size 1). */
void ref_block_reduce_arg_f64(const double* in, int64_t* out, int64_t n_out, int64_t n_red,
                              int want_max) {
  int64_t block_size, block_stride, nblk;
  ref_get_block_specs(n_out * n_red, n_out, 1, &block_size, &block_stride, &nblk);
  mm_t* sdata = (mm_t*)malloc(sizeof(mm_t) * (size_t)block_size);
  int64_t j_stride = block_size / block_stride;
  for (int64_t base = 0; base < n_out; base += block_stride) {
    for (int64_t tid = 0; tid < block_size; ++tid) {
      int64_t i = base + (tid % block_stride);
      mm_t s;
      s.value = 0;
      s.index = -1;
      if (i < n_out)
        for (int64_t j = tid / block_stride; j < n_red; j += j_stride) {
          mm_t a;
          a.value = in[i * n_red + j];
          a.index = j;
          s = mm_pick(s, a, want_max);
        }
      sdata[tid] = s;
    }
    for (int64_t blk = block_size / 2; blk >= block_stride; blk >>= 1)
      for (int64_t tid = 0; tid < blk; ++tid)
        sdata[tid] = mm_pick(sdata[tid], sdata[tid + blk], want_max);
    for (int64_t tid = 0; tid < block_stride; ++tid)
      if (base + tid < n_out) out[base + tid] = sdata[tid].index;
  }
  free(sdata);
}

/* z = a * x + y, float32, two roundings (build with -ffp-contract=off) */
void ref_saxpy_f32(float a, const float* x, const float* y, float* z, int64_t n) {
  for (int64_t i = 0; i < n; ++i) {
    volatile float p = a * x[i];
    z[i] = p + y[i];
  }
}
