"""RawKernel / RawModule on the device; cases follow the reference's
tests/cupy_tests/core_tests/test_raw.py (:510-557 basic / module / compiler
flag, :896-907 constant memory, :909-952 template specialisation, :985-999 raw
pointers, :677-686 loading a code object from a file)."""
import numpy as np
import pytest

import cupy_amd as cp
from cupy_amd.cuda import compiler, memory

pytestmark = pytest.mark.gpu

SRC_TWO = r'''
extern "C"{
__global__ void test_sum(const float* x1, const float* x2, float* y, unsigned int N) {
    unsigned int tid = blockDim.x * blockIdx.x + threadIdx.x;
    if (tid < N) y[tid] = x1[tid] + x2[tid];
}
__global__ void test_multiply(const float* x1, const float* x2, float* y, unsigned int N) {
    unsigned int tid = blockDim.x * blockIdx.x + threadIdx.x;
    if (tid < N) y[tid] = x1[tid] * x2[tid];
}
}
'''

SRC_MACRO = r'''
#ifndef PRECISION
    #define PRECISION 2
#endif
#if PRECISION == 2
    #define TYPE double
#elif PRECISION == 1
    #define TYPE float
#else
    #error precision not supported
#endif
extern "C" __global__ void test_sum(const TYPE* x1, const TYPE* x2, TYPE* y, unsigned int N) {
    unsigned int tid = blockDim.x * blockIdx.x + threadIdx.x;
    if (tid < N) y[tid] = x1[tid] + x2[tid];
}
'''

SRC_CONST = r'''
extern "C"{
__constant__ float some_array[100];
__global__ void multiply_by_const(float* x, int N) {
    int id = threadIdx.x + blockIdx.x * blockDim.x;
    if (id < N) x[id] *= some_array[id];
}
}
'''

SRC_TEMPLATE = r'''
template<typename T>
__global__ void my_sqrt(T* input, int N) {
  unsigned int x = blockDim.x * blockIdx.x + threadIdx.x;
  if (x < N) { input[x] *= input[x]; }
}
__global__ void my_func(double* input, int N) {
  unsigned int x = blockDim.x * blockIdx.x + threadIdx.x;
  if (x < N) { input[x] *= input[x]; }
}
'''

SRC_CAST = r'''
extern "C" __global__ void my_func(void* input, int N) {
  double* arr = (double*)(input);
  unsigned int x = blockDim.x * blockIdx.x + threadIdx.x;
  if (x < N) { arr[x] = 3.0 * arr[x] - 8.0; }
}
'''

SRC_SHARED = r'''
extern "C" __global__ void reverse_block(const int* in, int* out, int n) {
  extern __shared__ int buf[];
  int t = threadIdx.x, base = blockIdx.x * blockDim.x;
  if (base + t < n) buf[t] = in[base + t];
  __syncthreads();
  int src = blockDim.x - 1 - t;
  if (base + t < n && base + src < n) out[base + t] = buf[src];
}
'''


def _run(kernel, dtype, n=10, seed=0):
    rng = np.random.default_rng(seed)
    h1 = rng.standard_normal((n, n)).astype(dtype)
    h2 = rng.standard_normal((n, n)).astype(dtype)
    x1, x2 = cp.asarray(h1), cp.asarray(h2)
    y = cp.zeros((n, n), dtype)
    kernel((n,), (n,), (x1, x2, y, n * n))
    return h1, h2, y.get()


def test_raw_kernel_basic_and_attributes():
    ker = cp.RawKernel(SRC_TWO, 'test_sum')
    h1, h2, y = _run(ker, np.float32)
    assert np.array_equal(y, h1 + h2)
    attrs = ker.attributes
    for name in ('binary_version', 'const_size_bytes', 'local_size_bytes',
                 'max_threads_per_block', 'num_regs', 'shared_size_bytes'):
        assert name in attrs
    assert ker.max_threads_per_block > 0
    assert ker.shared_size_bytes == 0
    assert ker.num_regs > 0


def test_raw_module_two_kernels_and_macro_option():
    mod = cp.RawModule(code=SRC_TWO)
    h1, h2, y = _run(mod.get_function('test_sum'), np.float32, seed=1)
    assert np.array_equal(y, h1 + h2)
    h1, h2, y = _run(mod.get_function('test_multiply'), np.float32, seed=2)
    assert np.array_equal(y, h1 * h2)
    h1, h2, y = _run(cp.RawModule(code=SRC_MACRO).get_function('test_sum'), np.float64, seed=3)
    assert np.array_equal(y, h1 + h2)
    single = cp.RawModule(code=SRC_MACRO, options=('-DPRECISION=1',))
    h1, h2, y = _run(single.get_function('test_sum'), np.float32, seed=4)
    assert np.array_equal(y, h1 + h2)


def test_constant_memory_through_get_global():
    mod = cp.RawModule(code=SRC_CONST)
    ker = mod.get_function('multiply_by_const')
    ptr = mod.get_global('some_array')
    const_arr = cp.ndarray((100,), np.float32, ptr)
    data = np.arange(100, dtype=np.float32)
    const_arr.set(data)
    out = cp.ones((100,), np.float32)
    ker((1,), (100,), (out, np.int32(100)))
    assert np.array_equal(out.get(), data)


def test_template_specialisation_by_name_expression():
    exprs = ['my_sqrt<int>', 'my_sqrt<float>', 'my_sqrt<double>', 'my_func']
    mod = cp.RawModule(code=SRC_TEMPLATE, name_expressions=exprs)
    rng = np.random.default_rng(5)
    for expr, dtype in zip(exprs, (np.int32, np.float32, np.float64, np.float64)):
        ker = mod.get_function(expr)
        h = (rng.uniform(-9, 9, 10)).astype(dtype)
        d = cp.asarray(h)
        ker((1,), (10,), (d, 10))
        assert np.array_equal(d.get(), h * h)


def test_memory_pointer_argument():
    ker = cp.RawModule(code=SRC_CAST).get_function('my_func')
    a = np.ones(100, np.float64)
    memptr = memory.alloc(100 * 8)
    b = cp.ndarray((100,), np.float64, memptr)
    b.set(a)
    ker((1,), (100,), (memptr, 100))
    assert np.array_equal(b.get(), 3.0 * a - 8.0)


def test_dynamic_shared_memory_and_stream():
    ker = cp.RawKernel(SRC_SHARED, 'reverse_block')
    h = np.arange(1024, dtype=np.int32)
    d = cp.asarray(h)
    out = cp.zeros((1024,), np.int32)
    s = cp.cuda.Stream()
    ker((4,), (256,), (d, out, 1024), shared_mem=256 * 4, stream=s)
    s.synchronize()
    assert np.array_equal(out.get(), h.reshape(4, 256)[:, ::-1].ravel())


def test_load_code_object_from_file(tmp_path):
    code = compiler.compile_source(SRC_TWO, base_options=compiler._RAW_BASE_OPTIONS)
    path = tmp_path / 'two.hsaco'
    path.write_bytes(code)
    mod = cp.RawModule(path=str(path))
    h1, h2, y = _run(mod.get_function('test_multiply'), np.float32, seed=6)
    assert np.array_equal(y, h1 * h2)


GRID_SYNC_SRC = r'''
#include <hip/hip_cooperative_groups.h>
extern "C" __global__
void test_grid_sync(const float* x1, const float* x2, float* y, int n) {
    namespace cg = cooperative_groups;
    cg::grid_group grid = cg::this_grid();
    int size = gridDim.x * blockDim.x;
    int tid = blockDim.x * blockIdx.x + threadIdx.x;
    for (int i = tid; i < n; i += size) y[i] = x1[i];
    cg::sync(grid);
    for (int i = n - 1 - tid; i >= 0; i -= size) y[i] += x2[i];
}

// every workgroup adds up its share; after the grid-wide barrier workgroup 0
// adds up the shares of all workgroups
extern "C" __global__
void grid_sum(const int* x, long long* shares, long long* total, int n) {
    namespace cg = cooperative_groups;
    __shared__ long long sm[256];
    long long s = 0;
    for (int i = blockIdx.x * blockDim.x + threadIdx.x; i < n; i += gridDim.x * blockDim.x) s += x[i];
    sm[threadIdx.x] = s;
    __syncthreads();
    for (int w = blockDim.x / 2; w > 0; w >>= 1) {
        if (threadIdx.x < w) sm[threadIdx.x] += sm[threadIdx.x + w];
        __syncthreads();
    }
    if (threadIdx.x == 0) shares[blockIdx.x] = sm[0];
    cg::this_grid().sync();
    if (blockIdx.x == 0 && threadIdx.x == 0) {
        long long t = 0;
        for (int b = 0; b < gridDim.x; ++b) t += shares[b];
        total[0] = t;
    }
}
'''


@pytest.mark.parametrize('n,block', [(64, 64), (257, 128), (1024, 256)])
def test_grid_sync_rawkernel_and_rawmodule(n, block):
    """A grid-wide barrier inside a cooperatively launched kernel (reference:
    tests/cupy_tests/core_tests/test_raw.py:1364-1397, skipped there on HIP)."""
    x1 = np.arange(n * n, dtype=np.float32).reshape(n, n)
    x2 = np.ones((n, n), np.float32)
    grid = min((n * n + block - 1) // block, 512)
    ker = cp.RawKernel(GRID_SYNC_SRC, 'test_grid_sync', enable_cooperative_groups=True)
    y = cp.zeros((n, n), np.float32)
    ker((grid,), (block,), (cp.asarray(x1), cp.asarray(x2), y, n * n))
    assert np.array_equal(y.get(), x1 + x2)
    mod = cp.RawModule(code=GRID_SYNC_SRC, enable_cooperative_groups=True)
    y = cp.zeros((n, n), np.float32)
    mod.get_function('test_grid_sync')((grid,), (block,), (cp.asarray(x1), cp.asarray(x2), y, n * n))
    assert np.array_equal(y.get(), x1 + x2)


def test_sum_across_workgroups_after_a_grid_wide_barrier():
    rng = np.random.default_rng(21)
    h = rng.integers(-1000, 1000, (1 << 22) + 77).astype(np.int32)
    mod = cp.RawModule(code=GRID_SYNC_SRC, enable_cooperative_groups=True)
    ker = mod.get_function('grid_sum')
    shares = cp.zeros((512,), np.int64)
    total = cp.zeros((1,), np.int64)
    ker((512,), (256,), (cp.asarray(h), shares, total, h.size))
    assert int(total.get()[0]) == int(h.sum(dtype=np.int64))
    # a grid the device cannot hold at once is refused, and nothing is left broken
    with pytest.raises(cp.cuda.runtime.HIPError if hasattr(cp.cuda.runtime, 'HIPError') else Exception,
                       match='CooperativeLaunchTooLarge'):
        ker((1 << 16,), (256,), (cp.asarray(h), cp.zeros((1 << 16,), np.int64), total, h.size))
    total.fill(0)
    ker((256,), (256,), (cp.asarray(h), shares, total, h.size))
    assert int(total.get()[0]) == int(h.sum(dtype=np.int64))


LDS_SRC = r'''
extern "C" __global__ void reverse_through_lds(const int* x, int* y, int n) {
    extern __shared__ int buf[];
    for (int i = threadIdx.x; i < n; i += blockDim.x) buf[i] = x[i];
    __syncthreads();
    for (int i = threadIdx.x; i < n; i += blockDim.x) y[i] = buf[n - 1 - i];
}
'''


def test_more_than_64_kib_of_dynamic_lds_after_the_setter():
    """(reference: cupy/_core/raw.pyx:226-255; the setter is a stub on the
    reference's HIP build)"""
    ker = cp.RawKernel(LDS_SRC, 'reverse_through_lds')
    nbytes = 96 * 1024
    ker.max_dynamic_shared_size_bytes = nbytes
    assert ker.max_dynamic_shared_size_bytes >= nbytes
    ker.preferred_shared_memory_carveout = 100      # a hint; accepted
    n = nbytes // 4
    h = np.arange(n, dtype=np.int32)
    y = cp.zeros((n,), np.int32)
    ker((1,), (1024,), (cp.asarray(h), y, n), shared_mem=nbytes)
    assert np.array_equal(y.get(), h[::-1])
    # beyond the LDS of a compute unit the launch is refused
    with pytest.raises(Exception):
        ker((1,), (1024,), (cp.asarray(h), y, n), shared_mem=1 << 20)
        cp.cuda.Device().synchronize()
