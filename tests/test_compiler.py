"""Run-time compiler front end and the on-disk cache (CPU only: hiprtc
cross-compiles for gfx950 without a device)."""
import os
import pickle

import pytest

from cupy_amd.cuda import _codeobj
from cupy_amd.cuda import _compiler_cache
from cupy_amd.cuda import compiler


def test_kernel_name_rule(golden):
    for name in golden['kernel_names_valid']:
        assert compiler.is_valid_kernel_name(name)
    for name in golden['kernel_names_invalid']:
        assert not compiler.is_valid_kernel_name(name)


def test_compile_exception_is_picklable():
    e1 = compiler.CompileException('msg', 'fn.cu', 'fn', ('-ftz=true',))
    e2 = pickle.loads(pickle.dumps(e1))
    assert e1.args == e2.args
    assert str(e1) == str(e2) == 'msg'


def test_compile_for_gfx950_and_metadata():
    src = ('extern "C" __global__ void k(const float* x, float a, double* y, short n) '
           '{ y[threadIdx.x] = a * x[threadIdx.x] + n; }')
    code = compiler.compile_source(src)
    assert code[:4] == b'\x7fELF'
    meta = _codeobj.kernel_metadata(code)['k']
    assert [(o, s) for o, s, _ in meta['args']] == [(0, 8), (8, 4), (16, 8), (24, 2)]
    assert meta['explicit_size'] == 26


def test_compile_error_carries_log():
    with pytest.raises(compiler.CompileException) as info:
        compiler.compile_source('extern "C" __global__ void k() { a b; }')
    assert 'error' in str(info.value)
    assert 'k()' in info.value.source


def test_no_fp_contraction_and_no_packed_fp32():
    import subprocess
    src = ('extern "C" __global__ void k(const float2* x, const float2* y, float2* z, float a) {'
           ' int i = threadIdx.x; z[i].x = a * x[i].x + y[i].x; z[i].y = a * x[i].y + y[i].y; }')
    code = compiler.compile_source(src)
    path = os.path.join(os.environ.get('TMPDIR', '/tmp'), 'cupy_amd_test_k.co')
    with open(path, 'wb') as f:
        f.write(code)
    dis = subprocess.run(['/opt/rocm/llvm/bin/llvm-objdump', '-d', path],
                         capture_output=True, text=True).stdout
    os.unlink(path)
    assert 'v_mul_f32' in dis and 'v_add_f32' in dis
    assert 'v_fma' not in dis and 'v_pk_' not in dis and 'v_mac' not in dis


def test_cache_file_format_roundtrip(tmp_path):
    cache = _compiler_cache.DiskKernelCache(str(tmp_path))
    payload = b'\x00\x01binary payload' * 10
    cache.save('abc.hsaco', payload)
    blob = (tmp_path / 'abc.hsaco').read_bytes()
    import hashlib
    assert blob[:40] == hashlib.sha1(payload).hexdigest().encode('ascii')
    assert blob[40:] == payload
    assert cache.load('abc.hsaco') == payload
    assert not [p for p in os.listdir(tmp_path) if p.startswith('tmp_')]


def test_cache_rejects_damaged_entries(tmp_path):
    cache = _compiler_cache.DiskKernelCache(str(tmp_path))
    assert cache.load('missing.hsaco') is None
    (tmp_path / 'short.hsaco').write_bytes(b'deadbeef')
    assert cache.load('short.hsaco') is None
    cache.save('ok.hsaco', b'payload')
    blob = bytearray((tmp_path / 'ok.hsaco').read_bytes())
    blob[-1] ^= 0xFF
    (tmp_path / 'ok.hsaco').write_bytes(bytes(blob))
    assert cache.load('ok.hsaco') is None
    assert _compiler_cache.decode(b'') is None


def test_get_code_object_uses_disk_cache(tmp_path, monkeypatch):
    monkeypatch.setenv('CUPY_CACHE_DIR', str(tmp_path))
    monkeypatch.setenv('CUPY_CACHE_SAVE_CUDA_SOURCE', '1')
    src = 'extern "C" __global__ void cache_probe_kernel(int* x) { x[0] = 7; }'
    before = dict(compiler.stats)
    a = compiler.get_code_object(src)
    mid = dict(compiler.stats)
    b = compiler.get_code_object(src)
    after = dict(compiler.stats)
    assert a == b
    assert mid['compiled'] == before['compiled'] + 1
    assert after['compiled'] == mid['compiled']
    assert after['disk_hit'] == mid['disk_hit'] + 1
    names = os.listdir(tmp_path)
    assert any(n.endswith('.hsaco') for n in names)
    assert any(n.endswith('.hsaco.hip') for n in names)
    # a different option set is a different entry
    compiler.get_code_object(src, ('-DX=1',))
    assert len([n for n in os.listdir(tmp_path) if n.endswith('.hsaco')]) == 2


def test_compile_with_debug_switch(tmp_path, monkeypatch):
    """CUPY_CUDA_COMPILE_WITH_DEBUG (cupy/cuda/compiler.py:673 in the reference):
    debug information, no optimisation, and a cache entry of its own."""
    monkeypatch.setenv('CUPY_CACHE_DIR', str(tmp_path))
    src = ('extern "C" __global__ void debug_probe_kernel(float* x, float a) '
           '{ x[threadIdx.x] = x[threadIdx.x] * a + 1.0f; }')
    monkeypatch.delenv('CUPY_CUDA_COMPILE_WITH_DEBUG', raising=False)
    assert compiler._debug_options() == ()
    plain = compiler.compile_with_cache(src)
    monkeypatch.setenv('CUPY_CUDA_COMPILE_WITH_DEBUG', '1')
    assert compiler._debug_options() == ('-g', '-O0')
    debug = compiler.compile_with_cache(src)
    assert debug is not plain
    assert b'.debug_info' in debug.code and b'.debug_info' not in plain.code
    assert len([n for n in os.listdir(tmp_path) if n.endswith('.hsaco')]) == 2
    # header changes reach only the kernels that include the header
    a = compiler._cache_key('#include <cupy/carray.cuh>\n', (), 'gfx950')
    b = compiler._cache_key('#include <cupy/carray.cuh>\n#include <cupy/atomics.cuh>\n', (), 'gfx950')
    assert compiler._get_header_digest('int x;') != compiler._get_header_digest(
        '#include <cupy/carray.cuh>\n')
    assert a != b
    assert compiler._get_header_digest('#include <cupy/carray.cuh>') == \
        compiler._get_header_digest('#include "cupy/complex.cuh"\n#include <cupy/carray.cuh>')
