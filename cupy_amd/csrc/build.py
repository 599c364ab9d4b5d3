"""Builds ``_lib/libmi355rt.so`` (the C-ABI runtime shim) with hipcc.

Usage: ``python -m cupy_amd.csrc.build``.  Nothing is imported from the package
itself, so this also works before the library exists.
"""
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
PKG = os.path.dirname(HERE)
ROOT = os.path.dirname(PKG)
SOURCES = ['mi355rt.cpp', 'pool.cpp']
OUTPUT = os.path.join(PKG, '_lib', 'libmi355rt.so')


def build_shim(verbose=False):
    os.makedirs(os.path.dirname(OUTPUT), exist_ok=True)
    hipcc = os.environ.get('HIPCC', '/opt/rocm/bin/hipcc')
    cmd = [hipcc, '--offload-arch=gfx950', '-shared', '-fPIC', '-O2', '-std=c++17',
           '-Xclang', '-target-feature', '-Xclang', '-packed-fp32-ops',
           '-Wno-unused-command-line-argument',
           '-I' + os.path.join(ROOT, 'include')]
    cmd += [os.path.join(HERE, s) for s in SOURCES]
    cmd += ['-o', OUTPUT + '.tmp', '-lhiprtc']
    if verbose:
        print(' '.join(cmd))
    subprocess.check_call(cmd)
    os.replace(OUTPUT + '.tmp', OUTPUT)
    return OUTPUT


if __name__ == '__main__':
    print(build_shim(verbose=True))
    sys.exit(0)
