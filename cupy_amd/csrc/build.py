"""Builds ``_lib/libmi355rt.so`` (the C-ABI runtime shim) with hipcc and
``_lib/_hotpath.so`` (CPython extension: the per-launch calls into that
library without ctypes' argument conversion) with gcc.

Usage: ``python cupy_amd/csrc/build.py`` (run as a script, so that nothing of
the package is imported: importing the package needs what this builds).
"""
import os
import subprocess
import sys
import sysconfig

HERE = os.path.dirname(os.path.abspath(__file__))
PKG = os.path.dirname(HERE)
ROOT = os.path.dirname(PKG)
SOURCES = ['mi355rt.cpp', 'pool.cpp']
OUTPUT = os.path.join(PKG, '_lib', 'libmi355rt.so')
HOTPATH_OUTPUT = os.path.join(PKG, '_lib', '_hotpath.so')


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
    build_hotpath(verbose)
    return OUTPUT


def build_hotpath(verbose=False):
    """The extension module links against the shim beside it (found through
    ``$ORIGIN``) and is built for the interpreter that runs this script."""
    cc = os.environ.get('CC', 'gcc')
    cmd = [cc, '-shared', '-fPIC', '-O2', '-std=c11', '-Wall', '-Wextra',
           '-I' + os.path.join(ROOT, 'include'), '-I' + sysconfig.get_paths()['include'],
           os.path.join(HERE, 'hotpath.c'), '-o', HOTPATH_OUTPUT + '.tmp',
           '-L' + os.path.dirname(OUTPUT), '-lmi355rt', '-Wl,-rpath,$ORIGIN']
    if verbose:
        print(' '.join(cmd))
    subprocess.check_call(cmd)
    os.replace(HOTPATH_OUTPUT + '.tmp', HOTPATH_OUTPUT)
    return HOTPATH_OUTPUT


if __name__ == '__main__':
    print(build_shim(verbose=True))
    sys.exit(0)
