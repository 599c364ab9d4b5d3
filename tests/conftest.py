"""Test configuration.

``-m gpu`` tests need an MI355X; everything else runs on a machine without a
GPU.  There the package is switched to its compile-check mode (see
``cupy_amd/_dryrun.py``) before it is imported, so host logic, code generation
and the gfx950 compile of every kernel are still exercised.
"""
import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HAS_GPU = os.path.exists('/dev/kfd') and os.access('/dev/kfd', os.R_OK | os.W_OK)
if not HAS_GPU:
    os.environ.setdefault('CUPY_AMD_DRYRUN', '1')
# keep the kernel cache of a test run inside the tree: it travels with the
# sources, so kernels compiled on the CPU box are not compiled again on the GPU box
os.environ.setdefault('CUPY_CACHE_DIR', os.path.join(ROOT, 'cupy_amd', '_kernel_cache'))


def pytest_configure(config):
    config.addinivalue_line('markers', 'gpu: needs a real MI355X (run with -m gpu)')


def pytest_collection_modifyitems(config, items):
    if HAS_GPU:
        return
    skip = pytest.mark.skip(reason='no GPU on this machine')
    for item in items:
        if 'gpu' in item.keywords:
            item.add_marker(skip)


@pytest.fixture(scope='session')
def golden():
    import json
    with open(os.path.join(ROOT, 'tests', 'golden', 'reference_kats.json')) as f:
        return json.load(f)


@pytest.fixture(scope='session')
def small_configs():
    import numpy
    return numpy.load(os.path.join(ROOT, 'tests', 'golden', 'configs_small.npz'))
