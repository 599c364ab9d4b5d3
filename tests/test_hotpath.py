"""The extension module behind the per-launch host calls
(``cupy_amd/csrc/hotpath.c``): what it computes must be what the Python code it
replaced computed.  No test here launches anything: ``splice`` returns the
argument blocks ``replay`` would launch, and ``launch`` is only called with a
null function, which the library refuses before it reaches the GPU."""
import struct

import numpy as np
import pytest

import cupy_amd as cp
from cupy_amd import _dryrun, _rt
from cupy_amd._core import _launch_plan, _tuning

hot = _rt.hot


def test_module_exports():
    for name in ('launch', 'replay', 'splice', 'pool_malloc', 'pool_free', 'signature',
                 'setup', 'get_device'):
        assert callable(getattr(hot, name)), name


def python_signature(args, dev_id, version):
    """The rule the extension implements, written out."""
    sig = [dev_id, version]
    for a in args:
        t = type(a)
        if t is cp.ndarray:
            if a.data.device_id != dev_id:
                return None
            sig.append((a.dtype, a._shape, a._strides, a.data.ptr & 15))
        elif t in (float, bool, complex):
            sig.append(t)
        elif t is int:
            if not -2 ** 63 <= a < 2 ** 63:
                return None
            sig.append(t)
        elif isinstance(a, np.generic):
            sig.append(t)
        else:
            return None
    return tuple(sig)


needs_arrays = pytest.mark.skipif(not _dryrun.enabled(), reason='creates arrays without a GPU')


@needs_arrays
def test_signature_matches_the_rule():
    x = cp.zeros((3, 4), np.float32)
    y = cp.zeros((12,), np.float64)[1:7:2]
    cases = [
        (x,), (x, y), (x, 1.5, y), (x, True), (x, 2 + 1j), (x, 7), (x, -2 ** 63), (x, 2 ** 63 - 1),
        (x, 2 ** 63), (x, -2 ** 63 - 1), (x, 2 ** 70), (x, np.float32(1)), (x, np.int8(3)),
        (x, np.bool_(True)), (x, None), (x, 'text'), (x, [1, 2]), (x, np.zeros(3)), (),
        (x.T, x[1:], x[:, ::2]),
    ]
    for args in cases:
        want = python_signature(args, 0, 5)
        assert hot.signature(args, 0, 5) == want, args
        assert hot.signature(list(args), 0, 5) == want, args
    # an array of another device takes the full path
    assert hot.signature((x,), 1, 5) is None
    assert _launch_plan.call_signature((x, 2.0), 0) == python_signature(
        (x, 2.0), 0, _tuning.version())


@needs_arrays
def test_signature_tells_layouts_and_alignment_apart():
    base = cp.zeros((64,), np.float32)
    a, b = base[:16], base[1:17]                # same shape, other alignment
    assert hot.signature((a,), 0, 0) != hot.signature((b,), 0, 0)
    assert hot.signature((a,), 0, 0) == hot.signature((base[4:20],), 0, 0)
    assert hot.signature((a,), 0, 0) != hot.signature((a,), 0, 1)       # tuning changed
    assert hot.signature((a, 1), 0, 0) != hot.signature((a, 1.0), 0, 0)


def test_signature_rejects_wrong_calls():
    with pytest.raises(TypeError):
        hot.signature(5, 0, 0)
    with pytest.raises(TypeError):
        hot.signature((), 0)


class _Mem:
    def __init__(self, ptr):
        self.ptr = ptr


class _Arr:
    def __init__(self, ptr):
        self.data = _Mem(ptr)


def record_of(launches):
    """A launch record as ``_launch_plan._quick_launches`` lays it out."""
    out = [struct.pack('<II', len(launches), 0)]
    for function, grid, block, shmem, slots, blob in launches:
        out.append(struct.pack('<Q3I3IIIQ', function, *grid, *block, shmem, len(slots), len(blob)))
        out.append(b''.join(struct.pack('<II', off, ref) for off, ref in slots))
        out.append(blob + b'\0' * (-len(blob) % 8))
    return b''.join(out)


def test_splice_patches_addresses_of_arrays_and_temporaries():
    blob1 = bytes(range(40))
    blob2 = bytes(range(100, 124))
    big = bytes(i % 251 for i in range(6000))            # beyond the block kept on the stack
    rec = record_of([
        (0x1111, (7, 2, 1), (256, 1, 1), 0, [(8, 0), (24, 2)], blob1),
        (0x2222, (1, 1, 3), (64, 4, 1), 128, [(0, 2), (16, 1)], blob2),
        (0x3333, (5, 1, 1), (1024, 1, 1), 0, [(5992, 1)], big),
    ])
    refs = [_Arr(0xAAAA0000), _Arr(0xBBBB0010), _Mem(0xCCCC0200)]
    got = hot.splice(rec, refs, 2)

    def patched(blob, pairs):
        b = bytearray(blob)
        for off, value in pairs:
            b[off:off + 8] = struct.pack('<Q', value)
        return bytes(b)
    assert got == [
        (0x1111, (7, 2, 1), (256, 1, 1), 0, patched(blob1, [(8, 0xAAAA0000), (24, 0xCCCC0200)])),
        (0x2222, (1, 1, 3), (64, 4, 1), 128, patched(blob2, [(0, 0xCCCC0200), (16, 0xBBBB0010)])),
        (0x3333, (5, 1, 1), (1024, 1, 1), 0, patched(big, [(5992, 0xBBBB0010)])),
    ]
    # the record itself is never written to
    assert rec == record_of([
        (0x1111, (7, 2, 1), (256, 1, 1), 0, [(8, 0), (24, 2)], blob1),
        (0x2222, (1, 1, 3), (64, 4, 1), 128, [(0, 2), (16, 1)], blob2),
        (0x3333, (5, 1, 1), (1024, 1, 1), 0, [(5992, 1)], big),
    ])


@pytest.mark.parametrize('case', ['short', 'cut header', 'cut block', 'slot outside block',
                                  'ref outside refs', 'huge slot count'])
def test_malformed_records_are_refused(case):
    good = record_of([(1, (1, 1, 1), (1, 1, 1), 0, [(0, 0)], bytes(16))])
    refs = [_Arr(8)]
    if case == 'short':
        rec = good[:4]
    elif case == 'cut header':
        rec = good[:20]
    elif case == 'cut block':
        rec = good[:-8]
    elif case == 'slot outside block':
        rec = record_of([(1, (1, 1, 1), (1, 1, 1), 0, [(12, 0)], bytes(16))])
    elif case == 'ref outside refs':
        rec = record_of([(1, (1, 1, 1), (1, 1, 1), 0, [(0, 1)], bytes(16))])
    else:
        rec = bytearray(good)
        rec[8 + 36:8 + 40] = struct.pack('<I', 0xffffffff)       # n_slots
        rec = bytes(rec)
    with pytest.raises(ValueError):
        hot.splice(rec, refs, 1)
    with pytest.raises(ValueError):
        hot.replay(rec, refs, 1, 0)


def test_reference_without_an_address_raises():
    rec = record_of([(1, (1, 1, 1), (1, 1, 1), 0, [(0, 0)], bytes(16))])
    with pytest.raises(AttributeError):
        hot.splice(rec, [object()], 1)
    with pytest.raises(TypeError):
        hot.splice(rec, [_Arr('x')], 1)


def test_null_function_is_refused_before_any_launch():
    assert hot.launch(0, 1, 1, 1, 1, 1, 1, 0, 0, bytes(8)) == _rt.RT_ERR_INVALID
    rec = record_of([(0, (1, 1, 1), (1, 1, 1), 0, [(0, 0)], bytes(16))])
    assert hot.replay(rec, [_Arr(8)], 1, 0) == _rt.RT_ERR_INVALID
    with pytest.raises(OverflowError):
        hot.launch(1, 2 ** 32, 1, 1, 1, 1, 1, 0, 0, bytes(8))
    with pytest.raises(TypeError):
        hot.launch(1, 1, 1, 1, 1, 1, 1, 0, 0, 'not bytes')


@needs_arrays
def test_replayed_calls_go_through_the_extension():
    """In compile-check mode a replayed call is recorded from what ``splice``
    returns: it must equal what the full path recorded for the same call."""
    k = cp.ElementwiseKernel('T x', 'T y', 'y = x * 2', 'hotpath_double')
    x = cp.zeros((1000,), np.float32)
    y = cp.zeros((1000,), np.float32)
    n0 = len(_dryrun.launches)
    k(x, y)
    first = _dryrun.launches[n0:]
    fast = list(k._fast_calls.values())
    assert len(fast) == 1 and fast[0].quick is not None
    n1 = len(_dryrun.launches)
    k(x, y)
    assert _dryrun.launches[n1:] == first


@needs_arrays
def test_pool_calls_of_the_extension():
    pool = cp.cuda.MemoryPool()
    p = pool.malloc(1000)
    assert p.ptr != 0 and pool.used_bytes() == 1024
    address = p.ptr
    del p
    assert pool.used_bytes() == 0 and pool.free_bytes() == 1024
    q = pool.malloc(700)                  # the cached block comes back
    assert q.ptr == address
    # a failure comes back as minus the status
    assert hot.pool_malloc(0, 512, 0) == -_rt.RT_ERR_INVALID
