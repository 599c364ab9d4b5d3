"""Host side of the by-value kernel arguments ``CArray`` and ``CIndexer``
(reference: cupy/_core/_carray.pyx:90-184).  The byte layouts match the
classes in ``include/cupy/carray.cuh``:

* CArray<T, nd>:  data pointer, size, shape[nd], strides[nd]  (8 bytes each)
* CIndexer<nd>:   size, shape[nd], index[nd]                   (index = scratch)
"""
import ctypes

from cupy_amd._core import internal

MAX_NDIM = 64


class Indexer:
    """Shape of an index space handed to a kernel as ``CIndexer``."""
    __slots__ = ('shape', 'size', '_index_32_bits')

    def __init__(self, shape):
        self.shape = tuple(shape)
        self.size = internal.prod(self.shape)
        self._index_32_bits = self.size <= (1 << 31)

    @property
    def ndim(self):
        return len(self.shape)

    def _kernel_arg_bytes(self):
        nd = len(self.shape)
        return (ctypes.c_int64 * (1 + 2 * nd))(self.size, *self.shape)


def _indexer_init(shape):
    return Indexer(shape)


_byte_extent = None      # core._byte_extent, bound at the first call (core imports this module)


def may_share_bounds(a, b):
    """True if the byte ranges spanned by two arrays of one allocation
    intersect (reference: cupy/_core/_memory_range.pyx:46-59)."""
    global _byte_extent
    if _byte_extent is None:
        from cupy_amd._core.core import _byte_extent
    if (a.data.device_id != b.data.device_id
            or a.data.mem.ptr != b.data.mem.ptr
            or a.size == 0 or b.size == 0):
        return False
    alo, ahi = _byte_extent(a._shape, a._strides, a.dtype.itemsize)
    blo, bhi = _byte_extent(b._shape, b._strides, b.dtype.itemsize)
    alo += a.data.ptr
    ahi += a.data.ptr
    blo += b.data.ptr
    bhi += b.data.ptr
    return alo < bhi and blo < ahi
