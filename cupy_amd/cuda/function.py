"""Loaded code objects and kernel launch.

Counterpart of the reference's cupy/cuda/function.pyx (``Module`` :174-208,
``Function`` :134-171, ``_launch`` :92-131, argument conversion :53-82).
"""
import ctypes
import struct

import numpy

from cupy_amd import _dryrun
from cupy_amd import _rt
from cupy_amd.cuda import _codeobj
from cupy_amd.cuda import stream as _stream

# hipFunction_attribute values
_FUNC_ATTRIBUTES = {
    'max_threads_per_block': 0,
    'shared_size_bytes': 1,
    'const_size_bytes': 2,
    'local_size_bytes': 3,
    'num_regs': 4,
    'ptx_version': 5,
    'binary_version': 6,
    'cache_mode_ca': 7,
    'max_dynamic_shared_size_bytes': 8,
    'preferred_shared_memory_carveout': 9,
}


# cupy_amd.profiler.KernelTimer while one is active, else None
_kernel_timer = None


def _arg_to_bytes(arg):
    """Bytes of one kernel argument passed by value."""
    if hasattr(arg, '_kernel_arg_bytes'):      # ndarray, Indexer, CScalar
        return arg._kernel_arg_bytes()
    if isinstance(arg, bool):
        return struct.pack('?', arg)
    if isinstance(arg, int):
        return struct.pack('q', arg) if arg < (1 << 63) else struct.pack('Q', arg)
    if isinstance(arg, float):
        return struct.pack('d', arg)
    if isinstance(arg, complex):
        return struct.pack('dd', arg.real, arg.imag)
    if isinstance(arg, numpy.generic):
        return arg.tobytes()
    if isinstance(arg, numpy.ndarray):
        if arg.size != 1:
            raise TypeError(
                'You are trying to pass a numpy.ndarray of shape %s as a kernel '
                'parameter. Only numpy.ndarrays of size one can be passed by '
                'value. If you meant to pass a pointer to __global__ memory, '
                'you need to pass a cupy.ndarray instead.' % (arg.shape,))
        return arg.tobytes()
    if hasattr(arg, 'ptr'):                    # MemoryPointer and friends
        return struct.pack('Q', int(arg.ptr))
    raise TypeError('Unsupported type %s' % type(arg))


class Module:
    """A code object loaded on the current device."""

    def __init__(self):
        self.ptr = 0
        self.code = None
        self._metadata = None
        self.mapping = None       # name expression -> lowered symbol

    @property
    def metadata(self):
        """Per-kernel metadata of the code object (argument layout, register
        and LDS use)."""
        if self._metadata is None:
            self._metadata = _codeobj.kernel_metadata(self.code)
        return self._metadata

    def __del__(self):
        ptr, self.ptr = getattr(self, 'ptr', 0), 0
        if ptr:
            try:
                _rt.lib.rt_module_unload(ptr)
            except Exception:
                pass

    def load(self, code):
        self.code = bytes(code)
        if _dryrun.enabled():
            return
        p = ctypes.c_void_p()
        _rt.check(_rt.lib.rt_module_load(self.code, ctypes.byref(p)))
        self.ptr = p.value or 0

    def load_file(self, filename):
        """Loads a code object (.hsaco / .co) from a file."""
        with open(filename, 'rb') as f:
            self.load(f.read())

    def get_function(self, name):
        return Function(self, name)

    def get_global_var(self, name):
        """(device address, size in bytes) of a ``__device__`` variable."""
        if _dryrun.enabled():
            return 0, 0
        p = ctypes.c_void_p()
        n = ctypes.c_size_t(0)
        _rt.check(_rt.lib.rt_module_get_global(
            self.ptr, name.encode(), ctypes.byref(p), ctypes.byref(n)))
        return p.value or 0, n.value


class Function:
    """A ``__global__`` function of a module (keeps the module alive)."""

    def __init__(self, module, name):
        self.module = module
        self.name = name
        self.ptr = 0
        meta = module.metadata.get(name)
        if meta is None:
            raise _rt.HIPError(500, 'no kernel named %r in the module' % name)
        self.meta = meta
        # size of the explicit arguments, rounded as the packer may leave the
        # tail padding of the last argument off
        self._arg_size = meta['explicit_size']
        self._arg_min = (meta['args'][-1][0] + 1) if meta['args'] else 0
        if _dryrun.enabled():
            return
        p = ctypes.c_void_p()
        _rt.check(_rt.lib.rt_module_get_function(
            module.ptr, name.encode(), ctypes.byref(p)))
        self.ptr = p.value or 0

    def get_attribute(self, name):
        if _dryrun.enabled():
            return 0
        v = ctypes.c_int(0)
        _rt.check(_rt.lib.rt_func_get_attribute(
            _FUNC_ATTRIBUTES[name], self.ptr, ctypes.byref(v)))
        return v.value

    def set_attribute(self, name, value):
        """Sets 'max_dynamic_shared_size_bytes' or
        'preferred_shared_memory_carveout' (reference:
        cupy_backends/cuda/api/driver.pyx:322-330 ``funcSetAttribute``)."""
        if _dryrun.enabled():
            return
        _rt.check(_rt.lib.rt_func_set_attribute(self.ptr, _FUNC_ATTRIBUTES[name], int(value)))

    @property
    def attributes(self):
        out = {}
        for name in _FUNC_ATTRIBUTES:
            try:
                out[name] = self.get_attribute(name)
            except _rt.HIPError:
                pass
        return out

    def max_active_blocks_per_cu(self, block_size, dynamic_smem=0):
        if _dryrun.enabled():
            return 8
        v = ctypes.c_int(0)
        _rt.check(_rt.lib.rt_occupancy_max_active_blocks(
            self.ptr, block_size, dynamic_smem, ctypes.byref(v)))
        return v.value

    # -- launch -----------------------------------------------------------------
    def launch_packed(self, grid, block, arg_block, shared_mem=0, stream_ptr=None):
        """Launch with the argument block already laid out (bytes-like)."""
        if stream_ptr is None:
            stream_ptr = _stream.get_current_stream_ptr()
        gx, gy, gz = grid
        bx, by, bz = block
        if gx * bx > 0xffffffff or gy * by > 0xffffffff or gz * bz > 0xffffffff:
            # a dispatch holds its size in work-items in 32 bits per dimension
            raise ValueError(
                'kernel %s: grid %r x block %r exceeds 2**32 - 1 work-items in one dimension'
                % (self.name, grid, block))
        n = len(arg_block)
        if n > self._arg_size or n < self._arg_min:
            raise ValueError(
                'kernel %s expects an argument block of %d bytes, got %d'
                % (self.name, self._arg_size, n))
        if n < self._arg_size:
            arg_block = bytes(arg_block) + b'\0' * (self._arg_size - n)
        if _dryrun.enabled():
            _dryrun.record_launch(self.name, grid, block, shared_mem, bytes(arg_block))
            return
        if _kernel_timer is not None:
            start, stop = _kernel_timer._next(self.name)
            _rt.check(_rt.lib.rt_launch_packed_timed(
                self.ptr, gx, gy, gz, bx, by, bz, shared_mem, stream_ptr,
                bytes(arg_block), len(arg_block), start.ptr, stop.ptr))
            return
        status = _rt.hot.launch(
            self.ptr, gx, gy, gz, bx, by, bz, shared_mem, stream_ptr, arg_block)
        if status != 0:
            _rt.check(status)

    def launch_packed_scratch(self, grid, block, arg_block, scratch_arg_offset,
                              scratch_bytes, shared_mem=0, stream_ptr=None):
        """``launch_packed`` for a kernel whose scratch buffer is the runtime
        library's own static device array instead of an allocation: the
        pointer parameter at byte ``scratch_arg_offset`` of the argument block
        receives the array's address (``rt_launch_packed_scratch``).  Nothing
        is allocated on the way."""
        if stream_ptr is None:
            stream_ptr = _stream.get_current_stream_ptr()
        gx, gy, gz = grid
        bx, by, bz = block
        if gx * bx > 0xffffffff or gy * by > 0xffffffff or gz * bz > 0xffffffff:
            raise ValueError(
                'kernel %s: grid %r x block %r exceeds 2**32 - 1 work-items in one dimension'
                % (self.name, grid, block))
        n = len(arg_block)
        if n > self._arg_size or n < self._arg_min:
            raise ValueError(
                'kernel %s expects an argument block of %d bytes, got %d'
                % (self.name, self._arg_size, n))
        if n < self._arg_size:
            arg_block = bytes(arg_block) + b'\0' * (self._arg_size - n)
        if _dryrun.enabled():
            _dryrun.record_launch(self.name, grid, block, shared_mem, bytes(arg_block))
            return
        status = _rt.lib.rt_launch_packed_scratch(
            self.ptr, gx, gy, gz, bx, by, bz, shared_mem, stream_ptr,
            arg_block, len(arg_block), scratch_arg_offset, scratch_bytes)
        if status != 0:
            _rt.check(status)

    def launch_cooperative(self, grid, block, arg_block, shared_mem=0, stream_ptr=None):
        """``launch_packed`` as a cooperative launch: every workgroup of the
        grid is resident at once, so the kernel may synchronise the whole grid
        (reference: cupy/cuda/function.pyx:113-131 with
        ``enable_cooperative_groups``, driver.pyx:289-301).  The runtime
        refuses a grid larger than the device can hold at once."""
        if stream_ptr is None:
            stream_ptr = _stream.get_current_stream_ptr()
        gx, gy, gz = grid
        bx, by, bz = block
        if gx * bx > 0xffffffff or gy * by > 0xffffffff or gz * bz > 0xffffffff:
            raise ValueError(
                'kernel %s: grid %r x block %r exceeds 2**32 - 1 work-items in one dimension'
                % (self.name, grid, block))
        n = len(arg_block)
        if n > self._arg_size or n < self._arg_min:
            raise ValueError(
                'kernel %s expects an argument block of %d bytes, got %d'
                % (self.name, self._arg_size, n))
        arg_block = bytes(arg_block) + b'\0' * (self._arg_size - n)
        if _dryrun.enabled():
            _dryrun.record_launch(self.name, grid, block, shared_mem, arg_block)
            return
        # this launch takes one pointer per parameter: into a copy of the block
        buf = ctypes.create_string_buffer(arg_block, max(1, len(arg_block)))
        base = ctypes.addressof(buf)
        params = self.meta['args']
        pointers = (ctypes.c_void_p * max(1, len(params)))(
            *[base + offset for offset, _size, _kind in params])
        _rt.check(_rt.lib.rt_launch_cooperative(
            self.ptr, gx, gy, gz, bx, by, bz, shared_mem, stream_ptr, pointers))

    def __call__(self, grid, block, args, shared_mem=0, stream=None,
                 enable_cooperative_groups=False):
        """Launch with one Python object per kernel parameter.  Each object's
        bytes are placed at the parameter's offset in the argument block, cut
        or zero-padded to the parameter's size as recorded in the code object
        (an array passed for a pointer parameter contributes its address)."""
        grid = tuple(int(g) for g in grid) + (1,) * (3 - len(grid))
        block = tuple(int(b) for b in block) + (1,) * (3 - len(block))
        grid = tuple(max(1, g) for g in grid)
        block = tuple(max(1, b) for b in block)
        params = self.meta['args']
        if len(args) != len(params):
            raise TypeError('kernel %s takes %d arguments, %d given'
                            % (self.name, len(params), len(args)))
        blob = bytearray(self._arg_size)
        for a, (offset, size, _kind) in zip(args, params):
            b = bytes(_arg_to_bytes(a))
            n = min(len(b), size)
            blob[offset:offset + n] = b[:n]
        stream_ptr = (_stream.get_current_stream_ptr() if stream is None
                      else stream.ptr)
        if enable_cooperative_groups:
            self.launch_cooperative(grid, block, bytes(blob), shared_mem, stream_ptr)
        else:
            self.launch_packed(grid, block, bytes(blob), shared_mem, stream_ptr)

    def linear_launch(self, size, args, shared_mem=0, block_max_size=128,
                      stream=None):
        """1-D launch of ``size`` threads in blocks of at most
        ``block_max_size``; the grid is capped so that grid*block stays within
        the 2**32-1 work-items one dispatch may hold (kernels loop)."""
        block = max(1, min(block_max_size, size))
        grid = max(1, min((size + block - 1) // block, 0x7fffffff,
                          0xffffffff // block))
        self((grid,), (block,), args, shared_mem, stream)
