"""User-written kernels: ``RawKernel`` and ``RawModule``.

Counterpart of the reference's cupy/_core/raw.pyx (``RawKernel`` :10-303,
``RawModule`` :306-538, ``_get_raw_module`` :541-558).  The source is HIP C++
compiled by hiprtc for gfx950; precompiled modules are code objects
(``.hsaco``).  Compilation goes through the same two-level cache as the
generated kernels, launches through the same C-ABI entry points.
"""
from cupy_amd.cuda import compiler as _compiler
from cupy_amd.cuda import device as _device
from cupy_amd.cuda import function as _function
from cupy_amd.cuda import memory as _memory

_module_file_memo = {}


def _get_raw_module(code, path, options, name_expressions, log_stream,
                    enable_cooperative_groups=False):
    if code is not None:
        if enable_cooperative_groups:
            # <hip/hip_cooperative_groups.h> is not among the headers the
            # run-time compiler carries itself: it comes from the installation
            options = tuple(options) + ('-I' + _compiler.rocm_include_dir(),)
        return _compiler.compile_raw_with_cache(
            code, options, name_expressions=name_expressions, log_stream=log_stream)
    key = (_device.get_device_id(), path)
    mod = _module_file_memo.get(key)
    if mod is None:
        mod = _function.Module()
        mod.load_file(path)
        _module_file_memo[key] = mod
    return mod


class RawKernel:
    """User-defined kernel from raw HIP C++ source.

    Args:
        code (str): Source holding an ``extern "C" __global__`` function.
        name (str): Name of that function.
        options (tuple of str): Extra compiler options.
        backend (str): ``'nvrtc'`` (the run-time compiler, here hiprtc) is the
            only backend.
        translate_cucomplex (bool): Accepted for compatibility; no effect.
        enable_cooperative_groups (bool): Launch cooperatively (all
            workgroups resident at once), so that the kernel may use
            ``cooperative_groups::this_grid().sync()``; the installation's
            include directory is added for ``<hip/hip_cooperative_groups.h>``.

    ``kernel(grid, block, args, shared_mem=0, stream=None)`` launches; array
    arguments are passed as device pointers, NumPy scalars by value with their
    own type (a Python ``float`` is a C ``double``, a Python ``int`` a 64-bit
    integer).
    """

    def __init__(self, code, name, options=(), backend='nvrtc', *,
                 translate_cucomplex=False, enable_cooperative_groups=False,
                 jitify=None):
        if not isinstance(options, tuple):
            raise TypeError('options must be a tuple')
        if backend not in ('nvrtc', 'hiprtc'):
            raise ValueError('only the run-time compiler backend is available')
        if jitify:
            raise ValueError('jitify is not available')
        self.code = code
        self.name = name
        self.options = options
        self.backend = backend
        self.translate_cucomplex = translate_cucomplex
        self.enable_cooperative_groups = enable_cooperative_groups
        self.jitify = jitify
        self.file_path = None          # set when produced by a RawModule from a file
        self.name_expressions = None   # set when produced by a RawModule
        self._kernel_cache = {}
        self.__name__ = name

    def __call__(self, grid, block, args, **kwargs):
        """Compiles (first use) and launches.

        Args:
            grid (tuple): Grid size in workgroups.
            block (tuple): Workgroup size in threads.
            args (tuple): Kernel arguments.
            shared_mem (int): Dynamic LDS bytes per workgroup.
            stream: Stream to launch on (default: current stream).
        """
        self.kernel(grid, block, args,
                    enable_cooperative_groups=self.enable_cooperative_groups, **kwargs)

    @property
    def kernel(self):
        return self._kernel()

    def _kernel(self, log_stream=None):
        dev = _device.get_device_id()
        ker = self._kernel_cache.get(dev)
        if ker is None or log_stream is not None:
            assert (self.code is None) != (self.file_path is None)
            mod = _get_raw_module(self.code, self.file_path, self.options,
                                  self.name_expressions, log_stream,
                                  self.enable_cooperative_groups)
            ker = mod.get_function(self.name)
            self._kernel_cache[dev] = ker
        return ker

    def __getstate__(self):
        state = dict(self.__dict__)
        state['_kernel_cache'] = {}
        return state

    def compile(self, log_stream=None):
        """Compiles now instead of at the first call; the compiler's output
        goes to ``log_stream`` if given."""
        self._kernel_cache = {}
        self._kernel(log_stream)

    # -- function attributes (cupy/_core/raw.pyx:172-287) ---------------------------
    @property
    def attributes(self):
        """dict of the function attributes below (read-only)."""
        return dict(self.kernel.attributes)

    @property
    def max_threads_per_block(self):
        return self.kernel.get_attribute('max_threads_per_block')

    @property
    def shared_size_bytes(self):
        return self.kernel.get_attribute('shared_size_bytes')

    @property
    def const_size_bytes(self):
        return self.kernel.get_attribute('const_size_bytes')

    @property
    def local_size_bytes(self):
        return self.kernel.get_attribute('local_size_bytes')

    @property
    def num_regs(self):
        return self.kernel.get_attribute('num_regs')

    @property
    def ptx_version(self):
        return self.kernel.get_attribute('ptx_version')

    @property
    def binary_version(self):
        return self.kernel.get_attribute('binary_version')

    @property
    def cache_mode_ca(self):
        return self.kernel.get_attribute('cache_mode_ca')

    @property
    def max_dynamic_shared_size_bytes(self):
        return self.kernel.get_attribute('max_dynamic_shared_size_bytes')

    @max_dynamic_shared_size_bytes.setter
    def max_dynamic_shared_size_bytes(self, nbytes):
        self.kernel.set_attribute('max_dynamic_shared_size_bytes', nbytes)

    @property
    def preferred_shared_memory_carveout(self):
        return self.kernel.get_attribute('preferred_shared_memory_carveout')

    @preferred_shared_memory_carveout.setter
    def preferred_shared_memory_carveout(self, fraction):
        self.kernel.set_attribute('preferred_shared_memory_carveout', fraction)


class RawModule:
    """User-defined module: several kernels (and ``__device__`` variables)
    compiled from one source, or loaded from a code-object file.

    Args:
        code (str): HIP C++ source.  Mutually exclusive with ``path``.
        path (str): Path of a code object (``.hsaco``).
        options (tuple of str): Extra compiler options.
        name_expressions (sequence of str): C++ name expressions
            (``'func<float>'``) of template kernels to instantiate; pass the
            same strings to :meth:`get_function`.
    """

    def __init__(self, *, code=None, path=None, options=(), backend='nvrtc',
                 translate_cucomplex=False, enable_cooperative_groups=False,
                 name_expressions=None, jitify=None):
        if (code is None) == (path is None):
            raise TypeError(
                'Exactly one of `code` and `path` keyword arguments must be given.')
        if name_expressions is not None:
            if code is None:
                raise ValueError('need CUDA C++ code for the requested kernels')
            if backend not in ('nvrtc', 'hiprtc'):
                raise ValueError('only nvrtc supports retrieving the mangled '
                                 'names for the given name expressions')
            self.name_expressions = tuple(name_expressions)
        else:
            self.name_expressions = None
        if jitify:
            raise ValueError('jitify is not available')
        if not isinstance(options, tuple):
            raise TypeError('options must be a tuple')
        self.code = code
        self.file_path = path
        self.enable_cooperative_groups = enable_cooperative_groups
        self.jitify = jitify
        if code is not None:
            self.options = options
            self.backend = backend
            self.translate_cucomplex = translate_cucomplex
        else:
            self.options = ()
            self.backend = 'nvcc'
            self.translate_cucomplex = False

    @property
    def module(self):
        return self._module()

    def _module(self, log_stream=None):
        return _get_raw_module(self.code, self.file_path, self.options,
                               self.name_expressions, log_stream,
                               self.enable_cooperative_groups)

    def compile(self, log_stream=None):
        """Compiles now instead of at first use."""
        self._module(log_stream)

    def get_function(self, name):
        """RawKernel for the ``__global__`` function ``name`` (or for one of
        the name expressions given to the constructor)."""
        if self.name_expressions:
            mangled = self.module.mapping.get(name)
            if mangled is not None:
                name = mangled
        ker = RawKernel(self.code if self.code is not None else '', name, self.options,
                        'nvrtc', translate_cucomplex=self.translate_cucomplex,
                        enable_cooperative_groups=self.enable_cooperative_groups)
        if self.code is None:
            ker.code = None
        ker.file_path = self.file_path
        ker.name_expressions = self.name_expressions
        ker.kernel    # compile / look up now, as the reference does
        return ker

    def get_global(self, name):
        """MemoryPointer to the ``__device__`` / ``__constant__`` variable
        ``name``; wrap it in an ndarray of the known shape to use it."""
        mod = self.module
        ptr, size = mod.get_global_var(name)
        mem = _memory.UnownedMemory(ptr, size, mod, _device.get_device_id())
        return _memory.MemoryPointer(mem, 0)
