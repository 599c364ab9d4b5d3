"""Run-time compilation of generated HIP source for gfx950 with hiprtc.

Counterpart of the reference's cupy/cuda/compiler.py (``_compile_with_cache_hip``
:1003-1087, ``_NVRTCProgram`` :832-880, ``CompileException`` :793-829,
``is_valid_kernel_name`` :883-884) and of ``compile_with_cache`` in
cupy/_core/core.pyx:2621-2643.  Two cache levels: an in-process memo of loaded
modules per device, and code objects on disk.
"""
import ctypes
import hashlib
import os
import re
import struct
import sys
import threading

from cupy_amd import _dryrun
from cupy_amd import _rt
from cupy_amd.cuda import _compiler_cache
from cupy_amd.cuda import device as _device
from cupy_amd.cuda import function as _function

_INCLUDE_DIR = os.path.join(os.path.dirname(os.path.dirname(
    os.path.abspath(__file__))), 'include')

_kernel_name_re = re.compile(r'^[a-zA-Z_][a-zA-Z_0-9]*$')

# Options every generated kernel is compiled with.
#  * -ffp-contract=off: a*b+c must round twice, like the NumPy loops the
#    results are compared with.
#  * no denormal flushing (the default), for the same reason.
#  * packed-FP32 instructions are switched off.
_BASE_OPTIONS = (
    '-std=c++17', '-O3', '-ffp-contract=off',
    '-Xclang', '-target-feature', '-Xclang', '-packed-fp32-ops',
)


def is_valid_kernel_name(name):
    return _kernel_name_re.match(name) is not None


class CompileException(Exception):
    """hiprtc rejected the source; ``str()`` is the compiler log."""

    def __init__(self, msg, source, name, options, backend='hiprtc'):
        self._msg = msg
        self.source = source
        self.name = name
        self.options = options
        self.backend = backend
        super().__init__()

    def __reduce__(self):
        return (type(self), (self._msg, self.source, self.name, self.options,
                             self.backend))

    def __repr__(self):
        return str(self)

    def __str__(self):
        return self.get_message()

    def get_message(self):
        return self._msg

    def dump(self, f):
        lines = self.source.split('\n')
        digits = len(str(len(lines)))
        f.write('%s compilation error: %s\n' % (self.backend, self))
        f.write('-----\nName: %s\nOptions: %s\nSource:\n' % (
            self.name, ' '.join(self.options)))
        for i, line in enumerate(lines):
            f.write('%*d\t%s\n' % (digits, i + 1, line.rstrip()))
        f.write('-----\n')
        f.flush()


_rtc_version = None


def get_rtc_version():
    global _rtc_version
    if _rtc_version is None:
        major = ctypes.c_int(0)
        minor = ctypes.c_int(0)
        _rt.check(_rt.lib.rt_rtc_version(ctypes.byref(major), ctypes.byref(minor)))
        _rtc_version = (major.value, minor.value)
    return _rtc_version


_header_digest = None


_include_re = re.compile(r'#\s*include\s*[<"](cupy/[^>"]+)[>"]')
_header_files = {}          # relative name -> (bytes, names it includes)
_header_digests = {}        # frozenset of names -> digest


def _header_file(name):
    entry = _header_files.get(name)
    if entry is None:
        try:
            with open(os.path.join(_INCLUDE_DIR, name), 'rb') as f:
                data = f.read()
        except OSError:
            data = b''
        entry = (data, tuple(_include_re.findall(data.decode('utf-8', 'replace'))))
        _header_files[name] = entry
    return entry


def _get_header_digest(source=None):
    """Hash of the bundled device headers a source includes, directly or
    through other bundled headers: part of its cache key (a change to one
    header leaves the cached kernels that never saw it valid).  Without a
    source: of all bundled headers."""
    if source is None:
        names = set()
        for root, _, files in os.walk(_INCLUDE_DIR):
            for name in files:
                names.add(os.path.relpath(os.path.join(root, name), _INCLUDE_DIR))
    else:
        names = set()
        todo = list(_include_re.findall(source))
        while todo:
            name = todo.pop()
            if name not in names:
                names.add(name)
                todo.extend(_header_file(name)[1])
    key = frozenset(names)
    digest = _header_digests.get(key)
    if digest is None:
        h = hashlib.sha1()
        for name in sorted(names):
            h.update(name.encode())
            h.update(_header_file(name)[0])
        digest = _header_digests[key] = h.hexdigest()
    return digest


def get_arch(device_id=None):
    """Target processor for hiprtc, e.g. ``gfx950`` (feature suffixes dropped
    so the code object loads whatever the sramecc/xnack setting)."""
    if _dryrun.enabled():
        return 'gfx950'
    return _device.get_device_properties(device_id)['arch'].split(':')[0]


# Options of user-written (raw) kernels: no contraction override -- the source
# is the user's, so are its floating-point semantics.
_RAW_BASE_OPTIONS = (
    '-std=c++17', '-O3',
    '-Xclang', '-target-feature', '-Xclang', '-packed-fp32-ops',
)


def compile_source(source, options=(), arch='gfx950', name='kernel.hip',
                   base_options=_BASE_OPTIONS, name_expressions=None, with_log=False):
    """Compiles HIP source to a gfx950 code object (bytes); no caching.  With
    ``name_expressions`` or ``with_log`` returns ``(code, [lowered name per
    expression], compiler log)``."""
    opts = ('--offload-arch=' + arch,) + tuple(base_options) + (
        '-I' + _INCLUDE_DIR,) + tuple(options)
    enc = [o.encode() for o in opts]
    c_opts = (ctypes.c_char_p * len(enc))(*enc)
    code = ctypes.c_void_p()
    size = ctypes.c_size_t(0)
    log = ctypes.c_void_p()
    lowered = None
    if name_expressions:
        names = [n.encode() for n in name_expressions]
        c_names = (ctypes.c_char_p * len(names))(*names)
        lowered = (ctypes.c_void_p * len(names))()
        status = _rt.lib.rt_compile_named(
            source.encode(), name.encode(), len(enc), c_opts, 0, None, None,
            len(names), c_names, lowered,
            ctypes.byref(code), ctypes.byref(size), ctypes.byref(log))
    else:
        status = _rt.lib.rt_compile(
            source.encode(), name.encode(), len(enc), c_opts, 0, None, None,
            ctypes.byref(code), ctypes.byref(size), ctypes.byref(log))
    try:
        log_text = ctypes.string_at(log.value).decode(errors='replace') \
            if log.value else ''
        if status != 0:
            if _rt.RT_ERR_RTC_BASE <= status < _rt.RT_ERR_POOL_OOM:
                exc = CompileException(log_text or _rt.lib.rt_error_string(
                    status).decode(), source, name, opts)
                if os.environ.get('CUPY_DUMP_CUDA_SOURCE_ON_ERROR', '0') not in ('', '0'):
                    exc.dump(sys.stderr)
                raise exc
            _rt.check(status)
        binary = ctypes.string_at(code.value, size.value)
        if lowered is None:
            return (binary, [], log_text) if with_log else binary
        return binary, [ctypes.string_at(p).decode() for p in lowered], log_text
    finally:
        if code.value:
            _rt.lib.rt_free_buffer(code)
        if log.value:
            _rt.lib.rt_free_buffer(log)
        if lowered is not None:
            for p in lowered:
                if p:
                    _rt.lib.rt_free_buffer(p)


def _cache_key(source, options, arch):
    h = hashlib.sha1()
    for part in (arch, repr(_BASE_OPTIONS), repr(tuple(options)),
                 repr(get_rtc_version()), _get_header_digest(source), source):
        h.update(part.encode())
        h.update(b'\0')
    return h.hexdigest() + '.hsaco'


_disk_cache = None
_module_memo = {}
_memo_lock = threading.Lock()
# compile statistics, for tests and the launch-latency report
stats = {'memo_hit': 0, 'disk_hit': 0, 'compiled': 0}


def _get_disk_cache():
    global _disk_cache
    if _disk_cache is None or _disk_cache.cache_dir != _compiler_cache.get_cache_dir():
        _disk_cache = _compiler_cache.DiskKernelCache(
            extra_read_dirs=(_compiler_cache.bundled_cache_dir(),))
    return _disk_cache


def get_code_object(source, options=()):
    """Code object for ``source`` through the disk cache."""
    arch = get_arch()
    key = _cache_key(source, options, arch)
    use_disk = os.environ.get('CUPY_CACHE_IN_MEMORY', '0') in ('', '0')
    payload = _get_disk_cache().load(key) if use_disk else None
    if payload is None:
        payload = compile_source(source, options, arch)
        stats['compiled'] += 1
        if use_disk:
            save_src = os.environ.get('CUPY_CACHE_SAVE_CUDA_SOURCE', '0') not in ('', '0')
            _get_disk_cache().save(key, payload, source if save_src else None)
    else:
        stats['disk_hit'] += 1
    return payload


def _debug_options():
    """``CUPY_CUDA_COMPILE_WITH_DEBUG=1``: every kernel is compiled with debug
    information and without optimisation (the reference adds ``--device-debug
    --generate-line-info``, cupy/cuda/compiler.py:673-674).  The options are part
    of the cache key, so optimised and debug builds never mix."""
    if os.environ.get('CUPY_CUDA_COMPILE_WITH_DEBUG', '0') in ('', '0'):
        return ()
    return ('-g', '-O0')


def compile_with_cache(source, options=()):
    """Loaded module for ``source`` on the current device (memoised)."""
    options = tuple(options) + _debug_options()
    if 'cupy_struct_' in source:
        # structured element types: their definitions follow the device header
        from cupy_amd._core import _structured
        source = _structured.splice_definitions(source)
    dev = _device.get_device_id()
    key = (dev, source, options)
    mod = _module_memo.get(key)
    if mod is not None:
        stats['memo_hit'] += 1
        return mod
    code = get_code_object(source, options)
    mod = _function.Module()
    mod.load(code)
    with _memo_lock:
        mod = _module_memo.setdefault(key, mod)
    return mod


# Cache entries of modules built with name expressions store the lowered names
# ahead of the code object, in the reference's layout
# (cupy/cuda/compiler.py:545-621): magic, uint32 count, count x (uint32 length,
# UTF-8 bytes), code object; names ordered by sorted(name_expressions).
_PAYLOAD_MAGIC = b'\x93CUPYNE\x00'


def _encode_named_payload(lowered, code):
    parts = [_PAYLOAD_MAGIC, struct.pack('<I', len(lowered))]
    for n in lowered:
        e = n.encode('utf-8')
        parts.append(struct.pack('<I', len(e)))
        parts.append(e)
    parts.append(code)
    return b''.join(parts)


def _decode_named_payload(payload, count):
    if not payload.startswith(_PAYLOAD_MAGIC):
        return None
    pos = len(_PAYLOAD_MAGIC)
    if len(payload) < pos + 4:
        return None
    (stored,) = struct.unpack_from('<I', payload, pos)
    pos += 4
    if stored != count:
        return None
    names = []
    for _ in range(stored):
        if len(payload) < pos + 4:
            return None
        (size,) = struct.unpack_from('<I', payload, pos)
        pos += 4
        if len(payload) < pos + size:
            return None
        names.append(payload[pos:pos + size].decode('utf-8'))
        pos += size
    return names, payload[pos:]


def rocm_include_dir():
    """Include directory of the ROCm installation (``ROCM_HOME`` / ``ROCM_PATH``,
    else /opt/rocm; the reference looks for the installation the same way,
    cupy/_environment.py:214-230)."""
    for var in ('ROCM_HOME', 'ROCM_PATH'):
        root = os.environ.get(var)
        if root and os.path.isdir(os.path.join(root, 'include')):
            return os.path.join(root, 'include')
    return '/opt/rocm/include'


def compile_raw_with_cache(source, options=(), name_expressions=None, log_stream=None):
    """Loaded module for user-written source (cupy/_core/raw.pyx:541-558
    ``_get_raw_module``): no bundled headers are prepended, the user's options
    follow the target option, and ``module.mapping`` maps each name expression
    to its lowered symbol."""
    options = tuple(options)
    exprs = tuple(sorted(name_expressions)) if name_expressions else ()
    dev = _device.get_device_id()
    key = (dev, 'raw', source, options, exprs)
    mod = _module_memo.get(key)
    if mod is not None and log_stream is None:
        stats['memo_hit'] += 1
        return mod
    arch = get_arch()
    ckey = _cache_key(source, ('raw',) + options + exprs, arch)
    use_disk = (os.environ.get('CUPY_CACHE_IN_MEMORY', '0') in ('', '0')
                and log_stream is None)
    payload = _get_disk_cache().load(ckey) if use_disk else None
    lowered = None
    code = None
    if payload is not None:
        if exprs:
            dec = _decode_named_payload(payload, len(exprs))
            if dec is not None:
                lowered, code = dec
        else:
            code = payload
    if code is None:
        if exprs:
            code, lowered, log_text = compile_source(
                source, options, arch, base_options=_RAW_BASE_OPTIONS,
                name_expressions=exprs)
            payload = _encode_named_payload(lowered, code)
        else:
            code, _, log_text = compile_source(
                source, options, arch, base_options=_RAW_BASE_OPTIONS, with_log=True)
            payload = code
        if log_stream is not None and log_text:
            log_stream.write(log_text)
        stats['compiled'] += 1
        if use_disk:
            _get_disk_cache().save(ckey, payload, None)
    else:
        stats['disk_hit'] += 1
    mod = _function.Module()
    mod.load(code)
    mod.mapping = dict(zip(exprs, lowered)) if exprs else None
    with _memo_lock:
        _module_memo[key] = mod
    return mod


def clear_memo():
    with _memo_lock:
        _module_memo.clear()
