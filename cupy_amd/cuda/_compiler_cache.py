"""On-disk cache of compiled code objects.

File format (same as the reference's ``DiskKernelCacheBackend``,
cupy/cuda/_compiler_cache.py:78-182, pinned by
tests/cupy_tests/cuda_tests/test_compiler_cache.py:34-124): 40 ASCII hex
characters holding the SHA-1 of the payload, followed by the payload.  A file
that is missing, shorter than the digest or whose digest does not match is a
miss.  Writes go to a temporary file in the same directory and are moved into
place, so readers never see a half-written entry.
"""
import hashlib
import os
import tempfile

_DIGEST_LEN = 40


def get_cache_dir():
    """``$CUPY_CACHE_DIR`` or ``~/.cupy_amd/kernel_cache``."""
    return os.environ.get(
        'CUPY_CACHE_DIR', os.path.expanduser('~/.cupy_amd/kernel_cache'))


def bundled_cache_dir():
    """Read-only cache shipped inside the package tree (may not exist)."""
    return os.path.join(os.path.dirname(os.path.dirname(
        os.path.abspath(__file__))), '_kernel_cache')


def encode(payload):
    return hashlib.sha1(payload).hexdigest().encode('ascii') + payload


def decode(blob):
    """Payload of a cache file's contents, or None if it is damaged."""
    if blob is None or len(blob) < _DIGEST_LEN:
        return None
    digest, payload = blob[:_DIGEST_LEN], blob[_DIGEST_LEN:]
    if hashlib.sha1(payload).hexdigest().encode('ascii') != digest:
        return None
    return payload


class DiskKernelCache:

    def __init__(self, cache_dir=None, extra_read_dirs=()):
        self.cache_dir = cache_dir or get_cache_dir()
        self.extra_read_dirs = tuple(extra_read_dirs)

    def _path(self, directory, key):
        return os.path.join(directory, key)

    def load(self, key):
        for directory in (self.cache_dir,) + self.extra_read_dirs:
            try:
                with open(self._path(directory, key), 'rb') as f:
                    blob = f.read()
            except OSError:
                continue
            payload = decode(blob)
            if payload is not None:
                return payload
        return None

    def save(self, key, payload, source=None):
        try:
            os.makedirs(self.cache_dir, exist_ok=True)
            fd, tmp = tempfile.mkstemp(dir=self.cache_dir, prefix='tmp_')
            try:
                with os.fdopen(fd, 'wb') as f:
                    f.write(encode(payload))
                os.replace(tmp, self._path(self.cache_dir, key))
            except BaseException:
                try:
                    os.unlink(tmp)
                except OSError:
                    pass
                raise
            if source is not None:
                with open(self._path(self.cache_dir, key + '.hip'), 'w') as f:
                    f.write(source)
        except OSError:
            # An unwritable cache directory only costs recompilation.
            pass
