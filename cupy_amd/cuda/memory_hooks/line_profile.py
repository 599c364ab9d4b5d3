"""A memory hook that attributes device memory to lines of Python code
(reference: cupy/cuda/memory_hooks/line_profile.py; same report format)."""
import os
import sys
import traceback

from cupy_amd.cuda import memory_hook

_UNITS = ('', 'K', 'M', 'G', 'T', 'P', 'E')


def _humanized(nbytes):
    size = float(nbytes)
    for unit in _UNITS:
        if size < 1024.0:
            return '%3.2f%sB' % (size, unit)
        size /= 1024.0
    return '%.2f%sB' % (size, 'Z')


class _Node:
    """A call site (file, line, function) below its caller's node, with the
    bytes requested from the pool (``used``) and the bytes the pool took from
    the device (``acquired``) by everything called from there."""

    __slots__ = ('site', 'children', 'used', 'acquired')

    def __init__(self, site):
        self.site = site
        self.children = {}          # site -> _Node, in first-seen order
        self.used = 0
        self.acquired = 0

    def child(self, site):
        node = self.children.get(site)
        if node is None:
            node = self.children[site] = _Node(site)
        return node

    def write(self, file, depth):
        sizes = (_humanized(self.used), _humanized(self.acquired))
        if self.site is None:
            file.write('_root (%s, %s)\n' % sizes)
        else:
            file.write('%s%s:%s:%s (%s, %s)\n' % (('  ' * depth,) + self.site + sizes))
        for node in self.children.values():
            node.write(file, depth + 1)


class LineProfileHook(memory_hook.MemoryHook):
    """Line-by-line profile of device memory use.

    While the hook is active, every request served by the pool and every
    allocation the pool makes on the device is charged to each frame of the
    Python call stack that led to it.  ``print_report()`` shows the call tree::

        _root (4.00KB, 4.00KB)
          tests/test.py:37:test (1.00KB, 1.00KB)
          tests/test.py:38:test (1.00KB, 1.00KB)
          tests/test.py:39:test (2.00KB, 2.00KB)

    one line per call site: ``file:line:function (bytes requested from the
    pool, bytes the pool took from the device)``.

    Args:
        max_depth (int): levels of the report, the root line included: the
            outermost ``max_depth - 1`` frames of every stack (0: all).
    """

    name = 'LineProfileHook'

    def __init__(self, max_depth=0):
        self._root = _Node(None)
        self._max_depth = max_depth
        # frames of the package's own allocation path are left out: the
        # profile is about the caller's code
        self._skip = (os.path.abspath(__file__),)

    def malloc_preprocess(self, **kwargs):
        self._charge(used=kwargs['mem_size'])

    def alloc_preprocess(self, **kwargs):
        self._charge(acquired=kwargs['mem_size'])

    def _charge(self, used=0, acquired=0):
        node = self._root
        node.used += used
        node.acquired += acquired
        depth = 0
        for frame in traceback.extract_stack():
            if frame.filename in self._skip:
                continue
            depth += 1
            if 0 < self._max_depth <= depth:
                break
            node = node.child((frame.filename, frame.lineno, frame.name))
            node.used += used
            node.acquired += acquired

    def print_report(self, file=sys.stdout):
        """Writes the call tree with its byte counts to ``file``."""
        self._root.write(file, -1)
        file.flush()
