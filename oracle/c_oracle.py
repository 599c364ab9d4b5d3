"""ctypes access to the C restatement in ``ref_kernels.c`` -- TEST
INFRASTRUCTURE ONLY."""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB = os.path.join(_HERE, '_build', 'liboracle.so')
_lib = None


def load():
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB):
            subprocess.check_call(['make', '-C', _HERE], stdout=subprocess.DEVNULL)
        _lib = ctypes.CDLL(_LIB)
    return _lib


def _p(a):
    return a.ctypes.data_as(ctypes.c_void_p)


def get_block_specs(in_size, out_size, contiguous_size):
    lib = load()
    vals = [ctypes.c_int64(0) for _ in range(3)]
    lib.ref_get_block_specs(
        ctypes.c_int64(in_size), ctypes.c_int64(out_size),
        ctypes.c_int64(contiguous_size), *[ctypes.byref(v) for v in vals])
    return tuple(v.value for v in vals)


_SUM = {
    ('float32', 'float32'): 'ref_block_reduce_sum_f32',
    ('float64', 'float64'): 'ref_block_reduce_sum_f64',
    ('int32', 'int64'): 'ref_block_reduce_sum_i32_i64',
    ('int8', 'int64'): 'ref_block_reduce_sum_i8_i64',
}


def block_reduce_sum(a2d, axis):
    """Sum of a C-contiguous 2-d array along ``axis`` in the reference kernel's
    evaluation order."""
    lib = load()
    a2d = np.ascontiguousarray(a2d)
    rows, cols = a2d.shape
    out_dt = a2d.dtype if a2d.dtype.kind == 'f' else np.dtype('int64')
    fn = getattr(lib, _SUM[(a2d.dtype.name, out_dt.name)])
    if axis == 1:
        n_out, n_red, so, sr, contiguous = rows, cols, cols, 1, 1
    else:
        n_out, n_red, so, sr, contiguous = cols, rows, 1, cols, cols
    bs, stride, _ = get_block_specs(rows * cols, n_out, contiguous)
    out = np.empty(n_out, dtype=out_dt)
    fn(_p(a2d), _p(out), ctypes.c_int64(n_out), ctypes.c_int64(n_red),
       ctypes.c_int64(so), ctypes.c_int64(sr), ctypes.c_int64(bs),
       ctypes.c_int64(stride))
    return out


def block_reduce_arg(a2d, want_max):
    lib = load()
    a = np.ascontiguousarray(a2d, dtype=np.float64)
    out = np.empty(a.shape[0], dtype=np.int64)
    lib.ref_block_reduce_arg_f64(_p(a), _p(out), ctypes.c_int64(a.shape[0]),
                                 ctypes.c_int64(a.shape[1]), ctypes.c_int(int(want_max)))
    return out


def saxpy_f32(a, x, y):
    lib = load()
    x = np.ascontiguousarray(x, dtype=np.float32)
    y = np.ascontiguousarray(y, dtype=np.float32)
    z = np.empty_like(x)
    lib.ref_saxpy_f32(ctypes.c_float(a), _p(x), _p(y), _p(z), ctypes.c_int64(x.size))
    return z
