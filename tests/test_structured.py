"""Structured dtypes: type names, alignment rules and the aligned-dtype helper
(host logic; the kernels are compiled for gfx950 without being run).  The
cases follow the reference's tests/cupy_tests/core_tests/test_structured.py."""
import numpy as np
import pytest

import cupy_amd as cp
from cupy_amd._core import _structured
from cupy_amd._core._scalar import get_typename


def test_creation_keeps_dtype_and_shape():
    a = cp.empty((2, 3, 4), dtype='i,i')
    assert a.dtype == np.dtype('i,i') and a.shape == (2, 3, 4)
    z = cp.zeros((2, 3, 4), dtype='i,i')
    assert z.dtype == np.dtype('i,i') and z.nbytes == 2 * 3 * 4 * 8


def test_dtypes_that_hold_objects_are_rejected():
    arr = np.array([1, 2, 3], dtype='q,O')
    with pytest.raises(ValueError):
        cp.array(arr)
    with pytest.raises(ValueError):
        cp.asarray([arr, arr])
    with pytest.raises(ValueError):
        cp.empty(3, dtype='q,O')


def test_final_alignment_check():
    dt = np.dtype('f8,?')
    with pytest.raises(ValueError, match='Itemsize 9 is not a multiple'):
        get_typename(dt, None)
    with pytest.raises(ValueError, match='Itemsize 9 is not a multiple'):
        cp.ones(10, dtype=dt)            # building the kernel fails the same way


def test_bad_field():
    dt = np.dtype('?,f8')
    with pytest.raises(ValueError, match='Field f1 with offset 1 is not '):
        get_typename(dt, None)
    with pytest.raises(ValueError, match='Field f1 with offset 1 is not '):
        cp.ones(10, dtype=dt)


@pytest.mark.parametrize('dt,itemsize', [
    ('?,c8', 16), ('c8,?', 16),                       # complex is aligned to its full size
    ('?,(3,)c8', 32), ('(3,)c8,?', 32),               # sub-arrays by their base type
    (np.dtype([('a', 'c8,?'), ('b', '?')]), 24),
    (np.dtype([('a', '?'), ('b', 'c8,?')]), 24),
    ('?,(4,)V3', 13),                                 # raw bytes need no alignment
])
def test_make_aligned_dtype(dt, itemsize):
    assert cp.make_aligned_dtype(dt).itemsize == itemsize


@pytest.mark.parametrize('dt', ['c16', 'V3'])
def test_make_aligned_dtype_needs_a_structure(dt):
    with pytest.raises(ValueError, match='only supports structured dtypes'):
        cp.make_aligned_dtype(dt)


def test_make_aligned_dtype_alignment_argument():
    dt = cp.make_aligned_dtype('i4,f4', alignment=16)
    assert dt.itemsize == 16 and dt.metadata['__cuda_alignment__'] == 16
    with pytest.raises(ValueError, match='smaller than minimum alignment'):
        cp.make_aligned_dtype('i8,f8', alignment=4)
    with pytest.raises(ValueError, match='power of 2'):
        cp.make_aligned_dtype('i8,f8', alignment=12)
    name, align = _structured.struct_typename(dt)
    assert align == 16


def test_type_definitions_are_spliced_in_dependency_order():
    inner = np.dtype('i8,f8')
    outer = np.dtype([('a', 'f8'), ('b', inner)])
    name = get_typename(outer)
    inner_name = get_typename(inner)
    assert name.startswith('cupy_struct_') and name != inner_name
    src = _structured.splice_definitions('#include <cupy/carray.cuh>\ntypedef %s T;\n' % name)
    assert src.index('struct alignas(8) ' + inner_name) < src.index('struct alignas(8) ' + name)
    assert src.startswith('#include <cupy/carray.cuh>\n')
    # the same layout under other field names is the same type
    other = np.dtype([('x', 'i8'), ('y', 'f8')])
    assert get_typename(other) == inner_name


def test_field_views_and_their_errors():
    a = cp.zeros(4, dtype='i,i')
    v = a['f1']
    assert v.dtype == np.int32 and v.strides == (8,) and v.data.ptr == a.data.ptr + 4
    assert not v.flags.c_contiguous and not v.flags.f_contiguous
    assert a.flags.c_contiguous and a.flags.f_contiguous
    m = cp.ones(10, 'i,f,i')[['f2', 'f1']]
    assert m.dtype.names == ('f2', 'f1') and m.dtype.itemsize == 12
    assert m.dtype.fields['f2'][1] == 8 and m.dtype.fields['f1'][1] == 4
    for field, dtype in (('f1', '?,f8'), ('f0', 'f8,?')):
        b = cp.empty(4, dtype=dtype)
        with pytest.raises(ValueError, match='result array with.* sufficiently aligned for GPU'):
            b[field]
        with pytest.raises(ValueError, match='result array with.* sufficiently aligned for GPU'):
            b[field] = 1
        assert b[:0][field].shape == (0,)            # nothing to misalign
    with pytest.raises(ValueError, match='CuPy does not yet support accessing nested subarrays'):
        cp.zeros(10, dtype='i,(3,3)i')['f1']
    with pytest.raises(ValueError):
        a['nope']


def test_comparison_dtype_rules():
    a = cp.zeros(1, dtype='i8,f8')
    with pytest.raises(TypeError):
        a[['f1', 'f0']] == cp.zeros(3, dtype='f8,i8')     # field names in another order
    with pytest.raises(TypeError, match='structured and non-structured'):
        _structured.comparison_dtype(np.dtype('i8,f8'), np.dtype('V16'))
    common = _structured.comparison_dtype(np.dtype('f8,c8'), np.dtype('f8,f8'))
    assert np.result_type(np.dtype('f8,c8'), np.dtype('f8,f8')).itemsize == 24
    assert common.itemsize == 32                      # complex128 aligned to 16 bytes
    inner = np.dtype([('x', 'i4'), ('y', 'f4')])
    sub = cp.zeros(2, dtype=np.dtype([('a', inner, (3,))]))
    with pytest.raises(ValueError, match='.*subarray dtypes'):
        sub == sub
    with pytest.raises(TypeError):
        cp.zeros(2, dtype='i8,f8') + cp.zeros(2, dtype='i8,f8')
    with pytest.raises(TypeError):
        cp.zeros(2, dtype='i8,f8').astype('i8,f8,i8')
