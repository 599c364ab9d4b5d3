"""Structured dtypes in generated kernels.

The reference describes a structured element to its kernels with variadic
templates over (type, offset) pairs (cupy/_core/_scalar.pyx:195-256,
include/cupy/structview.cuh).  Here the kernel source is generated at run time
anyway, so every structured dtype gets a concrete C++ struct written out for
it: raw bytes of the dtype's size and alignment plus an accessor per field.
Assignment and comparison between different structured types go field by field
through two small generic templates; nested structures recurse.

The definitions are kept in a registry by type name and spliced into a kernel
source right before it is compiled (``splice_definitions``).
"""
import hashlib
import re

import numpy

_definitions = {}       # type name -> (source, names it depends on)
_names = {}             # dtype -> (type name, alignment)
_TOKEN = re.compile(r'cupy_struct_[0-9a-f]{16}')

_PRELUDE = '''
namespace cupy {
template <typename T> struct is_struct { static const bool value = false; };
template <typename D, typename S> __device__ __forceinline__ void sv_set(D& d, const S& s);
template <typename D, typename S, int I>
struct sv_fields {
  static __device__ __forceinline__ void assign(D& d, const S& s) {
    sv_set(d.template at<I - 1>(), s.template at<I - 1>());
    sv_fields<D, S, I - 1>::assign(d, s);
  }
  static __device__ __forceinline__ void broadcast(D& d, const S& s) {
    sv_set(d.template at<I - 1>(), s);
    sv_fields<D, S, I - 1>::broadcast(d, s);
  }
  static __device__ __forceinline__ bool equal(const D& d, const S& s) {
    return sv_fields<D, S, I - 1>::equal(d, s) && (d.template at<I - 1>() == s.template at<I - 1>());
  }
};
template <typename D, typename S>
struct sv_fields<D, S, 0> {
  static __device__ __forceinline__ void assign(D&, const S&) {}
  static __device__ __forceinline__ void broadcast(D&, const S&) {}
  static __device__ __forceinline__ bool equal(const D&, const S&) { return true; }
};
template <typename D, typename S, bool kDstStruct, bool kSrcStruct> struct sv_setter {
  static __device__ __forceinline__ void run(D& d, const S& s) { d = static_cast<D>(s); }
};
template <typename D, typename S> struct sv_setter<D, S, true, true> {
  static __device__ __forceinline__ void run(D& d, const S& s) {
    static_assert(D::n_fields == S::n_fields, "field counts differ");
    sv_fields<D, S, D::n_fields>::assign(d, s);
  }
};
template <typename D, typename S> struct sv_setter<D, S, true, false> {
  static __device__ __forceinline__ void run(D& d, const S& s) {
    sv_fields<D, S, D::n_fields>::broadcast(d, s);
  }
};
template <typename D, typename S> __device__ __forceinline__ void sv_set(D& d, const S& s) {
  sv_setter<D, S, is_struct<D>::value, is_struct<S>::value>::run(d, s);
}
}  // namespace cupy
'''


def is_structured(dtype):
    return dtype.kind == 'V' and dtype.fields is not None


def has_references(dtype):
    """True if ``dtype`` holds Python objects anywhere."""
    if dtype.kind == 'O':
        return True
    if dtype.fields is not None:
        return any(has_references(f[0]) for f in dtype.fields.values())
    if dtype.subdtype is not None:
        return has_references(dtype.subdtype[0])
    return False


def device_alignment(dtype):
    """Alignment kernels need for a non-structured ``dtype``: the element size
    (complex numbers are accessed whole), that of the base type for
    sub-arrays, 1 for raw bytes (cupy/_core/_scalar.pyx:137-190)."""
    if dtype.metadata and '__cuda_alignment__' in dtype.metadata:
        return dtype.metadata['__cuda_alignment__']
    if dtype.subdtype is not None:
        base = dtype.subdtype[0]
        if is_structured(base):
            return struct_typename(base)[1]
        return device_alignment(base)
    if dtype.kind == 'V':
        if is_structured(dtype):
            raise ValueError('device_alignment() only supports unstructured dtypes, got %s' % dtype)
        return 1
    return dtype.itemsize


def struct_typename(dtype):
    """(C++ type name, alignment) of a structured dtype; registers the type's
    definition.  Raises ValueError for layouts a kernel cannot address."""
    hit = _names.get(dtype)
    if hit is not None and (not dtype.metadata):
        return hit
    from cupy_amd._core._scalar import get_typename
    alignment = dtype.alignment
    if dtype.metadata:
        alignment = dtype.metadata.get('__cuda_alignment__', alignment)
    fields = []
    depends = []
    for name, info in dtype.fields.items():
        sub, offset = info[0], info[1]
        if sub.subdtype is not None:
            raise ValueError('structured dtypes with subarray dtypes are not supported in kernels')
        if is_structured(sub):
            sub_name, sub_align = struct_typename(sub)
            depends.append(sub_name)
        else:
            sub_name = get_typename(sub)
            sub_align = device_alignment(sub)
        alignment = max(alignment, sub_align)
        if offset % sub_align != 0:
            raise ValueError(
                f'Field {name} with offset {offset} is not aligned to {sub_align} in dtype '
                f'{dtype}. This is not supported by CuPy please ensure the structure is '
                'aligned. You can do so with the `make_aligned_dtype()` helper.')
        fields.append((sub_name, offset))
    if dtype.itemsize % alignment != 0:
        raise ValueError(
            f'Itemsize {dtype.itemsize} is not a multiple of alignment {alignment} for dtype '
            f'{dtype} and kernel launches are not supported. You can ensure compatibility with '
            'the `make_aligned_dtype()` helper (or try `align=True`).')
    layout = '%d/%d/' % (dtype.itemsize, alignment) + ';'.join('%s@%d' % f for f in fields)
    type_name = 'cupy_struct_' + hashlib.sha1(layout.encode()).hexdigest()[:16]
    if type_name not in _definitions:
        lines = ['struct alignas(%d) %s {' % (alignment, type_name),
                 '  char _d[%d];' % dtype.itemsize,
                 '  static const int n_fields = %d;' % len(fields),
                 '  static const int field_count = %d;' % len(fields)]
        for const in ('', 'const '):
            lines.append('  template <int I> __device__ __forceinline__ %sauto& at() %s{' % (const, const))
            for k, (sub_name, offset) in enumerate(fields):
                lines.append('    %sif constexpr (I == %d) return *reinterpret_cast<%s%s*>(_d + %d);' % (
                    'else ' if k else '', k, const, sub_name, offset))
            lines.append('  }')
        lines.append('  %s() = default;' % type_name)
        lines.append('  template <typename O> __device__ __forceinline__ explicit %s(const O& o) '
                     '{ cupy::sv_set(*this, o); }' % type_name)
        lines.append('  template <typename O> __device__ __forceinline__ %s& operator=(const O& o) '
                     '{ cupy::sv_set(*this, o); return *this; }' % type_name)
        lines.append('  template <typename O> __device__ __forceinline__ bool operator==(const O& o) const '
                     '{ static_assert(n_fields == O::n_fields, "field counts differ"); '
                     'return cupy::sv_fields<%s, O, n_fields>::equal(*this, o); }' % type_name)
        lines.append('  template <typename O> __device__ __forceinline__ bool operator!=(const O& o) const '
                     '{ return !(*this == o); }')
        lines.append('};')
        lines.append('namespace cupy { template <> struct is_struct<%s> '
                     '{ static const bool value = true; }; }' % type_name)
        _definitions[type_name] = ('\n'.join(lines), tuple(depends))
    if not dtype.metadata:
        _names[dtype] = (type_name, alignment)
    return type_name, alignment


def void_typename(itemsize):
    """C++ type of an unstructured void element: ``itemsize`` raw bytes that can
    be copied and compared (include/cupy/unstructured_void.cuh in the
    reference)."""
    type_name = 'cupy_struct_' + hashlib.sha1(b'void/%d' % itemsize).hexdigest()[:16]
    if type_name not in _definitions:
        _definitions[type_name] = ('''struct %(n)s {
  char _d[%(size)d];
  __device__ __forceinline__ bool operator==(const %(n)s& o) const {
    bool same = true;
    for (int k = 0; k < %(size)d; ++k) same = same && (_d[k] == o._d[k]);
    return same;
  }
  __device__ __forceinline__ bool operator!=(const %(n)s& o) const { return !(*this == o); }
};''' % dict(n=type_name, size=itemsize), ())
    return type_name


def splice_definitions(source):
    """``source`` with the definitions of the structured types it names put
    in after its first line (the include of the device header)."""
    found = _TOKEN.findall(source)
    if not found:
        return source
    ordered = []

    def visit(name):
        if name in ordered:
            return
        text, depends = _definitions[name]
        for d in depends:
            visit(d)
        ordered.append(name)
    for name in found:
        visit(name)
    head, _, rest = source.partition('\n')
    body = '\n'.join(_definitions[n][0] for n in ordered)
    return head + '\n' + _PRELUDE + body + '\n' + rest


def _aligned(dtype, alignment=-1, recurse=True):
    """(dtype, alignment): ``dtype`` re-laid with every field at a multiple of
    its device alignment and the size rounded up to the largest of them
    (cupy/_core/_dtype.pyx:211-298)."""
    descr = numpy.dtype(dtype, align=True)
    if alignment != -1 and (alignment <= 0 or alignment & (alignment - 1)):
        raise ValueError('Reasonable alignments must be >0 and a power of 2.')
    final = 1
    cursor = 0
    if not is_structured(descr):
        info = descr
        final = device_alignment(descr)
        cursor = descr.itemsize
    else:
        names, offsets, formats = [], [], []
        least = 0
        for name, field in descr.fields.items():
            sub, offset = field[0], field[1]
            if offset < least:
                raise ValueError('make_aligned_dtype() only supports well behaved in-order '
                                 'fields as it ignores field offsets.')
            least = offset + sub.itemsize
            sub_align = sub.metadata.get('__cuda_alignment__') if sub.metadata else None
            if sub_align is not None:
                pass
            elif not is_structured(sub):
                sub_align = device_alignment(sub)
            elif not recurse:
                sub_align = sub.alignment
            else:
                sub, sub_align = _aligned(sub, recurse=recurse)
            cursor += -cursor % sub_align
            final = max(final, sub_align)
            names.append(name)
            formats.append(sub)
            offsets.append(cursor)
            cursor += sub.itemsize
        info = dict(names=names, offsets=offsets, formats=formats, itemsize=0)
    metadata = {}
    if alignment != -1:
        if alignment < final:
            raise ValueError(f'make_aligned_dtype(): given alignment={alignment} smaller than '
                             f'minimum alignment {final}')
        final = alignment
        metadata = {'metadata': {'__cuda_alignment__': alignment}}
    itemsize = (cursor + final - 1) // final * final
    if not is_structured(descr):
        if descr.itemsize != itemsize:
            raise ValueError('Alignment larger than itemsize for non-structured dtype.')
    else:
        if descr.itemsize > itemsize:
            raise ValueError('Input descriptor had larger itemsize than inferred.')
        info['itemsize'] = itemsize
    return numpy.dtype(info, align=True, **metadata), final


def make_aligned_dtype(dtype, *, alignment=-1, recurse=True):
    """A structured dtype laid out as ``dtype`` but with every field aligned
    as kernels need it (complex fields to their full size) and the element size
    padded accordingly.

    .. seealso:: ``cupy.make_aligned_dtype`` (cupy/_core/_dtype.pyx:301-342)
    """
    descr = numpy.dtype(dtype, align=True)
    if not is_structured(descr):
        raise ValueError('make_aligned_dtype() only supports structured dtypes.')
    return _aligned(dtype, alignment=alignment, recurse=recurse)[0]


def comparison_dtype(dt1, dt2):
    """Common dtype two structured arrays are compared in
    (cupy/_core/_routines_logic.pyx:76-100)."""
    if dt1.fields is None and dt2.fields is None:
        if dt1.itemsize == dt2.itemsize and dt1.itemsize > 0:
            return dt1
        raise TypeError('cannot compare unstructured voids of different size '
                        f'({dt1.itemsize} vs {dt2.itemsize})')
    if dt1.fields is None or dt2.fields is None:
        raise TypeError('Cannot compare structured and non-structured dtypes')
    try:
        common = numpy.promote_types(dt1, dt2)
    except TypeError:
        raise TypeError('Cannot compare structured arrays unless they have a common dtype.  '
                        'I.e. `np.result_type(arr1, arr2)` must be defined.')
    return make_aligned_dtype(common)
