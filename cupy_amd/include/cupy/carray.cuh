// Device-side runtime of the generated kernels, written for gfx950 (CDNA4,
// wave64) only.  It provides the names that user kernel strings may use:
// CUPY_FOR, CArray, CIndexer, float16, _floor_divide, CUDART_INF/NAN, and the
// wave/block reduction helpers used by the reduction emitter.
//
// Counterpart of the reference's cupy/_core/include/cupy/carray.cuh (CArray
// :228-516, CIndexer :518-669, _floor_divide :671-700) and float16.cuh
// (:50-208); same user-visible interface, independent implementation.
#pragma once

#ifndef M_PI
#define M_PI 3.1415926535897932384626433832795
#endif

#define CUDART_INF_F __builtin_inff()
#define CUDART_INF __builtin_inf()
#define CUDART_NAN_F __builtin_nanf("")
#define CUDART_NAN __builtin_nan("")

#define _CUPY_DEV __device__ __forceinline__

// Grid-stride loop over [0, n).
#define CUPY_FOR(i, n)                                                         \
  for (ptrdiff_t i = static_cast<ptrdiff_t>(blockIdx.x) * blockDim.x +          \
                     threadIdx.x;                                               \
       i < static_cast<ptrdiff_t>(n);                                           \
       i += static_cast<ptrdiff_t>(blockDim.x) * gridDim.x)

namespace cupy {
template <bool B, class T, class F> struct conditional { typedef T type; };
template <class T, class F> struct conditional<false, T, F> { typedef F type; };
template <typename T, typename U> struct is_same { static const bool value = false; };
template <typename T> struct is_same<T, T> { static const bool value = true; };
}  // namespace cupy

// ---------------------------------------------------------------------------
// float16: IEEE binary16 storage; arithmetic happens in float (one rounding
// per operation, round-to-nearest-even), which is also what NumPy's half
// loops do.
// ---------------------------------------------------------------------------
class float16 {
  _Float16 v_;

 public:
  _CUPY_DEV float16() {}
  _CUPY_DEV float16(float x) : v_(static_cast<_Float16>(x)) {}
  _CUPY_DEV float16(double x) : v_(static_cast<_Float16>(x)) {}
  _CUPY_DEV float16(_Float16 x) : v_(x) {}
  _CUPY_DEV float16(bool x) : v_(static_cast<_Float16>(x ? 1.0f : 0.0f)) {}
  _CUPY_DEV float16(signed char x) : v_(static_cast<_Float16>(static_cast<float>(x))) {}
  _CUPY_DEV float16(unsigned char x) : v_(static_cast<_Float16>(static_cast<float>(x))) {}
  _CUPY_DEV float16(short x) : v_(static_cast<_Float16>(static_cast<float>(x))) {}
  _CUPY_DEV float16(unsigned short x) : v_(static_cast<_Float16>(static_cast<float>(x))) {}
  _CUPY_DEV float16(int x) : v_(static_cast<_Float16>(x)) {}
  _CUPY_DEV float16(unsigned int x) : v_(static_cast<_Float16>(x)) {}
  _CUPY_DEV float16(long x) : v_(static_cast<_Float16>(x)) {}
  _CUPY_DEV float16(unsigned long x) : v_(static_cast<_Float16>(x)) {}
  _CUPY_DEV float16(long long x) : v_(static_cast<_Float16>(x)) {}
  _CUPY_DEV float16(unsigned long long x) : v_(static_cast<_Float16>(x)) {}

  _CUPY_DEV operator float() const { return static_cast<float>(v_); }
  _CUPY_DEV _Float16 raw() const { return v_; }

  _CUPY_DEV float16& operator+=(const float16& r) { *this = float16(float(*this) + float(r)); return *this; }
  _CUPY_DEV float16& operator-=(const float16& r) { *this = float16(float(*this) - float(r)); return *this; }
  _CUPY_DEV float16& operator*=(const float16& r) { *this = float16(float(*this) * float(r)); return *this; }
  _CUPY_DEV float16& operator/=(const float16& r) { *this = float16(float(*this) / float(r)); return *this; }
  _CUPY_DEV float16 operator-() const { return float16(-float(*this)); }
  _CUPY_DEV float16 operator+() const { return *this; }

  _CUPY_DEV unsigned short bits() const { return __builtin_bit_cast(unsigned short, v_); }
  _CUPY_DEV bool isnan() const { return (bits() & 0x7fffu) > 0x7c00u; }
  _CUPY_DEV bool isinf() const { return (bits() & 0x7fffu) == 0x7c00u; }
  _CUPY_DEV bool isfinite() const { return (bits() & 0x7c00u) != 0x7c00u; }
  _CUPY_DEV int signbit() const { return (bits() & 0x8000u) != 0; }
  _CUPY_DEV static float16 copysign(float16 x, float16 y) {
    unsigned short b = (x.bits() & 0x7fffu) | (y.bits() & 0x8000u);
    return float16(__builtin_bit_cast(_Float16, b));
  }
};

_CUPY_DEV float16 min(float16 x, float16 y) { return float16(fminf(float(x), float(y))); }
_CUPY_DEV float16 max(float16 x, float16 y) { return float16(fmaxf(float(x), float(y))); }
_CUPY_DEV bool isnan(float16 x) { return x.isnan(); }
_CUPY_DEV bool isinf(float16 x) { return x.isinf(); }
_CUPY_DEV bool isfinite(float16 x) { return x.isfinite(); }
_CUPY_DEV int signbit(float16 x) { return x.signbit(); }
_CUPY_DEV float16 copysign(float16 x, float16 y) { return float16::copysign(x, y); }

#include <cupy/complex.cuh>

// ---------------------------------------------------------------------------
// CArray: strided N-d view passed by value to a kernel.
//   data pointer, element count, shape[ndim], strides[ndim] (strides in bytes)
// `c_contiguous` lets operator[](i) skip the index decomposition;
// `use_32bit` selects 32-bit offset arithmetic.
// ---------------------------------------------------------------------------
template <typename T, int _ndim, bool _c_contiguous = false, bool _use_32bit = false>
class CArray {
 public:
  static const int ndim = _ndim;
  static const bool c_contiguous = _c_contiguous;
  typedef typename cupy::conditional<_use_32bit, int, ptrdiff_t>::type index_t;

 private:
  T* data_;
  ptrdiff_t size_;
  ptrdiff_t shape_[_ndim];
  ptrdiff_t strides_[_ndim];

 public:
  _CUPY_DEV ptrdiff_t size() const { return size_; }
  _CUPY_DEV const ptrdiff_t* shape() const { return shape_; }
  _CUPY_DEV const ptrdiff_t* strides() const { return strides_; }
  _CUPY_DEV T* data() const { return data_; }

  // Multi-dimensional index -> element.
  template <typename Int>
  _CUPY_DEV T& operator[](const Int (&idx)[_ndim]) {
    return *element_(idx);
  }
  template <typename Int>
  _CUPY_DEV const T& operator[](const Int (&idx)[_ndim]) const {
    return *element_(idx);
  }

  // Linear (C-order) index -> element.
  _CUPY_DEV T& operator[](ptrdiff_t i) { return *linear_(i); }
  _CUPY_DEV const T& operator[](ptrdiff_t i) const { return *linear_(i); }

 private:
  template <typename Int>
  _CUPY_DEV T* element_(const Int (&idx)[_ndim]) const {
    index_t off = 0;
#pragma unroll
    for (int d = 0; d < _ndim; ++d)
      off += static_cast<index_t>(strides_[d]) * static_cast<index_t>(idx[d]);
    return reinterpret_cast<T*>(reinterpret_cast<char*>(data_) + off);
  }

  _CUPY_DEV T* linear_(ptrdiff_t i) const {
    if (_c_contiguous) return data_ + i;
    index_t rest = static_cast<index_t>(i);
    index_t off = 0;
#pragma unroll
    for (int d = _ndim - 1; d > 0; --d) {
      index_t extent = static_cast<index_t>(shape_[d]);
      index_t q = rest / extent;
      off += static_cast<index_t>(strides_[d]) * (rest - q * extent);
      rest = q;
    }
    off += static_cast<index_t>(strides_[0]) * rest;
    return reinterpret_cast<T*>(reinterpret_cast<char*>(data_) + off);
  }
};

template <typename T, bool _c_contiguous, bool _use_32bit>
class CArray<T, 0, _c_contiguous, _use_32bit> {
  T* data_;
  ptrdiff_t size_;

 public:
  static const int ndim = 0;
  static const bool c_contiguous = true;
  typedef typename cupy::conditional<_use_32bit, int, ptrdiff_t>::type index_t;
  _CUPY_DEV ptrdiff_t size() const { return size_; }
  _CUPY_DEV const ptrdiff_t* shape() const { return 0; }
  _CUPY_DEV const ptrdiff_t* strides() const { return 0; }
  _CUPY_DEV T* data() const { return data_; }
  template <typename U> _CUPY_DEV T& operator[](const U&) { return *data_; }
  template <typename U> _CUPY_DEV const T& operator[](const U&) const { return *data_; }
};

// ---------------------------------------------------------------------------
// CIndexer: maps a linear C-order index to a multi-dimensional one.
// The kernel argument carries size and shape; the decomposed index is
// per-thread state filled in by set().
// ---------------------------------------------------------------------------
template <int _ndim, bool _use_32bit = false>
class CIndexer {
 public:
  static const int ndim = _ndim;
  typedef ptrdiff_t index_t[_ndim];

 private:
  ptrdiff_t size_;
  ptrdiff_t shape_[_ndim];
  ptrdiff_t index_[_ndim];

 public:
  _CUPY_DEV ptrdiff_t size() const { return size_; }
  _CUPY_DEV const ptrdiff_t* shape() const { return shape_; }
  _CUPY_DEV const index_t& get() const { return index_; }

  _CUPY_DEV void set(ptrdiff_t i) {
    if (_use_32bit) {
      unsigned int rest = static_cast<unsigned int>(i);
#pragma unroll
      for (int d = _ndim - 1; d > 0; --d) {
        unsigned int extent = static_cast<unsigned int>(shape_[d]);
        unsigned int q = rest / extent;
        index_[d] = rest - q * extent;
        rest = q;
      }
      index_[0] = rest;
    } else {
      ptrdiff_t rest = i;
#pragma unroll
      for (int d = _ndim - 1; d > 0; --d) {
        ptrdiff_t extent = shape_[d];
        ptrdiff_t q = rest / extent;
        index_[d] = rest - q * extent;
        rest = q;
      }
      index_[0] = rest;
    }
  }
};

template <bool _use_32bit>
class CIndexer<0, _use_32bit> {
  ptrdiff_t size_;

 public:
  static const int ndim = 0;
  _CUPY_DEV ptrdiff_t size() const { return size_; }
  _CUPY_DEV void set(ptrdiff_t) {}
  _CUPY_DEV const ptrdiff_t* get() const { return 0; }
};

// ---------------------------------------------------------------------------
// Floor division with Python/NumPy semantics (division by zero yields 0 for
// integers).
// ---------------------------------------------------------------------------
_CUPY_DEV int _floor_divide(int x, int y) {
  if (y == 0) return 0;
  int q = x / y;
  return q - (((x < 0) != (y < 0)) && q * y != x);
}
_CUPY_DEV long long _floor_divide(long long x, long long y) {
  if (y == 0) return 0;
  long long q = x / y;
  return q - (((x < 0) != (y < 0)) && q * y != x);
}
_CUPY_DEV unsigned _floor_divide(unsigned x, unsigned y) { return y == 0 ? 0u : x / y; }
_CUPY_DEV unsigned long long _floor_divide(unsigned long long x, unsigned long long y) {
  return y == 0 ? 0ull : x / y;
}
_CUPY_DEV float _floor_divide(float x, float y) { return floorf(x / y); }
_CUPY_DEV double _floor_divide(double x, double y) { return floor(x / y); }

// ---------------------------------------------------------------------------
// Vector access: N consecutive elements moved with the widest instructions the
// alignment allows (up to 16 bytes each, i.e. global_load/store_dwordx4).
// The pointer needs the alignment of one element only: the device takes wide
// accesses at any address, at full speed when it is a multiple of 4.
// ---------------------------------------------------------------------------
namespace cupy {

template <typename T, int N>
struct alignas((sizeof(T) * N > 16) ? 16 : sizeof(T) * N) Vec {
  T v[N];
};

typedef unsigned int _u32x4 __attribute__((ext_vector_type(4)));
typedef unsigned int _u32x2 __attribute__((ext_vector_type(2)));

template <int kBytes> struct _RawChunk;
template <> struct _RawChunk<16> { typedef _u32x4 type; };
template <> struct _RawChunk<8> { typedef _u32x2 type; };
template <> struct _RawChunk<4> { typedef unsigned int type; };
template <> struct _RawChunk<2> { typedef unsigned short type; };
template <> struct _RawChunk<1> { typedef unsigned char type; };

// kStream = true marks the access non-temporal (data touched once: do not
// keep it in cache at the expense of other lines).
template <typename T, int N, bool kStream = false>
_CUPY_DEV Vec<T, N> load_vec(const T* p) {
  constexpr int kTotal = sizeof(T) * N;
  constexpr int kChunk = kTotal > 16 ? 16 : kTotal;
  typedef typename _RawChunk<kChunk>::type raw_t;
  typedef raw_t __attribute__((aligned(alignof(T)))) raw_at_t;
  Vec<T, N> out;
  const raw_at_t* src = reinterpret_cast<const raw_at_t*>(p);
#pragma unroll
  for (int c = 0; c < kTotal / kChunk; ++c) {
    raw_t r = kStream ? __builtin_nontemporal_load(src + c) : src[c];
    __builtin_memcpy(reinterpret_cast<char*>(&out) + c * kChunk, &r, kChunk);
  }
  return out;
}

template <typename T, int N, bool kStream = false>
_CUPY_DEV void store_vec(T* p, const Vec<T, N>& x) {
  constexpr int kTotal = sizeof(T) * N;
  constexpr int kChunk = kTotal > 16 ? 16 : kTotal;
  typedef typename _RawChunk<kChunk>::type raw_t;
  typedef raw_t __attribute__((aligned(alignof(T)))) raw_at_t;
  raw_at_t* dst = reinterpret_cast<raw_at_t*>(p);
#pragma unroll
  for (int c = 0; c < kTotal / kChunk; ++c) {
    raw_t r;
    __builtin_memcpy(&r, reinterpret_cast<const char*>(&x) + c * kChunk, kChunk);
    if (kStream) __builtin_nontemporal_store(r, dst + c);
    else dst[c] = r;
  }
}

}  // namespace cupy

// Stand-in for a CIndexer in kernels that address their operands directly:
// only the element count is available (``_in_ind.size() / _out_ind.size()`` is
// how reduction post-maps ask for the number of reduced elements).
struct SizeOnly {
  ptrdiff_t size_;
  __device__ __forceinline__ explicit SizeOnly(ptrdiff_t n) : size_(n) {}
  __device__ __forceinline__ ptrdiff_t size() const { return size_; }
};

// ---------------------------------------------------------------------------
// Wave64 / workgroup reduction helpers.
// ---------------------------------------------------------------------------
namespace cupy {

// Exchange an arbitrary trivially copyable value with lane (lane ^ mask).
template <typename T>
_CUPY_DEV T shfl_xor(const T& v, int mask) {
  constexpr int kWords = (sizeof(T) + 3) / 4;
  int w[kWords] = {};
  __builtin_memcpy(w, &v, sizeof(T));
#pragma unroll
  for (int k = 0; k < kWords; ++k) w[k] = __shfl_xor(w[k], mask, 64);
  T r = v;
  __builtin_memcpy(&r, w, sizeof(T));
  return r;
}

// Value of lane (lane - delta) within groups of `kWidth` adjacent lanes; the
// first `delta` lanes of a group keep their own value.
template <int kWidth = 64, typename T>
_CUPY_DEV T shfl_up(const T& v, int delta) {
  constexpr int kWords = (sizeof(T) + 3) / 4;
  int w[kWords] = {};
  __builtin_memcpy(w, &v, sizeof(T));
#pragma unroll
  for (int k = 0; k < kWords; ++k) w[k] = __shfl_up(w[k], delta, kWidth);
  T r = v;
  __builtin_memcpy(&r, w, sizeof(T));
  return r;
}

// Value of lane `src` of the caller's group of `kWidth` adjacent lanes.
template <int kWidth = 64, typename T>
_CUPY_DEV T shfl_idx(const T& v, int src) {
  constexpr int kWords = (sizeof(T) + 3) / 4;
  int w[kWords] = {};
  __builtin_memcpy(w, &v, sizeof(T));
#pragma unroll
  for (int k = 0; k < kWords; ++k) w[k] = __shfl(w[k], src, kWidth);
  T r = v;
  __builtin_memcpy(&r, w, sizeof(T));
  return r;
}

// `c ? a : b` for a value of any trivially copyable type, word by word.  The
// conditional operator on a structure of more than two words is compiled into
// stores of both operands to scratch memory and a load through a selected
// address; words selected one by one stay in registers.
template <typename T>
_CUPY_DEV T select_value(bool c, const T& a, const T& b) {
  constexpr int kWords = (sizeof(T) + 3) / 4;
  unsigned wa[kWords] = {}, wb[kWords] = {};
  __builtin_memcpy(wa, &a, sizeof(T));
  __builtin_memcpy(wb, &b, sizeof(T));
#pragma unroll
  for (int k = 0; k < kWords; ++k) wa[k] = c ? wa[k] : wb[k];
  T r = b;
  __builtin_memcpy(&r, wa, sizeof(T));
  return r;
}

// One value moved between lanes by a data-parallel-primitive modifier
// (`kCtrl`: quad permutation, row mirror / half mirror, row rotation), word by
// word.  These run in the vector ALU; a general shuffle goes through the LDS
// crossbar.  Every one of these modifiers is a permutation within a row of 16
// lanes, so no lane ever lacks a source; saying that such a lane would read
// zero (the last argument) is what lets the compiler fold the move into the
// instruction that consumes it (one `v_add_f32 ... row_mirror` instead of
// two moves and an add).
template <int kCtrl, typename T>
_CUPY_DEV T _dpp_move(const T& v) {
  constexpr int kWords = (sizeof(T) + 3) / 4;
  int w[kWords] = {};
  __builtin_memcpy(w, &v, sizeof(T));
#pragma unroll
  for (int k = 0; k < kWords; ++k) w[k] = __builtin_amdgcn_update_dpp(0, w[k], kCtrl, 0xf, 0xf, true);
  T r = v;
  __builtin_memcpy(&r, w, sizeof(T));
  return r;
}

// Exchange of 16-lane rows (kMask == 16) or wave halves (kMask == 32): `lo`
// receives the value of the lower partner of every pair, `hi` that of the
// upper one, in both partners alike.
template <int kMask, typename T>
_CUPY_DEV void _swap_halves(const T& v, T& lo, T& hi) {
  constexpr int kWords = (sizeof(T) + 3) / 4;
  unsigned w[kWords] = {}, a[kWords], b[kWords];
  __builtin_memcpy(w, &v, sizeof(T));
#pragma unroll
  for (int k = 0; k < kWords; ++k) {
    if (kMask == 16) {
      auto r = __builtin_amdgcn_permlane16_swap(w[k], w[k], false, false);
      a[k] = r[0]; b[k] = r[1];
    } else {
      auto r = __builtin_amdgcn_permlane32_swap(w[k], w[k], false, false);
      a[k] = r[0]; b[k] = r[1];
    }
  }
  lo = v; hi = v;
  __builtin_memcpy(&lo, a, sizeof(T));
  __builtin_memcpy(&hi, b, sizeof(T));
}

// One step of an all-reduce over lanes: combines the caller's value with that
// of a partner lane chosen so that the steps for masks 1, 2, 4, ... together
// cover the same lanes as exchanges with (lane ^ mask) would.
//   kKeepLow == false: the group is reduced down to mask 1 (row reductions):
//     masks 1 and 2 permute within quads, 4 and 8 mirror half rows / rows.
//   kKeepLow == true: lanes that differ in their low bits must stay apart
//     (column reductions, masks tx .. 32): masks below 16 rotate within rows.
// Masks 16 and 32 swap rows / wave halves and apply `op` to the same pair of
// operands, in the same order, in both partners.  `op` must be commutative
// and associative.
template <int kMask, bool kKeepLow, typename T, typename Op>
_CUPY_DEV T xor_combine(const T& v, Op op) {
  if (kMask >= 16) {
    T lo, hi;
    _swap_halves<kMask>(v, lo, hi);
    return op(lo, hi);
  }
  if (kKeepLow) return op(v, _dpp_move<0x120 + kMask>(v));          // row_ror:kMask
  if (kMask == 1) return op(v, _dpp_move<0xB1>(v));                  // quad_perm [1,0,3,2]
  if (kMask == 2) return op(v, _dpp_move<0x4E>(v));                  // quad_perm [2,3,0,1]
  if (kMask == 4) return op(v, _dpp_move<0x141>(v));                 // row_half_mirror
  return op(v, _dpp_move<0x140>(v));                                 // row_mirror
}

template <int kMask, int kTop, bool kKeepLow> struct _AllReduce {
  template <typename T, typename Op>
  static _CUPY_DEV T run(T v, Op op) {
    return _AllReduce<kMask * 2, kTop, kKeepLow>::run(xor_combine<kMask, kKeepLow>(v, op), op);
  }
};
template <int kTop, bool kKeepLow> struct _AllReduce<kTop, kTop, kKeepLow> {
  template <typename T, typename Op>
  static _CUPY_DEV T run(T v, Op) { return v; }
};

// All-reduce over groups of `kGroup` adjacent lanes (power of two <= 64):
// every lane of a group ends up holding the group's reduction.
template <int kGroup, typename T, typename Op>
_CUPY_DEV T group_allreduce(T v, Op op) {
  return _AllReduce<1, kGroup, false>::run(v, op);
}

// All-reduce over the lanes that share (lane % kStride): masks kStride .. 32.
template <int kStride, typename T, typename Op>
_CUPY_DEV T strided_allreduce(T v, Op op) {
  return _AllReduce<kStride, 64, true>::run(v, op);
}

// kBatch independent all-reduces over groups of kGroup adjacent lanes, step by
// step side by side: the exchanges of one step do not wait for each other.
template <int kMask, int kTop> struct _BatchAllReduce {
  template <typename T, int kBatch, typename Op>
  static _CUPY_DEV void run(T (&s)[kBatch], Op op) {
#pragma unroll
    for (int r = 0; r < kBatch; ++r) s[r] = xor_combine<kMask, false>(s[r], op);
    _BatchAllReduce<kMask * 2, kTop>::run(s, op);
  }
};
template <int kTop> struct _BatchAllReduce<kTop, kTop> {
  template <typename T, int kBatch, typename Op>
  static _CUPY_DEV void run(T (&)[kBatch], Op) {}
};
template <int kGroup, typename T, int kBatch, typename Op>
_CUPY_DEV void batch_allreduce(T (&s)[kBatch], Op op) {
  _BatchAllReduce<1, kGroup>::run(s, op);
}

}  // namespace cupy
