// bfloat16 for generated and user kernels: the upper 16 bits of an IEEE
// float32 (8 exponent bits, 7 stored mantissa bits).  Arithmetic goes through
// float; the conversion from float rounds to nearest, ties to even, and keeps
// NaNs quiet.  The interface follows the reference's device type
// (cupy/_core/include/cupy/bfloat16.cuh): construction from the numeric types,
// conversion to float, to_bits / from_bits, the classification functions,
// min / max / fmin / fmax, nextafter.  Include it after <cupy/carray.cuh>.
#pragma once

class bfloat16 {
 private:
  unsigned short bits_;

  static __device__ __forceinline__ unsigned short round_from(float v) {
    const unsigned int u = __builtin_bit_cast(unsigned int, v);
    if ((u & 0x7fffffffu) > 0x7f800000u) {            // NaN: keep it one, quiet
      return static_cast<unsigned short>((u >> 16) | 0x0040u);
    }
    const unsigned int bias = 0x7fffu + ((u >> 16) & 1u);
    return static_cast<unsigned short>((u + bias) >> 16);
  }

 public:
  __device__ bfloat16() : bits_(0) {}
  __device__ bfloat16(float v) : bits_(round_from(v)) {}
  explicit __device__ bfloat16(bool v) : bits_(round_from(float(v))) {}
  explicit __device__ bfloat16(double v) : bits_(round_from(float(v))) {}
  explicit __device__ bfloat16(int v) : bits_(round_from(float(v))) {}
  explicit __device__ bfloat16(unsigned int v) : bits_(round_from(float(v))) {}
  explicit __device__ bfloat16(long long v) : bits_(round_from(float(v))) {}
  explicit __device__ bfloat16(unsigned long long v) : bits_(round_from(float(v))) {}

  __device__ operator float() const {
    return __builtin_bit_cast(float, static_cast<unsigned int>(bits_) << 16);
  }

  template <typename T>
  __device__ bfloat16& operator=(const T& rhs) {
    bits_ = round_from(float(rhs));
    return *this;
  }
  bfloat16& operator=(const bfloat16&) = default;

  __device__ unsigned short to_bits() const { return bits_; }
  __device__ static bfloat16 from_bits(unsigned short v) {
    bfloat16 r;
    r.bits_ = v;
    return r;
  }

  __device__ int iszero() const { return (bits_ & 0x7fffu) == 0; }
  __device__ int isnan() const { return (bits_ & 0x7fffu) > 0x7f80u; }
  __device__ int isinf() const { return (bits_ & 0x7fffu) == 0x7f80u; }
  __device__ int isfinite() const { return (bits_ & 0x7f80u) != 0x7f80u; }
  __device__ int signbit() const { return (bits_ & 0x8000u) != 0; }
};

__device__ inline bfloat16 operator+(bfloat16 a, bfloat16 b) { return bfloat16(float(a) + float(b)); }
__device__ inline bfloat16 operator-(bfloat16 a, bfloat16 b) { return bfloat16(float(a) - float(b)); }
__device__ inline bfloat16 operator*(bfloat16 a, bfloat16 b) { return bfloat16(float(a) * float(b)); }
__device__ inline bfloat16 operator/(bfloat16 a, bfloat16 b) { return bfloat16(float(a) / float(b)); }
__device__ inline bfloat16 operator-(bfloat16 a) { return bfloat16::from_bits(a.to_bits() ^ 0x8000u); }
__device__ inline bfloat16& operator+=(bfloat16& a, bfloat16 b) { a = a + b; return a; }
__device__ inline bfloat16& operator-=(bfloat16& a, bfloat16 b) { a = a - b; return a; }
__device__ inline bfloat16& operator*=(bfloat16& a, bfloat16 b) { a = a * b; return a; }
__device__ inline bfloat16& operator/=(bfloat16& a, bfloat16 b) { a = a / b; return a; }
__device__ inline bool operator==(bfloat16 a, bfloat16 b) { return float(a) == float(b); }
__device__ inline bool operator!=(bfloat16 a, bfloat16 b) { return float(a) != float(b); }
__device__ inline bool operator<(bfloat16 a, bfloat16 b) { return float(a) < float(b); }
__device__ inline bool operator<=(bfloat16 a, bfloat16 b) { return float(a) <= float(b); }
__device__ inline bool operator>(bfloat16 a, bfloat16 b) { return float(a) > float(b); }
__device__ inline bool operator>=(bfloat16 a, bfloat16 b) { return float(a) >= float(b); }

// NaN propagates through min / max and loses against numbers in fmin / fmax
__device__ inline bfloat16 min(bfloat16 x, bfloat16 y) {
  return (x.isnan() || y.isnan()) ? (x.isnan() ? x : y) : (float(x) < float(y) ? x : y);
}
__device__ inline bfloat16 max(bfloat16 x, bfloat16 y) {
  return (x.isnan() || y.isnan()) ? (x.isnan() ? x : y) : (float(x) > float(y) ? x : y);
}
__device__ inline bfloat16 fmin(bfloat16 x, bfloat16 y) {
  return x.isnan() ? y : (y.isnan() ? x : (float(x) < float(y) ? x : y));
}
__device__ inline bfloat16 fmax(bfloat16 x, bfloat16 y) {
  return x.isnan() ? y : (y.isnan() ? x : (float(x) > float(y) ? x : y));
}
__device__ inline int iszero(bfloat16 x) { return x.iszero(); }
__device__ inline int isnan(bfloat16 x) { return x.isnan(); }
__device__ inline int isinf(bfloat16 x) { return x.isinf(); }
__device__ inline int isfinite(bfloat16 x) { return x.isfinite(); }
__device__ inline int signbit(bfloat16 x) { return x.signbit(); }

__device__ inline bfloat16 _floor_divide(bfloat16 x, bfloat16 y) {
  return bfloat16(_floor_divide(float(x), float(y)));
}

// the neighbour of x in the direction of y, stepping through the 16-bit patterns
__device__ inline bfloat16 nextafter(bfloat16 x, bfloat16 y) {
  if (x.isnan() || y.isnan()) return bfloat16::from_bits(0x7fc0u);
  if (float(x) == float(y)) return y;
  unsigned short b = x.to_bits();
  if (x.iszero()) return bfloat16::from_bits((y.to_bits() & 0x8000u) | 1u);
  const bool up = (float(x) < float(y)) == !(b & 0x8000u);
  b = up ? b + 1 : b - 1;
  return bfloat16::from_bits(b);
}
