// complex<T> for generated kernels (T = float or double): storage-compatible
// with NumPy's complex64 / complex128 (real part first), arithmetic and the
// elementary functions by their textbook formulas on top of the device math
// library.  Counterpart of the reference's cupy/_core/include/cupy/complex.cuh
// and complex/*.h (a copy of thrust::complex there); this one is written for
// this package and keeps to what the ufunc loops use.
#pragma once

template <typename T>
struct alignas(2 * sizeof(T)) complex {
  T re, im;

  complex() = default;                     // trivial: usable in __shared__ arrays
  __device__ __forceinline__ complex(T r) : re(r), im(0) {}
  __device__ __forceinline__ complex(T r, T i) : re(r), im(i) {}
  template <typename U>
  __device__ __forceinline__ complex(const complex<U>& z)
      : re(static_cast<T>(z.re)), im(static_cast<T>(z.im)) {}

  __device__ __forceinline__ T real() const { return re; }
  __device__ __forceinline__ T imag() const { return im; }
  __device__ __forceinline__ void real(T r) { re = r; }
  __device__ __forceinline__ void imag(T i) { im = i; }

  __device__ __forceinline__ complex& operator+=(const complex& z) {
    re += z.re; im += z.im; return *this;
  }
  __device__ __forceinline__ complex& operator-=(const complex& z) {
    re -= z.re; im -= z.im; return *this;
  }
  __device__ __forceinline__ complex& operator*=(const complex& z) {
    const T r = fma(re, z.re, -(im * z.im));
    im = fma(re, z.im, im * z.re);
    re = r;
    return *this;
  }
  __device__ __forceinline__ complex& operator/=(const complex& z);
  // NumPy's truth value of a complex number
  __device__ __forceinline__ explicit operator bool() const { return re != 0 || im != 0; }
  // conversion to a real type keeps the real part (NumPy's unsafe cast)
  template <typename U>
  __device__ __forceinline__ explicit operator U() const { return static_cast<U>(re); }
};

template <typename T>
__device__ __forceinline__ complex<T> operator+(const complex<T>& a, const complex<T>& b) {
  return complex<T>(a.re + b.re, a.im + b.im);
}
template <typename T>
__device__ __forceinline__ complex<T> operator-(const complex<T>& a, const complex<T>& b) {
  return complex<T>(a.re - b.re, a.im - b.im);
}
// One product rounded, the other fused into the sum: what NumPy's vectorised
// complex multiply computes on hosts with fused multiply-add (multiply, then
// multiply-add/subtract), and one rounding closer to the exact result than
// the four-product formula.
template <typename T>
__device__ __forceinline__ complex<T> operator*(const complex<T>& a, const complex<T>& b) {
  return complex<T>(fma(a.re, b.re, -(a.im * b.im)), fma(a.re, b.im, a.im * b.re));
}
// Smith's algorithm, the way NumPy divides: scale by the larger component of
// the divisor so that intermediate products neither overflow nor underflow.
template <typename T>
__device__ __forceinline__ complex<T> operator/(const complex<T>& a, const complex<T>& b) {
  const T abr = b.re < 0 ? -b.re : b.re;
  const T abi = b.im < 0 ? -b.im : b.im;
  if (abr >= abi) {
    if (abr == 0 && abi == 0) return complex<T>(a.re / abr, a.im / abr);
    const T rat = b.im / b.re;
    const T scl = T(1) / (b.re + b.im * rat);
    return complex<T>((a.re + a.im * rat) * scl, (a.im - a.re * rat) * scl);
  }
  const T rat = b.re / b.im;
  const T scl = T(1) / (b.re * rat + b.im);
  return complex<T>((a.re * rat + a.im) * scl, (a.im * rat - a.re) * scl);
}
template <typename T>
__device__ __forceinline__ complex<T>& complex<T>::operator/=(const complex<T>& z) {
  *this = *this / z;
  return *this;
}
template <typename T>
__device__ __forceinline__ complex<T> operator+(const complex<T>& a, T b) { return complex<T>(a.re + b, a.im); }
template <typename T>
__device__ __forceinline__ complex<T> operator+(T a, const complex<T>& b) { return complex<T>(a + b.re, b.im); }
template <typename T>
__device__ __forceinline__ complex<T> operator-(const complex<T>& a, T b) { return complex<T>(a.re - b, a.im); }
template <typename T>
__device__ __forceinline__ complex<T> operator-(T a, const complex<T>& b) { return complex<T>(a - b.re, -b.im); }
template <typename T>
__device__ __forceinline__ complex<T> operator*(const complex<T>& a, T b) { return complex<T>(a.re * b, a.im * b); }
template <typename T>
__device__ __forceinline__ complex<T> operator*(T a, const complex<T>& b) { return complex<T>(a * b.re, a * b.im); }
template <typename T>
__device__ __forceinline__ complex<T> operator/(const complex<T>& a, T b) { return complex<T>(a.re / b, a.im / b); }
template <typename T>
__device__ __forceinline__ complex<T> operator/(T a, const complex<T>& b) { return complex<T>(a) / b; }
template <typename T>
__device__ __forceinline__ complex<T> operator+(const complex<T>& a) { return a; }
template <typename T>
__device__ __forceinline__ complex<T> operator-(const complex<T>& a) { return complex<T>(-a.re, -a.im); }
template <typename T>
__device__ __forceinline__ bool operator==(const complex<T>& a, const complex<T>& b) {
  return a.re == b.re && a.im == b.im;
}
template <typename T>
__device__ __forceinline__ bool operator!=(const complex<T>& a, const complex<T>& b) {
  return !(a == b);
}
template <typename T>
__device__ __forceinline__ bool operator==(const complex<T>& a, T b) { return a.re == b && a.im == 0; }
template <typename T>
__device__ __forceinline__ bool operator!=(const complex<T>& a, T b) { return !(a == b); }
// NumPy orders complex numbers lexicographically (real part first); a NaN
// imaginary part makes the comparison of the real parts false
template <typename T>
__device__ __forceinline__ bool operator<(const complex<T>& a, const complex<T>& b) {
  return (a.re < b.re && a.im == a.im && b.im == b.im) || (a.re == b.re && a.im < b.im);
}
template <typename T>
__device__ __forceinline__ bool operator>(const complex<T>& a, const complex<T>& b) { return b < a; }
template <typename T>
__device__ __forceinline__ bool operator<=(const complex<T>& a, const complex<T>& b) {
  return (a.re < b.re && a.im == a.im && b.im == b.im) || (a.re == b.re && a.im <= b.im);
}
template <typename T>
__device__ __forceinline__ bool operator>=(const complex<T>& a, const complex<T>& b) { return b <= a; }

template <typename T> __device__ __forceinline__ T real(const complex<T>& z) { return z.re; }
template <typename T> __device__ __forceinline__ T imag(const complex<T>& z) { return z.im; }
template <typename T> __device__ __forceinline__ complex<T> conj(const complex<T>& z) { return complex<T>(z.re, -z.im); }
template <typename T> __device__ __forceinline__ T norm(const complex<T>& z) { return z.re * z.re + z.im * z.im; }
template <typename T> __device__ __forceinline__ T abs(const complex<T>& z) { return hypot(z.re, z.im); }
template <typename T> __device__ __forceinline__ T arg(const complex<T>& z) { return atan2(z.im, z.re); }
template <typename T> __device__ __forceinline__ bool isnan(const complex<T>& z) { return isnan(z.re) || isnan(z.im); }
template <typename T> __device__ __forceinline__ bool isinf(const complex<T>& z) { return isinf(z.re) || isinf(z.im); }
template <typename T> __device__ __forceinline__ bool isfinite(const complex<T>& z) { return isfinite(z.re) && isfinite(z.im); }

template <typename T>
__device__ __forceinline__ complex<T> polar(T rho, T theta) {
  return complex<T>(rho * cos(theta), rho * sin(theta));
}
// exp(x) * (c, s) where exp(x) alone may overflow although the products do
// not: above the threshold the exponential is taken in two factors.
template <typename T>
__device__ __forceinline__ complex<T> _exp_times(T x, T c, T s) {
  const T big = sizeof(T) == 4 ? T(88) : T(709);
  if (x > big) {
    const T e1 = exp(x - big / 2);
    const T e2 = exp(big / 2);
    return complex<T>(e1 * c * e2, e1 * s * e2);
  }
  const T e = exp(x);
  return complex<T>(e * c, e * s);
}
template <typename T>
__device__ __forceinline__ complex<T> exp(const complex<T>& z) {
  if (z.im == 0) return complex<T>(exp(z.re), z.im);    // keeps inf + 0j from turning into NaN
  return _exp_times(z.re, cos(z.im), sin(z.im));
}
template <typename T>
__device__ __forceinline__ complex<T> log(const complex<T>& z) {
  const T ax = z.re < 0 ? -z.re : z.re;
  const T ay = z.im < 0 ? -z.im : z.im;
  const T m = ax > ay ? ax : ay;
  const T n = ax > ay ? ay : ax;
  T re;
  if (m > T(0.5) && m < T(2)) {
    // |z| near 1: log|z| = log1p(|z|^2 - 1) / 2 without forming |z|
    re = log1p((m - 1) * (m + 1) + n * n) / 2;
  } else {
    re = log(hypot(z.re, z.im));
  }
  return complex<T>(re, atan2(z.im, z.re));
}
// log(1 + z) without forming 1 + z: |1 + z|^2 - 1 = x (2 + x) + y^2
template <typename T>
__device__ __forceinline__ complex<T> log1p(const complex<T>& z) {
  const T ax = z.re < 0 ? -z.re : z.re;
  const T ay = z.im < 0 ? -z.im : z.im;
  if (ax > T(0.5) || ay > T(0.5)) return log(complex<T>(1 + z.re, z.im));
  return complex<T>(log1p(z.re * (2 + z.re) + z.im * z.im) / 2, atan2(z.im, 1 + z.re));
}
// exp(z) - 1 = expm1(x) cos y - 2 sin^2(y / 2) + i exp(x) sin y
template <typename T>
__device__ __forceinline__ complex<T> expm1(const complex<T>& z) {
  const T ax = z.re < 0 ? -z.re : z.re;
  if (ax > T(1)) {
    const complex<T> e = exp(z);
    return complex<T>(e.re - 1, e.im);
  }
  const T sh = sin(z.im / 2);
  return complex<T>(expm1(z.re) * cos(z.im) - 2 * sh * sh, exp(z.re) * sin(z.im));
}
// 2^z = exp(z log 2).  The rounded product z log 2 alone would cost |z| eps
// (at |z| = 30 some 30 eps): both components keep the rounding error of their
// product (from an fma) and the part of log 2 beyond its leading digits, and
// the error term is applied to first order, e^(x + d) = e^x (1 + d),
// cos(y + d) = cos y - d sin y, sin(y + d) = sin y + d cos y.
template <typename T>
__device__ __forceinline__ complex<T> exp2(const complex<T>& z) {
  if (z.im == 0) return complex<T>(exp2(z.re), z.im);
  const T ln2 = T(0.69314718055994530942);
  const T ln2_rest = sizeof(T) == 4 ? T(-1.904654299957767878541823431924e-9)
                                    : T(2.319046813846299616e-17);
  const T x = z.re * ln2;
  const T dx = fma(z.re, ln2, -x) + z.re * ln2_rest;
  const T y = z.im * ln2;
  const T dy = fma(z.im, ln2, -y) + z.im * ln2_rest;
  T c = cos(y), s = sin(y);
  if (isfinite(dx) && isfinite(dy)) {
    const T c1 = c - dy * s, s1 = s + dy * c;
    c = c1 + c1 * dx;
    s = s1 + s1 * dx;
  }
  return _exp_times(x, c, s);
}
template <typename T>
__device__ __forceinline__ complex<T> rint(const complex<T>& z) {
  return complex<T>(rint(z.re), rint(z.im));
}
template <typename T>
__device__ __forceinline__ complex<T> log10(const complex<T>& z) {
  return log(z) * T(0.43429448190325182765);
}
template <typename T>
__device__ __forceinline__ complex<T> log2(const complex<T>& z) {
  return log(z) * T(1.44269504088896340736);
}
template <typename T>
__device__ __forceinline__ complex<T> sqrt(const complex<T>& z) {
  if (z.re == 0 && z.im == 0) return complex<T>(0, z.im);
  const T m = hypot(z.re, z.im);
  // the component computed without cancellation first
  if (z.re >= 0) {
    const T r = sqrt((m + z.re) / 2);
    return complex<T>(r, z.im / (2 * r));
  }
  const T i = sqrt((m - z.re) / 2);
  // below the cut (negative real axis approached with im = -0) the root is -i|..|
  const bool below = __builtin_signbit(z.im);
  return complex<T>((below ? -z.im : z.im) / (2 * i), below ? -i : i);
}
template <typename T>
__device__ __forceinline__ complex<T> pow(const complex<T>& a, const complex<T>& b) {
  if (b.re == 0 && b.im == 0) return complex<T>(1, 0);
  if (a.re == 0 && a.im == 0) return (b.re > 0) ? complex<T>(0, 0) : complex<T>(__builtin_nan(""), __builtin_nan(""));
  return exp(b * log(a));
}
template <typename T>
__device__ __forceinline__ complex<T> pow(const complex<T>& a, T b) { return pow(a, complex<T>(b)); }
// (cosh x, sinh x) scaled so that neither overflows before it is multiplied by
// a sine or cosine: for large |x| both are exp(|x|) / 2.
template <typename T>
__device__ __forceinline__ complex<T> sinh(const complex<T>& z) {
  const T ax = z.re < 0 ? -z.re : z.re;
  if (ax > (sizeof(T) == 4 ? T(80) : T(700))) {
    const complex<T> h = _exp_times(ax, cos(z.im) / 2, sin(z.im) / 2);
    return complex<T>(z.re < 0 ? -h.re : h.re, h.im);
  }
  return complex<T>(sinh(z.re) * cos(z.im), cosh(z.re) * sin(z.im));
}
template <typename T>
__device__ __forceinline__ complex<T> cosh(const complex<T>& z) {
  const T ax = z.re < 0 ? -z.re : z.re;
  if (ax > (sizeof(T) == 4 ? T(80) : T(700))) {
    const complex<T> h = _exp_times(ax, cos(z.im) / 2, sin(z.im) / 2);
    return complex<T>(h.re, z.re < 0 ? -h.im : h.im);
  }
  return complex<T>(cosh(z.re) * cos(z.im), sinh(z.re) * sin(z.im));
}
template <typename T>
__device__ __forceinline__ complex<T> tanh(const complex<T>& z) {
  // Kahan's form: with t = tan y, b = 1 + t^2, s = sinh x, r = sqrt(1 + s^2),
  //   tanh(x + iy) = (b r s + i t) / (1 + b s^2),
  // which has no cancellation near the poles (x = 0, y = pi/2 + k pi).
  const T ax = z.re < 0 ? -z.re : z.re;
  if (ax > (sizeof(T) == 4 ? T(11) : T(22))) {
    // |tanh| is 1 to working precision; the imaginary part underflows to a
    // zero with the sign of sin(2y)
    const T e = exp(-2 * ax);
    return complex<T>(z.re > 0 ? T(1) : T(-1), 4 * sin(z.im) * cos(z.im) * e);
  }
  const T t = tan(z.im);
  const T b = 1 + t * t;
  const T sh = sinh(z.re);
  const T r = sqrt(1 + sh * sh);
  const T d = 1 + b * sh * sh;
  return complex<T>(b * r * sh / d, t / d);
}
template <typename T>
__device__ __forceinline__ complex<T> sin(const complex<T>& z) {
  // sin z = -i sinh(i z)
  const complex<T> t = sinh(complex<T>(-z.im, z.re));
  return complex<T>(t.im, -t.re);
}
template <typename T>
__device__ __forceinline__ complex<T> cos(const complex<T>& z) {
  // cos z = cosh(i z)
  return cosh(complex<T>(-z.im, z.re));
}
template <typename T>
__device__ __forceinline__ complex<T> tan(const complex<T>& z) {
  // tan z = -i tanh(i z)
  const complex<T> t = tanh(complex<T>(-z.im, z.re));
  return complex<T>(t.im, -t.re);
}
template <typename T>
__device__ __forceinline__ complex<T> asinh(const complex<T>& z) {
  // asinh is odd: work in the half plane Re z >= 0, where w = z + sqrt(1 + z^2)
  // adds parts of equal sign.  log w is taken as log1p(w - 1), with
  // w - 1 = z + z^2 / (sqrt(1 + z^2) + 1) formed without cancellation, so small
  // arguments keep their relative accuracy.
  const bool neg = z.re < 0 || (z.re == 0 && __builtin_signbit(z.re));
  const T x = neg ? -z.re : z.re;
  const T y = neg ? -z.im : z.im;
  const T ay = y < 0 ? -y : y;
  complex<T> r;
  if (x > (sizeof(T) == 4 ? T(1e18) : T(1e150)) || ay > (sizeof(T) == 4 ? T(1e18) : T(1e150))) {
    // z^2 would overflow: asinh z = log(2 z)
    const complex<T> l = log(complex<T>(x, y));
    r = complex<T>(l.re + T(0.69314718055994530942), l.im);
  } else {
    const complex<T> u(x * x - y * y, 2 * x * y);
    const complex<T> s = sqrt(complex<T>(1 + u.re, u.im));
    const complex<T> q = u / complex<T>(s.re + 1, s.im);
    const T dr = x + q.re;
    const T di = y + q.im;
    r = complex<T>(log1p(dr * (2 + dr) + di * di) / 2, atan2(di, 1 + dr));
  }
  return neg ? complex<T>(-r.re, -r.im) : r;
}
template <typename T>
__device__ __forceinline__ complex<T> acosh(const complex<T>& z) {
  // log(z + sqrt(z + 1) * sqrt(z - 1))
  const complex<T> s = sqrt(complex<T>(z.re + 1, z.im)) * sqrt(complex<T>(z.re - 1, z.im));
  return log(complex<T>(z.re + s.re, z.im + s.im));
}
template <typename T>
__device__ __forceinline__ complex<T> atanh(const complex<T>& z) {
  // atanh is odd: with x >= 0,
  //   Re = log1p(4x / ((1-x)^2 + y^2)) / 4, Im = atan2(2y, (1-x)(1+x) - y^2) / 2
  // (the argument of log1p is then >= 0, away from its singularity at -1)
  const bool neg = z.re < 0 || (z.re == 0 && __builtin_signbit(z.re));
  const T x = neg ? -z.re : z.re;
  const T y = neg ? -z.im : z.im;
  const T ay = y < 0 ? -y : y;
  complex<T> r;
  if (x > (sizeof(T) == 4 ? T(1e18) : T(1e150)) || ay > (sizeof(T) == 4 ? T(1e18) : T(1e150))) {
    // far from the origin atanh z -> 1/z +- i pi/2
    const complex<T> inv = complex<T>(1) / complex<T>(x, y);
    r = complex<T>(inv.re, y < 0 || (y == 0 && __builtin_signbit(y))
                               ? T(-1.57079632679489661923) : T(1.57079632679489661923));
  } else {
    r = complex<T>(log1p(4 * x / ((1 - x) * (1 - x) + y * y)) / 4,
                   atan2(2 * y, (1 - x) * (1 + x) - y * y) / 2);
  }
  return neg ? complex<T>(-r.re, -r.im) : r;
}
template <typename T>
__device__ __forceinline__ complex<T> asin(const complex<T>& z) {
  // asin z = -i asinh(i z)
  const complex<T> t = asinh(complex<T>(-z.im, z.re));
  return complex<T>(t.im, -t.re);
}
template <typename T>
__device__ __forceinline__ complex<T> acos(const complex<T>& z) {
  // pi/2 - asin z
  const complex<T> t = asin(z);
  return complex<T>(T(1.57079632679489661923) - t.re, -t.im);
}
template <typename T>
__device__ __forceinline__ complex<T> atan(const complex<T>& z) {
  // atan z = -i atanh(i z)
  const complex<T> t = atanh(complex<T>(-z.im, z.re));
  return complex<T>(t.im, -t.re);
}
