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
    const T r = re * z.re - im * z.im;
    im = re * z.im + im * z.re;
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
template <typename T>
__device__ __forceinline__ complex<T> operator*(const complex<T>& a, const complex<T>& b) {
  return complex<T>(a.re * b.re - a.im * b.im, a.re * b.im + a.im * b.re);
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
template <typename T>
__device__ __forceinline__ complex<T> exp(const complex<T>& z) {
  const T e = exp(z.re);
  if (z.im == 0) return complex<T>(e, z.im);          // keeps inf + 0j from turning into NaN
  return complex<T>(e * cos(z.im), e * sin(z.im));
}
template <typename T>
__device__ __forceinline__ complex<T> log(const complex<T>& z) {
  return complex<T>(log(hypot(z.re, z.im)), atan2(z.im, z.re));
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
  return complex<T>((z.im < 0 ? -z.im : z.im) / (2 * i), z.im < 0 ? -i : i);
}
template <typename T>
__device__ __forceinline__ complex<T> pow(const complex<T>& a, const complex<T>& b) {
  if (b.re == 0 && b.im == 0) return complex<T>(1, 0);
  if (a.re == 0 && a.im == 0) return (b.re > 0) ? complex<T>(0, 0) : complex<T>(__builtin_nan(""), __builtin_nan(""));
  return exp(b * log(a));
}
template <typename T>
__device__ __forceinline__ complex<T> pow(const complex<T>& a, T b) { return pow(a, complex<T>(b)); }
template <typename T>
__device__ __forceinline__ complex<T> sinh(const complex<T>& z) {
  return complex<T>(sinh(z.re) * cos(z.im), cosh(z.re) * sin(z.im));
}
template <typename T>
__device__ __forceinline__ complex<T> cosh(const complex<T>& z) {
  return complex<T>(cosh(z.re) * cos(z.im), sinh(z.re) * sin(z.im));
}
template <typename T>
__device__ __forceinline__ complex<T> tanh(const complex<T>& z) {
  // tanh(x + iy) = (sinh 2x + i sin 2y) / (cosh 2x + cos 2y)
  const T tx = 2 * z.re, ty = 2 * z.im;
  if (tx > 40 || tx < -40) return complex<T>(tx > 0 ? 1 : -1, 0);     // cosh would overflow
  const T d = cosh(tx) + cos(ty);
  return complex<T>(sinh(tx) / d, sin(ty) / d);
}
template <typename T>
__device__ __forceinline__ complex<T> sin(const complex<T>& z) {
  return complex<T>(sin(z.re) * cosh(z.im), cos(z.re) * sinh(z.im));
}
template <typename T>
__device__ __forceinline__ complex<T> cos(const complex<T>& z) {
  return complex<T>(cos(z.re) * cosh(z.im), -sin(z.re) * sinh(z.im));
}
template <typename T>
__device__ __forceinline__ complex<T> tan(const complex<T>& z) {
  // tan z = -i tanh(i z)
  const complex<T> t = tanh(complex<T>(-z.im, z.re));
  return complex<T>(t.im, -t.re);
}
template <typename T>
__device__ __forceinline__ complex<T> asinh(const complex<T>& z) {
  // log(z + sqrt(z*z + 1))
  const complex<T> s = sqrt(complex<T>(z.re * z.re - z.im * z.im + 1, 2 * z.re * z.im));
  return log(complex<T>(z.re + s.re, z.im + s.im));
}
template <typename T>
__device__ __forceinline__ complex<T> acosh(const complex<T>& z) {
  // log(z + sqrt(z + 1) * sqrt(z - 1))
  const complex<T> s = sqrt(complex<T>(z.re + 1, z.im)) * sqrt(complex<T>(z.re - 1, z.im));
  return log(complex<T>(z.re + s.re, z.im + s.im));
}
template <typename T>
__device__ __forceinline__ complex<T> atanh(const complex<T>& z) {
  // (log(1 + z) - log(1 - z)) / 2
  const complex<T> a = log(complex<T>(1 + z.re, z.im));
  const complex<T> b = log(complex<T>(1 - z.re, -z.im));
  return complex<T>((a.re - b.re) / 2, (a.im - b.im) / 2);
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
