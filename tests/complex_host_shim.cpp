// Host build of the device header cupy/complex.cuh: the __device__ markers are
// defined away so that g++ compiles the same formulas against the host math
// library.  tests/test_complex_functions_host.py loads the result and compares
// every function with NumPy.
#include <cmath>
using namespace std;
#define __device__
#define __forceinline__ inline
#include "cupy/complex.cuh"
#define UN(name, fn) \
  extern "C" void c64_##name(const float* in, float* out, int n) { \
    for (int i = 0; i < n; ++i) { complex<float> z(in[2*i], in[2*i+1]); complex<float> r = fn(z); out[2*i] = r.re; out[2*i+1] = r.im; } } \
  extern "C" void c128_##name(const double* in, double* out, int n) { \
    for (int i = 0; i < n; ++i) { complex<double> z(in[2*i], in[2*i+1]); complex<double> r = fn(z); out[2*i] = r.re; out[2*i+1] = r.im; } }
UN(sqrt, sqrt) UN(exp, exp) UN(log, log) UN(log2, log2) UN(log10, log10) UN(sin, sin) UN(cos, cos) UN(tan, tan)
UN(sinh, sinh) UN(cosh, cosh) UN(tanh, tanh) UN(arcsin, asin) UN(arccos, acos) UN(arctan, atan)
UN(arcsinh, asinh) UN(arccosh, acosh) UN(arctanh, atanh)
UN(log1p, log1p) UN(expm1, expm1) UN(exp2, exp2)
#define BIN(name, expr) \
  extern "C" void c64_##name(const float* a_, const float* b_, float* out, int n) { \
    for (int i = 0; i < n; ++i) { complex<float> a(a_[2*i], a_[2*i+1]), b(b_[2*i], b_[2*i+1]); complex<float> r = expr; out[2*i] = r.re; out[2*i+1] = r.im; } } \
  extern "C" void c128_##name(const double* a_, const double* b_, double* out, int n) { \
    for (int i = 0; i < n; ++i) { complex<double> a(a_[2*i], a_[2*i+1]), b(b_[2*i], b_[2*i+1]); complex<double> r = expr; out[2*i] = r.re; out[2*i+1] = r.im; } }
BIN(multiply, a * b) BIN(divide, a / b) BIN(power, pow(a, b))
