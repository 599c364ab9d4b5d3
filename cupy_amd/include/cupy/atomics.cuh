// Atomic read-modify-write of one array element, for kernels in which several
// threads may update the same element (ufunc.at with repeated indices).
//
// cupy::atomic_update(p, f) replaces *p by f(*p) atomically for an element type
// of 1, 2, 4 or 8 bytes: a compare-and-swap loop on the aligned 32- or 64-bit
// word that holds the element (elements narrower than a word share theirs with
// neighbours, whose bytes are carried through unchanged).  The named
// operations use the hardware's own atomic instruction where gfx950 has one
// for the type (integer add / min / max / and / or / xor on 32 and 64 bits,
// float and double add) and the loop otherwise.
//
// Takes the place of cupy/_core/include/cupy/atomics.cuh in the reference
// (CUDA's atomicAdd overloads plus CAS fallbacks for float16 and 64-bit
// min/max); written for wave64 / gfx950, no CUDA intrinsics.
#pragma once

#include <cupy/carray.cuh>

namespace cupy {

template <int kBytes> struct _AtomicWord;
template <> struct _AtomicWord<4> { typedef unsigned int type; };
template <> struct _AtomicWord<8> { typedef unsigned long long type; };

// *p = f(*p) for an element that fills a whole 32- or 64-bit word
template <typename T, typename F>
_CUPY_DEV void _atomic_update_word(T* p, F f) {
  typedef typename _AtomicWord<sizeof(T)>::type word_t;
  word_t* wp = reinterpret_cast<word_t*>(p);
  word_t seen = __hip_atomic_load(wp, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  while (true) {
    T cur;
    __builtin_memcpy(&cur, &seen, sizeof(T));
    const T next = f(cur);
    word_t want;
    __builtin_memcpy(&want, &next, sizeof(T));
    if (want == seen) return;           // nothing to change (also ends NaN payload loops)
    if (__hip_atomic_compare_exchange_strong(wp, &seen, want, __ATOMIC_RELAXED,
                                             __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT))
      return;
  }
}

// the same for an element of 1 or 2 bytes inside its 32-bit word
template <typename T, typename F>
_CUPY_DEV void _atomic_update_part(T* p, F f) {
  const size_t address = reinterpret_cast<size_t>(p);
  unsigned int* wp = reinterpret_cast<unsigned int*>(address & ~size_t(3));
  const unsigned shift = static_cast<unsigned>(address & 3) * 8;
  const unsigned int mask = ((sizeof(T) == 1) ? 0xffu : 0xffffu) << shift;
  unsigned int seen = __hip_atomic_load(wp, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  while (true) {
    const unsigned int part = (seen & mask) >> shift;
    T cur;
    __builtin_memcpy(&cur, &part, sizeof(T));
    const T next = f(cur);
    unsigned int bits = 0;
    __builtin_memcpy(&bits, &next, sizeof(T));
    const unsigned int want = (seen & ~mask) | ((bits << shift) & mask);
    if (want == seen) return;
    if (__hip_atomic_compare_exchange_strong(wp, &seen, want, __ATOMIC_RELAXED,
                                             __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT))
      return;
  }
}

template <typename T, typename F>
_CUPY_DEV void atomic_update(T* p, F f) {
  if constexpr (sizeof(T) >= 4) {
    _atomic_update_word(p, f);
  } else {
    _atomic_update_part(p, f);
  }
}

// ---- named operations ----------------------------------------------------------

#define _CUPY_NATIVE_ATOMIC(NAME, T, BUILTIN)                                          \
  _CUPY_DEV void NAME(T* p, T v) {                                                      \
    (void)BUILTIN(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);                    \
  }

template <typename T> _CUPY_DEV void atomic_add(T* p, T v) {
  atomic_update(p, [v](T x) { return static_cast<T>(x + v); });
}
_CUPY_NATIVE_ATOMIC(atomic_add, int, __hip_atomic_fetch_add)
_CUPY_NATIVE_ATOMIC(atomic_add, unsigned int, __hip_atomic_fetch_add)
_CUPY_NATIVE_ATOMIC(atomic_add, long long, __hip_atomic_fetch_add)
_CUPY_NATIVE_ATOMIC(atomic_add, unsigned long long, __hip_atomic_fetch_add)
_CUPY_NATIVE_ATOMIC(atomic_add, float, __hip_atomic_fetch_add)
_CUPY_NATIVE_ATOMIC(atomic_add, double, __hip_atomic_fetch_add)
// complex values: the two parts are updated one after the other (an addition
// of complex numbers is two independent additions)
template <typename T> _CUPY_DEV void atomic_add(complex<T>* p, complex<T> v) {
  T* parts = reinterpret_cast<T*>(p);
  atomic_add(parts, v.real());
  atomic_add(parts + 1, v.imag());
}

template <typename T> _CUPY_DEV void atomic_sub(T* p, T v) {
  atomic_update(p, [v](T x) { return static_cast<T>(x - v); });
}
_CUPY_DEV void atomic_sub(int* p, int v) { atomic_add(p, static_cast<int>(0u - static_cast<unsigned>(v))); }
_CUPY_DEV void atomic_sub(unsigned int* p, unsigned int v) { atomic_add(p, 0u - v); }
_CUPY_DEV void atomic_sub(long long* p, long long v) {
  atomic_add(p, static_cast<long long>(0ull - static_cast<unsigned long long>(v)));
}
_CUPY_DEV void atomic_sub(unsigned long long* p, unsigned long long v) { atomic_add(p, 0ull - v); }
_CUPY_DEV void atomic_sub(float* p, float v) { atomic_add(p, -v); }
_CUPY_DEV void atomic_sub(double* p, double v) { atomic_add(p, -v); }
template <typename T> _CUPY_DEV void atomic_sub(complex<T>* p, complex<T> v) {
  atomic_add(p, complex<T>(-v.real(), -v.imag()));
}

// maximum / minimum as the ufuncs define them: a NaN operand wins
template <typename T> _CUPY_DEV T _nan_max(T x, T v) { return (x != x) ? x : ((v != v) ? v : (x < v ? v : x)); }
template <typename T> _CUPY_DEV T _nan_min(T x, T v) { return (x != x) ? x : ((v != v) ? v : (v < x ? v : x)); }
template <typename T> _CUPY_DEV void atomic_max(T* p, T v) {
  atomic_update(p, [v](T x) { return _nan_max(x, v); });
}
template <typename T> _CUPY_DEV void atomic_min(T* p, T v) {
  atomic_update(p, [v](T x) { return _nan_min(x, v); });
}
_CUPY_NATIVE_ATOMIC(atomic_max, int, __hip_atomic_fetch_max)
_CUPY_NATIVE_ATOMIC(atomic_max, unsigned int, __hip_atomic_fetch_max)
_CUPY_NATIVE_ATOMIC(atomic_max, long long, __hip_atomic_fetch_max)
_CUPY_NATIVE_ATOMIC(atomic_max, unsigned long long, __hip_atomic_fetch_max)
_CUPY_NATIVE_ATOMIC(atomic_min, int, __hip_atomic_fetch_min)
_CUPY_NATIVE_ATOMIC(atomic_min, unsigned int, __hip_atomic_fetch_min)
_CUPY_NATIVE_ATOMIC(atomic_min, long long, __hip_atomic_fetch_min)
_CUPY_NATIVE_ATOMIC(atomic_min, unsigned long long, __hip_atomic_fetch_min)

template <typename T> _CUPY_DEV void atomic_and(T* p, T v) {
  atomic_update(p, [v](T x) { return static_cast<T>(x & v); });
}
template <typename T> _CUPY_DEV void atomic_or(T* p, T v) {
  atomic_update(p, [v](T x) { return static_cast<T>(x | v); });
}
template <typename T> _CUPY_DEV void atomic_xor(T* p, T v) {
  atomic_update(p, [v](T x) { return static_cast<T>(x ^ v); });
}
_CUPY_DEV void atomic_and(bool* p, bool v) { atomic_update(p, [v](bool x) { return x && v; }); }
_CUPY_DEV void atomic_or(bool* p, bool v) { atomic_update(p, [v](bool x) { return x || v; }); }
_CUPY_DEV void atomic_xor(bool* p, bool v) { atomic_update(p, [v](bool x) { return x != v; }); }
_CUPY_NATIVE_ATOMIC(atomic_and, int, __hip_atomic_fetch_and)
_CUPY_NATIVE_ATOMIC(atomic_and, unsigned int, __hip_atomic_fetch_and)
_CUPY_NATIVE_ATOMIC(atomic_and, long long, __hip_atomic_fetch_and)
_CUPY_NATIVE_ATOMIC(atomic_and, unsigned long long, __hip_atomic_fetch_and)
_CUPY_NATIVE_ATOMIC(atomic_or, int, __hip_atomic_fetch_or)
_CUPY_NATIVE_ATOMIC(atomic_or, unsigned int, __hip_atomic_fetch_or)
_CUPY_NATIVE_ATOMIC(atomic_or, long long, __hip_atomic_fetch_or)
_CUPY_NATIVE_ATOMIC(atomic_or, unsigned long long, __hip_atomic_fetch_or)
_CUPY_NATIVE_ATOMIC(atomic_xor, int, __hip_atomic_fetch_xor)
_CUPY_NATIVE_ATOMIC(atomic_xor, unsigned int, __hip_atomic_fetch_xor)
_CUPY_NATIVE_ATOMIC(atomic_xor, long long, __hip_atomic_fetch_xor)
_CUPY_NATIVE_ATOMIC(atomic_xor, unsigned long long, __hip_atomic_fetch_xor)

#undef _CUPY_NATIVE_ATOMIC

}  // namespace cupy
