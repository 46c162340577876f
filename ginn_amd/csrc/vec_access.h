// Width-templated element access for the bandwidth-bound kernels: V = 8 moves
// eight consecutive elements with 16-byte memory operations (one for the
// 16-bit types, two for fp32), V = 1 is the scalar fallback for unaligned or
// odd-sized operands.
#ifndef GINN_HIP_VEC_ACCESS_H
#define GINN_HIP_VEC_ACCESS_H

#include "common.h"

namespace ginn_hip {

typedef uint32_t va_u32x4 __attribute__((ext_vector_type(4)));
typedef float va_f32x4 __attribute__((ext_vector_type(4)));

template <typename T, int V>
__device__ __forceinline__ void ld(const typename T::storage* p, float (&v)[V]) {
  if constexpr (V == 1) {
    v[0] = to_float<T>(p[0]);
  } else if constexpr (sizeof(typename T::storage) == 4 && V == 4) {
    const va_f32x4 q = *reinterpret_cast<const va_f32x4*>(p);
#pragma unroll
    for (int e = 0; e < 4; ++e) v[e] = q[e];
  } else if constexpr (sizeof(typename T::storage) == 4) {
    static_assert(V == 8, "vector width is 8");
    const va_f32x4 lo = *reinterpret_cast<const va_f32x4*>(p);
    const va_f32x4 hi = *reinterpret_cast<const va_f32x4*>(p + 4);
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      v[e] = lo[e];
      v[4 + e] = hi[e];
    }
  } else {
    static_assert(V == 8, "vector width is 8");
    const va_u32x4 raw = *reinterpret_cast<const va_u32x4*>(p);
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      v[2 * e] = to_float<T>(static_cast<uint16_t>(raw[e] & 0xffffu));
      v[2 * e + 1] = to_float<T>(static_cast<uint16_t>(raw[e] >> 16));
    }
  }
}

template <typename T, int V>
__device__ __forceinline__ void st(typename T::storage* p, const float (&v)[V]) {
  if constexpr (V == 1) {
    p[0] = from_float<T>(v[0]);
  } else if constexpr (sizeof(typename T::storage) == 4 && V == 4) {
    *reinterpret_cast<va_f32x4*>(p) = va_f32x4{v[0], v[1], v[2], v[3]};
  } else if constexpr (sizeof(typename T::storage) == 4) {
    va_f32x4 lo, hi;
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      lo[e] = v[e];
      hi[e] = v[4 + e];
    }
    *reinterpret_cast<va_f32x4*>(p) = lo;
    *reinterpret_cast<va_f32x4*>(p + 4) = hi;
  } else {
    va_u32x4 raw;
#pragma unroll
    for (int e = 0; e < 4; ++e)
      raw[e] = static_cast<uint32_t>(from_float<T>(v[2 * e])) |
               (static_cast<uint32_t>(from_float<T>(v[2 * e + 1])) << 16);
    *reinterpret_cast<va_u32x4*>(p) = raw;
  }
}

// All pointers 16-byte aligned and every extent in `extents` a multiple of 8.
inline bool vec8_ok(std::initializer_list<const void*> ptrs, std::initializer_list<size_t> extents) {
  for (const void* p : ptrs)
    if (p && reinterpret_cast<uintptr_t>(p) % 16) return false;
  for (size_t e : extents)
    if (e % 8) return false;
  return true;
}

}  // namespace ginn_hip

#endif  // GINN_HIP_VEC_ACCESS_H
