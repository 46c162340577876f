// Scalar and index types of the host layer (ginn/def.h:31-39).
//
// Half and BFloat16 are 16-bit storage types with float conversion; they are
// bit-compatible with what the device kernels read (IEEE binary16, and the
// upper half of an IEEE binary32).  BFloat16 has no counterpart in the
// reference.  GINN_ENABLE_GPU is always on: this build has a single code path.
#ifndef GINN_DEF_H
#define GINN_DEF_H

#include <cmath>
#include <cstdint>
#include <cstring>
#include <vector>

#include "ginn_hip.h"

#include <ginn/except.h>

#ifndef GINN_ENABLE_GPU
#define GINN_ENABLE_GPU
#endif

namespace ginn {

using Real = float;
using Int = int;
using Size = long;
using Shape = std::vector<Size>;

namespace detail {

inline uint32_t f32_bits(float f) {
  uint32_t u;
  std::memcpy(&u, &f, 4);
  return u;
}
inline float bits_f32(uint32_t u) {
  float f;
  std::memcpy(&f, &u, 4);
  return f;
}

// float -> binary16, round to nearest even.
inline uint16_t f32_to_f16(float f) {
  const uint32_t x = f32_bits(f);
  const uint32_t sign = (x >> 16) & 0x8000u;
  const uint32_t abs = x & 0x7fffffffu;
  if (abs >= 0x7f800000u) return sign | (abs > 0x7f800000u ? 0x7e00u : 0x7c00u);
  if (abs >= 0x477ff000u) return sign | 0x7c00u;  // rounds to infinity
  if (abs < 0x33000001u) return sign;             // rounds to zero
  int exp = static_cast<int>(abs >> 23) - 127;
  uint32_t mant = (abs & 0x7fffffu) | 0x800000u;
  int shift;
  uint32_t base;
  if (exp < -14) {  // subnormal result
    shift = 13 + (-14 - exp);
    base = 0;
  } else {
    shift = 13;
    base = static_cast<uint32_t>(exp + 15) << 10;
    mant &= 0x7fffffu;
  }
  uint32_t half = mant >> shift;
  const uint32_t rem = mant & ((1u << shift) - 1u), mid = 1u << (shift - 1);
  if (rem > mid || (rem == mid && (half & 1u))) ++half;
  return sign | (base + half);
}

inline float f16_to_f32(uint16_t h) {
  const uint32_t sign = static_cast<uint32_t>(h & 0x8000u) << 16;
  const uint32_t exp = (h >> 10) & 0x1fu, mant = h & 0x3ffu;
  if (exp == 0x1f) return bits_f32(sign | 0x7f800000u | (mant << 13));
  if (exp == 0) {
    if (mant == 0) return bits_f32(sign);
    const float v = std::ldexp(static_cast<float>(mant), -24);
    return sign ? -v : v;
  }
  return bits_f32(sign | ((exp + 112u) << 23) | (mant << 13));
}

inline uint16_t f32_to_bf16(float f) {
  uint32_t u = f32_bits(f);
  if ((u & 0x7fffffffu) > 0x7f800000u) return static_cast<uint16_t>((u >> 16) | 0x40u);
  u += 0x7fffu + ((u >> 16) & 1u);
  return static_cast<uint16_t>(u >> 16);
}

}  // namespace detail

struct Half {
  uint16_t bits = 0;
  Half() = default;
  Half(float f) : bits(detail::f32_to_f16(f)) {}
  Half(double f) : bits(detail::f32_to_f16(static_cast<float>(f))) {}
  Half(int i) : bits(detail::f32_to_f16(static_cast<float>(i))) {}
  operator float() const { return detail::f16_to_f32(bits); }
};

struct BFloat16 {
  uint16_t bits = 0;
  BFloat16() = default;
  BFloat16(float f) : bits(detail::f32_to_bf16(f)) {}
  BFloat16(double f) : bits(detail::f32_to_bf16(static_cast<float>(f))) {}
  BFloat16(int i) : bits(detail::f32_to_bf16(static_cast<float>(i))) {}
  operator float() const { return detail::bits_f32(static_cast<uint32_t>(bits) << 16); }
};

static_assert(sizeof(Half) == 2 && sizeof(BFloat16) == 2, "16-bit storage types");

template <typename Scalar>
struct is_floating_point : std::false_type {};
template <>
struct is_floating_point<float> : std::true_type {};
template <>
struct is_floating_point<Half> : std::true_type {};
template <>
struct is_floating_point<BFloat16> : std::true_type {};
template <typename Scalar>
inline constexpr bool is_floating_point_v = is_floating_point<Scalar>::value;

// Device dtype code of a floating-point Scalar.
template <typename Scalar>
inline ginn_hip_dtype dtype_of() {
  static_assert(is_floating_point_v<Scalar>, "device arithmetic exists for Real, Half and BFloat16 only");
  if constexpr (std::is_same_v<Scalar, float>) return GINN_HIP_F32;
  if constexpr (std::is_same_v<Scalar, Half>) return GINN_HIP_F16;
  return GINN_HIP_BF16;
}

// The same for the nodes that exist on Int as well (ginn/node/common.h: Add, Subtract, the scalar forms,
// CwiseProd, CwiseProdAdd, CwiseMax): their forward passes take GINN_HIP_I32, exact integer arithmetic;
// Int nodes carry no gradient.
template <typename Scalar>
inline ginn_hip_dtype arith_dtype_of() {
  if constexpr (std::is_same_v<Scalar, Int>) return GINN_HIP_I32;
  else return dtype_of<Scalar>();
}

namespace literals {
inline Real operator"" _r(long double x) { return static_cast<Real>(x); }
inline Real operator"" _r(unsigned long long x) { return static_cast<Real>(x); }
inline Half operator"" _h(long double x) { return Half(static_cast<float>(x)); }
inline Half operator"" _h(unsigned long long x) { return Half(static_cast<float>(x)); }
}  // namespace literals

}  // namespace ginn

#endif  // GINN_DEF_H
