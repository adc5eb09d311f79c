// 16-bit storage types and their conversions (device and host).
#ifndef PHIP_TYPES_H_
#define PHIP_TYPES_H_

#include <hip/hip_runtime.h>

#include <cstdint>

namespace phip {

typedef _Float16 f16_t;

// bfloat16 kept as its bit pattern; arithmetic always happens in fp32.
struct bf16_t {
  uint16_t bits;
};

__host__ __device__ inline float to_f32(float x) { return x; }
__host__ __device__ inline float to_f32(f16_t x) { return static_cast<float>(x); }
__host__ __device__ inline float to_f32(bf16_t x) {
  return __builtin_bit_cast(float, static_cast<uint32_t>(x.bits) << 16);
}

template <typename T>
__host__ __device__ inline T from_f32(float x);

template <>
__host__ __device__ inline float from_f32<float>(float x) {
  return x;
}

// Round to nearest even (the conversion's default rounding).
template <>
__host__ __device__ inline f16_t from_f32<f16_t>(float x) {
  return static_cast<f16_t>(x);
}

template <>
__host__ __device__ inline bf16_t from_f32<bf16_t>(float x) {
  uint32_t u = __builtin_bit_cast(uint32_t, x);
  bf16_t r;
  if ((u & 0x7fffffffu) > 0x7f800000u) {  // NaN stays NaN
    r.bits = static_cast<uint16_t>((u >> 16) | 0x0040u);
  } else {
    u += 0x7fffu + ((u >> 16) & 1u);  // round to nearest even
    r.bits = static_cast<uint16_t>(u >> 16);
  }
  return r;
}

}  // namespace phip

#endif  // PHIP_TYPES_H_
