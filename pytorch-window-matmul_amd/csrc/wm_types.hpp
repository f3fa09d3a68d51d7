// Storage types and conversions used by every kernel family.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace wm {

struct bf16_t {
  uint16_t bits;
};
typedef _Float16 f16_t;

template <typename T>
struct Acc {
  typedef float type;
};
template <>
struct Acc<double> {
  typedef double type;
};

__device__ __forceinline__ float bf16_bits_to_float(uint32_t bits) { return __uint_as_float(bits << 16); }

// Round to nearest even; NaN stays NaN (quiet), Inf stays Inf.
__device__ __forceinline__ uint32_t float_to_bf16_bits(float f) {
  uint32_t u = __float_as_uint(f);
  if ((u & 0x7fffffffu) > 0x7f800000u) return (u >> 16) | 0x40u;
  u += 0x7fffu + ((u >> 16) & 1u);
  return u >> 16;
}

template <typename T>
__device__ __forceinline__ typename Acc<T>::type to_acc(T v);
template <>
__device__ __forceinline__ float to_acc<float>(float v) { return v; }
template <>
__device__ __forceinline__ double to_acc<double>(double v) { return v; }
template <>
__device__ __forceinline__ float to_acc<f16_t>(f16_t v) { return (float)v; }
template <>
__device__ __forceinline__ float to_acc<bf16_t>(bf16_t v) { return bf16_bits_to_float(v.bits); }

template <typename T>
__device__ __forceinline__ T from_acc(typename Acc<T>::type v);
template <>
__device__ __forceinline__ float from_acc<float>(float v) { return v; }
template <>
__device__ __forceinline__ double from_acc<double>(double v) { return v; }
template <>
__device__ __forceinline__ f16_t from_acc<f16_t>(float v) { return (f16_t)v; }
template <>
__device__ __forceinline__ bf16_t from_acc<bf16_t>(float v) {
  bf16_t r;
  r.bits = (uint16_t)float_to_bf16_bits(v);
  return r;
}

}  // namespace wm
