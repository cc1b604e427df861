// Operand vectors of the bfloat16 matrix instructions and guarded stores of four results,
// shared by the weight-streaming products.
#pragma once

#include <hip/hip_runtime.h>

#include <cstdint>

#include "device_utils.h"

namespace kvc {

typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef float f32x4_t __attribute__((ext_vector_type(4)));

__device__ __forceinline__ bf16x8_t zero8() {
  bf16x8_t z;
#pragma unroll
  for (int e = 0; e < 8; ++e) z[e] = static_cast<__bf16>(0.f);
  return z;
}

template <typename OutT>
__device__ __forceinline__ void store4(OutT* p, f32x4_t v, int n_left);
template <>
__device__ __forceinline__ void store4<float>(float* p, f32x4_t v, int n_left) {
  if (n_left >= 4 && (reinterpret_cast<uintptr_t>(p) & 15) == 0) {
    *reinterpret_cast<f32x4_t*>(p) = v;
  } else {
    for (int i = 0; i < 4 && i < n_left; ++i) p[i] = v[i];
  }
}
template <>
__device__ __forceinline__ void store4<bf16_t>(bf16_t* p, f32x4_t v, int n_left) {
  if (n_left >= 4 && (reinterpret_cast<uintptr_t>(p) & 7) == 0) {
    uint2 packed;
    packed.x = f32_to_bf16_bits(v[0]) | (static_cast<uint32_t>(f32_to_bf16_bits(v[1])) << 16);
    packed.y = f32_to_bf16_bits(v[2]) | (static_cast<uint32_t>(f32_to_bf16_bits(v[3])) << 16);
    *reinterpret_cast<uint2*>(p) = packed;
  } else {
    for (int i = 0; i < 4 && i < n_left; ++i) p[i].bits = f32_to_bf16_bits(v[i]);
  }
}

}  // namespace kvc
