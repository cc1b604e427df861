// Device helpers shared by the gfx950 kernels: storage types, 64-lane wave
// reductions, block reductions.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace kvc {

constexpr int kWave = 64;

// bfloat16 as stored in memory.  Conversions are written out so that rounding is
// the same everywhere: to float is exact, from float rounds to nearest even.
struct bf16_t {
  uint16_t bits;
};

__device__ __forceinline__ float to_float(float x) { return x; }
__device__ __forceinline__ float to_float(bf16_t x) {
  return __uint_as_float(static_cast<uint32_t>(x.bits) << 16);
}

__device__ __forceinline__ uint16_t f32_to_bf16_bits(float f) {
  uint32_t u = __float_as_uint(f);
  if ((u & 0x7fffffffu) > 0x7f800000u) return static_cast<uint16_t>((u >> 16) | 0x0040u);  // NaN
  u += 0x7fffu + ((u >> 16) & 1u);
  return static_cast<uint16_t>(u >> 16);
}

template <typename T>
__device__ __forceinline__ T from_float(float x);
template <>
__device__ __forceinline__ float from_float<float>(float x) { return x; }
template <>
__device__ __forceinline__ bf16_t from_float<bf16_t>(float x) {
  bf16_t r;
  r.bits = f32_to_bf16_bits(x);
  return r;
}

// One rotary pair (x0, x1) turned by the angle whose cosine and sine are c and s:
// (x0 c - x1 s, x1 c + x0 s), each as one product and one fused multiply-add, so that every
// kernel that rotates gives the same bits.
__device__ __forceinline__ float rotate_first(float x0, float x1, float c, float s) {
  return __builtin_fmaf(-x1, s, x0 * c);
}
__device__ __forceinline__ float rotate_second(float x0, float x1, float c, float s) {
  return __builtin_fmaf(x0, s, x1 * c);
}

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int o = kWave / 2; o > 0; o >>= 1) v += __shfl_xor(v, o, kWave);
  return v;
}

__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
  for (int o = kWave / 2; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, kWave));
  return v;
}

// Sum over a block of up to 1024 threads; every thread gets the result.  The order
// of the additions is fixed by the block size alone.
__device__ __forceinline__ float block_sum(float v, float* scratch /* >= 16 floats in LDS */) {
  const int lane = threadIdx.x & (kWave - 1);
  const int wave = threadIdx.x / kWave;
  const int nwaves = (blockDim.x + kWave - 1) / kWave;
  v = wave_sum(v);
  __syncthreads();
  if (lane == 0) scratch[wave] = v;
  __syncthreads();
  float total = 0.f;
  for (int w = 0; w < nwaves; ++w) total += scratch[w];
  return total;
}

}  // namespace kvc

// Dispatch on the storage type code of the C interface: 0 = float32, 1 = bfloat16.
#define KVC_DISPATCH_DTYPE(code, T, ...)        \
  do {                                          \
    if ((code) == 0) {                          \
      using T = float;                          \
      __VA_ARGS__;                              \
    } else if ((code) == 1) {                   \
      using T = kvc::bf16_t;                    \
      __VA_ARGS__;                              \
    } else {                                    \
      return kvc_fail("unknown dtype code");    \
    }                                           \
  } while (0)

// Every entry point returns 0 on success, or a negative code after recording a
// message that kvc_last_error() returns.
int kvc_fail(const char* message);
int kvc_check_launch(const char* what);
// Compute units of the current device (asked of the runtime once per device; 256, an MI355X's,
// if it will not say).  Launch plans count blocks against this, not against a constant.
int kvc_device_compute_units(void);
// Kernel families that have several variants to choose from at launch.  The entry points note
// which one they launched (kvc_note_variant), and kvc_last_variant() tells the caller's thread:
// for tests and tuning that must know which code ran.
enum { kVariantPrefillAttention = 0, kVariantRopeKvWrite = 1, kVariantDecodeAttention = 2, kVariantFamilies = 3 };
void kvc_note_variant(int family, const char* name);
