// Two kernels that only measure the chip: how fast it reads memory when a kernel does nothing
// else, and how fast its matrix cores run when their operands are already in registers.  The
// benchmark prices its steps against the data sheet's peaks and, beside them, against these.

#include <hip/hip_runtime.h>

#include "device_utils.h"
#include "kvcore_hip.h"

using namespace kvc;

namespace {

typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef float f32x16_t __attribute__((ext_vector_type(16)));

// 16-byte loads, four in flight a thread, nothing stored (the condition practically never holds)
__global__ __launch_bounds__(256) void read_only_kernel(const uint4* __restrict__ p, int64_t n16,
                                                        uint32_t* __restrict__ sink) {
  const int64_t stride = static_cast<int64_t>(gridDim.x) * 256;
  int64_t i = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x;
  uint32_t acc = 0;
  for (; i + 3 * stride < n16; i += 4 * stride) {
    const uint4 a = p[i], b = p[i + stride], c = p[i + 2 * stride], d = p[i + 3 * stride];
    acc ^= a.x ^ a.y ^ a.z ^ a.w ^ b.x ^ b.y ^ b.z ^ b.w ^ c.x ^ c.y ^ c.z ^ c.w ^ d.x ^ d.y ^ d.z ^ d.w;
  }
  for (; i < n16; i += stride) {
    const uint4 a = p[i];
    acc ^= a.x ^ a.y ^ a.z ^ a.w;
  }
  if (acc == 0x12345678u) sink[0] = acc;
}

// four independent 32x32x16 bfloat16 products a round, `rounds` times, per wave: the shape
// with which the matrix cores were measured fastest here (2.47 PFLOP/s with four waves a SIMD;
// 16x16x32 products reach 2.17 with sixteen sums in flight a wave)
__global__ __launch_bounds__(256) void mfma_rate_kernel(float* __restrict__ out, int rounds) {
  bf16x8_t a[4], b[4];
  for (int j = 0; j < 4; ++j)
    for (int e = 0; e < 8; ++e) {
      a[j][e] = static_cast<__bf16>(threadIdx.x * 0.001f + j);
      b[j][e] = static_cast<__bf16>(e * 0.01f + j);
    }
  f32x16_t acc[4];
  for (int i = 0; i < 4; ++i)
    for (int e = 0; e < 16; ++e) acc[i][e] = 0.f;
  for (int r = 0; r < rounds; ++r) {
#pragma unroll
    for (int i = 0; i < 4; ++i)
      acc[i] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[i], b[(i + 1) & 3], acc[i], 0, 0, 0);
  }
  float s = 0.f;
  for (int i = 0; i < 4; ++i) s += acc[i][0];
  out[static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x] = s;
}

}  // namespace

extern "C" int kvc_peak_read(const void* buffer, int64_t bytes, int blocks, void* sink, kvc_stream stream) {
  if (buffer == nullptr || sink == nullptr || bytes < 16 || blocks <= 0 ||
      (reinterpret_cast<uintptr_t>(buffer) & 15))
    return kvc_fail("kvc_peak_read: a 16-byte aligned buffer, a sink and a positive number of blocks");
  hipLaunchKernelGGL(read_only_kernel, dim3(blocks), dim3(256), 0, reinterpret_cast<hipStream_t>(stream),
                     static_cast<const uint4*>(buffer), bytes / 16, static_cast<uint32_t*>(sink));
  return kvc_check_launch("kvc_peak_read");
}

extern "C" int kvc_peak_mfma_bf16(float* out, int blocks, int rounds, kvc_stream stream) {
  if (out == nullptr || blocks <= 0 || rounds <= 0)
    return kvc_fail("kvc_peak_mfma_bf16: room for blocks x 256 floats, and positive counts");
  hipLaunchKernelGGL(mfma_rate_kernel, dim3(blocks), dim3(256), 0, reinterpret_cast<hipStream_t>(stream), out,
                     rounds);
  return kvc_check_launch("kvc_peak_mfma_bf16");
}
