// Seeded normal variates whose bits do not depend on where they are made.
//
// Element i of a tensor is a function of (seed_lo, seed_hi, i) alone: 32-bit integer mixing
// gives two 24-bit uniforms, and a Box-Muller step turns them into one normal variate.  The
// logarithm, the cosine and every other step are written out in single float32 operations
// (products, sums, one correctly rounded square root, polynomials by Horner's rule, a
// 32-entry table) with fused multiply-adds switched off for this file, so that a host
// program doing the same operations one by one in IEEE float32 arrives at the same bits
// (kvcore_amd/weights/random_normal.py does, and a test compares them).  The random-weights
// mode of the loader draws with this on the GPU and writes model folders with the host
// twin; both give the same model for one seed.

#include <hip/hip_runtime.h>

#include "device_utils.h"
#include "kvcore_hip.h"

#pragma clang fp contract(off)

using namespace kvc;

namespace {

__device__ __forceinline__ uint32_t mix32(uint32_t x) {
  x ^= x >> 16;
  x *= 0x85EBCA6Bu;
  x ^= x >> 13;
  x *= 0xC2B2AE35u;
  x ^= x >> 16;
  return x;
}

// float32(1 / c_i) and float32(ln c_i) for c_i = 1 + (i + 0.5) / 32, as bit patterns
__device__ const uint32_t kInvC[32] = {
    0x3F7C0FC1u, 0x3F74898Du, 0x3F6D7304u, 0x3F66C2B4u, 0x3F607038u, 0x3F5A740Eu, 0x3F54C77Bu, 0x3F4F6475u,
    0x3F4A4588u, 0x3F4565C8u, 0x3F40C0C1u, 0x3F3C5264u, 0x3F381703u, 0x3F340B41u, 0x3F302C0Bu, 0x3F2C7692u,
    0x3F28E83Fu, 0x3F257EB5u, 0x3F2237C3u, 0x3F1F1166u, 0x3F1C09C1u, 0x3F191F1Au, 0x3F164FDAu, 0x3F139A86u,
    0x3F10FDBCu, 0x3F0E7835u, 0x3F0C08C1u, 0x3F09AE41u, 0x3F0767ABu, 0x3F053408u, 0x3F03126Fu, 0x3F010204u};
__device__ const uint32_t kLnC[32] = {
    0x3C7E0546u, 0x3D3BA2C8u, 0x3D9A0EBDu, 0x3DD4936Au, 0x3E06BBF4u, 0x3E22695Bu, 0x3E3D5C48u, 0x3E579E4Au,
    0x3E71383Bu, 0x3E851927u, 0x3E914A10u, 0x3E9D3263u, 0x3EA8D56Cu, 0x3EB43641u, 0x3EBF57C2u, 0x3ECA3CA1u,
    0x3ED4E765u, 0x3EDF5A6Du, 0x3EE997F4u, 0x3EF3A213u, 0x3EFD7AC4u, 0x3F0391F3u, 0x3F084F9Du, 0x3F0CF736u,
    0x3F118987u, 0x3F16074Fu, 0x3F1A7145u, 0x3F1EC813u, 0x3F230C5Eu, 0x3F273EC1u, 0x3F2B5FCFu, 0x3F2F7015u};

__device__ __forceinline__ float bits(uint32_t b) { return __uint_as_float(b); }

// One standard normal variate from the element's index.  Every line is one rounded float32
// operation (or exact integer work); the host twin follows it line by line.
__device__ float normal_variate(uint32_t key, uint32_t i_lo, uint32_t i_hi) {
  uint32_t x = mix32(key ^ i_lo);
  x = mix32(x + i_hi + 0x9E3779B9u);
  const uint32_t k1 = mix32(x ^ 0x68E31DA4u) >> 8;  // 24 bits
  const uint32_t k2 = mix32(x ^ 0xB5297A4Du) >> 8;

  // ln(u1), u1 = (k1 + 1) / 2^24 in (0, 1]
  const float u1 = static_cast<float>(k1 + 1u) * bits(0x33800000u);  // * 2^-24, exact
  const uint32_t ub = __float_as_uint(u1);
  const float e = static_cast<float>(static_cast<int>(ub >> 23) - 127);
  const uint32_t mant = ub & 0x7FFFFFu;
  const uint32_t idx = mant >> 18;
  const float m = bits(mant | 0x3F800000u);  // in [1, 2)
  float r = m * bits(kInvC[idx]);
  r = r - 1.0f;  // |r| <= 1/64: ln(1 + r) by four terms
  float p = r * bits(0xBE800000u);   // -1/4
  p = p + bits(0x3EAAAAABu);         // + 1/3
  p = p * r;
  p = p + bits(0xBF000000u);         // - 1/2
  p = p * r;
  p = p + 1.0f;
  p = p * r;
  float ln_u = bits(kLnC[idx]) + p;
  const float e_ln2 = e * bits(0x3F317218u);
  ln_u = e_ln2 + ln_u;
  float t = ln_u * -2.0f;
  t = t > 0.f ? t : 0.f;
  const float radius = __builtin_sqrtf(t);  // correctly rounded: built with -fhip-fp32-correctly-rounded-divide-sqrt

  // cos(2 pi k2 / 2^24): the quadrant from the two top bits, polynomials on [0, pi/2)
  const uint32_t quadrant = k2 >> 22;
  const float f = static_cast<float>(k2 & 0x3FFFFFu) * bits(0x34800000u);  // * 2^-22, exact
  const float a = f * bits(0x3FC90FDBu);                                   // * pi/2
  const float a2 = a * a;
  float s = a2 * bits(0xB2D7322Bu);  // -1/11!
  s = s + bits(0x3638EF1Du);         // + 1/9!
  s = s * a2;
  s = s + bits(0xB9500D01u);         // - 1/7!
  s = s * a2;
  s = s + bits(0x3C088889u);         // + 1/5!
  s = s * a2;
  s = s + bits(0xBE2AAAABu);         // - 1/3!
  s = s * a2;
  s = s + 1.0f;
  s = s * a;
  float c = a2 * bits(0x310F76C7u);  // + 1/12!
  c = c + bits(0xB493F27Eu);         // - 1/10!
  c = c * a2;
  c = c + bits(0x37D00D01u);         // + 1/8!
  c = c * a2;
  c = c + bits(0xBAB60B61u);         // - 1/6!
  c = c * a2;
  c = c + bits(0x3D2AAAABu);         // + 1/4!
  c = c * a2;
  c = c + bits(0xBF000000u);         // - 1/2!
  c = c * a2;
  c = c + 1.0f;
  float cosine = c;
  if (quadrant == 1u) cosine = -s;
  if (quadrant == 2u) cosine = -c;
  if (quadrant == 3u) cosine = s;
  return radius * cosine;
}

template <typename T>
__global__ void fill_normal_kernel(T* __restrict__ out, int64_t n, uint32_t seed_lo, uint32_t seed_hi,
                                   float mean, float std) {
  const uint32_t key = mix32(seed_lo ^ mix32(seed_hi + 0x9E3779B9u));
  const int64_t stride = static_cast<int64_t>(gridDim.x) * blockDim.x;
  for (int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x; i < n; i += stride) {
    const float z = normal_variate(key, static_cast<uint32_t>(i & 0xFFFFFFFF), static_cast<uint32_t>(i >> 32));
    float v = z * std;
    v = v + mean;
    out[i] = from_float<T>(v);
  }
}

}  // namespace

extern "C" int kvc_fill_normal(void* out, int64_t n, int dtype, uint32_t seed_lo, uint32_t seed_hi,
                               float mean, float std, kvc_stream stream) {
  if (n < 0) return kvc_fail("kvc_fill_normal: bad size");
  if (n == 0) return 0;
  const int64_t want = (n + 255) / 256;
  const unsigned blocks = static_cast<unsigned>(want < 65536 ? want : 65536);
  KVC_DISPATCH_DTYPE(dtype, Tp,
                     hipLaunchKernelGGL(fill_normal_kernel<Tp>, dim3(blocks), dim3(256), 0,
                                        reinterpret_cast<hipStream_t>(stream), static_cast<Tp*>(out), n,
                                        seed_lo, seed_hi, mean, std));
  return kvc_check_launch("kvc_fill_normal");
}
