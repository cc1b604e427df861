// Paged attention, general kernel: one 64-lane wave per (token, query head).
//
// Serves every batch shape (portions of prompts beside single decoded tokens), both
// storage types and every head size that is a multiple of 16 up to 256.  A token at
// position p reads keys first..p of its request through the block table, 64 keys a
// tile: each lane scores one key (a float32 dot product over the head in index
// order), the tile is folded into a running softmax (float32 max, sum and output
// accumulators), then the lanes split the head's elements to add p_j * V_j in key
// order.  K pages are [kv head, page_size, d], V pages [kv head, d, page_size].  What a token computes depends on its position, window and cache content
// only: not on the batch it is in nor on how its request was cut into steps.

#include <hip/hip_runtime.h>

#include "device_utils.h"
#include "kvcore_hip.h"

using namespace kvc;

namespace {

constexpr int kWavesPerBlock = 4;
constexpr int kMaxHeadDim = 256;

template <typename T>
struct Vec16;  // 16 bytes of T
template <>
struct Vec16<float> {
  static constexpr int N = 4;
  float4 v;
  __device__ __forceinline__ float get(int i) const { return (&v.x)[i]; }
};
template <>
struct Vec16<bf16_t> {
  static constexpr int N = 8;
  uint4 v;
  __device__ __forceinline__ float get(int i) const {
    const uint32_t word = (&v.x)[i >> 1];
    return __uint_as_float((i & 1) ? (word & 0xffff0000u) : (word << 16));
  }
};

template <typename T>
__global__ __launch_bounds__(kWavesPerBlock* kWave) void paged_attention_wave_kernel(
    T* __restrict__ out, const T* __restrict__ q, int64_t q_stride, const T* __restrict__ k_cache,
    const T* __restrict__ v_cache, const int32_t* __restrict__ table, int table_stride,
    const int32_t* __restrict__ positions, const int32_t* __restrict__ token_req,
    const int32_t* __restrict__ slots, int nh, int nkv, int d, int page_size, int num_pages,
    float scale, int window) {
  __shared__ float q_s[kWavesPerBlock][kMaxHeadDim];
  __shared__ float p_s[kWavesPerBlock][kWave];
  __shared__ int64_t off_s[kWavesPerBlock][kWave];   // K row of each key of the tile
  __shared__ int64_t voff_s[kWavesPerBlock][kWave];  // V column of each key of the tile

  const int t = blockIdx.x;
  const int wave = threadIdx.x / kWave;
  const int lane = threadIdx.x & (kWave - 1);
  const int h_raw = blockIdx.y * kWavesPerBlock + wave;
  const bool head_live = h_raw < nh;
  const int h = head_live ? h_raw : nh - 1;
  T* o = out + (static_cast<int64_t>(t) * nh + h) * d;

  const int req = token_req[t];
  if (req < 0) {  // padding token: the whole block takes this branch
    if (head_live)
      for (int i = lane; i < d; i += kWave) o[i] = from_float<T>(0.f);
    return;
  }
  const int pos = positions[t];
  const int first = (window > 0 && pos - window + 1 > 0) ? pos - window + 1 : 0;
  const int32_t* row = table + static_cast<int64_t>(slots[req]) * table_stride;
  const int hk = h / (nh / nkv);

  const T* qh = q + static_cast<int64_t>(t) * q_stride + static_cast<int64_t>(h) * d;
  for (int i = lane; i < d; i += kWave) q_s[wave][i] = to_float(qh[i]);
  __syncthreads();

  float m = -INFINITY, l = 0.f;
  float acc[kMaxHeadDim / kWave];
#pragma unroll
  for (int i = 0; i < kMaxHeadDim / kWave; ++i) acc[i] = 0.f;

  constexpr int VN = Vec16<T>::N;
  const int64_t head_off = static_cast<int64_t>(hk) * page_size * d;
  const int64_t page_elems = static_cast<int64_t>(nkv) * page_size * d;

  for (int tile = first; tile <= pos; tile += kWave) {
    const int key = tile + lane;
    const bool valid = key <= pos;
    float s = -INFINITY;
    int64_t off = -1, voff = -1;
    if (valid) {
      const int page = row[key / page_size];
      if (page > 0 && page < num_pages) {
        off = static_cast<int64_t>(page) * page_elems + head_off +
              static_cast<int64_t>(key % page_size) * d;
        voff = static_cast<int64_t>(page) * page_elems + head_off + key % page_size;
        const T* kr = k_cache + off;
        float dot = 0.f;
        for (int i = 0; i < d; i += VN) {
          const Vec16<T> kv = *reinterpret_cast<const Vec16<T>*>(kr + i);
#pragma unroll
          for (int e = 0; e < VN; ++e) dot = fmaf(q_s[wave][i + e], kv.get(e), dot);
        }
        s = dot * scale;
      }
    }
    const float tile_max = wave_max(s);
    const float m_new = fmaxf(m, tile_max);
    // a tile with no readable key (pages given back behind a window) leaves the state alone
    const float p = (s == -INFINITY) ? 0.f : expf(s - m_new);
    const float alpha = (m == -INFINITY) ? 0.f : expf(m - m_new);
    const float tile_sum = wave_sum(p);
    l = l * alpha + tile_sum;
    m = m_new;
    __syncthreads();
    p_s[wave][lane] = p;
    off_s[wave][lane] = off;
    voff_s[wave][lane] = voff;
    __syncthreads();
    const int n_keys = (pos - tile + 1 < kWave) ? pos - tile + 1 : kWave;
#pragma unroll
    for (int i = 0; i < kMaxHeadDim / kWave; ++i) acc[i] *= alpha;
    for (int j = 0; j < n_keys; ++j) {
      const int64_t vo = voff_s[wave][j];
      if (vo < 0) continue;
      const float pj = p_s[wave][j];
      const T* vr = v_cache + vo;  // element e of this key is at vr[e * page_size]
#pragma unroll
      for (int i = 0; i < kMaxHeadDim / kWave; ++i) {
        const int e = lane + i * kWave;
        if (e < d) acc[i] = fmaf(pj, to_float(vr[static_cast<int64_t>(e) * page_size]), acc[i]);
      }
    }
  }
  if (!head_live) return;
  const float inv = (l > 0.f) ? 1.f / l : 0.f;
#pragma unroll
  for (int i = 0; i < kMaxHeadDim / kWave; ++i) {
    const int e = lane + i * kWave;
    if (e < d) o[e] = from_float<T>(acc[i] * inv);
  }
}

}  // namespace

extern "C" int kvc_paged_attention(void* out, const void* q, int64_t q_stride, const void* k_cache,
                                   const void* v_cache, const int32_t* table, int table_stride,
                                   const int32_t* positions, const int32_t* token_req,
                                   const int32_t* slots, int T, int nh, int nkv, int d,
                                   int page_size, int num_pages, float scale, int window,
                                   int dtype, kvc_stream stream) {
  if (T < 0 || nh <= 0 || nkv <= 0 || page_size <= 0 || num_pages <= 0 || table_stride <= 0)
    return kvc_fail("kvc_paged_attention: bad sizes");
  if (nh % nkv) return kvc_fail("kvc_paged_attention: heads must be a multiple of kv heads");
  if (d <= 0 || d % 16 || d > kMaxHeadDim)
    return kvc_fail("kvc_paged_attention: head size must be a multiple of 16, at most 256");
  if (q_stride < static_cast<int64_t>(nh) * d || q_stride % 8)
    return kvc_fail("kvc_paged_attention: q stride too small or not a multiple of 8");
  if (T == 0) return 0;
  const dim3 grid(T, (nh + kWavesPerBlock - 1) / kWavesPerBlock);
  KVC_DISPATCH_DTYPE(
      dtype, Tp,
      hipLaunchKernelGGL(paged_attention_wave_kernel<Tp>, grid, dim3(kWavesPerBlock * kWave), 0,
                         reinterpret_cast<hipStream_t>(stream), static_cast<Tp*>(out),
                         static_cast<const Tp*>(q), q_stride, static_cast<const Tp*>(k_cache),
                         static_cast<const Tp*>(v_cache), table, table_stride, positions,
                         token_req, slots, nh, nkv, d, page_size, num_pages, scale, window));
  return kvc_check_launch("kvc_paged_attention");
}
