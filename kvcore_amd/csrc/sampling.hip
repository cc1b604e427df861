// Sampling over float32 logits: one block of 1024 threads per row.
//
// Greedy is the argmax (lowest index among equals).  Otherwise the row is divided by
// its temperature; top-k and top-p become a value threshold found digit by digit (four
// digits of eight bits, a histogram in LDS each: counts for top-k, probability mass in
// fixed point for top-p) over the order-preserving integer image of float32, without a
// sort and with sums that do not depend on the order of addition; the token is
// argmax_v(z_v - log(e_v)) with e_v = -log(u_v) exponential noise, which is the same
// draw as argmax_v(softmax(z)_v / e_v).  u_v comes from 32-bit integer mixing of
// (seed, output index, v), so a row's draw depends on nothing else in the batch.

#include <hip/hip_runtime.h>

#include "device_utils.h"
#include "kvcore_hip.h"

using namespace kvc;

namespace {

constexpr int kThreads = 1024;
constexpr float kGreedyEps = 1e-5f;

__device__ __forceinline__ uint32_t fmix(uint32_t x) {
  x ^= x >> 16;
  x *= 0x85EBCA6Bu;
  x ^= x >> 13;
  x *= 0xC2B2AE35u;
  x ^= x >> 16;
  return x;
}

__device__ __forceinline__ uint32_t noise_key(uint32_t lo, uint32_t hi, uint32_t index) {
  const uint32_t key = fmix(lo ^ fmix(hi + 0x9E3779B9u));
  return fmix(key ^ fmix(index + 0x7F4A7C15u));
}

__device__ __forceinline__ float uniform_noise(uint32_t key, uint32_t v) {
  uint32_t x = fmix(key + v * 0x9E3779B1u);
  x = fmix(x ^ key);
  return (static_cast<float>(x >> 9) + 0.5f) * (1.0f / 8388608.0f);
}

// float32 -> unsigned key with the same order
__device__ __forceinline__ uint32_t order_key(float f) {
  const uint32_t b = __float_as_uint(f);
  return (b & 0x80000000u) ? ~b : (b | 0x80000000u);
}

// f(v, row[v]) for every v < V, this thread's share: four values a load where the row is
// aligned, several loads in flight
template <typename F>
__device__ __forceinline__ void for_each_logit(const float* __restrict__ row, int V, F f) {
  if ((reinterpret_cast<uintptr_t>(row) & 15) == 0) {
    const int V4 = V >> 2;
    const float4* row4 = reinterpret_cast<const float4*>(row);
#pragma unroll 4
    for (int i = threadIdx.x; i < V4; i += kThreads) {
      const float4 x = row4[i];
      f(4 * i, x.x);
      f(4 * i + 1, x.y);
      f(4 * i + 2, x.z);
      f(4 * i + 3, x.w);
    }
    for (int v = 4 * V4 + threadIdx.x; v < V; v += kThreads) f(v, row[v]);
  } else {
#pragma unroll 4
    for (int v = threadIdx.x; v < V; v += kThreads) f(v, row[v]);
  }
}

struct Best {
  float val;
  int idx;
};

__device__ __forceinline__ Best better(Best a, Best b) {
  if (b.idx < 0) return a;
  if (a.idx < 0) return b;
  if (b.val > a.val || (b.val == a.val && b.idx < a.idx)) return b;
  return a;
}

__device__ Best block_best(Best mine, Best* scratch) {
#pragma unroll
  for (int o = kWave / 2; o > 0; o >>= 1) {
    Best other;
    other.val = __shfl_xor(mine.val, o, kWave);
    other.idx = __shfl_xor(mine.idx, o, kWave);
    mine = better(mine, other);
  }
  const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
  __syncthreads();
  if (lane == 0) scratch[wave] = mine;
  __syncthreads();
  Best total = scratch[0];
  for (int w = 1; w < kThreads / kWave; ++w) total = better(total, scratch[w]);
  return total;
}

__device__ float block_max(float v, float* scratch) {
  v = wave_max(v);
  const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
  __syncthreads();
  if (lane == 0) scratch[wave] = v;
  __syncthreads();
  float total = scratch[0];
  for (int w = 1; w < kThreads / kWave; ++w) total = fmaxf(total, scratch[w]);
  return total;
}

__global__ __launch_bounds__(kThreads) void argmax_kernel(int32_t* __restrict__ out,
                                                          const float* __restrict__ logits, int V,
                                                          int64_t row_stride) {
  __shared__ Best scratch[kThreads / kWave];
  const float* row = logits + static_cast<int64_t>(blockIdx.x) * row_stride;
  Best mine{-INFINITY, -1};
  for_each_logit(row, V, [&](int v, float x) { mine = better(mine, Best{x, v}); });
  const Best total = block_best(mine, scratch);
  if (threadIdx.x == 0) out[blockIdx.x] = total.idx < 0 ? 0 : total.idx;
}

// Two-stage argmax for long rows: stage one takes the best of a chunk of the row per
// block, stage two the best of the chunk results (same order of preference: larger value,
// then lower index).
__global__ __launch_bounds__(kThreads) void argmax_chunk_kernel(float* __restrict__ part_val,
                                                                int32_t* __restrict__ part_idx,
                                                                const float* __restrict__ logits,
                                                                int V, int64_t row_stride,
                                                                int chunk) {
  __shared__ Best scratch[kThreads / kWave];
  const float* row = logits + static_cast<int64_t>(blockIdx.x) * row_stride;
  const int begin = blockIdx.y * chunk;
  const int end = (begin + chunk < V) ? begin + chunk : V;
  Best mine{-INFINITY, -1};
  for (int v = begin + threadIdx.x; v < end; v += kThreads) mine = better(mine, Best{row[v], v});
  const Best total = block_best(mine, scratch);
  if (threadIdx.x == 0) {
    part_val[blockIdx.x * gridDim.y + blockIdx.y] = total.val;
    part_idx[blockIdx.x * gridDim.y + blockIdx.y] = total.idx;
  }
}

__global__ void argmax_final_kernel(int32_t* __restrict__ out, const float* __restrict__ part_val,
                                    const int32_t* __restrict__ part_idx, int chunks) {
  const int s = blockIdx.x;
  Best mine{-INFINITY, -1};
  for (int c = threadIdx.x; c < chunks; c += kWave)
    mine = better(mine, Best{part_val[s * chunks + c], part_idx[s * chunks + c]});
#pragma unroll
  for (int o = kWave / 2; o > 0; o >>= 1) {
    Best other;
    other.val = __shfl_xor(mine.val, o, kWave);
    other.idx = __shfl_xor(mine.idx, o, kWave);
    mine = better(mine, other);
  }
  if (threadIdx.x == 0) out[s] = mine.idx < 0 ? 0 : mine.idx;
}

__global__ __launch_bounds__(kThreads) void sample_kernel(
    int32_t* __restrict__ out, const float* __restrict__ logits, int V, int64_t row_stride,
    const float* __restrict__ temperature, const int32_t* __restrict__ top_k,
    const float* __restrict__ top_p, const uint32_t* __restrict__ seed_lo,
    const uint32_t* __restrict__ seed_hi, const uint32_t* __restrict__ index) {
  __shared__ Best best_scratch[kThreads / kWave];
  __shared__ float f_scratch[kThreads / kWave];
  const int s = blockIdx.x;
  const float* row = logits + static_cast<int64_t>(s) * row_stride;
  const float temp = temperature[s];

  if (temp < kGreedyEps) {
    Best mine{-INFINITY, -1};
    for_each_logit(row, V, [&](int v, float x) { mine = better(mine, Best{x, v}); });
    const Best total = block_best(mine, best_scratch);
    if (threadIdx.x == 0) out[s] = total.idx < 0 ? 0 : total.idx;
    return;
  }
  const float inv_t = 1.0f / temp;
  int k = top_k[s];
  if (k <= 0 || k > V) k = V;
  const float p_keep = top_p[s];

  // threshold key: entries with order_key(z) >= keep_key stay
  __shared__ unsigned long long hist[256];
  __shared__ uint32_t chosen_prefix;
  __shared__ unsigned long long chosen_sum;
  uint32_t keep_key = 0u;
  if (k < V) {
    // the k-th largest key, digit by digit from the top: among the entries that share the
    // digits found so far, the highest digit with at least `need` entries at or above it
    uint32_t prefix = 0u;
    unsigned long long need = static_cast<unsigned long long>(k);
    for (int shift = 24; shift >= 0; shift -= 8) {
      for (int b = threadIdx.x; b < 256; b += kThreads) hist[b] = 0ull;
      __syncthreads();
      const uint32_t high_mask = (shift == 24) ? 0u : (0xFFFFFFFFu << (shift + 8));
      for_each_logit(row, V, [&](int, float x) {
        const uint32_t key = order_key(x * inv_t);
        if ((key & high_mask) == (prefix & high_mask)) atomicAdd(&hist[(key >> shift) & 255u], 1ull);
      });
      __syncthreads();
      if (threadIdx.x == 0) {
        unsigned long long above = 0ull;
        int d = 255;
        for (; d > 0; --d) {
          if (above + hist[d] >= need) break;
          above += hist[d];
        }
        chosen_prefix = prefix | (static_cast<uint32_t>(d) << shift);
        chosen_sum = need - above;  // still to find among the entries of this digit
      }
      __syncthreads();
      prefix = chosen_prefix;
      need = chosen_sum;
    }
    keep_key = prefix;
  }
  if (p_keep < 1.0f) {
    float zmax = -INFINITY;
    for_each_logit(row, V, [&](int, float x) { zmax = fmaxf(zmax, x * inv_t); });
    zmax = block_max(zmax, f_scratch);
    const uint32_t max_key = order_key(zmax);
    // probability mass in fixed point (2^-40 of the largest entry's), so that sums are exact
    // integers whatever the order of addition
    constexpr float kFix = 1099511627776.0f;  // 2^40
    unsigned long long den = 0ull;
    for_each_logit(row, V, [&](int, float x) {
      const float z = x * inv_t;
      if (order_key(z) >= keep_key) den += static_cast<unsigned long long>(expf(z - zmax) * kFix);
    });
    for (int b = threadIdx.x; b < 256; b += kThreads) hist[b] = 0ull;
    __syncthreads();
    atomicAdd(&hist[0], den);
    __syncthreads();
    den = hist[0];
    const unsigned long long limit =
        static_cast<unsigned long long>((1.0 - static_cast<double>(p_keep)) * static_cast<double>(den));
    // the largest key whose strictly-smaller kept entries weigh at most `limit`, digit by digit
    uint32_t prefix = 0u;
    unsigned long long below = 0ull;  // mass of the kept entries whose key is under `prefix`
    for (int shift = 24; shift >= 0; shift -= 8) {
      __syncthreads();
      for (int b = threadIdx.x; b < 256; b += kThreads) hist[b] = 0ull;
      __syncthreads();
      const uint32_t high_mask = (shift == 24) ? 0u : (0xFFFFFFFFu << (shift + 8));
      for_each_logit(row, V, [&](int, float x) {
        const float z = x * inv_t;
        const uint32_t key = order_key(z);
        if (key >= keep_key && (key & high_mask) == (prefix & high_mask)) {
          const unsigned long long m = static_cast<unsigned long long>(expf(z - zmax) * kFix);
          if (m) atomicAdd(&hist[(key >> shift) & 255u], m);
        }
      });
      __syncthreads();
      if (threadIdx.x == 0) {
        unsigned long long run = below;
        int d = 0;
        for (; d < 255; ++d) {
          if (run + hist[d] > limit) break;
          run += hist[d];
        }
        chosen_prefix = prefix | (static_cast<uint32_t>(d) << shift);
        chosen_sum = run;
      }
      __syncthreads();
      prefix = chosen_prefix;
      below = chosen_sum;
    }
    uint32_t lo = prefix;
    if (lo > max_key) lo = max_key;  // the largest entry is never dropped
    if (lo > keep_key) keep_key = lo;
  }

  const uint32_t key = noise_key(seed_lo[s], seed_hi[s], index[s]);
  Best mine{-INFINITY, -1};
  for_each_logit(row, V, [&](int v, float x) {
    const float z = x * inv_t;
    if (order_key(z) < keep_key) return;
    const float e = -logf(uniform_noise(key, static_cast<uint32_t>(v)));
    mine = better(mine, Best{z - logf(e), v});
  });
  const Best total = block_best(mine, best_scratch);
  if (threadIdx.x == 0) out[s] = total.idx < 0 ? 0 : total.idx;
}

}  // namespace

extern "C" int kvc_argmax(int32_t* out, const float* logits, int S_, int V, int64_t row_stride,
                          float* part_val, int32_t* part_idx, int part_capacity,
                          kvc_stream stream) {
  if (S_ < 0 || V <= 0 || row_stride < V) return kvc_fail("kvc_argmax: bad sizes");
  if (S_ == 0) return 0;
  constexpr int kChunk = 8192;
  const int chunks = (V + kChunk - 1) / kChunk;
  if (chunks > 1 && part_val != nullptr && part_idx != nullptr && part_capacity >= S_ * chunks &&
      chunks <= 65535) {
    hipStream_t st = reinterpret_cast<hipStream_t>(stream);
    hipLaunchKernelGGL(argmax_chunk_kernel, dim3(S_, chunks), dim3(kThreads), 0, st, part_val,
                       part_idx, logits, V, row_stride, kChunk);
    hipLaunchKernelGGL(argmax_final_kernel, dim3(S_), dim3(kWave), 0, st, out, part_val, part_idx,
                       chunks);
    return kvc_check_launch("kvc_argmax");
  }
  hipLaunchKernelGGL(argmax_kernel, dim3(S_), dim3(kThreads), 0,
                     reinterpret_cast<hipStream_t>(stream), out, logits, V, row_stride);
  return kvc_check_launch("kvc_argmax");
}

extern "C" int kvc_sample(int32_t* out, const float* logits, int S_, int V, int64_t row_stride,
                          const float* temperature, const int32_t* top_k, const float* top_p,
                          const uint32_t* seed_lo, const uint32_t* seed_hi, const uint32_t* index,
                          kvc_stream stream) {
  if (S_ < 0 || V <= 0 || row_stride < V) return kvc_fail("kvc_sample: bad sizes");
  if (S_ == 0) return 0;
  hipLaunchKernelGGL(sample_kernel, dim3(S_), dim3(kThreads), 0,
                     reinterpret_cast<hipStream_t>(stream), out, logits, V, row_stride,
                     temperature, top_k, top_p, seed_lo, seed_hi, index);
  return kvc_check_launch("kvc_sample");
}
