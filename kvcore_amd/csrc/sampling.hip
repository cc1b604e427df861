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

#include <mutex>

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

// the float32 that order_key made the key from
__device__ __forceinline__ float key_value(uint32_t key) {
  return __uint_as_float((key & 0x80000000u) ? (key & 0x7FFFFFFFu) : ~key);
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


// ------------------------------------------------------------------ several blocks a row
// The same sampling with a row's work dealt to blocks of 256 threads, a chunk of the row
// each, for batches too small to fill the chip with one block a row.  What a pass needs
// from the passes before it is in a workspace of 64-bit words per row, added up with
// integer atomics (so the sums do not depend on the order of addition either):
//
//   [0] largest key of the row   [1] probability mass of the kept entries (2^-40 units)
//   [2] best draw, packed        [3] unused
//   [4 ..)        four histograms of 256 counts: top-k's digits from the top
//   [4 + 1024 ..) four histograms of 256 masses: top-p's digits from the top
//
// A pass starts by working out, from the histograms before it, which digits have been
// chosen so far: every wave does that for itself with a scan over the wave, which costs
// less than handing the result round.  The draws are those of sample_kernel, bit for bit.
constexpr int kSplitThreads = 256;
constexpr int kSplitChunk = 8192;
constexpr int kRowWords = 4 + 2 * 4 * 256;
constexpr float kFixedOne = 1099511627776.0f;  // 2^40

typedef unsigned long long u64;

__device__ __forceinline__ u64 shfl_up_u64(u64 v, int o) {
  const uint32_t lo = __shfl_up(static_cast<uint32_t>(v), o, kWave);
  const uint32_t hi = __shfl_up(static_cast<uint32_t>(v >> 32), o, kWave);
  return (static_cast<u64>(hi) << 32) | lo;
}
__device__ __forceinline__ u64 shfl_u64(u64 v, int src) {
  const uint32_t lo = __shfl(static_cast<uint32_t>(v), src, kWave);
  const uint32_t hi = __shfl(static_cast<uint32_t>(v >> 32), src, kWave);
  return (static_cast<u64>(hi) << 32) | lo;
}
__device__ __forceinline__ u64 wave_inclusive_sum(u64 v) {
  const int lane = threadIdx.x & (kWave - 1);
#pragma unroll
  for (int o = 1; o < kWave; o <<= 1) {
    const u64 t = shfl_up_u64(v, o);
    if (lane >= o) v += t;
  }
  return v;
}

// The highest digit d with (entries of higher digits) + hist[d] >= need, and need less the
// entries of higher digits; digit 0 if none.  The whole wave calls it and gets the result.
__device__ void pick_from_top(const u64* __restrict__ hist, u64 need, int* digit, u64* still) {
  const int lane = threadIdx.x & (kWave - 1);
  u64 h[4];  // digits 255 - 4*lane - i
  u64 mine = 0;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    h[i] = hist[255 - 4 * lane - i];
    mine += h[i];
  }
  const u64 incl = wave_inclusive_sum(mine);
  const u64 before = incl - mine;
  const u64 hit = __ballot(incl >= need);
  const int first = hit ? __ffsll(static_cast<long long>(hit)) - 1 : kWave - 1;
  int d = 0;
  u64 above = before;
  if (lane == first) {
    int i = 0;
    for (; i < 4; ++i) {
      d = 255 - 4 * lane - i;
      if (d == 0 || above + h[i] >= need) break;
      above += h[i];
    }
  }
  *digit = __shfl(d, first, kWave);
  *still = need - shfl_u64(above, first);
}

// The lowest digit d with below + (mass of lower digits) + hist[d] > limit, and below plus
// the mass of the lower digits; digit 255 if none.
__device__ void pick_from_bottom(const u64* __restrict__ hist, u64 below, u64 limit, int* digit, u64* run_out) {
  const int lane = threadIdx.x & (kWave - 1);
  u64 h[4];  // digits 4*lane + i
  u64 mine = 0;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    h[i] = hist[4 * lane + i];
    mine += h[i];
  }
  const u64 incl = wave_inclusive_sum(mine) + below;
  const u64 before = incl - mine;
  const u64 hit = __ballot(incl > limit);
  const int first = hit ? __ffsll(static_cast<long long>(hit)) - 1 : kWave - 1;
  int d = 255;
  u64 run = before;
  if (lane == first) {
    int i = 0;
    for (; i < 4; ++i) {
      d = 4 * lane + i;
      if (d == 255 || run + h[i] > limit) break;
      run += h[i];
    }
  }
  *digit = __shfl(d, first, kWave);
  *run_out = shfl_u64(run, first);
}

struct RowPlan {
  float inv_t;
  int k;         // V when top-k is off
  float p_keep;  // 1 when top-p is off
  bool greedy;
};

__device__ __forceinline__ RowPlan row_plan(const float* temperature, const int32_t* top_k,
                                            const float* top_p, int s, int V) {
  RowPlan r;
  const float temp = temperature[s];
  r.greedy = temp < kGreedyEps;
  r.inv_t = r.greedy ? 1.f : 1.0f / temp;
  int k = top_k[s];
  r.k = (k <= 0 || k > V) ? V : k;
  r.p_keep = top_p[s];
  return r;
}

// top-k's digits chosen by the first `passes` histograms: the prefix and what is still to find
__device__ void topk_state(const u64* __restrict__ w, int k, int passes, uint32_t* prefix, u64* need) {
  uint32_t pre = 0u;
  u64 n = static_cast<u64>(k);
  for (int p = 0; p < passes; ++p) {
    int d;
    pick_from_top(w + 4 + 256 * p, n, &d, &n);
    pre |= static_cast<uint32_t>(d) << (24 - 8 * p);
  }
  *prefix = pre;
  *need = n;
}

__device__ void topp_state(const u64* __restrict__ w, float p_keep, int passes, uint32_t* prefix, u64* below) {
  const u64 den = w[1];
  const u64 limit = static_cast<u64>((1.0 - static_cast<double>(p_keep)) * static_cast<double>(den));
  uint32_t pre = 0u;
  u64 run = 0;
  for (int p = 0; p < passes; ++p) {
    int d;
    pick_from_bottom(w + 4 + 1024 + 256 * p, run, limit, &d, &run);
    pre |= static_cast<uint32_t>(d) << (24 - 8 * p);
  }
  *prefix = pre;
  *below = run;
}

__global__ void split_clear_kernel(u64* __restrict__ ws, int64_t words) {
  const int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (i < words) ws[i] = 0ull;
}

// this block's chunk of the row
template <typename F>
__device__ __forceinline__ void for_each_in_chunk(const float* __restrict__ row, int V, F f) {
  const int begin = blockIdx.y * kSplitChunk;
  const int end = (begin + kSplitChunk < V) ? begin + kSplitChunk : V;
  if ((reinterpret_cast<uintptr_t>(row + begin) & 15) == 0) {
    const int n4 = (end - begin) >> 2;
    const float4* row4 = reinterpret_cast<const float4*>(row + begin);
#pragma unroll 4
    for (int i = threadIdx.x; i < n4; i += kSplitThreads) {
      const float4 x = row4[i];
      f(begin + 4 * i, x.x);
      f(begin + 4 * i + 1, x.y);
      f(begin + 4 * i + 2, x.z);
      f(begin + 4 * i + 3, x.w);
    }
    for (int v = begin + 4 * n4 + threadIdx.x; v < end; v += kSplitThreads) f(v, row[v]);
  } else {
    for (int v = begin + threadIdx.x; v < end; v += kSplitThreads) f(v, row[v]);
  }
}

__device__ __forceinline__ void flush_hist(u64* __restrict__ dst, const u64* lds_hist) {
  for (int b = threadIdx.x; b < 256; b += kSplitThreads)
    if (lds_hist[b]) atomicAdd(&dst[b], lds_hist[b]);
}

// PASS 0..3: top-k's histogram of digit PASS (and the row's largest key in pass 0).
// PASS 4..7: top-p's histogram of digit PASS - 4 (and the kept mass in pass 4).
template <int PASS>
__global__ __launch_bounds__(kSplitThreads) void split_hist_kernel(
    u64* __restrict__ ws, const float* __restrict__ logits, int V, int64_t row_stride,
    const float* __restrict__ temperature, const int32_t* __restrict__ top_k,
    const float* __restrict__ top_p) {
  __shared__ u64 hist[256];
  const int s = blockIdx.x;
  const RowPlan plan = row_plan(temperature, top_k, top_p, s, V);
  if (plan.greedy) return;
  u64* w = ws + static_cast<int64_t>(s) * kRowWords;
  const float* row = logits + static_cast<int64_t>(s) * row_stride;
  const float inv_t = plan.inv_t;
  for (int b = threadIdx.x; b < 256; b += kSplitThreads) hist[b] = 0ull;
  __syncthreads();
  if constexpr (PASS < 4) {
    const bool counting = plan.k < V;
    if (PASS > 0 && !counting) return;
    uint32_t prefix = 0u;
    u64 need = 0;
    if (PASS > 0) topk_state(w, plan.k, PASS, &prefix, &need);
    constexpr int shift = 24 - 8 * PASS;
    constexpr uint32_t high_mask = (PASS == 0) ? 0u : (0xFFFFFFFFu << (shift + 8));
    uint32_t max_key = 0u;
    for_each_in_chunk(row, V, [&](int, float x) {
      const uint32_t key = order_key(x * inv_t);
      if (PASS == 0) max_key = key > max_key ? key : max_key;
      if (counting && (key & high_mask) == (prefix & high_mask)) atomicAdd(&hist[(key >> shift) & 255u], 1ull);
    });
    if (PASS == 0) {
#pragma unroll
      for (int o = kWave / 2; o > 0; o >>= 1) {
        const uint32_t other = __shfl_xor(max_key, o, kWave);
        max_key = other > max_key ? other : max_key;
      }
      if ((threadIdx.x & (kWave - 1)) == 0) atomicMax(&w[0], static_cast<u64>(max_key));
    }
    __syncthreads();
    if (counting) flush_hist(w + 4 + 256 * PASS, hist);
  } else {
    if (!(plan.p_keep < 1.0f)) return;
    constexpr int P = PASS - 4;
    uint32_t keep_key = 0u;
    if (plan.k < V) {
      u64 unused;
      topk_state(w, plan.k, 4, &keep_key, &unused);
    }
    uint32_t prefix = 0u;
    u64 below = 0;
    if (P > 0) topp_state(w, plan.p_keep, P, &prefix, &below);
    const float zmax = key_value(static_cast<uint32_t>(w[0]));
    constexpr int shift = 24 - 8 * P;
    constexpr uint32_t high_mask = (P == 0) ? 0u : (0xFFFFFFFFu << (shift + 8));
    u64 den = 0ull;
    for_each_in_chunk(row, V, [&](int, float x) {
      const float z = x * inv_t;
      const uint32_t key = order_key(z);
      if (key < keep_key) return;
      const u64 m = static_cast<u64>(expf(z - zmax) * kFixedOne);
      if (P == 0) den += m;
      if (m && (key & high_mask) == (prefix & high_mask)) atomicAdd(&hist[(key >> shift) & 255u], m);
    });
    if (P == 0) {
      // one atomic a wave
#pragma unroll
      for (int o = kWave / 2; o > 0; o >>= 1) den += shfl_u64(den, (threadIdx.x & (kWave - 1)) ^ o);
      if ((threadIdx.x & (kWave - 1)) == 0 && den) atomicAdd(&w[1], den);
    }
    __syncthreads();
    flush_hist(w + 4 + 1024 + 256 * P, hist);
  }
}

// the draw over this block's chunk; the best of all blocks gathers in the row's word 2
__global__ __launch_bounds__(kSplitThreads) void split_draw_kernel(
    u64* __restrict__ ws, const float* __restrict__ logits, int V, int64_t row_stride,
    const float* __restrict__ temperature, const int32_t* __restrict__ top_k,
    const float* __restrict__ top_p, const uint32_t* __restrict__ seed_lo,
    const uint32_t* __restrict__ seed_hi, const uint32_t* __restrict__ index) {
  const int s = blockIdx.x;
  const RowPlan plan = row_plan(temperature, top_k, top_p, s, V);
  u64* w = ws + static_cast<int64_t>(s) * kRowWords;
  const float* row = logits + static_cast<int64_t>(s) * row_stride;
  uint32_t keep_key = 0u;
  if (!plan.greedy) {
    if (plan.k < V) {
      u64 unused;
      topk_state(w, plan.k, 4, &keep_key, &unused);
    }
    if (plan.p_keep < 1.0f) {
      uint32_t lo;
      u64 unused;
      topp_state(w, plan.p_keep, 4, &lo, &unused);
      const uint32_t max_key = static_cast<uint32_t>(w[0]);
      if (lo > max_key) lo = max_key;  // the largest entry is never dropped
      if (lo > keep_key) keep_key = lo;
    }
  }
  const float inv_t = plan.inv_t;
  const uint32_t key = plan.greedy ? 0u : noise_key(seed_lo[s], seed_hi[s], index[s]);
  Best mine{-INFINITY, -1};
  if (plan.greedy) {
    for_each_in_chunk(row, V, [&](int v, float x) { mine = better(mine, Best{x, v}); });
  } else {
    for_each_in_chunk(row, V, [&](int v, float x) {
      const float z = x * inv_t;
      if (order_key(z) < keep_key) return;
      const float e = -logf(uniform_noise(key, static_cast<uint32_t>(v)));
      mine = better(mine, Best{z - logf(e), v});
    });
  }
#pragma unroll
  for (int o = kWave / 2; o > 0; o >>= 1) {
    Best other;
    other.val = __shfl_xor(mine.val, o, kWave);
    other.idx = __shfl_xor(mine.idx, o, kWave);
    mine = better(mine, other);
  }
  if ((threadIdx.x & (kWave - 1)) == 0 && mine.idx >= 0 && mine.val == mine.val) {
    // larger value first, then the lower index: one word whose maximum is the winner
    const u64 packed = (static_cast<u64>(order_key(mine.val)) << 32) |
                       static_cast<u64>(0xFFFFFFFFu - static_cast<uint32_t>(mine.idx));
    atomicMax(&w[2], packed);
  }
}

__global__ void split_final_kernel(int32_t* __restrict__ out, const u64* __restrict__ ws, int S_) {
  const int s = blockIdx.x * blockDim.x + threadIdx.x;
  if (s >= S_) return;
  const u64 packed = ws[static_cast<int64_t>(s) * kRowWords + 2];
  out[s] = packed ? static_cast<int32_t>(0xFFFFFFFFu - static_cast<uint32_t>(packed)) : 0;
}

// ------------------------------------------------------- argmax without a workspace argument
// Partial results of the two-stage argmax for callers that can neither allocate nor bring a
// workspace.  Every GPU that the library runs on holds its own copy of this array until the
// process ends (128 KB).  In host code the array's name is a stand-in, not a device address:
// only the pointer that hipGetSymbolAddress returns for the current device is passed on.
// All calls on one GPU share that GPU's copy, so calls that overlap there (two streams, two
// threads) race; calls on one stream follow each other and do not.
constexpr int kStaticArgmaxEntries = 16384;
constexpr int kStaticArgmaxDevices = 64;
// values in the first half (float32), indices in the second (int32)
static __device__ __align__(256) uint32_t scratch[2 * kStaticArgmaxEntries];

uint32_t* g_static_scratch[kStaticArgmaxDevices];  // per device: its copy's address, once known
std::mutex g_static_scratch_mutex;

// The current device's copy of `scratch`, looked up once per device with that device current.
int static_scratch_pointer(uint32_t** out) {
  int device = -1;
  if (hipGetDevice(&device) != hipSuccess || device < 0 || device >= kStaticArgmaxDevices)
    return kvc_fail("kvc_argmax_static: cannot tell the current device");
  std::lock_guard<std::mutex> lock(g_static_scratch_mutex);
  if (g_static_scratch[device] == nullptr) {
    void* ptr = nullptr;
    const hipError_t err = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
    if (err != hipSuccess || ptr == nullptr) {
      (void)hipGetLastError();
      return kvc_fail("kvc_argmax_static: hipGetSymbolAddress failed for the scratch array");
    }
    g_static_scratch[device] = static_cast<uint32_t*>(ptr);
  }
  *out = g_static_scratch[device];
  return 0;
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

extern "C" int kvc_argmax_static_capacity(void) { return kStaticArgmaxEntries; }

extern "C" int kvc_argmax_static(int32_t* out, const float* logits, int S_, int V,
                                 int64_t row_stride, kvc_stream stream) {
  if (S_ < 0 || V <= 0 || row_stride < V) return kvc_fail("kvc_argmax_static: bad sizes");
  if (out == nullptr || logits == nullptr) return kvc_fail("kvc_argmax_static: null pointer");
  if (S_ == 0) return 0;
  constexpr int kChunk = 8192;
  const int chunks = (V + kChunk - 1) / kChunk;
  hipStream_t st = reinterpret_cast<hipStream_t>(stream);
  if (chunks == 1) {  // a short row is one block's work and needs no partial results
    hipLaunchKernelGGL(argmax_kernel, dim3(S_), dim3(kThreads), 0, st, out, logits, V, row_stride);
    return kvc_check_launch("kvc_argmax_static");
  }
  if (chunks > 65535 || static_cast<int64_t>(S_) * chunks > kStaticArgmaxEntries)
    return kvc_fail("kvc_argmax_static: rows x ceil(V / 8192) exceeds the 16384 partial results "
                    "that the static scratch array holds; use kvc_argmax with a workspace");
  uint32_t* ptr = nullptr;
  if (static_scratch_pointer(&ptr) != 0) return -1;
  float* part_val = reinterpret_cast<float*>(ptr);
  int32_t* part_idx = reinterpret_cast<int32_t*>(ptr + kStaticArgmaxEntries);
  // every partial result that stage two reads was written by stage one of this call, so the
  // array's old contents need no clearing
  hipLaunchKernelGGL(argmax_chunk_kernel, dim3(S_, chunks), dim3(kThreads), 0, st, part_val,
                     part_idx, logits, V, row_stride, kChunk);
  hipLaunchKernelGGL(argmax_final_kernel, dim3(S_), dim3(kWave), 0, st, out, part_val, part_idx,
                     chunks);
  return kvc_check_launch("kvc_argmax_static");
}

extern "C" int kvc_sample_workspace_words(int S_, int V) {
  if (S_ <= 0 || V <= kSplitChunk) return 0;  // short rows: one block a row does
  return S_ * kRowWords;
}

extern "C" int kvc_sample(int32_t* out, const float* logits, int S_, int V, int64_t row_stride,
                          const float* temperature, const int32_t* top_k, const float* top_p,
                          const uint32_t* seed_lo, const uint32_t* seed_hi, const uint32_t* index,
                          void* workspace, int64_t workspace_words, int filters, kvc_stream stream) {
  if (S_ < 0 || V <= 0 || row_stride < V) return kvc_fail("kvc_sample: bad sizes");
  if (S_ == 0) return 0;
  hipStream_t st = reinterpret_cast<hipStream_t>(stream);
  const int64_t words = static_cast<int64_t>(S_) * kRowWords;
  if (workspace == nullptr || workspace_words < words || V <= kSplitChunk ||
      (reinterpret_cast<uintptr_t>(workspace) & 7)) {
    hipLaunchKernelGGL(sample_kernel, dim3(S_), dim3(kThreads), 0, st, out, logits, V, row_stride,
                       temperature, top_k, top_p, seed_lo, seed_hi, index);
    return kvc_check_launch("kvc_sample");
  }
  u64* ws = static_cast<u64*>(workspace);
  const int chunks = (V + kSplitChunk - 1) / kSplitChunk;
  if (chunks > 65535) return kvc_fail("kvc_sample: the rows are too long");
  const dim3 grid(S_, chunks), block(kSplitThreads);
  hipLaunchKernelGGL(split_clear_kernel, dim3(static_cast<unsigned>((words + 255) / 256)), dim3(256), 0, st,
                     ws, words);
  const bool any_k = (filters & 1) != 0, any_p = (filters & 2) != 0;
#define KVC_SPLIT_PASS(P_)                                                                          \
  hipLaunchKernelGGL(split_hist_kernel<P_>, grid, block, 0, st, ws, logits, V, row_stride, temperature, \
                     top_k, top_p)
  if (any_k || any_p) KVC_SPLIT_PASS(0);
  if (any_k) {
    KVC_SPLIT_PASS(1);
    KVC_SPLIT_PASS(2);
    KVC_SPLIT_PASS(3);
  }
  if (any_p) {
    KVC_SPLIT_PASS(4);
    KVC_SPLIT_PASS(5);
    KVC_SPLIT_PASS(6);
    KVC_SPLIT_PASS(7);
  }
#undef KVC_SPLIT_PASS
  hipLaunchKernelGGL(split_draw_kernel, grid, block, 0, st, ws, logits, V, row_stride, temperature, top_k,
                     top_p, seed_lo, seed_hi, index);
  hipLaunchKernelGGL(split_final_kernel, dim3((S_ + 255) / 256), dim3(256), 0, st, out, ws, S_);
  return kvc_check_launch("kvc_sample");
}
