// Paged attention for single tokens (decode), bfloat16, on the matrix cores.
//
// One 64-lane wave per (token, kv head, split of the key range).  The query heads that
// share the kv head are the columns of one 16-wide MFMA tile, so every key and value
// is fetched once for the whole group, straight from global memory:
//
//   S^T[16 keys, 16 heads]  = K[16 keys, d]       * Q^T[d, 16 heads]     (16x16x32)
//   O^T[d, 16 heads]       += V^T[d, 16 keys]     * P^T[16 keys, 16 heads] (16x16x16)
//
// K pages are [page_size, d] (d contiguous) and V pages are [d, page_size] (keys
// contiguous), which are exactly the A-operand layouts of the two products; the
// accumulator layout of S^T is the B-operand layout of the second product, so the
// probabilities never leave registers.  Softmax state (max, sum) is float32, one per
// head, kept redundantly by the four lanes that hold a head's column.
//
// With more than one split each wave writes an unnormalised partial (max, sum,
// output) and a second kernel combines them; split boundaries depend on the
// request's length only.

#include <hip/hip_runtime.h>

#include "device_utils.h"
#include "kvcore_hip.h"

using namespace kvc;

namespace {

typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef short s16x4_t __attribute__((ext_vector_type(4)));
typedef float f32x4_t __attribute__((ext_vector_type(4)));

constexpr float kLog2e = 1.4426950408889634f;

template <int D>
__global__ __launch_bounds__(64) void decode_attention_kernel(
    bf16_t* __restrict__ out, float* __restrict__ part_o, float* __restrict__ part_ml,
    const bf16_t* __restrict__ q, int64_t q_stride, const bf16_t* __restrict__ k_cache,
    const bf16_t* __restrict__ v_cache, const int32_t* __restrict__ table, int table_stride,
    const int32_t* __restrict__ positions, const int32_t* __restrict__ token_req,
    const int32_t* __restrict__ slots, int nh, int nkv, int page_size, int num_pages,
    float scale_log2e, int window, int nsplit) {
  const int t = blockIdx.x;
  const int hk = blockIdx.y;
  const int split = blockIdx.z;
  const int lane = threadIdx.x;
  const int col = lane & 15;   // head within the group (B/C column)
  const int quad = lane >> 4;  // 0..3
  const int g = nh / nkv;
  const int head = hk * g + col;
  const bool head_live = col < g;

  const int req = token_req[t];
  constexpr int NJ = D / 16;  // output row blocks
  constexpr int NC = D / 32;  // 32-wide chunks of the head for Q.K
  if (req < 0) {  // padding token
    if (nsplit == 1 && head_live) {
      bf16_t* o = out + (static_cast<int64_t>(t) * nh + head) * D;
      for (int j = 0; j < NJ; ++j)
        for (int i = 0; i < 4; ++i) o[16 * j + 4 * quad + i] = from_float<bf16_t>(0.f);
    } else if (head_live && quad == 0) {
      float* ml = part_ml + ((static_cast<int64_t>(t) * nh + head) * nsplit + split) * 2;
      ml[0] = -INFINITY;
      ml[1] = 0.f;
    }
    return;
  }
  const int pos = positions[t];
  const int first = (window > 0 && pos - window + 1 > 0) ? pos - window + 1 : 0;
  const int32_t* row = table + static_cast<int64_t>(slots[req]) * table_stride;

  // the 16-key blocks this wave owns: blocks [b0, b1) of the range that holds keys first..pos
  const int blk_first = first / 16;
  const int blk_end = pos / 16 + 1;
  const int nblk = blk_end - blk_first;
  const int per = (nblk + nsplit - 1) / nsplit;
  const int b0 = blk_first + split * per;
  const int b1 = (b0 + per < blk_end) ? b0 + per : blk_end;

  // Q^T as B operand: lane holds head `col`, elements 32c + 8*quad .. +8
  bf16x8_t bq[NC];
  {
    const bf16_t* qh = q + static_cast<int64_t>(t) * q_stride + static_cast<int64_t>(head_live ? head : 0) * D;
#pragma unroll
    for (int c = 0; c < NC; ++c) {
      if (head_live) {
        bq[c] = *reinterpret_cast<const bf16x8_t*>(qh + 32 * c + 8 * quad);
      } else {
#pragma unroll
        for (int e = 0; e < 8; ++e) bq[c][e] = static_cast<__bf16>(0.f);
      }
    }
  }

  f32x4_t o[NJ];
#pragma unroll
  for (int j = 0; j < NJ; ++j) o[j] = f32x4_t{0.f, 0.f, 0.f, 0.f};
  float m = -INFINITY, l = 0.f;

  const int blocks_per_page = page_size / 16;
  for (int b = b0; b < b1; ++b) {
    const int page_idx = b / blocks_per_page;
    const int sub = b - page_idx * blocks_per_page;
    const int page = row[page_idx];
    if (page <= 0 || page >= num_pages) continue;  // a page given back behind the window
    const bf16_t* kb = k_cache + ((static_cast<int64_t>(page) * nkv + hk) * page_size + sub * 16) * D;
    const bf16_t* vb = v_cache + (static_cast<int64_t>(page) * nkv + hk) * D * page_size + sub * 16;

    // S^T = K Q^T: A operand row = key `col`, elements 32c + 8*quad .. +8
    f32x4_t s = f32x4_t{0.f, 0.f, 0.f, 0.f};
    const bf16_t* krow = kb + static_cast<int64_t>(col) * D + 8 * quad;
#pragma unroll
    for (int c = 0; c < NC; ++c) {
      const bf16x8_t a = *reinterpret_cast<const bf16x8_t*>(krow + 32 * c);
      s = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, bq[c], s, 0, 0, 0);
    }
    // V^T rows for the second product, fetched early: row = element 16j + col, keys 4*quad .. +4
    s16x4_t va[NJ];
    const bf16_t* vrow = vb + static_cast<int64_t>(col) * page_size + 4 * quad;
#pragma unroll
    for (int j = 0; j < NJ; ++j)
      va[j] = *reinterpret_cast<const s16x4_t*>(vrow + static_cast<int64_t>(16 * j) * page_size);

    // s[i] belongs to key 16b + 4*quad + i and head `col`
    const int key0 = 16 * b + 4 * quad;
    float sv[4];
    bool ok[4];
    float mx = -INFINITY;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int key = key0 + i;
      ok[i] = key >= first && key <= pos;
      sv[i] = ok[i] ? s[i] * scale_log2e : -INFINITY;
      mx = fmaxf(mx, sv[i]);
    }
    mx = fmaxf(mx, __shfl_xor(mx, 16, 64));
    mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
    const float m_new = fmaxf(m, mx);
    const float m_safe = (m_new == -INFINITY) ? 0.f : m_new;
    const float alpha = __builtin_amdgcn_exp2f(m - m_safe);
    float p[4];
    float ps = 0.f;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      p[i] = __builtin_amdgcn_exp2f(sv[i] - m_safe);  // exp2(-inf) = 0 for masked keys
      ps += p[i];
    }
    ps += __shfl_xor(ps, 16, 64);
    ps += __shfl_xor(ps, 32, 64);
    l = l * alpha + ps;
    m = m_new;

    // P^T as B operand of the 16x16x16 product: k = key 4*quad + i, column = head
    s16x4_t pb;
#pragma unroll
    for (int i = 0; i < 4; ++i) pb[i] = static_cast<short>(f32_to_bf16_bits(p[i]));
    // values of masked keys may be anything (a reused page, NaN): they must not meet the
    // product even with weight zero
    const bool edge = (16 * b + 15 > pos) || (16 * b < first);
#pragma unroll
    for (int j = 0; j < NJ; ++j) {
      s16x4_t a = va[j];
      if (edge) {
#pragma unroll
        for (int i = 0; i < 4; ++i)
          if (!ok[i]) a[i] = 0;
      }
      o[j] = o[j] * alpha;
      o[j] = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(a, pb, o[j], 0, 0, 0);
    }
  }

  if (!head_live) return;
  // o[j][i] = O^T[element 16j + 4*quad + i, head col]
  if (nsplit == 1) {
    const float inv = (l > 0.f) ? 1.f / l : 0.f;
    bf16_t* op = out + (static_cast<int64_t>(t) * nh + head) * D + 4 * quad;
#pragma unroll
    for (int j = 0; j < NJ; ++j) {
      uint2 packed;
      packed.x = f32_to_bf16_bits(o[j][0] * inv) | (static_cast<uint32_t>(f32_to_bf16_bits(o[j][1] * inv)) << 16);
      packed.y = f32_to_bf16_bits(o[j][2] * inv) | (static_cast<uint32_t>(f32_to_bf16_bits(o[j][3] * inv)) << 16);
      *reinterpret_cast<uint2*>(op + 16 * j) = packed;
    }
  } else {
    const int64_t slot_idx = (static_cast<int64_t>(t) * nh + head) * nsplit + split;
    float* po = part_o + slot_idx * D + 4 * quad;
#pragma unroll
    for (int j = 0; j < NJ; ++j) *reinterpret_cast<f32x4_t*>(po + 16 * j) = o[j];
    if (quad == 0) {
      part_ml[slot_idx * 2] = m;
      part_ml[slot_idx * 2 + 1] = l;
    }
  }
}

// out[t, head, :] = sum_s w_s * part_o[s] / sum_s w_s * l_s with w_s = exp2(m_s - max m)
__global__ void decode_combine_kernel(bf16_t* __restrict__ out, const float* __restrict__ part_o,
                                      const float* __restrict__ part_ml, int D, int nsplit) {
  const int64_t th = blockIdx.x;  // token * nh + head
  const float* ml = part_ml + th * nsplit * 2;
  float mmax = -INFINITY;
  for (int s = 0; s < nsplit; ++s) mmax = fmaxf(mmax, ml[2 * s]);
  const float m_safe = (mmax == -INFINITY) ? 0.f : mmax;
  float denom = 0.f;
  for (int s = 0; s < nsplit; ++s) denom += __builtin_amdgcn_exp2f(ml[2 * s] - m_safe) * ml[2 * s + 1];
  const float inv = (denom > 0.f) ? 1.f / denom : 0.f;
  for (int e = threadIdx.x; e < D; e += blockDim.x) {
    float acc = 0.f;
    for (int s = 0; s < nsplit; ++s) {
      const float w = __builtin_amdgcn_exp2f(ml[2 * s] - m_safe);
      if (w > 0.f) acc += w * part_o[(th * nsplit + s) * D + e];
    }
    out[th * D + e] = from_float<bf16_t>(acc * inv);
  }
}

template <int D>
int launch_decode(bf16_t* out, float* part_o, float* part_ml, const bf16_t* q, int64_t q_stride,
                  const bf16_t* k_cache, const bf16_t* v_cache, const int32_t* table,
                  int table_stride, const int32_t* positions, const int32_t* token_req,
                  const int32_t* slots, int T, int nh, int nkv, int page_size, int num_pages,
                  float scale, int window, int nsplit, hipStream_t stream) {
  hipLaunchKernelGGL(decode_attention_kernel<D>, dim3(T, nkv, nsplit), dim3(64), 0, stream, out,
                     part_o, part_ml, q, q_stride, k_cache, v_cache, table, table_stride, positions,
                     token_req, slots, nh, nkv, page_size, num_pages, scale * kLog2e, window, nsplit);
  if (nsplit > 1)
    hipLaunchKernelGGL(decode_combine_kernel, dim3(T * nh), dim3(D < 64 ? 64 : D), 0, stream, out,
                       part_o, part_ml, D, nsplit);
  return kvc_check_launch("kvc_decode_attention");
}

}  // namespace

extern "C" int kvc_decode_attention_supported(int nh, int nkv, int d, int page_size, int dtype) {
  if (dtype != 1) return 0;
  if (nkv <= 0 || nh % nkv || nh / nkv > 16) return 0;
  if (page_size % 16) return 0;
  return d == 32 || d == 64 || d == 96 || d == 128 || d == 160 || d == 192 || d == 224 || d == 256;
}

extern "C" int kvc_decode_attention(void* out, void* part_o, void* part_ml, const void* q,
                                    int64_t q_stride, const void* k_cache, const void* v_cache,
                                    const int32_t* table, int table_stride,
                                    const int32_t* positions, const int32_t* token_req,
                                    const int32_t* slots, int T, int nh, int nkv, int d,
                                    int page_size, int num_pages, float scale, int window,
                                    int nsplit, kvc_stream stream) {
  if (!kvc_decode_attention_supported(nh, nkv, d, page_size, 1))
    return kvc_fail("kvc_decode_attention: unsupported shape (bfloat16, head size a multiple of 32 "
                    "up to 256, at most 16 query heads per kv head, page size a multiple of 16)");
  if (T < 0 || nsplit < 1 || nsplit > 65535 || nkv > 65535 || table_stride <= 0 || num_pages <= 0)
    return kvc_fail("kvc_decode_attention: bad sizes");
  if (q_stride % 8) return kvc_fail("kvc_decode_attention: q rows must be 16-byte aligned");
  if (nsplit > 1 && (part_o == nullptr || part_ml == nullptr))
    return kvc_fail("kvc_decode_attention: splits need a workspace");
  if (T == 0) return 0;
  hipStream_t s = reinterpret_cast<hipStream_t>(stream);
#define KVC_DECODE_CASE(DD)                                                                       \
  case DD:                                                                                        \
    return launch_decode<DD>(static_cast<bf16_t*>(out), static_cast<float*>(part_o),              \
                             static_cast<float*>(part_ml), static_cast<const bf16_t*>(q),         \
                             q_stride, static_cast<const bf16_t*>(k_cache),                       \
                             static_cast<const bf16_t*>(v_cache), table, table_stride, positions, \
                             token_req, slots, T, nh, nkv, page_size, num_pages, scale, window,   \
                             nsplit, s)
  switch (d) {
    KVC_DECODE_CASE(32);
    KVC_DECODE_CASE(64);
    KVC_DECODE_CASE(96);
    KVC_DECODE_CASE(128);
    KVC_DECODE_CASE(160);
    KVC_DECODE_CASE(192);
    KVC_DECODE_CASE(224);
    KVC_DECODE_CASE(256);
  }
#undef KVC_DECODE_CASE
  return kvc_fail("kvc_decode_attention: unsupported head size");
}
