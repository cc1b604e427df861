// Paged attention for single tokens (decode), bfloat16, on the matrix cores, with the
// rotation of the token's query and key and the write of its key and value into the cache
// done by the same kernel.
//
// One block of W waves per (token, kv head, split of the key range); the waves take the
// 16-key blocks of the range in turn.  The query heads that share the kv head are the
// columns of one 16-wide MFMA tile, so every key and value is fetched once for the whole
// group, straight from global memory:
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
// The block first rotates the group's query heads into LDS.  The block whose range holds
// the token's own position also rotates the key, stores key and value in their cache slot
// and keeps both in LDS; the wave that meets the position's 16-key block takes them from
// there, so nothing is read back from global memory in the kernel that wrote it.
//
// The waves' partial results (max, sum, output) are merged through LDS in wave order.
// With more than one split each block writes an unnormalised partial and a second kernel
// combines them; split boundaries depend on the request's length only.  (Letting the last
// block to finish do that combination needs a device-wide fence per block, which costs
// more than the second kernel.)

#include <hip/hip_runtime.h>

#include "attention_combine.h"
#include "device_utils.h"
#include "kvcore_hip.h"

using namespace kvc;

namespace {

typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef short s16x4_t __attribute__((ext_vector_type(4)));
typedef float f32x4_t __attribute__((ext_vector_type(4)));

constexpr float kLog2e = 1.4426950408889634f;
constexpr int kMaxWaves = 8;
constexpr int kQPad = 8;    // bf16 elements between query rows in LDS beyond d
constexpr int kOPad = 16;   // floats between output rows in LDS beyond d
constexpr size_t kLdsLimit = 64 * 1024;

struct DecodeArgs {
  bf16_t* out;
  float* part_o;
  float* part_ml;
  const bf16_t* qkv;  // rows [nh q heads | nkv k heads | nkv v heads] of d
  int64_t qkv_stride;
  bf16_t* k_cache;
  bf16_t* v_cache;
  const int32_t* table;
  int table_stride;
  const int32_t* positions;
  const int32_t* token_req;
  const int32_t* slots;
  const int32_t* token_rows;  // [T] block-table row of each token (-1: padding), or null
  const float* cos_tab;  // [T, rot_dim / 2]
  const float* sin_tab;
  int rot_dim;
  int interleaved;
  int write_kv;  // store the token's key and value (and attend to them from LDS)
  int nh, nkv, page_size, num_pages;
  float scale_log2e;
  int window;
  int nsplit;
  int lds_pages;  // page ids of a block's range that fit in LDS
};

__host__ __device__ inline size_t lds_q_bytes(int g, int d) {
  return (static_cast<size_t>(g) * (d + kQPad) * 2 + 15) / 16 * 16;
}
__host__ __device__ inline size_t lds_kv_bytes(int d) { return static_cast<size_t>(2) * d * 2; }
__host__ __device__ inline size_t lds_ml_bytes(int waves) { return static_cast<size_t>(waves) * 16 * 8; }
__host__ __device__ inline size_t lds_o_bytes(int waves, int g, int d) {
  return static_cast<size_t>(waves) * g * (d + kOPad) * 4;
}
constexpr int kMaxLdsPages = 1024;  // what the choice of waves per block leaves room for
inline size_t lds_total(int waves, int g, int d, int lds_pages) {
  return lds_q_bytes(g, d) + lds_kv_bytes(d) + lds_ml_bytes(waves) + lds_o_bytes(waves, g, d) +
         static_cast<size_t>(lds_pages) * 4;
}

// wide heads keep more registers per lane, so fewer waves fit in a block
template <int D>
constexpr int max_waves() { return D > 128 ? 4 : kMaxWaves; }

template <int D>
__global__ __launch_bounds__(max_waves<D>() * 64) void decode_attention_kernel(const DecodeArgs a) {
  extern __shared__ __attribute__((aligned(16))) unsigned char lds[];
  const int t = blockIdx.x;
  const int hk = blockIdx.y;
  const int split = blockIdx.z;
  const int tid = threadIdx.x;
  const int nthreads = blockDim.x;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int waves = nthreads >> 6;
  const int lane = tid & 63;
  const int col = lane & 15;   // head within the group (B/C column)
  const int quad = lane >> 4;  // 0..3
  const int nh = a.nh, nkv = a.nkv, nsplit = a.nsplit, page_size = a.page_size;
  const int g = nh / nkv;
  const bool head_live = col < g;
  constexpr int NJ = D / 16;  // output row blocks
  constexpr int NC = D / 32;  // 32-wide chunks of the head for Q.K
  constexpr int NBUF = 3;     // 16-key blocks a wave holds: one in work, two on their way

  bf16_t* sq = reinterpret_cast<bf16_t*>(lds);                       // [g][D + kQPad]
  bf16_t* sk = reinterpret_cast<bf16_t*>(lds + lds_q_bytes(g, D));   // [D] key, then [D] value
  bf16_t* sv = sk + D;
  float* sml = reinterpret_cast<float*>(lds + lds_q_bytes(g, D) + lds_kv_bytes(D));  // [waves][16][2]
  float* so = sml + waves * 32;                                      // [waves][g][D + kOPad]
  int32_t* spage = reinterpret_cast<int32_t*>(so + static_cast<int64_t>(waves) * g * (D + kOPad));  // [lds_pages]

  // which row of the block table: one load if the caller resolved it, else two in a chain
  const int pos = __builtin_amdgcn_readfirstlane(a.positions[t]);
  int trow_idx;
  if (a.token_rows != nullptr) {
    trow_idx = a.token_rows[t];
  } else {
    const int req = a.token_req[t];
    trow_idx = req < 0 ? -1 : a.slots[req];
  }
  trow_idx = __builtin_amdgcn_readfirstlane(trow_idx);
  if (trow_idx < 0) {  // padding token
    if (nsplit == 1) {
      for (int idx = tid; idx < g * D; idx += nthreads)
        a.out[(static_cast<int64_t>(t) * nh + hk * g) * D + idx] = from_float<bf16_t>(0.f);
    } else if (tid < g) {
      float* ml = a.part_ml + ((static_cast<int64_t>(t) * nh + hk * g + tid) * nsplit + split) * 2;
      ml[0] = -INFINITY;
      ml[1] = 0.f;
    }
    return;
  }
  const int window = a.window;
  const int first = (window > 0 && pos - window + 1 > 0) ? pos - window + 1 : 0;
  const int32_t* row = a.table + static_cast<int64_t>(trow_idx) * a.table_stride;

  // the 16-key blocks this block owns: [b0, b1) of the range that holds keys first..pos
  const int blk_first = first / 16;
  const int blk_end = pos / 16 + 1;
  const int nblk = blk_end - blk_first;
  const int per = (nblk + nsplit - 1) / nsplit;
  const int b0 = blk_first + split * per;
  const int b1 = (b0 + per < blk_end) ? b0 + per : blk_end;
  const int blk_own = pos / 16;  // the block of the token's own key
  const bool owner = a.write_kv && b0 <= blk_own && blk_own < b1;
  const int blocks_per_page = page_size / 16;

  // the page ids of the range go to LDS, where the walk below reads them
  const int page_lo = b0 / blocks_per_page;
  const int n_range_pages = (b1 > b0) ? (b1 - 1) / blocks_per_page - page_lo + 1 : 0;
  for (int i = tid; i < n_range_pages && i < a.lds_pages; i += nthreads)
    spage[i] = (page_lo + i < a.table_stride) ? row[page_lo + i] : 0;

  // One 16-key block: K rows as A operand (row = key `col`, elements 32c + 8*quad .. +8) and
  // V^T rows (row = element 16j + col, keys 4*quad .. +4).  The loads are issued without any
  // branch around them, so that the waits the compiler places count them exactly and a
  // block's loads stay in flight while earlier blocks are worked on.
  bf16x8_t kb[NBUF][NC];
  s16x4_t vb[NBUF][NJ];
  bool okb[NBUF];
  auto issue_block = [&](int bn, int page, bf16x8_t (&ka)[NC], s16x4_t (&va)[NJ]) -> bool {
    const bool in_range = bn < b1;
    const bool page_ok = page > 0 && page < a.num_pages;  // else given back behind the window
    const bool real = in_range && page_ok;
    const int sub = bn % blocks_per_page;
    // a block that is not there reads one line of the null page with every lane
    const bf16_t* krow = real ? a.k_cache + ((static_cast<int64_t>(page) * nkv + hk) * page_size +
                                             sub * 16 + col) * D + 8 * quad
                              : a.k_cache;
    const bf16_t* vrow = real ? a.v_cache + ((static_cast<int64_t>(page) * nkv + hk) * D + col) * page_size +
                                    sub * 16 + 4 * quad
                              : a.v_cache;
    const int64_t v_step = real ? static_cast<int64_t>(16) * page_size : 0;
    const int k_step = real ? 32 : 0;
#pragma unroll
    for (int c = 0; c < NC; ++c) ka[c] = *reinterpret_cast<const bf16x8_t*>(krow + k_step * c);
#pragma unroll
    for (int j = 0; j < NJ; ++j) va[j] = *reinterpret_cast<const s16x4_t*>(vrow + v_step * j);
    return real;
  };
  auto clamp_block = [&](int bn) -> int { return bn < b1 ? bn : b1 - 1; };

  // the first blocks of this wave are asked for at once, before anything else waits
  const int b_wave = b0 + wave;
  const bool has_work = b_wave < b1;
#pragma unroll
  for (int s = 0; s < NBUF; ++s) okb[s] = false;
  if (has_work) {
    int first_pages[NBUF - 1];
#pragma unroll
    for (int s = 0; s < NBUF - 1; ++s) {
      const int page_idx = clamp_block(b_wave + s * waves) / blocks_per_page;
      first_pages[s] = __builtin_amdgcn_readfirstlane((page_idx < a.table_stride) ? row[page_idx] : 0);
    }
#pragma unroll
    for (int s = 0; s < NBUF - 1; ++s) okb[s] = issue_block(b_wave + s * waves, first_pages[s], kb[s], vb[s]);
  }

  // ---- rotation of the group's queries (and the key) into LDS; key and value into the cache
  {
    const bf16_t* trow = a.qkv + static_cast<int64_t>(t) * a.qkv_stride;
    const int rot_dim = a.rot_dim, half = rot_dim / 2;
    const float* cs = a.cos_tab + static_cast<int64_t>(t) * half;
    const float* sn = a.sin_tab + static_cast<int64_t>(t) * half;
    int64_t k_off = -1, v_off = -1;
    if (owner) {
      const int page = (pos / page_size < a.table_stride) ? row[pos / page_size] : 0;
      if (page > 0 && page < a.num_pages) {
        const int off = pos % page_size;
        k_off = ((static_cast<int64_t>(page) * nkv + hk) * page_size + off) * D;
        v_off = (static_cast<int64_t>(page) * nkv + hk) * D * page_size + off;
      }
    }
    const int n_heads = owner ? g + 1 : g;  // the key is one more head to rotate
    for (int idx = tid; idx < n_heads * D; idx += nthreads) {
      const int hh = idx / D;
      const int e = idx - hh * D;
      const bf16_t* src = (hh < g) ? trow + static_cast<int64_t>(hk * g + hh) * D
                                   : trow + static_cast<int64_t>(nh + hk) * D;
      bf16_t y = src[e];
      if (e < rot_dim) {
        int j, partner;
        bool is_first;
        if (a.interleaved) {
          j = e >> 1;
          is_first = (e & 1) == 0;
          partner = is_first ? e + 1 : e - 1;
        } else {
          is_first = e < half;
          j = is_first ? e : e - half;
          partner = is_first ? e + half : e - half;
        }
        const float c = cs[j], s_ = sn[j];
        const float xe = to_float(y), xp = to_float(src[partner]);
        y = from_float<bf16_t>(is_first ? rotate_first(xe, xp, c, s_) : rotate_second(xp, xe, c, s_));
      }
      if (hh < g) {
        sq[hh * (D + kQPad) + e] = y;
      } else {
        sk[e] = y;
        if (k_off >= 0) a.k_cache[k_off + e] = y;
      }
    }
    if (owner) {
      const bf16_t* vsrc = trow + static_cast<int64_t>(nh + nkv + hk) * D;
      for (int e = tid; e < D; e += nthreads) {
        const bf16_t v = vsrc[e];
        sv[e] = v;
        if (v_off >= 0) a.v_cache[v_off + static_cast<int64_t>(e) * page_size] = v;
      }
    }
  }
  __syncthreads();

  // Q^T as B operand: lane holds head `col`, elements 32c + 8*quad .. +8
  bf16x8_t bq[NC];
#pragma unroll
  for (int c = 0; c < NC; ++c) {
    if (head_live) {
      bq[c] = *reinterpret_cast<const bf16x8_t*>(sq + col * (D + kQPad) + 32 * c + 8 * quad);
    } else {
#pragma unroll
      for (int e = 0; e < 8; ++e) bq[c][e] = static_cast<__bf16>(0.f);
    }
  }

  f32x4_t o[NJ];
#pragma unroll
  for (int j = 0; j < NJ; ++j) o[j] = f32x4_t{0.f, 0.f, 0.f, 0.f};
  float m = -INFINITY, l = 0.f;

  auto work_block = [&](int b, bf16x8_t (&ka)[NC], s16x4_t (&va)[NJ]) {
    if (owner && b == blk_own) {
      // the token's own key and value come from LDS, not from the cache line just written
      const int kk = pos & 15;
      if (col == kk) {
#pragma unroll
        for (int c = 0; c < NC; ++c) ka[c] = *reinterpret_cast<const bf16x8_t*>(sk + 32 * c + 8 * quad);
      }
      if (quad == (kk >> 2)) {
#pragma unroll
        for (int j = 0; j < NJ; ++j) {
          const short bits = static_cast<short>(sv[16 * j + col].bits);
          if ((kk & 3) == 0) va[j][0] = bits;
          if ((kk & 3) == 1) va[j][1] = bits;
          if ((kk & 3) == 2) va[j][2] = bits;
          if ((kk & 3) == 3) va[j][3] = bits;
        }
      }
    }
    f32x4_t s = f32x4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int c = 0; c < NC; ++c) s = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ka[c], bq[c], s, 0, 0, 0);

    // s[i] belongs to key 16b + 4*quad + i and head `col`
    const int key0 = 16 * b + 4 * quad;
    float sv4[4];
    bool ok[4];
    float mx = -INFINITY;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int key = key0 + i;
      ok[i] = key >= first && key <= pos;
      sv4[i] = ok[i] ? s[i] * a.scale_log2e : -INFINITY;
      mx = fmaxf(mx, sv4[i]);
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
      p[i] = __builtin_amdgcn_exp2f(sv4[i] - m_safe);  // exp2(-inf) = 0 for masked keys
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
      s16x4_t vv = va[j];
      if (edge) {
#pragma unroll
        for (int i = 0; i < 4; ++i)
          if (!ok[i]) vv[i] = 0;
      }
      o[j] = o[j] * alpha;
      o[j] = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(vv, pb, o[j], 0, 0, 0);
    }
  };

  // the wave's blocks b_wave, b_wave + waves, ...: while one is worked on, the next two load
  if (has_work) {
    for (int b = b_wave; b < b1; b += NBUF * waves) {
#pragma unroll
      for (int s = 0; s < NBUF; ++s) {
        const int bc = b + s * waves;
        constexpr int kAhead = NBUF - 1;
        const int bn = bc + kAhead * waves;
        const int sn = (s + kAhead) % NBUF;
        const int page = __builtin_amdgcn_readfirstlane(spage[clamp_block(bn) / blocks_per_page - page_lo]);
        okb[sn] = issue_block(bn, page, kb[sn], vb[sn]);
        if (bc < b1 && okb[s]) work_block(bc, kb[s], vb[s]);  // the same for the whole wave
      }
    }
  }

  // ---- merge the waves' partials in wave order
  // o[j][i] = O^T[element 16j + 4*quad + i, head col]
  if (head_live) {
    float* wo = so + (static_cast<int64_t>(wave) * g + col) * (D + kOPad) + 4 * quad;
#pragma unroll
    for (int j = 0; j < NJ; ++j) *reinterpret_cast<f32x4_t*>(wo + 16 * j) = o[j];
    if (quad == 0) {
      sml[(wave * 16 + col) * 2] = m;
      sml[(wave * 16 + col) * 2 + 1] = l;
    }
  }
  __syncthreads();
  for (int idx = tid; idx < g * D; idx += nthreads) {
    const int h = idx / D;
    const int e = idx - h * D;
    float mmax = -INFINITY;
    for (int w = 0; w < waves; ++w) mmax = fmaxf(mmax, sml[(w * 16 + h) * 2]);
    const float m_safe = (mmax == -INFINITY) ? 0.f : mmax;
    float denom = 0.f, acc = 0.f;
    for (int w = 0; w < waves; ++w) {
      const float wgt = __builtin_amdgcn_exp2f(sml[(w * 16 + h) * 2] - m_safe);
      if (wgt > 0.f) {
        denom += wgt * sml[(w * 16 + h) * 2 + 1];
        acc += wgt * so[(static_cast<int64_t>(w) * g + h) * (D + kOPad) + e];
      }
    }
    const int64_t th = static_cast<int64_t>(t) * nh + hk * g + h;
    if (nsplit == 1) {
      a.out[th * D + e] = from_float<bf16_t>(denom > 0.f ? acc / denom : 0.f);
    } else {
      a.part_o[(th * nsplit + split) * D + e] = acc;
      if (e == 0) {
        a.part_ml[(th * nsplit + split) * 2] = mmax;
        a.part_ml[(th * nsplit + split) * 2 + 1] = denom;
      }
    }
  }
}

// out[t, head, :] = sum_s w_s * part_o[s] / sum_s w_s * l_s with w_s = exp2(m_s - max m).
// Every wave works the weights out for itself (lane s holds split s), so nothing waits on
// another wave; the partial outputs are asked for before the weights are known.
constexpr int kMaxSplits = kMaxAttentionSplits;
__global__ void decode_combine_kernel(bf16_t* __restrict__ out, const float* __restrict__ part_o,
                                      const float* __restrict__ part_ml, int D, int nsplit) {
  const int64_t th = blockIdx.x;  // token * nh + head
  const int lane = threadIdx.x & 63;
  const float* ml = part_ml + th * nsplit * 2;
  const float* po = part_o + th * nsplit * D;
  float m_s = -INFINITY, l_s = 0.f;
  if (lane < nsplit) {
    m_s = ml[2 * lane];
    l_s = ml[2 * lane + 1];
  }
  for (int e0 = 0; e0 < D; e0 += blockDim.x) {
    const int e = e0 + threadIdx.x;
    const bool live = e < D;
    float acc = 0.f;
    float mmax = wave_max(m_s);
    const float m_safe = (mmax == -INFINITY) ? 0.f : mmax;
    const float w_lane = __builtin_amdgcn_exp2f(m_s - m_safe);  // 0 for lanes beyond nsplit
    const float denom = wave_sum(w_lane * l_s);
    for (int s0 = 0; s0 < nsplit; s0 += 4) {
      float v[4];
#pragma unroll
      for (int i = 0; i < 4; ++i)
        v[i] = (live && s0 + i < nsplit) ? po[static_cast<int64_t>(s0 + i) * D + e] : 0.f;
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const float w = __shfl(w_lane, (s0 + i) & 63, 64);
        if (s0 + i < nsplit && w > 0.f) acc += w * v[i];
      }
    }
    if (live) out[th * D + e] = from_float<bf16_t>(denom > 0.f ? acc / denom : 0.f);
  }
}

int decode_waves(int g, int d) {
  int waves = d > 128 ? 4 : kMaxWaves;
  while (waves > 1 && lds_total(waves, g, d, kMaxLdsPages) > kLdsLimit) waves /= 2;
  return waves;
}

template <int D>
int launch_decode(DecodeArgs& args, int T, hipStream_t stream) {
  const int g = args.nh / args.nkv;
  // a split's range of pages always fits: the table's width cut into nsplit parts, and slack
  args.lds_pages = (args.table_stride + args.nsplit - 1) / args.nsplit + 2;
  if (args.lds_pages > args.table_stride) args.lds_pages = args.table_stride;
  int waves = decode_waves(g, D);
  // more blocks than compute units: smaller blocks pack better
  if (static_cast<int64_t>(T) * args.nkv * args.nsplit > kvc_device_compute_units() && waves > 4) waves = 4;
  while (waves > 1 && lds_total(waves, g, D, args.lds_pages) > kLdsLimit) waves /= 2;
  if (lds_total(waves, g, D, args.lds_pages) > kLdsLimit)
    return kvc_fail("kvc_decode_attention: the block table is wider than kvc_decode_attention_max_table "
                    "allows for one split");
  hipLaunchKernelGGL(decode_attention_kernel<D>, dim3(T, args.nkv, args.nsplit), dim3(waves * 64),
                     lds_total(waves, g, D, args.lds_pages), stream, args);
  if (args.nsplit > 1)
    hipLaunchKernelGGL(decode_combine_kernel, dim3(T * args.nh), dim3((D + 63) / 64 * 64), 0, stream,
                       args.out, args.part_o, args.part_ml, D, args.nsplit);
  return kvc_check_launch("kvc_decode_attention");
}

}  // namespace

int kvc::launch_attention_combine(bf16_t* out, const float* part_o, const float* part_ml, int64_t rows,
                                  int d, int nsplit, hipStream_t stream) {
  if (rows <= 0) return 0;
  if (rows > 0x7fffffff || nsplit < 1 || nsplit > kMaxAttentionSplits)
    return kvc_fail("attention combine: bad sizes");
  hipLaunchKernelGGL(decode_combine_kernel, dim3(static_cast<unsigned>(rows)), dim3((d + 63) / 64 * 64), 0,
                     stream, out, part_o, part_ml, d, nsplit);
  return kvc_check_launch("attention combine");
}

extern "C" int kvc_decode_attention_supported(int nh, int nkv, int d, int page_size, int dtype) {
  if (dtype != 1) return 0;
  if (nkv <= 0 || nh % nkv || nh / nkv > 16) return 0;
  if (page_size % 16) return 0;
  return d == 32 || d == 64 || d == 96 || d == 128 || d == 160 || d == 192 || d == 224 || d == 256;
}

extern "C" int kvc_decode_attention_max_table(int nh, int nkv, int d) {
  if (nkv <= 0 || nh % nkv || d <= 0) return 0;
  const size_t fixed = lds_total(1, nh / nkv, d, 0);
  if (fixed >= kLdsLimit) return 0;
  // launch_decode keeps two entries of slack beyond a split's share of the table
  return static_cast<int>((kLdsLimit - fixed) / 4) - 2;
}

extern "C" int kvc_decode_attention_waves(int nh, int nkv, int d) {
  if (nkv <= 0 || nh % nkv || d <= 0) return 0;
  return decode_waves(nh / nkv, d);
}

extern "C" int kvc_decode_attention(void* out, void* part_o, void* part_ml, const void* qkv,
                                    int64_t qkv_stride, void* k_cache, void* v_cache,
                                    const int32_t* table, int table_stride,
                                    const int32_t* positions, const int32_t* token_req,
                                    const int32_t* slots, const int32_t* token_rows,
                                    const float* cos_tab, const float* sin_tab, int rot_dim, int interleaved, int write_kv, int T, int nh,
                                    int nkv, int d, int page_size, int num_pages, float scale,
                                    int window, int nsplit, kvc_stream stream) {
  if (!kvc_decode_attention_supported(nh, nkv, d, page_size, 1))
    return kvc_fail("kvc_decode_attention: unsupported shape (bfloat16, head size a multiple of 32 "
                    "up to 256, at most 16 query heads per kv head, page size a multiple of 16)");
  if (T < 0 || nsplit < 1 || nsplit > kMaxSplits || nkv > 65535 || table_stride <= 0 || num_pages <= 0)
    return kvc_fail("kvc_decode_attention: bad sizes (at most 64 splits)");
  if (qkv_stride % 8 || qkv_stride < static_cast<int64_t>(nh + (write_kv ? 2 * nkv : 0)) * d)
    return kvc_fail("kvc_decode_attention: token rows must be 16-byte aligned and hold q (and k, v)");
  if (rot_dim < 0 || rot_dim > d || rot_dim % 2)
    return kvc_fail("kvc_decode_attention: the rotated width must be even and at most the head size");
  if (rot_dim > 0 && (cos_tab == nullptr || sin_tab == nullptr))
    return kvc_fail("kvc_decode_attention: rotation needs its cos and sin tables");
  if (nsplit > 1 && (part_o == nullptr || part_ml == nullptr))
    return kvc_fail("kvc_decode_attention: splits need a workspace");
  if (T == 0) return 0;
  DecodeArgs args;
  args.out = static_cast<bf16_t*>(out);
  args.part_o = static_cast<float*>(part_o);
  args.part_ml = static_cast<float*>(part_ml);
  args.qkv = static_cast<const bf16_t*>(qkv);
  args.qkv_stride = qkv_stride;
  args.k_cache = static_cast<bf16_t*>(k_cache);
  args.v_cache = static_cast<bf16_t*>(v_cache);
  args.table = table;
  args.table_stride = table_stride;
  args.positions = positions;
  args.token_req = token_req;
  args.slots = slots;
  args.token_rows = token_rows;
  args.cos_tab = cos_tab;
  args.sin_tab = sin_tab;
  args.rot_dim = rot_dim;
  args.interleaved = interleaved;
  args.write_kv = write_kv;
  args.nh = nh;
  args.nkv = nkv;
  args.page_size = page_size;
  args.num_pages = num_pages;
  args.scale_log2e = scale * kLog2e;
  args.window = window;
  args.nsplit = nsplit;
  hipStream_t s = reinterpret_cast<hipStream_t>(stream);
  switch (d) {
    case 32: return launch_decode<32>(args, T, s);
    case 64: return launch_decode<64>(args, T, s);
    case 96: return launch_decode<96>(args, T, s);
    case 128: return launch_decode<128>(args, T, s);
    case 160: return launch_decode<160>(args, T, s);
    case 192: return launch_decode<192>(args, T, s);
    case 224: return launch_decode<224>(args, T, s);
    case 256: return launch_decode<256>(args, T, s);
  }
  return kvc_fail("kvc_decode_attention: unsupported head size");
}
