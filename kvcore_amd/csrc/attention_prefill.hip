// Paged attention for portions of prompts, bfloat16, on the matrix cores.
//
// A block of W = 4 or 8 waves owns up to 16*W*CT query rows of one request and one kv head:
// BQ = 16*W*CT / g consecutive tokens times the g query heads that share the kv head.
// It walks the request's keys in tiles of 64 (128 for eight waves on heads of 64), staged
// once through LDS for all its waves (two tiles of LDS: while one is read, the next is
// written, one barrier a tile):
// K pages as they lie in the cache ([key, d], rows padded against bank conflicts) and V
// pages ([d, key]) regrouped so that operand reads are contiguous.  Per wave:
//
//   S^T[16 keys, 16 rows]  = K[16 keys, d]   * Q^T[d, 16 rows]        (16x16x32, per key block)
//   O^T[d, 16 rows]       += V^T[d, 32 keys] * P^T[32 keys, 16 rows]  (16x16x32, per two key blocks)
//
// A lane's four accumulator values of S^T for key blocks a and b are the eight values of
// the B operand of the second product, if the product's k index 8*quad + e stands for key
// 4*quad + e of block a (e < 4) or key 4*quad + e - 4 of block b: V is laid out in LDS to
// match, so the probabilities stay in registers.  Softmax state is float32 per row; the
// running output is rescaled only when a row's maximum moved by more than 2^8.
// A key is visible to a row iff first <= key <= the row's position; keys beyond the
// request's last position and pages given back behind a window are zeroed on their way
// into LDS, so nothing that was not written by this request reaches a product.

#include <hip/hip_runtime.h>

#include <cstdio>

#include <cstdlib>

#include "attention_combine.h"
#include "device_utils.h"
#include "kvcore_hip.h"

using namespace kvc;

namespace {

typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef short s16x4_t __attribute__((ext_vector_type(4)));
typedef float f32x4_t __attribute__((ext_vector_type(4)));

constexpr float kLog2e = 1.4426950408889634f;

// four float32 to four bfloat16 (round to nearest even) with the hardware's packed convert
__device__ __forceinline__ s16x4_t pack_bf16x4(const float* p) {
  typedef __bf16 bf16x4_t __attribute__((ext_vector_type(4)));
  bf16x4_t v;
#pragma unroll
  for (int i = 0; i < 4; ++i) v[i] = static_cast<__bf16>(p[i]);
  return *reinterpret_cast<s16x4_t*>(&v);
}


// A row of S^T lies in the four lanes col, col + 16, col + 32 and col + 48.  Their maximum and
// their sum by the two lane-swap instructions of gfx950: registers only, where a shuffle goes
// through LDS and back.
typedef unsigned u32x2_t __attribute__((ext_vector_type(2)));
__device__ __forceinline__ float quad_max(float v) {
  const unsigned u = __float_as_uint(v);
  const u32x2_t a = __builtin_amdgcn_permlane16_swap(u, u, false, false);
  const unsigned w = __float_as_uint(fmaxf(__uint_as_float(a[0]), __uint_as_float(a[1])));
  const u32x2_t b = __builtin_amdgcn_permlane32_swap(w, w, false, false);
  return fmaxf(__uint_as_float(b[0]), __uint_as_float(b[1]));
}
__device__ __forceinline__ float quad_sum(float v) {
  const unsigned u = __float_as_uint(v);
  const u32x2_t a = __builtin_amdgcn_permlane16_swap(u, u, false, false);
  const unsigned w = __float_as_uint(__uint_as_float(a[0]) + __uint_as_float(a[1]));
  const u32x2_t b = __builtin_amdgcn_permlane32_swap(w, w, false, false);
  return __uint_as_float(b[0]) + __uint_as_float(b[1]);
}

// KB: 16-key blocks per LDS tile
template <int D, int KB>
constexpr int tile_bytes() {
  return KB * 16 * (D + 16) * 2 + KB * D * 16 * 2;  // K rows padded, then V
}

// W: waves of a block (4 or 8).  Eight waves stage each key tile for twice the rows, which
// halves the block's loads and LDS writes per row; a compute unit then holds one block.
template <int D, int CT, int KB, int W>
__global__ __launch_bounds__(W * 64, (W == 4) ? 2 : 1) void prefill_attention_kernel(
    bf16_t* __restrict__ out, const bf16_t* __restrict__ q, int64_t q_stride,
    const bf16_t* __restrict__ k_cache, const bf16_t* __restrict__ v_cache,
    const int32_t* __restrict__ table, int table_stride, const int32_t* __restrict__ positions,
    const int32_t* __restrict__ q_start, const int32_t* __restrict__ slots, int num_reqs, int nh,
    int nkv, int page_size, int num_pages, float scale_log2e, int window,
    float* __restrict__ part_o, float* __restrict__ part_ml, int single,
    const float* __restrict__ cos_tab, const float* __restrict__ sin_tab, int rot_dim, int interleaved) {
  constexpr int kKeyBlocks = KB;
  constexpr int NJ = D / 16;
  constexpr int NC = D / 32;
  // padded K row in LDS (elements): with 32 bytes of padding the operand reads (16 rows x 4
  // pieces of 16 bytes a wave) meet no bank conflict; with 16 they took 1.45 times as long
  constexpr int KROW = D + 16;
  constexpr int K_ELEMS = kKeyBlocks * 16 * KROW;
  constexpr int TILE_ELEMS = tile_bytes<D, KB>() / 2;
  extern __shared__ __attribute__((aligned(16))) bf16_t tiles[];  // two tiles: [K | V] each

  const int g = nh / nkv;
  const int bq = (16 * W * CT) / g;  // tokens per block
  // Workgroups go to the chip's eight dies in turn (workgroup id modulo 8) and every die has
  // an L2 of its own, while all blocks of a kv head read the same keys and values.  So a kv
  // head's blocks get ids that land on one die (with fewer than eight kv heads, on 8 / nkv
  // dies): the die's L2 then holds one head's keys and values instead of every head's.
  // Head counts that neither divide eight nor are divided by it are dealt out plainly.
  int hk, block_index;
  {
    const int lin = blockIdx.x;  // the grid is a multiple of 8 wide
    const int die = lin & 7, turn = lin >> 3;
    if ((nkv & 7) == 0) {
      const int per_die = nkv >> 3;
      hk = die + 8 * (turn % per_die);
      block_index = turn / per_die;
    } else if (8 % nkv == 0) {
      hk = die % nkv;
      block_index = turn * (8 / nkv) + die / nkv;
    } else {
      hk = lin % nkv;
      block_index = lin / nkv;
    }
  }
  const int tid = threadIdx.x;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int lane = tid & 63;
  const int col = lane & 15;
  const int quad = lane >> 4;

  // Which request and which two of its token tiles.  Under the causal mask a request's late
  // tiles see many keys and its early tiles few, so a block takes tile n-1-p and then tile p
  // (p < n/2; the middle tile of an odd count once): every block of a request then walks
  // about the same number of key tiles.  Pairs are numbered request by request.
  int req = -1, pair = 0, n_tiles = 0, q_begin = 0, q_end = 0;
  {
    int idx = block_index;
    for (int r = 0; r < num_reqs; ++r) {
      const int b = q_start[r], e = q_start[r + 1];
      const int tiles_r = (e - b + bq - 1) / bq;
      const int pairs_r = single ? tiles_r : (tiles_r + 1) / 2;
      if (idx < pairs_r) {
        req = r;
        pair = idx;
        n_tiles = tiles_r;
        q_begin = b;
        q_end = e;
        break;
      }
      idx -= pairs_r;
    }
  }
  if (req < 0) return;  // the grid is an upper bound on the number of pairs
  const int32_t* row_table = table + static_cast<int64_t>(slots[req]) * table_stride;
  for (int turn = 0; turn < 2; ++turn) {
  const int tile = (turn == 0) ? n_tiles - 1 - pair : pair;
  if (turn == 1 && (single || tile == n_tiles - 1 - pair)) break;  // the middle tile was the first turn
  if (turn == 1) __syncthreads();  // the first turn's last tile has been consumed by every wave
  const int t0 = q_begin + tile * bq;
  const int t_end = (t0 + bq < q_end) ? t0 + bq : q_end;
  const int n_tok = t_end - t0;
  const int pos_lo = positions[t0];
  const int pos_hi = pos_lo + n_tok - 1;  // positions rise by one along a request's tokens
  const int first_lo = (window > 0 && pos_lo - window + 1 > 0) ? pos_lo - window + 1 : 0;

  // this lane's rows: column `col` of tile ct is row (wave*CT + ct)*16 + col of the block
  int my_pos[CT], my_first[CT], my_tok[CT], my_head[CT];
  bool live[CT];
  bf16x8_t qb[CT][NC];
#pragma unroll
  for (int ct = 0; ct < CT; ++ct) {
    const int rho = (wave * CT + ct) * 16 + col;
    const int tq = rho / g;
    live[ct] = tq < n_tok;
    my_tok[ct] = t0 + (live[ct] ? tq : 0);
    my_head[ct] = hk * g + rho % g;
    my_pos[ct] = live[ct] ? pos_lo + tq : -1;  // positions rise by one along a request's tokens
    my_first[ct] = (window > 0 && my_pos[ct] - window + 1 > 0) ? my_pos[ct] - window + 1 : 0;
    const bf16_t* qp = q + static_cast<int64_t>(my_tok[ct]) * q_stride +
                       static_cast<int64_t>(my_head[ct]) * D + 8 * quad;
#pragma unroll
    for (int c = 0; c < NC; ++c) {
      if (live[ct]) {
        qb[ct][c] = *reinterpret_cast<const bf16x8_t*>(qp + 32 * c);
      } else {
#pragma unroll
        for (int e = 0; e < 8; ++e) qb[ct][c][e] = static_cast<__bf16>(0.f);
      }
    }
    // With tables the queries arrive unrotated and are rotated here, in registers, exactly as
    // the kernel that rotates in memory would have (float32 products, rounded once): a lane
    // holds both elements of every pair, since rot_dim is a multiple of 64 (of 32 for
    // neighbouring pairs).  The query rows then need not be written and read again.
    if (cos_tab != nullptr && live[ct]) {
      const int half = rot_dim >> 1;
      const float* cs = cos_tab + static_cast<int64_t>(my_tok[ct]) * half;
      const float* sn = sin_tab + static_cast<int64_t>(my_tok[ct]) * half;
      if (interleaved) {
#pragma unroll
        for (int c = 0; c < NC; ++c) {
          if (32 * c < rot_dim) {  // uniform
            const int j0 = 16 * c + 4 * quad;
            const f32x4_t cv = *reinterpret_cast<const f32x4_t*>(cs + j0);
            const f32x4_t sv = *reinterpret_cast<const f32x4_t*>(sn + j0);
#pragma unroll
            for (int e = 0; e < 4; ++e) {
              const float x0 = static_cast<float>(qb[ct][c][2 * e]);
              const float x1 = static_cast<float>(qb[ct][c][2 * e + 1]);
              qb[ct][c][2 * e] = static_cast<__bf16>(rotate_first(x0, x1, cv[e], sv[e]));
              qb[ct][c][2 * e + 1] = static_cast<__bf16>(rotate_second(x0, x1, cv[e], sv[e]));
            }
          }
        }
      } else {
        // element j < half pairs with j + half: register c with register c + half / 32
#pragma unroll
        for (int span = 1; span <= NC / 2; ++span) {
          if (half == 32 * span) {  // uniform
#pragma unroll
            for (int c = 0; c < span; ++c) {
              const int j0 = 32 * c + 8 * quad;
#pragma unroll
              for (int e4 = 0; e4 < 2; ++e4) {
                const f32x4_t cv = *reinterpret_cast<const f32x4_t*>(cs + j0 + 4 * e4);
                const f32x4_t sv = *reinterpret_cast<const f32x4_t*>(sn + j0 + 4 * e4);
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                  const float x0 = static_cast<float>(qb[ct][c][4 * e4 + e]);
                  const float x1 = static_cast<float>(qb[ct][c + span][4 * e4 + e]);
                  qb[ct][c][4 * e4 + e] = static_cast<__bf16>(rotate_first(x0, x1, cv[e], sv[e]));
                  qb[ct][c + span][4 * e4 + e] = static_cast<__bf16>(rotate_second(x0, x1, cv[e], sv[e]));
                }
              }
            }
          }
        }
      }
    }
  }
  // Bounds of what this wave's live rows can see, from the wave's first and last row alone
  // (positions rise by one along the tokens).  They are scalars, so that the conditions on
  // them below are scalar branches: matrix instructions must be skipped by a branch, never by
  // a lane mask.
  const int wave_tq_lo = (wave * CT * 16) / g;
  const int wave_tq_hi = ((wave * CT + CT) * 16 - 1) / g;
  const bool wave_live = wave_tq_lo < n_tok;
  const int wave_pos_hi = wave_live ? pos_lo + (wave_tq_hi < n_tok ? wave_tq_hi : n_tok - 1) : -1;
  const int wave_pos_lo = wave_live ? pos_lo + wave_tq_lo : 0x7fffffff;
  const int wave_first_hi = (wave_live && window > 0 && wave_pos_hi - window + 1 > 0) ? wave_pos_hi - window + 1 : 0;

  f32x4_t o_acc[CT][NJ];
  // m: the reference maximum of the raw (unscaled) scores, the same in the four lanes of a row;
  // l: the sum of this lane's probabilities
  float m[CT], l[CT];
#pragma unroll
  for (int ct = 0; ct < CT; ++ct) {
    m[ct] = -INFINITY;
    l[ct] = 0.f;
#pragma unroll
    for (int j = 0; j < NJ; ++j) o_acc[ct][j] = f32x4_t{0.f, 0.f, 0.f, 0.f};
  }

  const int blocks_per_page = page_size / 16;
  const int kb_first = first_lo / 16;
  const int kb_end = pos_hi / 16 + 1;
  constexpr int K_CHUNKS = kKeyBlocks * 16 * (D / 8);  // 16-byte pieces of a K tile
  constexpr int V_CHUNKS = kKeyBlocks * D * 2;         // 16-byte pieces of a V tile
  constexpr int THREADS = W * 64;
  constexpr int K_PER_THREAD = K_CHUNKS / THREADS;
  constexpr int V_PER_THREAD = V_CHUNKS / THREADS;
  uint4 kreg[K_PER_THREAD], vreg[V_PER_THREAD];

  // Fetch the tile that starts at key block kb0 into registers.  Keys beyond the request's
  // last position, key blocks beyond the range and pages that are gone arrive as zeros.
  // The key blocks that a thread fetches from are the same for its whole wave (K: 16 rows of
  // 16-byte pieces are 128 or 256 threads; V: a key block takes 2 * D threads), so a wave looks
  // up the pages of its own key blocks only, as scalars.
  constexpr int PIECES = D / 8;                    // 16-byte pieces of a K row
  constexpr int ROWS_PER_STEP = THREADS / PIECES;  // K rows that the block fetches per step
  // V: a key block's rows of the head times its two halves of 8 keys take V_THREADS threads;
  // the block's threads form V_GROUPS such groups, each with an even number of key blocks
  constexpr int V_THREADS = 2 * D;
  constexpr int V_GROUPS = THREADS / V_THREADS;
  static_assert(THREADS % V_THREADS == 0 && kKeyBlocks % (2 * V_GROUPS) == 0 &&
                    V_PER_THREAD == kKeyBlocks / V_GROUPS && (kKeyBlocks * 16) % ROWS_PER_STEP == 0 &&
                    V_THREADS % 64 == 0 && (16 * PIECES) % 64 == 0,
                "tile shape and block size do not fit");
  const int v_group = (V_GROUPS == 1) ? 0 : __builtin_amdgcn_readfirstlane(tid / V_THREADS);  // key blocks v_group * V_PER_THREAD ...
  const int v_rem = tid % V_THREADS;                                    // (row of the head) * 2 + half
  const int k_row0 = tid / PIECES;  // this thread's K row within a step
  const int k_piece = tid % PIECES;
  // the key block within a step's rows that this wave fetches K from (steps of more than 16 rows)
  const int k_block0 = (ROWS_PER_STEP <= 16) ? 0 : __builtin_amdgcn_readfirstlane(k_row0 >> 4);
  // element offsets of this thread's pieces within a key block's K rows and V rows
  int k_off[K_PER_THREAD], v_off[V_PER_THREAD];
#pragma unroll
  for (int i = 0; i < K_PER_THREAD; ++i)
    k_off[i] = ((i * ROWS_PER_STEP + k_row0) & 15) * D + k_piece * 8;
#pragma unroll
  for (int i = 0; i < V_PER_THREAD; ++i) {
    v_off[i] = (v_rem >> 1) * page_size + (v_rem & 1) * 8;
  }
  // Where the key blocks of a tile lie.  Lane i of every wave looks up key block kb0 + i of
  // the tile with one vector load (`lookup_issue`), one tile before the tile is fetched; the
  // page comes back while the tile before is worked on, and `lookup_finish` turns it into the
  // element offsets of the block's K rows and V rows in their planes (-1: no such block, or
  // not a page), which the fetch then reads as scalars from the lanes of its own key blocks.
  // (Scalar loads, one per key block with a wait and three branches each, cost a tenth of the
  // kernel.)
  const int sub_mask = blocks_per_page - 1;
  const int sub_shift = (blocks_per_page & sub_mask) == 0 ? __builtin_ctz(blocks_per_page) : -1;
  const int64_t page_elems = static_cast<int64_t>(nkv) * page_size * D;  // of one plane
  const int64_t head_elems = static_cast<int64_t>(hk) * page_size * D;
  const int lk_lane = lane & 15;
  int lk_page = 0, lk_sub = 0;
  auto lookup_issue = [&](int kb0) {
    const int kb = kb0 + lk_lane;
    const bool there = lk_lane < kKeyBlocks && kb < kb_end;
    int page_index;
    if (sub_shift >= 0) {  // uniform
      page_index = kb >> sub_shift;
      lk_sub = kb & sub_mask;
    } else {
      page_index = kb / blocks_per_page;
      lk_sub = kb - page_index * blocks_per_page;
    }
    lk_sub = there ? lk_sub : -1;
    lk_page = row_table[there ? page_index : 0];
  };
  // whether step i of the K fetch and piece i of the V fetch lie in the same key block for all i
  constexpr bool kSameBlocks = ROWS_PER_STEP == 16 && V_GROUPS == 1;
  auto lookup_finish = [&](int64_t (&kbase)[K_PER_THREAD], int64_t (&vbase)[V_PER_THREAD]) -> bool {
    const bool ok = lk_sub >= 0 && lk_page > 0 && lk_page < num_pages;
    const int64_t at = lk_page * page_elems + head_elems;
    const int64_t k_at = ok ? at + lk_sub * (16 * D) : -1;
    const int64_t v_at = ok ? at + lk_sub * 16 : -1;
    auto pick = [&](int64_t v, int from) -> int64_t {
      const uint32_t lo = __builtin_amdgcn_readlane(static_cast<int>(static_cast<uint64_t>(v) & 0xffffffffu), from);
      const uint32_t hi = __builtin_amdgcn_readlane(static_cast<int>(static_cast<uint64_t>(v) >> 32), from);
      return static_cast<int64_t>((static_cast<uint64_t>(hi) << 32) | lo);
    };
#pragma unroll
    for (int i = 0; i < K_PER_THREAD; ++i)
      kbase[i] = pick(k_at, kSameBlocks ? i : (i * ROWS_PER_STEP) / 16 + k_block0);
#pragma unroll
    for (int i = 0; i < V_PER_THREAD; ++i) vbase[i] = pick(v_at, kSameBlocks ? i : v_group * V_PER_THREAD + i);
    // every key block of the tile is there (lanes beyond the tile's blocks do not count)
    return __ballot(ok || lk_lane >= kKeyBlocks) == ~0ull;
  };
  auto fetch_tile = [&](int kb0, const int64_t (&kbase)[K_PER_THREAD], const int64_t (&vbase)[V_PER_THREAD],
                        bool all_there) {
    const bool tail = (kb0 + kKeyBlocks) * 16 > pos_hi + 1;  // uniform: some keys are not the request's
    if (!tail && all_there) {
      // every key of the tile is the request's and on a page: a scalar base and a fixed offset
      // per piece, and no branch between the loads
#pragma unroll
      for (int i = 0; i < K_PER_THREAD; ++i)
        kreg[i] = *reinterpret_cast<const uint4*>(k_cache + kbase[i] + k_off[i]);
#pragma unroll
      for (int i = 0; i < V_PER_THREAD; ++i)
        vreg[i] = *reinterpret_cast<const uint4*>(v_cache + vbase[i] + v_off[i]);
      return;
    }
#pragma unroll
    for (int i = 0; i < K_PER_THREAD; ++i) {
      const int key_row = i * ROWS_PER_STEP + k_row0;  // within the tile
      uint4 val = make_uint4(0u, 0u, 0u, 0u);
      if (kbase[i] >= 0 && kb0 * 16 + key_row <= pos_hi)
        val = *reinterpret_cast<const uint4*>(k_cache + kbase[i] + k_off[i]);
      kreg[i] = val;
    }
#pragma unroll
    for (int i = 0; i < V_PER_THREAD; ++i) {
      // this thread's pieces: both key blocks of a pair, one row of the head, one half of 16 keys
      const int kbi = v_group * V_PER_THREAD + i;
      const int half = v_rem & 1;
      uint4 val = make_uint4(0u, 0u, 0u, 0u);
      const int key0 = (kb0 + kbi) * 16 + half * 8;
      if (vbase[i] >= 0 && key0 <= pos_hi) {
        val = *reinterpret_cast<const uint4*>(v_cache + vbase[i] + v_off[i]);
        const int n_ok = pos_hi - key0 + 1;  // keys key0 .. key0+7 beyond pos_hi are not this request's
        if (n_ok < 8) {
          uint32_t w[4] = {val.x, val.y, val.z, val.w};
#pragma unroll
          for (int e = 0; e < 8; ++e)
            if (e >= n_ok) w[e >> 1] &= (e & 1) ? 0x0000ffffu : 0xffff0000u;
          val = make_uint4(w[0], w[1], w[2], w[3]);
        }
      }
      vreg[i] = val;
    }
  };
  // Registers to LDS.  K: [key][KROW].  V: [pair of key blocks][16-row group j][quad][row in
  // group, flipped by 8 for quads 2 and 3][8 keys], the eight keys being 4*quad .. +4 of the
  // pair's first block and then of its second, so that the 64 lanes of an A-operand read
  // (lane = quad*16 + row) touch 1024 consecutive bytes.
  auto store_tile = [&](int buf) {
    bf16_t* k_lds = tiles + buf * TILE_ELEMS;
    bf16_t* v_lds = k_lds + K_ELEMS;
#pragma unroll
    for (int i = 0; i < K_PER_THREAD; ++i)
      *reinterpret_cast<uint4*>(k_lds + (i * ROWS_PER_STEP + k_row0) * KROW + k_piece * 8) = kreg[i];
    // A thread holds the same eight keys of both key blocks of a pair (head size 128: two
    // pairs), so it stores whole 16-byte slots: [4 keys of the first block | 4 of the second]
    // for quad 2*half and for quad 2*half + 1.  The row within the 16-row group is flipped by
    // 8 for quads 2 and 3, so that the 16 lanes that store together (8 rows x 2 halves) hit
    // 16 different slots; the reads flip it back.
#pragma unroll
    for (int pr = 0; pr < V_PER_THREAD / 2; ++pr) {
      const int pair = v_group * (V_PER_THREAD / 2) + pr;
      const int drow = v_rem >> 1;
      const int half = v_rem & 1;
      const uint4 a = vreg[2 * pr], b = vreg[2 * pr + 1];
      bf16_t* dst = v_lds + (((pair * NJ + (drow >> 4)) * 4 + 2 * half) * 16 + ((drow & 15) ^ (8 * half))) * 8;
      *reinterpret_cast<uint4*>(dst) = make_uint4(a.x, a.y, b.x, b.y);
      *reinterpret_cast<uint4*>(dst + 16 * 8) = make_uint4(a.z, a.w, b.z, b.w);
    }
  };

  const float unit = 8.f / scale_log2e;  // 2^8 in units of the raw scores
  auto work_tile = [&](int kb0, int buf) {
    const bf16_t* k_lds = tiles + buf * TILE_ELEMS;
    const bf16_t* v_lds = k_lds + K_ELEMS;
    // ---- raw scores of the tile for this wave's rows.  The operand reads of two key blocks
    // are asked for while the matrix instructions of the two before them run (left to itself
    // the compiler asks for each read one instruction before its use, and every matrix
    // instruction then waits out the latency of LDS); the two blocks' sums are interleaved so
    // that no instruction waits for the one before it.
    f32x4_t s[CT][kKeyBlocks];
    constexpr int GK = (CT == 1) ? 2 : 1;  // key blocks a group
    static_assert(kKeyBlocks % GK == 0, "the key blocks of a tile must come in whole groups");
    bf16x8_t ka[2][GK][NC];
    auto read_keys = [&](int grp, bf16x8_t (&dst)[GK][NC]) {
#pragma unroll
      for (int b = 0; b < GK; ++b)
#pragma unroll
        for (int c = 0; c < NC; ++c)
          dst[b][c] = *reinterpret_cast<const bf16x8_t*>(k_lds + ((grp * GK + b) * 16 + col) * KROW + 32 * c + 8 * quad);
    };
    read_keys(0, ka[0]);
#pragma unroll
    for (int grp = 0; grp < kKeyBlocks / GK; ++grp) {
      if (grp + 1 < kKeyBlocks / GK) read_keys(grp + 1, ka[(grp + 1) & 1]);
      __builtin_amdgcn_sched_barrier(0);
      f32x4_t acc[CT][GK];
#pragma unroll
      for (int c = 0; c < NC; ++c)
#pragma unroll
        for (int ct = 0; ct < CT; ++ct)
#pragma unroll
          for (int b = 0; b < GK; ++b)
            acc[ct][b] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(
                ka[grp & 1][b][c], qb[ct][c], c == 0 ? f32x4_t{0.f, 0.f, 0.f, 0.f} : acc[ct][b], 0, 0, 0);
#pragma unroll
      for (int ct = 0; ct < CT; ++ct)
#pragma unroll
        for (int b = 0; b < GK; ++b) s[ct][grp * GK + b] = acc[ct][b];
      __builtin_amdgcn_sched_barrier(0);
    }
    // with registers to spare the first value operands are asked for now: they do not depend
    // on the softmax
    constexpr bool kEarlyValues = CT == 1;
    constexpr int GJ = NJ / (2 * CT);  // operand reads a group
    constexpr int NG = NJ / GJ;        // groups a pair of key blocks
    static_assert(GJ > 0 && NJ % GJ == 0,
                  "a head size whose column groups do not divide into whole read groups would "
                  "leave columns of the output without their sums");
    bf16x8_t va[2][GJ];
    auto read_values = [&](int pr, int grp, bf16x8_t (&dst)[GJ]) {
#pragma unroll
      for (int jj = 0; jj < GJ; ++jj) {
        const int j = grp * GJ + jj;
        dst[jj] = *reinterpret_cast<const bf16x8_t*>(v_lds + (((pr * NJ + j) * 4 + quad) * 16 + (col ^ (8 * (quad >> 1)))) * 8);
      }
    };
    if constexpr (kEarlyValues) {
      read_values(0, 0, va[0]);
      __builtin_amdgcn_sched_barrier(0);
    }
    // ---- softmax update per row over the 64 keys of the tile; a tile that every live row of
    // the wave sees whole needs no masks
    const bool whole = (kb0 + kKeyBlocks) * 16 - 1 <= wave_pos_lo && kb0 * 16 >= wave_first_hi;
    // The reference maximum of a row only moves when the tile's maximum exceeds it by more
    // than 2^8 (after scaling): probabilities then stay below 256, which bfloat16 and the
    // float32 sums hold easily, and the running output is rescaled rarely instead of at
    // every tile.  The scale is applied inside the exponent's multiply-add.
    float mx[CT];
    bool moved = false;
#pragma unroll
    for (int ct = 0; ct < CT; ++ct) {
      if (!whole) {
#pragma unroll
        for (int kbi = 0; kbi < kKeyBlocks; ++kbi) {
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            const int key = (kb0 + kbi) * 16 + 4 * quad + i;
            const bool ok = key >= my_first[ct] && key <= my_pos[ct];
            s[ct][kbi][i] = ok ? s[ct][kbi][i] : -INFINITY;
          }
        }
      }
      float v = -INFINITY;
#pragma unroll
      for (int kbi = 0; kbi < kKeyBlocks; ++kbi)
#pragma unroll
        for (int i = 0; i < 4; ++i) v = fmaxf(v, s[ct][kbi][i]);
      v = quad_max(v);
      mx[ct] = v;
      moved = moved || (v > m[ct] + unit);  // also true for the first visible key (m = -inf)
    }
    if (__any(moved)) {
#pragma unroll
      for (int ct = 0; ct < CT; ++ct) {
        if (mx[ct] > m[ct] + unit) {
          const float alpha = __builtin_amdgcn_exp2f((m[ct] - mx[ct]) * scale_log2e);  // 0 when m was -inf
          m[ct] = mx[ct];
          l[ct] *= alpha;
#pragma unroll
          for (int j = 0; j < NJ; ++j) o_acc[ct][j] = o_acc[ct][j] * alpha;
        }
      }
    }
    bf16x8_t pb[CT][kKeyBlocks / 2];
#pragma unroll
    for (int ct = 0; ct < CT; ++ct) {
      const float neg_mc = (m[ct] == -INFINITY) ? 0.f : -m[ct] * scale_log2e;
      float ps = 0.f;
#pragma unroll
      for (int kbi = 0; kbi < kKeyBlocks; ++kbi) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const float p = __builtin_amdgcn_exp2f(__builtin_fmaf(s[ct][kbi][i], scale_log2e, neg_mc));
          ps += p;
          pb[ct][kbi >> 1][4 * (kbi & 1) + i] = static_cast<__bf16>(p);
        }
      }
      l[ct] += ps;  // this lane's keys only: the four lanes of a row are added up at the end
    }
    // ---- O^T += V^T P^T, two key blocks a product; the operand reads run half a pair ahead
    if constexpr (!kEarlyValues) read_values(0, 0, va[0]);
#pragma unroll
    for (int pr = 0; pr < kKeyBlocks / 2; ++pr) {
      if ((kb0 + 2 * pr) * 16 > wave_pos_hi) break;  // scalar: later blocks weigh nothing
#pragma unroll
      for (int grp = 0; grp < NG; ++grp) {
        const int step = pr * NG + grp;
        if (grp + 1 < NG) read_values(pr, grp + 1, va[(step + 1) & 1]);
        else if (pr + 1 < kKeyBlocks / 2) read_values(pr + 1, 0, va[(step + 1) & 1]);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int jj = 0; jj < GJ; ++jj)
#pragma unroll
          for (int ct = 0; ct < CT; ++ct)
            o_acc[ct][grp * GJ + jj] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(va[step & 1][jj], pb[ct][pr], o_acc[ct][grp * GJ + jj], 0, 0, 0);
        __builtin_amdgcn_sched_barrier(0);
      }
    }
  };

  // With gridDim.z > 1 the key tiles of the rows are dealt to that many blocks in
  // consecutive runs; each leaves its unnormalised sums for the combining kernel.
  const int tiles_all = (kb_end - kb_first + kKeyBlocks - 1) / kKeyBlocks;
  const int tiles_mine = (tiles_all + static_cast<int>(gridDim.z) - 1) / static_cast<int>(gridDim.z);
  const int kb_mine = kb_first + static_cast<int>(blockIdx.z) * tiles_mine * kKeyBlocks;
  const int kb_mine_end = (kb_mine + tiles_mine * kKeyBlocks < kb_end) ? kb_mine + tiles_mine * kKeyBlocks : kb_end;
  if (kb_mine < kb_mine_end) {  // the same for the whole block
    int64_t kbase[K_PER_THREAD], vbase[V_PER_THREAD];
    lookup_issue(kb_mine);
    bool all_there = lookup_finish(kbase, vbase);
    fetch_tile(kb_mine, kbase, vbase, all_there);
    lookup_issue(kb_mine + kKeyBlocks);
    store_tile(0);
    __syncthreads();
    int buf = 0;
    for (int kb0 = kb_mine; kb0 < kb_mine_end; kb0 += kKeyBlocks, buf ^= 1) {
      const bool more = kb0 + kKeyBlocks < kb_mine_end;
      if (more) {
        all_there = lookup_finish(kbase, vbase);
        fetch_tile(kb0 + kKeyBlocks, kbase, vbase, all_there);  // in flight while this tile is used
        lookup_issue(kb0 + 2 * kKeyBlocks);                     // answered by the time it is fetched
      }
      if (kb0 * 16 <= wave_pos_hi) work_tile(kb0, buf);  // scalar: else nothing here is visible to this wave
      if (more) store_tile(buf ^ 1);
      __syncthreads();  // the next tile is whole, and this one has been consumed
    }
  }

#pragma unroll
  for (int ct = 0; ct < CT; ++ct) {
    const float l_row = quad_sum(l[ct]);
    if (!live[ct]) continue;
    if (gridDim.z > 1) {
      // sums relative to m, and m in the exponent's units, as the combining kernel expects
      const int64_t slot =
          (static_cast<int64_t>(my_tok[ct]) * nh + my_head[ct]) * gridDim.z + blockIdx.z;
      float* po = part_o + slot * D + 4 * quad;
#pragma unroll
      for (int j = 0; j < NJ; ++j) *reinterpret_cast<f32x4_t*>(po + 16 * j) = o_acc[ct][j];
      if (quad == 0) {
        part_ml[2 * slot] = (m[ct] == -INFINITY) ? -INFINITY : m[ct] * scale_log2e;
        part_ml[2 * slot + 1] = l_row;
      }
      continue;
    }
    const float inv = (l_row > 0.f) ? 1.f / l_row : 0.f;
    bf16_t* op = out + (static_cast<int64_t>(my_tok[ct]) * nh + my_head[ct]) * D + 4 * quad;
#pragma unroll
    for (int j = 0; j < NJ; ++j) {
      const f32x4_t v = o_acc[ct][j] * inv;
      const float vv[4] = {v[0], v[1], v[2], v[3]};
      *reinterpret_cast<s16x4_t*>(op + 16 * j) = pack_bf16x4(vv);
    }
  }
  }  // turn
}

template <int D, int CT, int W>
int launch_prefill_ct(bf16_t* out, const bf16_t* q, int64_t q_stride, const bf16_t* k_cache,
                      const bf16_t* v_cache, const int32_t* table, int table_stride,
                      const int32_t* positions, const int32_t* q_start, const int32_t* slots, int T,
                      int R, int nh, int nkv, int page_size, int num_pages, float scale, int window,
                      float* part_o, float* part_ml, int nsplit, int single, const float* cos_tab,
                      const float* sin_tab, int rot_dim, int interleaved, hipStream_t stream) {
  const int g = nh / nkv;
  const int bq = (16 * W * CT) / g;
  // every request may end in a ragged tile and have an odd number of tiles
  const int max_pairs = single ? (T + bq - 1) / bq + R : ((T + bq - 1) / bq + R) / 2 + R;
  // key tiles of 64 for four waves (tiles of 32, with which more blocks would fit a compute
  // unit, were slower: 2,048 tokens 121 against 90 us); a block of eight waves has the compute
  // unit's LDS to itself and takes tiles of 128 keys: half the barriers and page lookups per key
  // (16,384 tokens 2.52 against 2.39 ms), and on heads of 64 a thread then still stages whole
  // pairs of key blocks
  constexpr int KB = (W == 8) ? 8 : 4;
  constexpr int lds_bytes = 2 * tile_bytes<D, KB>();
  static const hipError_t attr = hipFuncSetAttribute(
      reinterpret_cast<const void*>(&prefill_attention_kernel<D, CT, KB, W>),
      hipFuncAttributeMaxDynamicSharedMemorySize, lds_bytes);
  if (attr != hipSuccess) return kvc_fail("kvc_prefill_attention: the kernel's LDS size was refused");
  // see the kernel on how block ids map to (kv head, pair)
  const int64_t wide = (8 % nkv == 0) ? static_cast<int64_t>((max_pairs + 8 / nkv - 1) / (8 / nkv)) * 8
                                      : (static_cast<int64_t>(max_pairs) * nkv + 7) / 8 * 8;
  if (wide > 0x7fffffff) return kvc_fail("kvc_prefill_attention: too many blocks");
  char variant[64];
  snprintf(variant, sizeof(variant), "prefill_attention_kernel<%d,%d,%d,%d>%s x%d", D, CT, KB, W,
           single ? " one tile a block" : "", nsplit);
  kvc_note_variant(kVariantPrefillAttention, variant);
  hipLaunchKernelGGL((prefill_attention_kernel<D, CT, KB, W>), dim3(static_cast<unsigned>(wide), 1, nsplit), dim3(W * 64),
                     lds_bytes, stream, out, q, q_stride, k_cache, v_cache, table, table_stride, positions,
                     q_start, slots, R, nh, nkv, page_size, num_pages, scale * kLog2e, window, part_o,
                     part_ml, single, cos_tab, sin_tab, rot_dim, interleaved);
  if (nsplit > 1) return launch_attention_combine(out, part_o, part_ml, static_cast<int64_t>(T) * nh, D, nsplit, stream);
  return kvc_check_launch("kvc_prefill_attention");
}

template <int D>
int launch_prefill(bf16_t* out, const bf16_t* q, int64_t q_stride, const bf16_t* k_cache,
                   const bf16_t* v_cache, const int32_t* table, int table_stride,
                   const int32_t* positions, const int32_t* q_start, const int32_t* slots, int T,
                   int R, int nh, int nkv, int page_size, int num_pages, float scale, int window,
                   float* part_o, float* part_ml, int nsplit, const float* cos_tab, const float* sin_tab,
                   int rot_dim, int interleaved, hipStream_t stream) {
  const int g = nh / nkv;
  // Blocks of four waves lie two to a compute unit, blocks of eight waves one.  Tiles of 64
  // query rows, two a block one after the other (a late and an early one), are the fastest as
  // long as all their blocks find room at once; more rows than that take tiles of 128 rows,
  // which stage each key tile for twice the rows (and so does a launch that splits the keys,
  // unless its rows are very few: its caller splits until there are blocks enough).  Few rows
  // take one tile of 64 a block, for twice the blocks.  Where the requests are long, blocks of
  // eight waves (tiles of 128 or 256 rows) halve the loads and LDS writes per row once more.
  // Measured at 32 heads over 8 kv heads of 128, one request, four waves against eight:
  // 1,024 tokens 36 against 38 us, 1,536 tokens 64 against 56, 2,048 tokens 83 against 77,
  // 3,072 tokens 149 against 144, 8,192 tokens 699 against 672; four requests of 512 tokens 29
  // (tiles of 64 rows) and 33 (tiles of 128) against 40 (eight waves, tiles of 256).  Heads
  // of 64: 1,024 tokens 27 against 23, 2,048 tokens 54 against 43, 8,192 tokens 445 against 393.
  // (every request but one may add a ragged tile)
  const int bq1 = 64 / g > 0 ? 64 / g : 1;
  const int tiles1 = (T + bq1 - 1) / bq1 + (R - 1);
  const int64_t pairs1 = static_cast<int64_t>((tiles1 + 1) / 2) * nkv;
  const int64_t small_tiles = static_cast<int64_t>(tiles1) * nkv;
  const bool long_requests = T / R >= (D == 64 ? 512 : 1024);
  // the thresholds below were measured on 256 compute units and are kept as multiples of them
  const int cu = kvc_device_compute_units();
  int ct = 1, single = 0, waves = 4;
  if (g > 64) {
    ct = 2;
  } else if (nsplit > 1) {
    // very few rows: small tiles one a block reach the blocks wanted with a quarter of the
    // splits (128 rows at 1,024 keys: 21 against 39 us)
    if (small_tiles <= cu / 2) {
      single = 1;
    } else {
      ct = 2;
      if (long_requests) waves = 8;  // 2,048 tokens after 30,000: 1.38 against 1.32 ms
    }
  } else if (pairs1 > 2 * cu) {
    ct = 2;
    if (long_requests) waves = 8;
  } else if (pairs1 > cu) {
    if (long_requests) {
      waves = 8;
      single = pairs1 <= 7 * cu / 4;
    }
  } else {
    single = 1;
    if (D == 64 && pairs1 > cu / 2 && long_requests) waves = 8;
  }
  // KVC_PREFILL_MODE = 1p | 1s | 2p | 2s, then 4 or 8 (waves), overrides the choice for tuning
  static const char* mode = getenv("KVC_PREFILL_MODE");
  if (mode && (mode[0] == '1' || mode[0] == '2')) {
    ct = mode[0] == '2' ? 2 : 1;
    single = mode[1] == 's';
    waves = (mode[1] && mode[2] == '8') ? 8 : 4;
  }
  if (g > 16 * waves * ct) return kvc_fail("kvc_prefill_attention: too many query heads per kv head");
#define KVC_LAUNCH_PREFILL(CT_, W_)                                                                      \
  return launch_prefill_ct<D, CT_, W_>(out, q, q_stride, k_cache, v_cache, table, table_stride, positions, \
                                       q_start, slots, T, R, nh, nkv, page_size, num_pages, scale, window, \
                                       part_o, part_ml, nsplit, single, cos_tab, sin_tab, rot_dim,     \
                                       interleaved, stream)
  if (waves == 8) {
    if (ct == 2) KVC_LAUNCH_PREFILL(2, 8);
    KVC_LAUNCH_PREFILL(1, 8);
  }
  if (ct == 2) KVC_LAUNCH_PREFILL(2, 4);
  KVC_LAUNCH_PREFILL(1, 4);
#undef KVC_LAUNCH_PREFILL
}

}  // namespace

extern "C" int kvc_prefill_attention_supported(int nh, int nkv, int d, int page_size, int dtype) {
  if (dtype != 1) return 0;
  if (nkv <= 0 || nh % nkv || nh / nkv > 64) return 0;
  if (page_size % 16) return 0;
  return d == 64 || d == 128;
}

extern "C" int kvc_prefill_attention(void* out, const void* q, int64_t q_stride,
                                     const void* k_cache, const void* v_cache,
                                     const int32_t* table, int table_stride,
                                     const int32_t* positions, const int32_t* q_start,
                                     const int32_t* slots, int T, int R, int nh, int nkv, int d,
                                     int page_size, int num_pages, float scale, int window,
                                     void* part_o, void* part_ml, int nsplit, const float* cos_tab,
                                     const float* sin_tab, int rot_dim, int interleaved,
                                     kvc_stream stream) {
  if (!kvc_prefill_attention_supported(nh, nkv, d, page_size, 1))
    return kvc_fail("kvc_prefill_attention: unsupported shape (bfloat16, head size 64 or 128, at "
                    "most 64 query heads per kv head, page size a multiple of 16)");
  if (T < 0 || R <= 0 || nkv > 65535 || table_stride <= 0 || num_pages <= 0)
    return kvc_fail("kvc_prefill_attention: bad sizes");
  if (!(scale > 0.f)) return kvc_fail("kvc_prefill_attention: the scale must be positive");
  if (q_stride % 8) return kvc_fail("kvc_prefill_attention: q rows must be 16-byte aligned");
  if (nsplit < 1 || nsplit > kMaxAttentionSplits)
    return kvc_fail("kvc_prefill_attention: between 1 and 64 splits");
  if (nsplit > 1 && (part_o == nullptr || part_ml == nullptr))
    return kvc_fail("kvc_prefill_attention: splits need a workspace");
  if ((cos_tab == nullptr) != (sin_tab == nullptr))
    return kvc_fail("kvc_prefill_attention: cosines and sines come together");
  if (cos_tab != nullptr &&
      (rot_dim <= 0 || rot_dim > d || rot_dim % (interleaved ? 32 : 64)))
    return kvc_fail("kvc_prefill_attention: rotating the queries here needs rot_dim to be a multiple "
                    "of 64 (32 for neighbouring pairs) and at most the head size");
  if (T == 0) return 0;
  float* po = static_cast<float*>(part_o);
  float* pml = static_cast<float*>(part_ml);
  hipStream_t s = reinterpret_cast<hipStream_t>(stream);
  const bf16_t* qq = static_cast<const bf16_t*>(q);
  const bf16_t* kc = static_cast<const bf16_t*>(k_cache);
  const bf16_t* vc = static_cast<const bf16_t*>(v_cache);
  if (d == 64)
    return launch_prefill<64>(static_cast<bf16_t*>(out), qq, q_stride, kc, vc, table, table_stride,
                              positions, q_start, slots, T, R, nh, nkv, page_size, num_pages, scale,
                              window, po, pml, nsplit, cos_tab, sin_tab, rot_dim, interleaved, s);
  return launch_prefill<128>(static_cast<bf16_t*>(out), qq, q_stride, kc, vc, table, table_stride,
                             positions, q_start, slots, T, R, nh, nkv, page_size, num_pages, scale,
                             window, po, pml, nsplit, cos_tab, sin_tab, rot_dim, interleaved, s);
}
