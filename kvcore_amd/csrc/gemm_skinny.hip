// C[M, N] = A[M, K] * W[N, K]^T (+ bias) for few rows (M <= 64), bfloat16 operands,
// float32 sums: the decode-time shape, where the weight matrix is read once from HBM
// and everything else is small.
//
// The weight rows are the A operand of v_mfma_f32_16x16x32_bf16 and the activations
// its B operand, so a lane loads 16 bytes of one weight row per instruction and a
// wave walks 16 rows along K:
//
//   C^T[16 weight rows, 16 tokens] += W[16 rows, 32 k] * A^T[32 k, 16 tokens]
//
// A block owns 16 weight rows; its waves split K and their partial tiles are added in
// wave order through LDS, so every element is summed in an order that K and the launch
// shape fix, whatever M is and whatever else is in the batch.  With N/16 blocks times
// KS waves there are enough 16-byte loads in flight to keep HBM busy.

#include <hip/hip_runtime.h>

#include <cstdio>
#include <cstdlib>

#include "device_utils.h"
#include "gemm_common.h"
#include "kvcore_hip.h"

using namespace kvc;

namespace {

// Optional work around the product, all of it by the wave that holds the finished sums:
//  - in_ss: the rows of A are activations not yet normalised (a gain is already applied);
//    row m's products are multiplied by rsqrt(sum_p in_ss[m][p] / in_width + in_eps), which
//    is what normalising the row first would have given;
//  - residual: the product (+ bias) is added into the float32 residual stream, C receives
//    bfloat16(residual * gain) and out_ss[m][block] the sum of squares of the new residual
//    over this block's columns: the next product's in_ss.
struct SkinnyExtras {
  const float* in_ss;
  int in_parts;
  float in_width;
  float in_eps;
  float* residual;
  int64_t ldr;
  const float* gain;
  float* out_ss;
};

// GATED: the two row tiles of a wave are rows n of the first N weight rows (gate) and rows
// N + n (up), and the stored value is silu(gate) * up, each factor rounded to bfloat16
// first as if it had been stored.
// FOLD: bit 0, the rows of A carry a scale factor still to be applied (ex.in_ss); bit 1, the
// result goes into the residual stream (ex.residual).  Kernels without these keep their
// register count, on which the number of waves in flight depends.
template <int RT, int NT, int U, int MAXW, typename OutT, bool GATED, int FOLD = 0>
__global__ __launch_bounds__(MAXW * 64) void gemm_skinny_kernel(OutT* __restrict__ C, const bf16_t* __restrict__ A,
                                   const bf16_t* __restrict__ W, const bf16_t* __restrict__ bias,
                                   int M, int N, int K, int64_t lda, int64_t ldc, int k_per_wave,
                                   const SkinnyExtras ex, int packed) {
  static_assert(!GATED || RT == 2, "the gated form pairs one gate tile with one up tile");
  extern __shared__ float red[];  // [waves - 1][RT * NT][64][4], then 16 row scales and [16][256] parts of their sums if FOLD & 1
  // wave-uniform values are made scalar on purpose: a condition on them becomes a scalar
  // branch, and matrix instructions are only ever skipped by branches (they do not honour
  // the lane mask that a vector condition would leave)
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int waves = blockDim.x >> 6;
  const int lane = threadIdx.x & 63;
  const int col = lane & 15;
  const int quad = lane >> 4;
  const int n0 = blockIdx.x * (GATED ? 16 : 16 * RT);
  const int k_begin = wave * k_per_wave;
  const int k_end = (k_begin + k_per_wave < K) ? k_begin + k_per_wave : K;

  const int ks = packed ? 16 : 1;  // elements between a row's 32-wide steps, in units of 32
  const bf16_t* wp[RT];
#pragma unroll
  for (int rt = 0; rt < RT; ++rt) {
    const int r = GATED ? n0 + col : n0 + rt * 16 + col;
    const int64_t row = (r < N ? r : N - 1) + ((GATED && rt == 1) ? N : 0);
    // packed: tiles of 16 rows x 32 k stored one after the other along K, so that the 64 lanes
    // of a load read 1 KB in one piece (see kvc_pack_weight)
    wp[rt] = packed ? W + (row >> 4) * (static_cast<int64_t>(K) * 16) + (row & 15) * 32 + 8 * quad
                    : W + row * K + 8 * quad;
  }
  const bf16_t* ap[NT];
  bool tok_ok[NT];
#pragma unroll
  for (int nt = 0; nt < NT; ++nt) {
    const int tok = nt * 16 + col;
    tok_ok[nt] = tok < M;
    ap[nt] = A + static_cast<int64_t>(tok_ok[nt] ? tok : 0) * lda + 8 * quad;
  }
  f32x4_t acc[RT][NT];
#pragma unroll
  for (int rt = 0; rt < RT; ++rt)
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) acc[rt][nt] = f32x4_t{0.f, 0.f, 0.f, 0.f};

  float row_scale[NT];
#pragma unroll
  for (int nt = 0; nt < NT; ++nt) row_scale[nt] = 1.f;

  // the residual rows this block will add into, asked for now by the wave that adds at the
  // end: they were written by the kernel before and come from far
  f32x4_t res_pre[RT][NT];
  bool res_vec[RT][NT];
  if constexpr ((FOLD & 2) != 0) {
#pragma unroll
    for (int rt = 0; rt < RT; ++rt)
#pragma unroll
      for (int nt = 0; nt < NT; ++nt) {
        const int n_first = n0 + rt * 16 + 4 * quad;
        const int tok = nt * 16 + col;
        const float* rp = ex.residual + static_cast<int64_t>(tok < M ? tok : 0) * ex.ldr + n_first;
        res_vec[rt][nt] = wave == 0 && tok < M && N - n_first >= 4 &&
                          (reinterpret_cast<uintptr_t>(rp) & 15) == 0;
        res_pre[rt][nt] = f32x4_t{0.f, 0.f, 0.f, 0.f};
        if (res_vec[rt][nt]) res_pre[rt][nt] = *reinterpret_cast<const f32x4_t*>(rp);
      }
  }

  // Whole steps of 64 along K first, software-pipelined: the loads of the next STAGES - 1
  // steps are in flight while a step is multiplied (a lane reads 2 x 16 bytes = a row reads
  // 128 contiguous bytes a step).  Then whole 32-wide steps, then one guarded step for a
  // tail (a multiple of 8).
  constexpr int STAGES = U;  // steps in flight, the one being multiplied included
  bf16x8_t abuf[STAGES][RT][2], bbuf[STAGES][NT][2];
  const int n64 = (k_end - k_begin) / 64;
  auto load_step = [&](int stage, int step) {
    const int k = k_begin + 64 * step;
#pragma unroll
    for (int rt = 0; rt < RT; ++rt) {
      abuf[stage][rt][0] = *reinterpret_cast<const bf16x8_t*>(wp[rt] + static_cast<int64_t>(k) * ks);
      abuf[stage][rt][1] = *reinterpret_cast<const bf16x8_t*>(wp[rt] + static_cast<int64_t>(k + 32) * ks);
    }
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) {
      bbuf[stage][nt][0] = *reinterpret_cast<const bf16x8_t*>(ap[nt] + k);
      bbuf[stage][nt][1] = *reinterpret_cast<const bf16x8_t*>(ap[nt] + k + 32);
    }
  };
  auto mma_step = [&](int stage) {
#pragma unroll
    for (int h = 0; h < 2; ++h)
#pragma unroll
      for (int rt = 0; rt < RT; ++rt)
#pragma unroll
        for (int nt = 0; nt < NT; ++nt)
          acc[rt][nt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(abuf[stage][rt][h], bbuf[stage][nt][h],
                                                                 acc[rt][nt], 0, 0, 0);
  };
  // (Loads without a branch around them would let the waits count them exactly and keep
  // all STAGES steps in flight; measured inside a decode step that is slower than this form,
  // whose waits drain more often but which needs fewer registers and so runs more waves.)
  // The rows' scale factors.  Where a row's parts fit one 16-byte load a lane, every wave
  // asks for the parts of its share of the rows now, before its weights, straight into LDS
  // (no registers wait for them), and adds them up only after its walk along K: loads
  // complete in the order of their issue, so by then they have long arrived.
  float* scale_lds = red + static_cast<int64_t>(waves - 1) * (RT * NT) * 256;  // [16] row scales,
  float* parts_lds = scale_lds + 16;                                           // then [16][256] parts
  bool ss_late = false;
  if constexpr ((FOLD & 1) != 0 && NT == 1) {
    // (one or two rows cost the old way nothing: a single round of loads while the weights come)
    ss_late = M > 2 && ex.in_parts % 4 == 0 && ex.in_parts <= 256 && (reinterpret_cast<uintptr_t>(ex.in_ss) & 15) == 0;
    if (ss_late) {
      for (int t = wave; t < M; t += waves) {  // scalar
        if (4 * lane < ex.in_parts)
          __builtin_amdgcn_global_load_lds(
              (const __attribute__((address_space(1))) void*)(ex.in_ss + static_cast<int64_t>(t) * ex.in_parts + 4 * lane),
              (__attribute__((address_space(3))) void*)(parts_lds + t * 256), 16, 0, 0);
      }
    }
  }
  int k = k_begin;
#pragma unroll
  for (int st = 0; st < STAGES - 1; ++st)
    if (st < n64) load_step(st, st);
  // Otherwise they are worked out by the wave that will need them at the end while its
  // first weight loads are on their way, four tokens at a time (more would cost registers and
  // with them waves in flight).  Token by token the wave reads the row's parts (four a lane)
  // and adds them up in the fixed order of a butterfly, so the result does not depend on
  // anything but the parts.
  if ((FOLD & 1) && wave == 0 && !ss_late) {
    const bool vec = (ex.in_parts % 4 == 0) && ((reinterpret_cast<uintptr_t>(ex.in_ss) & 15) == 0);
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) {
      const int n_tok = (M - nt * 16 < 16) ? M - nt * 16 : 16;  // scalar
      // all loads of a batch first, then its sums
      float mine = 0.f;
      for (int t0 = 0; t0 < n_tok; t0 += 4) {
        float part[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          part[i] = 0.f;
          if (t0 + i < n_tok) {
            const float* parts = ex.in_ss + static_cast<int64_t>(nt * 16 + t0 + i) * ex.in_parts;
            if (vec) {
              for (int p = 4 * lane; p < ex.in_parts; p += 256) {
                const f32x4_t v = *reinterpret_cast<const f32x4_t*>(parts + p);
                part[i] += (v[0] + v[1]) + (v[2] + v[3]);
              }
            } else {
              for (int p = lane; p < ex.in_parts; p += 64) part[i] += parts[p];
            }
          }
        }
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          if (t0 + i < n_tok) {
            const float total = wave_sum(part[i]);
            if (col == t0 + i) mine = total;
          }
        }
      }
      row_scale[nt] = rsqrtf(mine / ex.in_width + ex.in_eps);
    }
  }

  for (int i = 0; i < n64; i += STAGES) {
#pragma unroll
    for (int j = 0; j < STAGES; ++j) {
      if (i + j < n64) {  // the same for the whole wave, and a scalar branch
        if constexpr (STAGES == 4) {
          // two steps asked for together: a row's 256 contiguous bytes reach the memory
          // close in time
          if ((j & 1) == 0) {
            if (i + j + 2 < n64 && i + j + 2 >= STAGES - 1) load_step((j + 2) % STAGES, i + j + 2);
            if (i + j + 3 < n64) load_step((j + 3) % STAGES, i + j + 3);
          }
        } else {
          if (i + j + STAGES - 1 < n64) load_step((j + STAGES - 1) % STAGES, i + j + STAGES - 1);
        }
        mma_step(j);
      }
    }
  }
  k = k_begin + 64 * n64;
  const int k_full = k + ((k_end - k) / 32) * 32;
  for (; k < k_full; k += 32) {
    bf16x8_t a[RT], b[NT];
#pragma unroll
    for (int rt = 0; rt < RT; ++rt) a[rt] = *reinterpret_cast<const bf16x8_t*>(wp[rt] + static_cast<int64_t>(k) * ks);
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) b[nt] = *reinterpret_cast<const bf16x8_t*>(ap[nt] + k);
#pragma unroll
    for (int rt = 0; rt < RT; ++rt)
#pragma unroll
      for (int nt = 0; nt < NT; ++nt)
        acc[rt][nt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[rt], b[nt], acc[rt][nt], 0, 0, 0);
  }
  if (k_full < k_end) {
    const bool valid = k_full + 8 * quad < k_end;
    bf16x8_t a[RT], b[NT];
#pragma unroll
    for (int rt = 0; rt < RT; ++rt)
      a[rt] = valid ? *reinterpret_cast<const bf16x8_t*>(wp[rt] + static_cast<int64_t>(k_full) * ks) : zero8();
#pragma unroll
    for (int nt = 0; nt < NT; ++nt)
      b[nt] = valid ? *reinterpret_cast<const bf16x8_t*>(ap[nt] + k_full) : zero8();
#pragma unroll
    for (int rt = 0; rt < RT; ++rt)
#pragma unroll
      for (int nt = 0; nt < NT; ++nt)
        acc[rt][nt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[rt], b[nt], acc[rt][nt], 0, 0, 0);
  }

  if constexpr ((FOLD & 1) != 0 && NT == 1) {
    if (ss_late) {
      // the wave's own loads into LDS have all landed once its load counter is at zero
      __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0)
      for (int t = wave; t < M; t += waves) {
        f32x4_t v = f32x4_t{0.f, 0.f, 0.f, 0.f};
        if (4 * lane < ex.in_parts) v = *reinterpret_cast<const f32x4_t*>(parts_lds + t * 256 + 4 * lane);
        const float total = wave_sum((v[0] + v[1]) + (v[2] + v[3]));
        if (lane == 0) scale_lds[t] = rsqrtf(total / ex.in_width + ex.in_eps);
      }
    }
  }
  constexpr int TILES = RT * NT;
  if (wave > 0) {
#pragma unroll
    for (int rt = 0; rt < RT; ++rt)
#pragma unroll
      for (int nt = 0; nt < NT; ++nt)
        *reinterpret_cast<f32x4_t*>(
            red + ((static_cast<int64_t>(wave - 1) * TILES + rt * NT + nt) * 64 + lane) * 4) = acc[rt][nt];
  }
  __syncthreads();
  if (wave != 0) return;
  if constexpr ((FOLD & 1) != 0 && NT == 1) {
    if (ss_late && tok_ok[0]) row_scale[0] = scale_lds[col];
  }
  for (int w = 1; w < waves; ++w) {
#pragma unroll
    for (int rt = 0; rt < RT; ++rt)
#pragma unroll
      for (int nt = 0; nt < NT; ++nt)
        acc[rt][nt] += *reinterpret_cast<const f32x4_t*>(
            red + ((static_cast<int64_t>(w - 1) * TILES + rt * NT + nt) * 64 + lane) * 4);
  }
  // acc[rt][nt][i] = C[token nt*16 + col][n0 + rt*16 + 4*quad + i]; columns of unused tokens
  // multiplied whatever row 0 of A holds and are dropped here
  if constexpr (GATED) {
    const int n_first = n0 + 4 * quad;
    const int n_left = N - n_first;
    if (n_left <= 0) return;
    f32x4_t bg = f32x4_t{0.f, 0.f, 0.f, 0.f}, bu = bg;
    if (bias != nullptr)
      for (int i = 0; i < 4 && i < n_left; ++i) {
        bg[i] = to_float(bias[n_first + i]);
        bu[i] = to_float(bias[N + n_first + i]);
      }
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) {
      const int tok = nt * 16 + col;
      if (tok >= M) continue;
      f32x4_t y;
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const float gv = to_float(from_float<bf16_t>(acc[0][nt][i] * row_scale[nt] + bg[i]));
        const float uv = to_float(from_float<bf16_t>(acc[1][nt][i] * row_scale[nt] + bu[i]));
        y[i] = gv / (1.f + expf(-gv)) * uv;
      }
      store4<OutT>(C + static_cast<int64_t>(tok) * ldc + n_first, y, n_left);
    }
    return;
  }
  if constexpr ((FOLD & 2) != 0 && sizeof(OutT) == 2) {
    {
      float ss[NT];
#pragma unroll
      for (int nt = 0; nt < NT; ++nt) ss[nt] = 0.f;
#pragma unroll
      for (int rt = 0; rt < RT; ++rt) {
        const int n_first = n0 + rt * 16 + 4 * quad;
        const int n_left = N - n_first;
#pragma unroll
        for (int nt = 0; nt < NT; ++nt) {
          const int tok = nt * 16 + col;
          if (tok >= M || n_left <= 0) continue;
          float* rp = ex.residual + static_cast<int64_t>(tok) * ex.ldr + n_first;
          bf16_t* cp = reinterpret_cast<bf16_t*>(C) + static_cast<int64_t>(tok) * ldc + n_first;
          if (res_vec[rt][nt] && (reinterpret_cast<uintptr_t>(ex.gain + n_first) & 15) == 0 &&
              (reinterpret_cast<uintptr_t>(cp) & 7) == 0) {
            f32x4_t b = f32x4_t{0.f, 0.f, 0.f, 0.f};
            if (bias != nullptr)
              for (int i = 0; i < 4; ++i) b[i] = to_float(bias[n_first + i]);
            const f32x4_t r = res_pre[rt][nt] + (acc[rt][nt] * row_scale[nt] + b);
            *reinterpret_cast<f32x4_t*>(rp) = r;
            store4<bf16_t>(cp, r * *reinterpret_cast<const f32x4_t*>(ex.gain + n_first), 4);
            ss[nt] += (r[0] * r[0] + r[1] * r[1]) + (r[2] * r[2] + r[3] * r[3]);
          } else {
            for (int i = 0; i < 4 && i < n_left; ++i) {
              const float b = (bias != nullptr) ? to_float(bias[n_first + i]) : 0.f;
              const float r = rp[i] + (acc[rt][nt][i] * row_scale[nt] + b);
              rp[i] = r;
              cp[i] = from_float<bf16_t>(r * ex.gain[n_first + i]);
              ss[nt] += r * r;
            }
          }
        }
      }
#pragma unroll
      for (int nt = 0; nt < NT; ++nt) {
        float v = ss[nt];
        v += __shfl_xor(v, 16, 64);
        v += __shfl_xor(v, 32, 64);
        const int tok = nt * 16 + col;
        if (quad == 0 && tok < M) ex.out_ss[static_cast<int64_t>(tok) * gridDim.x + blockIdx.x] = v;
      }
    }
    return;
  }
#pragma unroll
  for (int rt = 0; rt < RT; ++rt) {
    const int n_first = n0 + rt * 16 + 4 * quad;
    const int n_left = N - n_first;
    if (n_left <= 0) continue;
    f32x4_t bv = f32x4_t{0.f, 0.f, 0.f, 0.f};
    if (bias != nullptr)
      for (int i = 0; i < 4 && i < n_left; ++i) bv[i] = to_float(bias[n_first + i]);
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) {
      const int tok = nt * 16 + col;
      if (tok >= M) continue;
      store4<OutT>(C + static_cast<int64_t>(tok) * ldc + n_first, acc[rt][nt] * row_scale[nt] + bv, n_left);
    }
  }
}

template <int RT, int NT, typename OutT, bool GATED = false>
void launch(OutT* C, const bf16_t* A, const bf16_t* W, const bf16_t* bias, int M, int N, int K,
            int64_t lda, int64_t ldc, int waves, int k_per_wave, const SkinnyExtras& ex, int packed,
            hipStream_t stream) {
  // steps in flight by what fits in registers beside the accumulators
  constexpr int STAGES = (RT + NT <= 5) ? 4 : ((RT + NT <= 6) ? 3 : 2);
  constexpr int MAXW = (RT >= 2) ? 4 : 8;
  const size_t lds = static_cast<size_t>(waves - 1) * RT * NT * 64 * 4 * sizeof(float) +
                     (ex.in_ss != nullptr ? (16 + 16 * 256) * sizeof(float) : 0);
  const int rows_per_block = GATED ? 16 : 16 * RT;
  const dim3 grid((N + rows_per_block - 1) / rows_per_block), block(waves * 64);
  const int fold = (ex.in_ss != nullptr ? 1 : 0) | (ex.residual != nullptr ? 2 : 0);
#define KVC_SKINNY_LAUNCH(FOLD_)                                                                   \
  hipLaunchKernelGGL((gemm_skinny_kernel<RT, NT, STAGES, MAXW, OutT, GATED, FOLD_>), grid, block, \
                     lds, stream, C, A, W, bias, M, N, K, lda, ldc, k_per_wave, ex, packed)
  if constexpr (NT == 1 && sizeof(OutT) == 2) {  // folded norms are for steps of few rows
    switch (fold) {
      case 0: KVC_SKINNY_LAUNCH(0); break;
      case 1: KVC_SKINNY_LAUNCH(1); break;
      case 2: if constexpr (!GATED) KVC_SKINNY_LAUNCH(2); break;
      default: if constexpr (!GATED) KVC_SKINNY_LAUNCH(3); break;
    }
  } else {
    KVC_SKINNY_LAUNCH(0);
  }
#undef KVC_SKINNY_LAUNCH
}

// The launch shape is a function of N and K alone, so that a row's sums do not depend on
// how many rows come with it.  Measured on MI355X at 1 to 16 rows: 4 waves along K; outputs
// wider than 4096 want 32 weight rows a wave, narrower ones 16.  Row-major matrices whose rows
// lie a multiple of 16 KB apart (K a multiple of 8192: the 70B shape's qkv, o and head) are
// the exception: a wave's two row tiles are then two streams at a distance that maps to the
// same memory channels, and 16 rows a wave read faster, with 8 waves along K at K = 8192
// (10240 x 8192: 42.7 against 51.2 us; 8192 x 8192: 28.8 against 33.8; 16384 x 8192: 52.6
// against 59.8; 8192 x 16384 with 4 waves: 55.1 against 61.5; 8192 x 12288 and 8192 x 28672
// are faster as they were, 38.3 against 41.9 and 80.4 against 88.5).
// KVC_SKINNY_RT / KVC_SKINNY_WAVES override the choice for tuning.
// From a packed matrix a wave takes 16 rows whatever N is: its second 16 rows would be a
// second stream 16 * K elements behind the first, and the two together read slower than one
// (128256 x 4096: 199 against 172 us; 28672 x 4096: 50.5 against 40.6 us).
inline void pick_shape(int N, int K, int packed, int* rt_out, int* waves_out) {
  int rt, waves;
  // the waves along K are the same for a matrix and its packed copy, so that both give the
  // same sums in the same order
  const bool aligned_rows = N > 4096 && K % 8192 == 0;
  waves = (aligned_rows && K <= 8192) ? 8 : 4;
  rt = (N > 4096 && !packed && !aligned_rows) ? 2 : 1;
  while (waves > 1 && K / waves < 128) waves /= 2;
  if (const char* e = getenv("KVC_SKINNY_RT")) rt = atoi(e);
  if (const char* e = getenv("KVC_SKINNY_WAVES")) waves = atoi(e);
  if (rt != 1 && rt != 2) rt = 1;
  const int max_waves = (rt >= 2) ? 4 : 8;
  if (waves < 1) waves = 1;
  if (waves > max_waves) waves = max_waves;
  *rt_out = rt;
  *waves_out = waves;
}

template <typename OutT>
int dispatch(OutT* C, const bf16_t* A, const bf16_t* W, const bf16_t* bias, int M, int N, int K,
             int64_t lda, int64_t ldc, const SkinnyExtras& ex, int packed, hipStream_t stream) {
  int rt, waves;
  pick_shape(N, K, packed, &rt, &waves);
  const int nt = (M + 15) / 16 == 3 ? 4 : (M + 15) / 16;
  int k_per_wave = (K + waves - 1) / waves;
  k_per_wave = (k_per_wave + 63) / 64 * 64;
#define KVC_SKINNY(RT_, NT_) \
  launch<RT_, NT_, OutT>(C, A, W, bias, M, N, K, lda, ldc, waves, k_per_wave, ex, packed, stream)
  switch (rt * 10 + nt) {
    case 11: KVC_SKINNY(1, 1); break;
    case 12: KVC_SKINNY(1, 2); break;
    case 14: KVC_SKINNY(1, 4); break;
    case 21: KVC_SKINNY(2, 1); break;
    case 22: KVC_SKINNY(2, 2); break;
    case 24: KVC_SKINNY(2, 4); break;
    default: return kvc_fail("kvc_gemm_skinny_bf16: unsupported launch shape");
  }
#undef KVC_SKINNY
  return kvc_check_launch("kvc_gemm_skinny_bf16");
}

// silu(A Wg^T) * (A Wu^T) with Wg the first N rows of W and Wu the next N
int dispatch_gated(bf16_t* C, const bf16_t* A, const bf16_t* W, const bf16_t* bias, int M, int N,
                   int K, int64_t lda, int64_t ldc, const SkinnyExtras& ex, int packed, hipStream_t stream) {
  int waves = 4;
  if (const char* e = getenv("KVC_SKINNY_GATED_WAVES")) waves = atoi(e) == 2 ? 2 : 4;  // for tuning
  while (waves > 1 && K / waves < 128) waves /= 2;
  const int nt = (M + 15) / 16 == 3 ? 4 : (M + 15) / 16;
  int k_per_wave = (K + waves - 1) / waves;
  k_per_wave = (k_per_wave + 63) / 64 * 64;
#define KVC_SKINNY_GATED(NT_) \
  launch<2, NT_, bf16_t, true>(C, A, W, bias, M, N, K, lda, ldc, waves, k_per_wave, ex, packed, stream)
  switch (nt) {
    case 1: KVC_SKINNY_GATED(1); break;
    case 2: KVC_SKINNY_GATED(2); break;
    case 4: KVC_SKINNY_GATED(4); break;
    default: return kvc_fail("kvc_gemm_skinny_silu_mul_bf16: unsupported launch shape");
  }
#undef KVC_SKINNY_GATED
  return kvc_check_launch("kvc_gemm_skinny_silu_mul_bf16");
}

}  // namespace

namespace {

int check_operands(const char* who, const void* A, const void* W, int M, int N, int K, int64_t lda,
                   int64_t ldc, int packed) {
  static thread_local char msg[160];
  if (M < 0 || M > 64 || N <= 0 || K <= 0 || lda < K || ldc < N) {
    snprintf(msg, sizeof(msg), "%s: bad sizes (1 to 64 rows)", who);
    return kvc_fail(msg);
  }
  if (K % 8 || lda % 8) {
    snprintf(msg, sizeof(msg), "%s: K and the row stride must be multiples of 8", who);
    return kvc_fail(msg);
  }
  if (packed && (N % 16 || K % 64)) {
    snprintf(msg, sizeof(msg), "%s: packed weights have a multiple of 16 rows of a multiple of 64", who);
    return kvc_fail(msg);
  }
  if ((reinterpret_cast<uintptr_t>(A) & 15) || (reinterpret_cast<uintptr_t>(W) & 15)) {
    snprintf(msg, sizeof(msg), "%s: operands must be 16-byte aligned", who);
    return kvc_fail(msg);
  }
  return 0;
}

const SkinnyExtras kNoExtras = {nullptr, 0, 1.f, 0.f, nullptr, 0, nullptr, nullptr};

}  // namespace

extern "C" int kvc_gemm_skinny_silu_mul_bf16(void* C, const void* A, const void* W, const void* bias,
                                             int M, int N, int K, int64_t lda, int64_t ldc,
                                             int packed, kvc_stream stream) {
  if (int rc = check_operands("kvc_gemm_skinny_silu_mul_bf16", A, W, M, N, K, lda, ldc, packed)) return rc;
  if (M == 0) return 0;
  return dispatch_gated(static_cast<bf16_t*>(C), static_cast<const bf16_t*>(A),
                        static_cast<const bf16_t*>(W), static_cast<const bf16_t*>(bias), M, N, K,
                        lda, ldc, kNoExtras, packed, reinterpret_cast<hipStream_t>(stream));
}

extern "C" int kvc_gemm_skinny_bf16(void* C, const void* A, const void* W, const void* bias, int M,
                                    int N, int K, int64_t lda, int64_t ldc, int out_dtype,
                                    int packed, kvc_stream stream) {
  if (int rc = check_operands("kvc_gemm_skinny_bf16", A, W, M, N, K, lda, ldc, packed)) return rc;
  if (M == 0) return 0;
  hipStream_t s = reinterpret_cast<hipStream_t>(stream);
  if (out_dtype == 0)
    return dispatch<float>(static_cast<float*>(C), static_cast<const bf16_t*>(A),
                           static_cast<const bf16_t*>(W), static_cast<const bf16_t*>(bias), M, N,
                           K, lda, ldc, kNoExtras, packed, s);
  if (out_dtype == 1)
    return dispatch<bf16_t>(static_cast<bf16_t*>(C), static_cast<const bf16_t*>(A),
                            static_cast<const bf16_t*>(W), static_cast<const bf16_t*>(bias), M, N,
                            K, lda, ldc, kNoExtras, packed, s);
  return kvc_fail("kvc_gemm_skinny_bf16: unknown output dtype code");
}

namespace {

// dst tile (n / 16, k / 32) holds src[16 rows][32 k] in one piece of 1 KB, the tiles of a row
// block one after the other along K
__global__ void pack_weight_kernel(bf16_t* __restrict__ dst, const bf16_t* __restrict__ src, int N, int K) {
  const int64_t piece = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;  // 8 elements
  const int per_row = K / 8;
  if (piece >= static_cast<int64_t>(N) * per_row) return;
  const int n = static_cast<int>(piece / per_row);
  const int k = static_cast<int>(piece % per_row) * 8;
  const int64_t at = (static_cast<int64_t>(n >> 4) * (K / 32) + (k >> 5)) * 512 + (n & 15) * 32 + (k & 31);
  *reinterpret_cast<uint4*>(dst + at) = *reinterpret_cast<const uint4*>(src + static_cast<int64_t>(n) * K + k);
}

}  // namespace

extern "C" int kvc_pack_weight(void* dst, const void* src, int N, int K, kvc_stream stream) {
  if (N <= 0 || K <= 0 || N % 16 || K % 64)
    return kvc_fail("kvc_pack_weight: a multiple of 16 rows of a multiple of 64");
  if ((reinterpret_cast<uintptr_t>(dst) & 15) || (reinterpret_cast<uintptr_t>(src) & 15) || dst == src)
    return kvc_fail("kvc_pack_weight: two different 16-byte aligned matrices");
  const int64_t pieces = static_cast<int64_t>(N) * (K / 8);
  hipLaunchKernelGGL(pack_weight_kernel, dim3(static_cast<unsigned>((pieces + 255) / 256)), dim3(256), 0,
                     reinterpret_cast<hipStream_t>(stream), static_cast<bf16_t*>(dst),
                     static_cast<const bf16_t*>(src), N, K);
  return kvc_check_launch("kvc_pack_weight");
}

extern "C" int kvc_gemm_skinny_blocks(int N, int K, int gated, int packed) {
  if (N <= 0 || K <= 0) return 0;
  if (gated) return (N + 15) / 16;
  int rt, waves;
  pick_shape(N, K, packed, &rt, &waves);
  return (N + 16 * rt - 1) / (16 * rt);
}

extern "C" int kvc_gemm_skinny_fused_bf16(void* C, const void* A, const void* W, const void* bias,
                                          int M, int N, int K, int64_t lda, int64_t ldc, int gated,
                                          const float* in_ss, int in_parts, int in_width,
                                          float in_eps, float* residual, int64_t ldr,
                                          const float* gain, float* out_ss, int packed,
                                          kvc_stream stream) {
  if (int rc = check_operands("kvc_gemm_skinny_fused_bf16", A, W, M, N, K, lda, ldc, packed)) return rc;
  if ((in_ss != nullptr || residual != nullptr) && M > 16)
    return kvc_fail("kvc_gemm_skinny_fused_bf16: norms are folded in for at most 16 rows");
  if (in_ss != nullptr && (in_parts <= 0 || in_width <= 0))
    return kvc_fail("kvc_gemm_skinny_fused_bf16: row scaling needs its part count and width");
  if (residual != nullptr && (gain == nullptr || out_ss == nullptr || ldr < N || gated))
    return kvc_fail("kvc_gemm_skinny_fused_bf16: the residual form needs gain and out_ss, rows of "
                    "at least N, and is not gated");
  if (M == 0) return 0;
  SkinnyExtras ex = {in_ss, in_parts, static_cast<float>(in_width), in_eps,
                     residual, ldr, gain, out_ss};
  hipStream_t s = reinterpret_cast<hipStream_t>(stream);
  if (gated)
    return dispatch_gated(static_cast<bf16_t*>(C), static_cast<const bf16_t*>(A),
                          static_cast<const bf16_t*>(W), static_cast<const bf16_t*>(bias), M, N, K,
                          lda, ldc, ex, packed, s);
  return dispatch<bf16_t>(static_cast<bf16_t*>(C), static_cast<const bf16_t*>(A),
                          static_cast<const bf16_t*>(W), static_cast<const bf16_t*>(bias), M, N, K,
                          lda, ldc, ex, packed, s);
}
