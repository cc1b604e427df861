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

#include <cstdlib>

#include "device_utils.h"
#include "kvcore_hip.h"

using namespace kvc;

namespace {

typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef float f32x4_t __attribute__((ext_vector_type(4)));

__device__ __forceinline__ bf16x8_t zero8() {
  bf16x8_t z;
#pragma unroll
  for (int e = 0; e < 8; ++e) z[e] = static_cast<__bf16>(0.f);
  return z;
}

template <typename OutT>
__device__ __forceinline__ void store4(OutT* p, f32x4_t v, int n_left);
template <>
__device__ __forceinline__ void store4<float>(float* p, f32x4_t v, int n_left) {
  if (n_left >= 4 && (reinterpret_cast<uintptr_t>(p) & 15) == 0) {
    *reinterpret_cast<f32x4_t*>(p) = v;
  } else {
    for (int i = 0; i < 4 && i < n_left; ++i) p[i] = v[i];
  }
}
template <>
__device__ __forceinline__ void store4<bf16_t>(bf16_t* p, f32x4_t v, int n_left) {
  if (n_left >= 4 && (reinterpret_cast<uintptr_t>(p) & 7) == 0) {
    uint2 packed;
    packed.x = f32_to_bf16_bits(v[0]) | (static_cast<uint32_t>(f32_to_bf16_bits(v[1])) << 16);
    packed.y = f32_to_bf16_bits(v[2]) | (static_cast<uint32_t>(f32_to_bf16_bits(v[3])) << 16);
    *reinterpret_cast<uint2*>(p) = packed;
  } else {
    for (int i = 0; i < 4 && i < n_left; ++i) p[i].bits = f32_to_bf16_bits(v[i]);
  }
}

// GATED: the two row tiles of a wave are rows n of the first N weight rows (gate) and rows
// N + n (up), and the stored value is silu(gate) * up, each factor rounded to bfloat16
// first as if it had been stored.
template <int RT, int NT, int U, int MAXW, typename OutT, bool GATED>
__global__ __launch_bounds__(MAXW * 64) void gemm_skinny_kernel(OutT* __restrict__ C, const bf16_t* __restrict__ A,
                                   const bf16_t* __restrict__ W, const bf16_t* __restrict__ bias,
                                   int M, int N, int K, int64_t lda, int64_t ldc, int k_per_wave) {
  static_assert(!GATED || RT == 2, "the gated form pairs one gate tile with one up tile");
  extern __shared__ float red[];  // [waves - 1][RT * NT][64][4]
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

  const bf16_t* wp[RT];
#pragma unroll
  for (int rt = 0; rt < RT; ++rt) {
    const int r = GATED ? n0 + col : n0 + rt * 16 + col;
    const int64_t row = (r < N ? r : N - 1) + ((GATED && rt == 1) ? N : 0);
    wp[rt] = W + row * K + 8 * quad;
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
      abuf[stage][rt][0] = *reinterpret_cast<const bf16x8_t*>(wp[rt] + k);
      abuf[stage][rt][1] = *reinterpret_cast<const bf16x8_t*>(wp[rt] + k + 32);
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
  int k = k_begin;
#pragma unroll
  for (int st = 0; st < STAGES - 1; ++st)
    if (st < n64) load_step(st, st);
  for (int i = 0; i < n64; i += STAGES) {
#pragma unroll
    for (int j = 0; j < STAGES; ++j) {
      if (i + j < n64) {  // the same for the whole wave, and a scalar branch
        if (i + j + STAGES - 1 < n64) load_step((j + STAGES - 1) % STAGES, i + j + STAGES - 1);
        mma_step(j);
      }
    }
  }
  k = k_begin + 64 * n64;
  const int k_full = k + ((k_end - k) / 32) * 32;
  for (; k < k_full; k += 32) {
    bf16x8_t a[RT], b[NT];
#pragma unroll
    for (int rt = 0; rt < RT; ++rt) a[rt] = *reinterpret_cast<const bf16x8_t*>(wp[rt] + k);
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
      a[rt] = valid ? *reinterpret_cast<const bf16x8_t*>(wp[rt] + k_full) : zero8();
#pragma unroll
    for (int nt = 0; nt < NT; ++nt)
      b[nt] = valid ? *reinterpret_cast<const bf16x8_t*>(ap[nt] + k_full) : zero8();
#pragma unroll
    for (int rt = 0; rt < RT; ++rt)
#pragma unroll
      for (int nt = 0; nt < NT; ++nt)
        acc[rt][nt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[rt], b[nt], acc[rt][nt], 0, 0, 0);
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
        const float gv = to_float(from_float<bf16_t>(acc[0][nt][i] + bg[i]));
        const float uv = to_float(from_float<bf16_t>(acc[1][nt][i] + bu[i]));
        y[i] = gv / (1.f + expf(-gv)) * uv;
      }
      store4<OutT>(C + static_cast<int64_t>(tok) * ldc + n_first, y, n_left);
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
      store4<OutT>(C + static_cast<int64_t>(tok) * ldc + n_first, acc[rt][nt] + bv, n_left);
    }
  }
}

template <int RT, int NT, typename OutT, bool GATED = false>
void launch(OutT* C, const bf16_t* A, const bf16_t* W, const bf16_t* bias, int M, int N, int K,
            int64_t lda, int64_t ldc, int waves, int k_per_wave, hipStream_t stream) {
  // steps in flight by what fits in registers beside the accumulators
  constexpr int STAGES = (RT + NT <= 5) ? 4 : ((RT + NT <= 6) ? 3 : 2);
  constexpr int MAXW = (RT >= 2) ? 4 : 8;
  const size_t lds = static_cast<size_t>(waves - 1) * RT * NT * 64 * 4 * sizeof(float);
  const int rows_per_block = GATED ? 16 : 16 * RT;
  hipLaunchKernelGGL((gemm_skinny_kernel<RT, NT, STAGES, MAXW, OutT, GATED>),
                     dim3((N + rows_per_block - 1) / rows_per_block), dim3(waves * 64), lds, stream,
                     C, A, W, bias, M, N, K, lda, ldc, k_per_wave);
}

// The launch shape is a function of N and K alone, so that a row's sums do not depend on
// how many rows come with it.  Measured on MI355X at 1 to 16 rows: 4 waves along K; outputs
// wider than 4096 want 32 weight rows a wave, narrower ones 16.
// KVC_SKINNY_RT / KVC_SKINNY_WAVES override the choice for tuning.
inline void pick_shape(int N, int K, int* rt_out, int* waves_out) {
  int rt, waves;
  if (N > 4096) {
    rt = 2;
    waves = 4;
  } else {
    rt = 1;
    waves = 4;
  }
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
             int64_t lda, int64_t ldc, hipStream_t stream) {
  int rt, waves;
  pick_shape(N, K, &rt, &waves);
  const int nt = (M + 15) / 16 == 3 ? 4 : (M + 15) / 16;
  int k_per_wave = (K + waves - 1) / waves;
  k_per_wave = (k_per_wave + 63) / 64 * 64;
#define KVC_SKINNY(RT_, NT_) \
  launch<RT_, NT_, OutT>(C, A, W, bias, M, N, K, lda, ldc, waves, k_per_wave, stream)
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
                   int K, int64_t lda, int64_t ldc, hipStream_t stream) {
  int waves = 4;
  while (waves > 1 && K / waves < 128) waves /= 2;
  const int nt = (M + 15) / 16 == 3 ? 4 : (M + 15) / 16;
  int k_per_wave = (K + waves - 1) / waves;
  k_per_wave = (k_per_wave + 63) / 64 * 64;
#define KVC_SKINNY_GATED(NT_) \
  launch<2, NT_, bf16_t, true>(C, A, W, bias, M, N, K, lda, ldc, waves, k_per_wave, stream)
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

extern "C" int kvc_gemm_skinny_silu_mul_bf16(void* C, const void* A, const void* W, const void* bias,
                                             int M, int N, int K, int64_t lda, int64_t ldc,
                                             kvc_stream stream) {
  if (M < 0 || M > 64 || N <= 0 || K <= 0 || lda < K || ldc < N)
    return kvc_fail("kvc_gemm_skinny_silu_mul_bf16: bad sizes (1 to 64 rows)");
  if (K % 8 || lda % 8)
    return kvc_fail("kvc_gemm_skinny_silu_mul_bf16: K and the row stride must be multiples of 8");
  if ((reinterpret_cast<uintptr_t>(A) & 15) || (reinterpret_cast<uintptr_t>(W) & 15))
    return kvc_fail("kvc_gemm_skinny_silu_mul_bf16: operands must be 16-byte aligned");
  if (M == 0) return 0;
  return dispatch_gated(static_cast<bf16_t*>(C), static_cast<const bf16_t*>(A),
                        static_cast<const bf16_t*>(W), static_cast<const bf16_t*>(bias), M, N, K,
                        lda, ldc, reinterpret_cast<hipStream_t>(stream));
}

extern "C" int kvc_gemm_skinny_bf16(void* C, const void* A, const void* W, const void* bias, int M,
                                    int N, int K, int64_t lda, int64_t ldc, int out_dtype,
                                    kvc_stream stream) {
  if (M < 0 || M > 64 || N <= 0 || K <= 0 || lda < K || ldc < N)
    return kvc_fail("kvc_gemm_skinny_bf16: bad sizes (1 to 64 rows)");
  if (K % 8 || lda % 8)
    return kvc_fail("kvc_gemm_skinny_bf16: K and the row stride must be multiples of 8");
  if ((reinterpret_cast<uintptr_t>(A) & 15) || (reinterpret_cast<uintptr_t>(W) & 15))
    return kvc_fail("kvc_gemm_skinny_bf16: operands must be 16-byte aligned");
  if (M == 0) return 0;
  hipStream_t s = reinterpret_cast<hipStream_t>(stream);
  if (out_dtype == 0)
    return dispatch<float>(static_cast<float*>(C), static_cast<const bf16_t*>(A),
                           static_cast<const bf16_t*>(W), static_cast<const bf16_t*>(bias), M, N,
                           K, lda, ldc, s);
  if (out_dtype == 1)
    return dispatch<bf16_t>(static_cast<bf16_t*>(C), static_cast<const bf16_t*>(A),
                            static_cast<const bf16_t*>(W), static_cast<const bf16_t*>(bias), M, N,
                            K, lda, ldc, s);
  return kvc_fail("kvc_gemm_skinny_bf16: unknown output dtype code");
}
