// C[M, N] = A[M, K] * W[N, K]^T (+ bias) for up to 192 rows of bfloat16 (used from 17 on),
// float32 sums: the decode step of a few dozen requests.  The weight matrix is still read
// once from HBM, but the activations are no longer small beside a wave's share of it, so the
// waves of a block share them through LDS instead of each reading its own copy from the cache.
//
// A block of WAVES waves owns WAVES * 16 * RT weight rows and a slice of K.  Each wave
// walks its 16 * RT rows along the slice in steps of 64, with the weights of the next two
// to four steps on their way into registers (a lane loads 16 bytes of one row, a row reads
// 128 contiguous bytes a step, and the two steps of a chunk are asked for together).  The
// rows of A of the slice pass through two LDS buffers in chunks of 128 along K, fetched by
// all waves together as far ahead as the weights: one barrier a chunk.  All loads are issued
// without a branch around them (addresses beyond the slice are bent back into it and their
// values never multiplied), so that the waits can count them exactly and none drains the queue.
// Four steps in flight and chunks of 128 keep a block of four waves within 36 KB of LDS and
// half the registers, so that two blocks share a compute unit: measured against eight steps
// and chunks of 256 (one block a unit), the wide products at K = 4096 take 4 to 11% less time
// and those at K = 8192 the same.
//
//   C^T[16 weight rows, 16 tokens] += W[16 rows, 32 k] * A^T[32 k, 16 tokens]   (16x16x32)
//
// With one slice the results are stored at once (plain, or silu(gate) * up for a pair of
// row tiles); with several, each slice leaves float32 partial sums [slice, M, N] that the
// caller adds up, in slice order, in the kernel that consumes them.  The launch shape
// depends on N and K alone, so a row's sums do not depend on what else is in the batch.

#include <hip/hip_runtime.h>

#include <cstdio>
#include <cstdlib>

#include "device_utils.h"
#include "gemm_common.h"
#include "kvcore_hip.h"

using namespace kvc;

namespace {

constexpr int kChunk = 128;             // k per LDS chunk
constexpr int kChunkSteps = kChunk / 64;
constexpr int kRowElems = kChunk + 8;   // padded against bank conflicts
constexpr int kStages = 4;              // steps of weights in flight per wave, the current one included
constexpr int kRound = 64 * kStages;    // a slice of K is whole rounds of this many
constexpr int kKMultiple = 512;         // what callers are promised: K is a multiple of this
constexpr int kMaxRows = 192;           // rows of A: up to twelve 16-row tiles a wave (sixteen were measured slower than the vendor's product)
static_assert(kKMultiple % kRound == 0, "every K that is accepted must be whole rounds");

template <int WAVES, int RT, int NT, bool GATED, typename OutT>
__global__ __launch_bounds__(WAVES * 64) void gemm_mid_kernel(
    OutT* __restrict__ C, float* __restrict__ partial, const bf16_t* __restrict__ A,
    const bf16_t* __restrict__ W, const bf16_t* __restrict__ bias, int M, int N, int K, int64_t lda,
    int64_t ldc, int k_per_block, int packed) {
  static_assert(!GATED || RT == 2, "the gated form pairs one gate tile with one up tile");
  static_assert(kStages % (2 * kChunkSteps) == 0, "a round of stages must cover whole pairs of chunks");
  __shared__ __attribute__((aligned(16))) bf16_t a_lds[2][NT * 16 * kRowElems];
  constexpr int THREADS = WAVES * 64;
  constexpr int PIECES = NT * 16 * (kChunk / 8);  // 16-byte pieces of a chunk
  constexpr int PER_THREAD = PIECES / THREADS;
  static_assert(PIECES % THREADS == 0, "a chunk must divide among the threads");

  const int tid = threadIdx.x;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);  // scalar: see gemm_skinny.hip
  const int lane = tid & 63;
  const int col = lane & 15;
  const int quad = lane >> 4;
  constexpr int COLS_PER_WAVE = GATED ? 16 : 16 * RT;
  const int n0 = (blockIdx.x * WAVES + wave) * COLS_PER_WAVE;
  const int k_begin = blockIdx.y * k_per_block;
  const int k_end = (k_begin + k_per_block < K) ? k_begin + k_per_block : K;
  const int n_steps = (k_end - k_begin) / 64;  // the host makes slices whole rounds of steps

  const int ks = packed ? 16 : 1;
  const bf16_t* wp[RT];
#pragma unroll
  for (int rt = 0; rt < RT; ++rt) {
    const int r = GATED ? n0 + col : n0 + rt * 16 + col;
    const int64_t row = (r < N ? r : N - 1) + ((GATED && rt == 1) ? N : 0);
    // packed: what kvc_pack_weight made of W (tiles of 16 rows x 32 k, 1 KB each, along K)
    wp[rt] = packed ? W + (row >> 4) * (static_cast<int64_t>(K) * 16) + (row & 15) * 32 +
                          static_cast<int64_t>(k_begin) * 16 + 8 * quad
                    : W + row * K + k_begin + 8 * quad;
  }
  // this thread's pieces of a chunk of A: rows beyond M read the last row and are dropped
  // at the end
  const bf16_t* a_src[PER_THREAD];
  int a_dst[PER_THREAD];
  const int piece_k = (tid % (kChunk / 8)) * 8;
#pragma unroll
  for (int i = 0; i < PER_THREAD; ++i) {
    const int row = (i * THREADS + tid) / (kChunk / 8);
    a_src[i] = A + static_cast<int64_t>(row < M ? row : M - 1) * lda + k_begin + piece_k;
    a_dst[i] = row * kRowElems + piece_k;
  }

  f32x4_t acc[RT][NT];
#pragma unroll
  for (int rt = 0; rt < RT; ++rt)
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) acc[rt][nt] = f32x4_t{0.f, 0.f, 0.f, 0.f};

  bf16x8_t wbuf[kStages][RT][2];
  constexpr int AHEAD = kStages / kChunkSteps;  // chunks of A on their way, as far ahead as the weights
  bf16x8_t areg[AHEAD][PER_THREAD];
  // Blocks start their walk along the slice at different rounds and wrap: all of them at
  // the same k at the same time would ask the same memory channels.
  const int rot = static_cast<int>(blockIdx.x % static_cast<unsigned>(n_steps / kStages)) * kStages;
  auto where = [&](int step) {  // the 64-wide step of the slice that is this block's step-th
    const int s = (step < n_steps) ? step : n_steps - 1;
    return (s + rot < n_steps) ? s + rot : s + rot - n_steps;
  };
  auto load_w = [&](int stage, int step) {
    const int k = 64 * where(step);
#pragma unroll
    for (int rt = 0; rt < RT; ++rt) {
      wbuf[stage][rt][0] = *reinterpret_cast<const bf16x8_t*>(wp[rt] + k * ks);
      wbuf[stage][rt][1] = *reinterpret_cast<const bf16x8_t*>(wp[rt] + (k + 32) * ks);
    }
  };
  auto fetch_chunk = [&](int slot, int chunk) {
    // a chunk beyond the slice: the last whole chunk again, never multiplied.  (The start is
    // bent back by whole chunks, so that all columns of it that are read lie inside the slice:
    // rounds, and with them the rotation, are whole chunks.)
    const int first = (chunk * kChunkSteps < n_steps) ? chunk * kChunkSteps : n_steps - kChunkSteps;
    const int k = 64 * where(first);
#pragma unroll
    for (int i = 0; i < PER_THREAD; ++i) areg[slot][i] = *reinterpret_cast<const bf16x8_t*>(a_src[i] + k);
  };
  auto store_chunk = [&](int slot, int buf) {
#pragma unroll
    for (int i = 0; i < PER_THREAD; ++i) *reinterpret_cast<bf16x8_t*>(&a_lds[buf][a_dst[i]]) = areg[slot][i];
  };
  auto mma_step = [&](int stage, int buf, int part) {
#pragma unroll
    for (int h = 0; h < 2; ++h) {
      // the tiles of A four at a time: with many tiles, all of them at once cost registers
      constexpr int G = NT < 4 ? NT : 4;
#pragma unroll
      for (int n0 = 0; n0 < NT; n0 += G) {
        bf16x8_t b[G];
#pragma unroll
        for (int j = 0; j < G; ++j)
          if (n0 + j < NT)
            b[j] = *reinterpret_cast<const bf16x8_t*>(
                &a_lds[buf][((n0 + j) * 16 + col) * kRowElems + part * 64 + h * 32 + 8 * quad]);
#pragma unroll
        for (int rt = 0; rt < RT; ++rt)
#pragma unroll
          for (int j = 0; j < G; ++j)
            if (n0 + j < NT)
              acc[rt][n0 + j] =
                  __builtin_amdgcn_mfma_f32_16x16x32_bf16(wbuf[stage][rt][h], b[j], acc[rt][n0 + j], 0, 0, 0);
      }
    }
  };

  // Loads complete in the order of their issue, so a chunk of A is asked for when the weights
  // of its steps are: by the time it is wanted in LDS it is the oldest load in flight and
  // waiting for it drains nothing.
#pragma unroll
  for (int st = 0; st < kStages; ++st) {
    if (st % kChunkSteps == 0) fetch_chunk(st / kChunkSteps, st / kChunkSteps);
    load_w(st, st);
  }
  store_chunk(0, 0);
  __syncthreads();
  // A slice is whole rounds of kStages steps (the host sees to it), so the body is one
  // straight line: a branch inside it would make the waits at the loop's head assume the
  // worst and drain every load in flight once a round.  The weights of a whole chunk's steps
  // are asked for together, when the chunk before them has been multiplied: a row's 256
  // contiguous bytes then reach the memory close in time.
  for (int s0 = 0; s0 < n_steps; s0 += kStages) {
#pragma unroll
    for (int j = 0; j < kStages; ++j) {
      const int step = s0 + j;
      const int cj = j / kChunkSteps;  // the chunk's number within the round
      mma_step(j, cj & 1, j % kChunkSteps);
      if (j % kChunkSteps == kChunkSteps - 1) {
        // this chunk's registers are free: the chunk a round ahead, rows of A first
        fetch_chunk(cj % AHEAD, step / kChunkSteps + AHEAD);
#pragma unroll
        for (int t = 0; t < kChunkSteps; ++t) load_w(cj * kChunkSteps + t, step + 1 - kChunkSteps + t + kStages);
        // the chunk after this one goes into the buffer that was read a chunk ago
        store_chunk((cj + 1) % AHEAD, (cj + 1) & 1);
        __syncthreads();
      }
    }
  }

  // acc[rt][nt][i] = C[token nt*16 + col][n0 + rt*16 + 4*quad + i]
  if (partial != nullptr) {
#pragma unroll
    for (int rt = 0; rt < RT; ++rt) {
      const int n_first = n0 + rt * 16 + 4 * quad;
      const int n_left = N - n_first;
      if (n_left <= 0) continue;
#pragma unroll
      for (int nt = 0; nt < NT; ++nt) {
        const int tok = nt * 16 + col;
        if (tok >= M) continue;
        store4<float>(partial + (static_cast<int64_t>(blockIdx.y) * M + tok) * N + n_first, acc[rt][nt], n_left);
      }
    }
    return;
  }
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

// C[M, N] = sum over slices of partial[slice, M, N] (+ bias), four columns a thread
template <typename OutT>
__global__ void sum_slices_kernel(OutT* __restrict__ C, const float* __restrict__ partial,
                                  const bf16_t* __restrict__ bias, int M, int N, int64_t ldc, int slices) {
  const int n4 = (N + 3) / 4;
  const int64_t idx = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (idx >= static_cast<int64_t>(M) * n4) return;
  const int tok = static_cast<int>(idx / n4);
  const int n_first = static_cast<int>(idx % n4) * 4;
  const int n_left = N - n_first;
  f32x4_t sum = f32x4_t{0.f, 0.f, 0.f, 0.f};
  for (int s = 0; s < slices; ++s) {
    const float* p = partial + (static_cast<int64_t>(s) * M + tok) * N + n_first;
    if (n_left >= 4 && (reinterpret_cast<uintptr_t>(p) & 15) == 0) {
      sum += *reinterpret_cast<const f32x4_t*>(p);
    } else {
      for (int i = 0; i < 4 && i < n_left; ++i) sum[i] += p[i];
    }
  }
  if (bias != nullptr)
    for (int i = 0; i < 4 && i < n_left; ++i) sum[i] += to_float(bias[n_first + i]);
  store4<OutT>(C + static_cast<int64_t>(tok) * ldc + n_first, sum, n_left);
}

struct MidPlan {
  int waves;   // per block
  int rt;      // 16-row tiles per wave
  int slices;  // along K
  int k_per_block;
  int packed;  // W is in kvc_pack_weight's order
};

// Blocks enough for every compute unit, from N and K alone.  Narrow outputs are cut along K
// (at least 512 of it a slice, in whole chunks); wide ones are not.
// KVC_MID_WAVES / KVC_MID_RT / KVC_MID_SLICES override the choice for tuning.
MidPlan plan_mid(int N, int K, bool gated, bool may_slice) {
  MidPlan p;
  p.packed = 0;
  // two waves a block where four would leave compute units without one
  p.waves = (gated && (N + 63) / 64 < 192) ? 2 : 4;
  p.rt = gated ? 2 : (N >= 16384 ? 2 : 1);
  if (const char* e = getenv("KVC_MID_WAVES")) p.waves = atoi(e);
  if (const char* e = getenv("KVC_MID_RT")) p.rt = atoi(e);
  if (gated) p.rt = 2;
  if (p.rt != 1 && p.rt != 2) p.rt = 1;
  if (p.waves != 2 && p.waves != 4) p.waves = 4;
  const int cols_per_block = p.waves * (gated ? 16 : 16 * p.rt);
  const int blocks_n = (N + cols_per_block - 1) / cols_per_block;
  int slices = 1;
  if (may_slice) {
    slices = (256 + blocks_n - 1) / blocks_n;
    const int most = K / 512 > 0 ? K / 512 : 1;
    if (slices > most) slices = most;
    if (const char* e = getenv("KVC_MID_SLICES")) slices = atoi(e);
    if (slices < 1) slices = 1;
    if (slices > 64) slices = 64;
  }
  int per = (K + slices - 1) / slices;
  per = (per + kRound - 1) / kRound * kRound;
  p.k_per_block = per;
  p.slices = (K + per - 1) / per;
  return p;
}

template <int WAVES, int RT, int NT, bool GATED, typename OutT>
void launch_mid(OutT* C, float* partial, const bf16_t* A, const bf16_t* W, const bf16_t* bias, int M,
                int N, int K, int64_t lda, int64_t ldc, const MidPlan& p, hipStream_t stream) {
  const int cols_per_block = WAVES * (GATED ? 16 : 16 * RT);
  const dim3 grid((N + cols_per_block - 1) / cols_per_block, p.slices), block(WAVES * 64);
  hipLaunchKernelGGL((gemm_mid_kernel<WAVES, RT, NT, GATED, OutT>), grid, block, 0, stream, C,
                     p.slices > 1 ? partial : nullptr, A, W, bias, M, N, K, lda, ldc, p.k_per_block, p.packed);
}

template <bool GATED, typename OutT>
int dispatch_mid(OutT* C, float* partial, const bf16_t* A, const bf16_t* W, const bf16_t* bias, int M,
                 int N, int K, int64_t lda, int64_t ldc, const MidPlan& p, hipStream_t stream) {
  const int nt = (M + 15) / 16;
  // with more than eight tiles of rows a block of two waves would hold a chunk of A in more
  // registers than there are: four waves then (the slices along K, and with them the order of
  // every sum, stay as planned)
  const int waves = nt > 8 ? 4 : p.waves;
#define KVC_MID(W_, RT_, NT_) \
  launch_mid<W_, RT_, NT_, GATED, OutT>(C, partial, A, W, bias, M, N, K, lda, ldc, p, stream)
#define KVC_MID_NT(W_, RT_)                                   \
  switch (nt) {                                               \
    case 1: KVC_MID(W_, RT_, 1); break;                       \
    case 2: KVC_MID(W_, RT_, 2); break;                       \
    case 3: KVC_MID(W_, RT_, 3); break;                       \
    case 4: KVC_MID(W_, RT_, 4); break;                       \
    case 5:                                                   \
    case 6: KVC_MID(W_, RT_, 6); break;                       \
    case 7:                                                   \
    case 8: KVC_MID(W_, RT_, 8); break;                       \
    case 9:                                                   \
    case 10:                                                  \
    case 11:                                                  \
    default: KVC_MID(W_, RT_, 12); break;                     \
  }
  if constexpr (GATED) {
    switch (waves) {
      case 2: KVC_MID_NT(2, 2); break;
      default: KVC_MID_NT(4, 2); break;
    }
  } else {
    switch (waves * 10 + p.rt) {
      case 21: KVC_MID_NT(2, 1); break;
      case 22: KVC_MID_NT(2, 2); break;
      case 42: KVC_MID_NT(4, 2); break;
      default: KVC_MID_NT(4, 1); break;
    }
  }
#undef KVC_MID_NT
#undef KVC_MID
  return kvc_check_launch("kvc_gemm_mid_bf16");
}

int check_mid(const void* A, const void* W, int M, int N, int K, int64_t lda, int64_t ldc) {
  if (M < 0 || M > kMaxRows || N <= 0 || K <= 0 || lda < K || ldc < N)
    return kvc_fail("kvc_gemm_mid_bf16: bad sizes (1 to 192 rows)");
  if (K % kKMultiple || lda % 8)
    return kvc_fail("kvc_gemm_mid_bf16: K must be a multiple of 512 and the row stride of 8");
  if ((reinterpret_cast<uintptr_t>(A) & 15) || (reinterpret_cast<uintptr_t>(W) & 15))
    return kvc_fail("kvc_gemm_mid_bf16: operands must be 16-byte aligned");
  return 0;
}

}  // namespace

extern "C" int kvc_gemm_mid_slices(int N, int K) {
  if (N <= 0 || K <= 0 || K % kKMultiple) return 0;
  return plan_mid(N, K, false, true).slices;
}

extern "C" int kvc_gemm_mid_bf16(void* C, void* partial, const void* A, const void* W, const void* bias,
                                 int M, int N, int K, int64_t lda, int64_t ldc, int out_dtype, int mode,
                                 int packed, kvc_stream stream) {
  if (int rc = check_mid(A, W, M, N, K, lda, ldc)) return rc;
  if (packed && N % 16) return kvc_fail("kvc_gemm_mid_bf16: packed weights have a multiple of 16 rows");
  if (mode < 0 || mode > 3) return kvc_fail("kvc_gemm_mid_bf16: unknown mode");
  if (M == 0) return 0;
  hipStream_t s = reinterpret_cast<hipStream_t>(stream);
  const bf16_t* a = static_cast<const bf16_t*>(A);
  const bf16_t* w = static_cast<const bf16_t*>(W);
  const bf16_t* b = static_cast<const bf16_t*>(bias);
  float* part = static_cast<float*>(partial);
  if (mode == 1) {  // silu(A Wg^T) * (A Wu^T): one slice, bfloat16
    if (out_dtype != 1) return kvc_fail("kvc_gemm_mid_bf16: the gated form stores bfloat16");
    MidPlan p = plan_mid(N, K, true, false);
    p.packed = packed;
    return dispatch_mid<true>(static_cast<bf16_t*>(C), nullptr, a, w, b, M, N, K, lda, ldc, p, s);
  }
  if (mode == 2) {  // only the slices' partial sums
    if (part == nullptr) return kvc_fail("kvc_gemm_mid_bf16: the partial sums need their buffer");
    MidPlan p = plan_mid(N, K, false, true);
    p.packed = packed;
    if (p.slices == 1) {  // a single slice is the result: float32 [M, N]
      return dispatch_mid<false>(part, nullptr, a, w, nullptr, M, N, K, lda, N, p, s);
    }
    return dispatch_mid<false>(part, part, a, w, nullptr, M, N, K, lda, N, p, s);
  }
  // plain product: one slice at once, or (mode 3, given a buffer) slices and their sum
  MidPlan p = plan_mid(N, K, false, mode == 3 && part != nullptr);
  p.packed = packed;
  if (out_dtype != 0 && out_dtype != 1) return kvc_fail("kvc_gemm_mid_bf16: unknown output dtype code");
  if (p.slices == 1) {
    if (out_dtype == 0)
      return dispatch_mid<false>(static_cast<float*>(C), nullptr, a, w, b, M, N, K, lda, ldc, p, s);
    return dispatch_mid<false>(static_cast<bf16_t*>(C), nullptr, a, w, b, M, N, K, lda, ldc, p, s);
  }
  if (int rc = dispatch_mid<false>(part, part, a, w, nullptr, M, N, K, lda, N, p, s)) return rc;
  const int64_t work = static_cast<int64_t>(M) * ((N + 3) / 4);
  const dim3 grid(static_cast<unsigned>((work + 255) / 256));
  if (out_dtype == 0)
    hipLaunchKernelGGL(sum_slices_kernel<float>, grid, dim3(256), 0, s, static_cast<float*>(C), part, b, M,
                       N, ldc, p.slices);
  else
    hipLaunchKernelGGL(sum_slices_kernel<bf16_t>, grid, dim3(256), 0, s, static_cast<bf16_t*>(C), part, b,
                       M, N, ldc, p.slices);
  return kvc_check_launch("kvc_gemm_mid_bf16");
}
