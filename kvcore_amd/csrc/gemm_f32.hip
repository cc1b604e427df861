// C[M, N] = A[M, K] * W[N, K]^T (+ bias) in true float32: float32 products,
// float32 sums, no matrix-core mode of reduced precision.
//
// A 64x64 tile of C per block of 256 threads, each thread a 4x4 patch; K is walked in
// steps of 16 through LDS.  Every element of C is one accumulator that takes its
// products in the order k = 0, 1, ..., K-1, so its value does not depend on M, on the
// tile it falls in or on its row's place in the batch.

#include <hip/hip_runtime.h>

#include "device_utils.h"
#include "kvcore_hip.h"

namespace {

constexpr int BM = 64, BN = 64, BK = 16;

__global__ __launch_bounds__(256) void gemm_f32_kernel(float* __restrict__ C,
                                                       const float* __restrict__ A,
                                                       const float* __restrict__ W,
                                                       const float* __restrict__ bias, int M,
                                                       int N, int K, int64_t lda, int64_t ldc) {
  __shared__ float As[BK][BM + 4];
  __shared__ float Ws[BK][BN + 4];
  const int tid = threadIdx.x;
  const int tx = tid & 15;   // column patch
  const int ty = tid >> 4;   // row patch
  const int m0 = blockIdx.y * BM;
  const int n0 = blockIdx.x * BN;

  float acc[4][4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) acc[i][j] = 0.f;

  // loader mapping: 256 threads fetch 64 rows x 16 k: thread -> (row = tid / 4, k4 = tid % 4)
  const int lrow = tid >> 2;
  const int lk = (tid & 3) * 4;

  for (int k0 = 0; k0 < K; k0 += BK) {
    float a[4], w[4];
    const int am = m0 + lrow;
    const int wn = n0 + lrow;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int k = k0 + lk + i;
      a[i] = (am < M && k < K) ? A[static_cast<int64_t>(am) * lda + k] : 0.f;
      w[i] = (wn < N && k < K) ? W[static_cast<int64_t>(wn) * K + k] : 0.f;
    }
    __syncthreads();
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      As[lk + i][lrow] = a[i];
      Ws[lk + i][lrow] = w[i];
    }
    __syncthreads();
#pragma unroll
    for (int k = 0; k < BK; ++k) {
      float av[4], wv[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) av[i] = As[k][ty * 4 + i];
#pragma unroll
      for (int j = 0; j < 4; ++j) wv[j] = Ws[k][tx * 4 + j];
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = fmaf(av[i], wv[j], acc[i][j]);
    }
  }

#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int m = m0 + ty * 4 + i;
    if (m >= M) continue;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int n = n0 + tx * 4 + j;
      if (n >= N) continue;
      float v = acc[i][j];
      if (bias != nullptr) v += bias[n];
      C[static_cast<int64_t>(m) * ldc + n] = v;
    }
  }
}

}  // namespace

extern "C" int kvc_gemm_f32(float* C, const float* A, const float* W, const float* bias, int M,
                            int N, int K, int64_t lda, int64_t ldc, kvc_stream stream) {
  if (M < 0 || N <= 0 || K <= 0 || lda < K || ldc < N) return kvc_fail("kvc_gemm_f32: bad sizes");
  if (M == 0) return 0;
  const dim3 grid((N + BN - 1) / BN, (M + BM - 1) / BM);
  if (grid.y > 65535) return kvc_fail("kvc_gemm_f32: M too large for one launch");
  hipLaunchKernelGGL(gemm_f32_kernel, grid, dim3(256), 0, reinterpret_cast<hipStream_t>(stream),
                     C, A, W, bias, M, N, K, lda, ldc);
  return kvc_check_launch("kvc_gemm_f32");
}
