// True 32-bit matrix product  C[M,N] = A[M,K] . W[N,K]^T  (both operands K-major).
//
// This is the projection kernel of the 32-bit path of the model: no reduced
// precision anywhere, and every output element is added up in one fixed order:
// a chain of fused multiply-adds over each 16 consecutive k (from k = 0 on), the
// sums of sixteen such chains added in ascending order into the sum of 256 k, and
// those in ascending order into the result.  (One chain over all of K loses about
// sqrt(K) roundings, 50 at K = 2,560 and 100 at K = 9,728, and at 36 layers of
// such products the logits sat at 1.1e-5 of their largest; three levels lose about
// 4 + 4 + sqrt(K / 256).)  The order does not depend on M, on the tile an element
// falls into, or on what else is in the batch, so a token's result is bit-identical
// however the work is cut into steps.
// Reference counterpart (bf16, library): crates/cuda-kernels/csrc/gemm/gemv.cu:240-330.
#include "common.h"

namespace arle {

constexpr int kBM = 64, kBN = 64, kBK = 16;
constexpr int kGemmThreads = 256;
constexpr int kMidTiles = 16;  // tiles of kBK whose sums are added up before they join the result

__global__ __launch_bounds__(kGemmThreads) void gemm_f32_kernel(
    const float* __restrict__ a, int64_t lda, const float* __restrict__ w, int64_t ldw,
    float* __restrict__ c, int64_t ldc, int M, int N, int K) {
  __shared__ float as[kBK][kBM + 4];
  __shared__ float ws[kBK][kBN + 4];
  const int m0 = blockIdx.y * kBM;
  const int n0 = blockIdx.x * kBN;
  const int tx = threadIdx.x % 16;  // columns tx*4 .. tx*4+3
  const int ty = threadIdx.x / 16;  // rows    ty*4 .. ty*4+3
  float acc[4][4] = {}, mid[4][4] = {};

  for (int k0 = 0; k0 < K; k0 += kBK) {
#pragma unroll
    for (int i = 0; i < (kBM * kBK) / kGemmThreads; ++i) {
      const int idx = threadIdx.x + i * kGemmThreads;
      const int row = idx / kBK, col = idx % kBK;
      const int gm = m0 + row, gn = n0 + row, gk = k0 + col;
      as[col][row] = (gm < M && gk < K) ? a[static_cast<int64_t>(gm) * lda + gk] : 0.f;
      ws[col][row] = (gn < N && gk < K) ? w[static_cast<int64_t>(gn) * ldw + gk] : 0.f;
    }
    __syncthreads();
    float part[4][4] = {};
#pragma unroll
    for (int kk = 0; kk < kBK; ++kk) {
      float av[4], wv[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) av[i] = as[kk][ty * 4 + i];
#pragma unroll
      for (int j = 0; j < 4; ++j) wv[j] = ws[kk][tx * 4 + j];
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) part[i][j] = fmaf(av[i], wv[j], part[i][j]);
    }
    const bool flush = ((k0 / kBK) % kMidTiles) == kMidTiles - 1 || k0 + kBK >= K;
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        mid[i][j] += part[i][j];
        if (flush) {
          acc[i][j] += mid[i][j];
          mid[i][j] = 0.f;
        }
      }
    __syncthreads();
  }
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int gm = m0 + ty * 4 + i;
    if (gm >= M) continue;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int gn = n0 + tx * 4 + j;
      if (gn < N) c[static_cast<int64_t>(gm) * ldc + gn] = acc[i][j];
    }
  }
}

}  // namespace arle

using namespace arle;

extern "C" int arle_gemm_f32(const float* a, long long lda, const float* w, long long ldw, float* c,
                             long long ldc, int M, int N, int K, void* stream) {
  if (M == 0 || N == 0) return 0;
  dim3 grid((N + kBN - 1) / kBN, (M + kBM - 1) / kBM);
  gemm_f32_kernel<<<grid, kGemmThreads, 0, static_cast<hipStream_t>(stream)>>>(a, lda, w, ldw, c,
                                                                               ldc, M, N, K);
  return launch_status();
}
