// Skinny bfloat16 matrix product for decode steps:  C[M,N] = X[M,K] . W[N,K]^T, M <= 64.
//
// With few rows the product is a stream of W through the chip: every weight is read once
// and HBM bandwidth is the bound, so the kernel is built around keeping many 16-byte loads
// in flight and nothing else.  A workgroup owns 16*NT rows of W (output columns) and all M
// rows of X; its waves split K among themselves and add their partial sums through LDS at
// the end.  Each wave feeds v_mfma_f32_16x16x32_bf16 straight from global memory:
//   A = W tile (16 n x 32 k), lane (i, g) loads W[n0 + i][32 s + 8 g .. +7]   (16 bytes)
//   B = X tile (16 m x 32 k), lane (j, g) loads X[m0 + j][32 s + 8 g .. +7]
//   C lane (j, g) register r = C[m0 + j][n0 + 4 g + r]
// X is small and is served by the L2; W comes from HBM.  Rows past N or M are clamped for
// the loads and skipped at the store; K must be a multiple of 8 (16-byte loads), any other
// size is fine.  Accumulation is float32; the output is bfloat16 or float32.
//
// Epilogue kSiluMul: W holds gate and up rows interleaved in blocks of 16 (rows 32b..32b+15
// are gate rows 16b.., rows 32b+16..32b+31 the matching up rows), NT is 2, and the
// workgroup writes out[m][16 b + c] = silu(gate) * up: the SwiGLU activation never goes
// through memory as two separate vectors (the reference runs two products and an
// elementwise kernel, or one product and crates/cuda-kernels/csrc/misc/split_qkv.cu:35-52).
// Reference counterpart of the plain product: crates/cuda-kernels/csrc/gemm/gemv.cu:45-,240-330.
#include "common.h"

namespace arle {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x4 __attribute__((ext_vector_type(4)));

constexpr int kEpiNone = 0, kEpiSiluMul = 1;

__device__ __forceinline__ bf16x8 ldg_bf16x8(const uint16_t* p) {
  return __builtin_bit_cast(bf16x8, *reinterpret_cast<const uint4*>(p));
}

// A workgroup has at most 16 waves with one 16-row tile of X, at most 8 with more (registers).
template <int MT, int NT, int EPI, typename TOut>
__global__ __launch_bounds__(MT == 1 ? 1024 : 512) void gemm_skinny_kernel(const uint16_t* __restrict__ x, int64_t ldx,
                                   const uint16_t* __restrict__ w, int64_t ldw,
                                   TOut* __restrict__ out, int64_t ldo, int M, int N, int K) {
  extern __shared__ float red[];  // [waves][NT*MT][64 lanes][4]
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, waves = blockDim.x >> 6;
  const int li = lane & 15, g = lane >> 4;
  const int n0 = blockIdx.x * (16 * NT);

  const uint16_t* wp[NT];
#pragma unroll
  for (int t = 0; t < NT; ++t) wp[t] = w + static_cast<int64_t>(min(n0 + 16 * t + li, N - 1)) * ldw;
  const uint16_t* xp[MT];
#pragma unroll
  for (int t = 0; t < MT; ++t) xp[t] = x + static_cast<int64_t>(min(16 * t + li, M - 1)) * ldx;

  f32x4 acc[NT][MT];
#pragma unroll
  for (int a = 0; a < NT; ++a)
#pragma unroll
    for (int b = 0; b < MT; ++b) acc[a][b] = f32x4{0.f, 0.f, 0.f, 0.f};

  // this wave's share of the k steps (32 k each)
  const int steps = (K + 31) / 32;
  const int per = (steps + waves - 1) / waves;
  const int s0 = wave * per, s1 = min(s0 + per, steps);
  const uint4 zero = {0u, 0u, 0u, 0u};

  // Loads of kChunk steps are issued together before any of them is used, so that a wave keeps
  // kChunk * (NT + MT) 16-byte loads in flight: the kernel lives on memory-level parallelism.
  constexpr int kChunk = MT == 4 ? 4 : 8;
  for (int base = s0; base < s1; base += kChunk) {
    bf16x8 wv[kChunk][NT], xv[kChunk][MT];
#pragma unroll
    for (int u = 0; u < kChunk; ++u) {
      const int k = 32 * (base + u) + 8 * g;
      const bool in = base + u < s1 && k < K;  // K % 8 == 0: a chunk of 8 is inside or outside as a whole
#pragma unroll
      for (int t = 0; t < NT; ++t) wv[u][t] = in ? ldg_bf16x8(wp[t] + k) : __builtin_bit_cast(bf16x8, zero);
#pragma unroll
      for (int t = 0; t < MT; ++t) xv[u][t] = in ? ldg_bf16x8(xp[t] + k) : __builtin_bit_cast(bf16x8, zero);
    }
#pragma unroll
    for (int u = 0; u < kChunk; ++u)
#pragma unroll
      for (int a = 0; a < NT; ++a)
#pragma unroll
        for (int b = 0; b < MT; ++b)
          acc[a][b] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wv[u][a], xv[u][b], acc[a][b], 0, 0, 0);
  }

  // add the waves' partial sums: wave w > 0 parks its registers in LDS, wave 0 sums in wave order
  if (waves > 1) {
    if (wave > 0) {
#pragma unroll
      for (int a = 0; a < NT; ++a)
#pragma unroll
        for (int b = 0; b < MT; ++b)
          *reinterpret_cast<f32x4*>(red + ((static_cast<size_t>(wave) * (NT * MT) + a * MT + b) * 64 + lane) * 4) = acc[a][b];
    }
    __syncthreads();
    if (wave > 0) return;
    for (int v = 1; v < waves; ++v) {
#pragma unroll
      for (int a = 0; a < NT; ++a)
#pragma unroll
        for (int b = 0; b < MT; ++b) {
          const f32x4 p = *reinterpret_cast<const f32x4*>(red + ((static_cast<size_t>(v) * (NT * MT) + a * MT + b) * 64 + lane) * 4);
          acc[a][b][0] += p[0];
          acc[a][b][1] += p[1];
          acc[a][b][2] += p[2];
          acc[a][b][3] += p[3];
        }
    }
  }

  // acc[a][b][r] = C[m = 16 b + li][n = n0 + 16 a + 4 g + r]
  if constexpr (EPI == kEpiSiluMul) {
    static_assert(NT == 2, "the fused activation needs the gate and the up tile side by side");
    const int c0 = (n0 / 2) + 4 * g;  // output column of register 0
#pragma unroll
    for (int b = 0; b < MT; ++b) {
      const int mrow = 16 * b + li;
      if (mrow >= M) continue;
      TOut* o = out + static_cast<int64_t>(mrow) * ldo + c0;
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        if (n0 + 16 + 4 * g + r >= N) continue;
        const float gate = acc[0][b][r], up = acc[1][b][r];
        o[r] = from_float<TOut>(gate / (1.0f + expf(-gate)) * up);
      }
    }
  } else {
#pragma unroll
    for (int a = 0; a < NT; ++a)
#pragma unroll
      for (int b = 0; b < MT; ++b) {
        const int mrow = 16 * b + li;
        if (mrow >= M) continue;
        const int ncol = n0 + 16 * a + 4 * g;
        TOut* o = out + static_cast<int64_t>(mrow) * ldo + ncol;
#pragma unroll
        for (int r = 0; r < 4; ++r)
          if (ncol + r < N) o[r] = from_float<TOut>(acc[a][b][r]);
      }
  }
}

template <int MT, int NT, int EPI, typename TOut>
int launch_skinny(const uint16_t* x, int64_t ldx, const uint16_t* w, int64_t ldw, void* out, int64_t ldo,
                  int M, int N, int K, int waves, hipStream_t s) {
  const int tiles = (N + 16 * NT - 1) / (16 * NT);
  const size_t lds = waves > 1 ? static_cast<size_t>(waves) * NT * MT * 64 * 4 * sizeof(float) : 0;
  gemm_skinny_kernel<MT, NT, EPI, TOut><<<tiles, waves * 64, lds, s>>>(x, ldx, w, ldw, static_cast<TOut*>(out),
                                                                      ldo, M, N, K);
  return launch_status();
}

template <int MT, int NT, int EPI>
int launch_skinny_out(const uint16_t* x, int64_t ldx, const uint16_t* w, int64_t ldw, void* out, int64_t ldo,
                      int out_dtype, int M, int N, int K, int waves, hipStream_t s) {
  if (out_dtype == kF32) return launch_skinny<MT, NT, EPI, float>(x, ldx, w, ldw, out, ldo, M, N, K, waves, s);
  return launch_skinny<MT, NT, EPI, bf16>(x, ldx, w, ldw, out, ldo, M, N, K, waves, s);
}

}  // namespace arle

using namespace arle;

// x [M, K] and w [N, K] bfloat16 with row strides in elements (multiples of 8), out [M, N]
// (or [M, N/2] with the fused activation) bfloat16 or float32.  1 <= M <= 64, K % 8 == 0.
// `waves` (1..16) split K inside a workgroup; the caller picks it from N and K.
extern "C" int arle_gemm_bf16_skinny(const void* x, long long ldx, const void* w, long long ldw, void* out,
                                     long long ldo, int out_dtype, int M, int N, int K, int epilogue,
                                     int waves, void* stream) {
  if (M <= 0 || N <= 0) return 0;
  if (M > 64 || K % 8 != 0 || K <= 0 || ldx % 8 != 0 || ldw % 8 != 0 || waves < 1 || waves > 16)
    return static_cast<int>(hipErrorInvalidValue);
  hipStream_t s = static_cast<hipStream_t>(stream);
  const uint16_t* xp = static_cast<const uint16_t*>(x);
  const uint16_t* wp = static_cast<const uint16_t*>(w);
  const int mt = M <= 16 ? 1 : (M <= 32 ? 2 : 4);
  if (mt > 1 && waves > 8) return static_cast<int>(hipErrorInvalidValue);
  if (epilogue == kEpiSiluMul) {
    if (N % 32 != 0) return static_cast<int>(hipErrorInvalidValue);
    if (mt == 1) return launch_skinny_out<1, 2, kEpiSiluMul>(xp, ldx, wp, ldw, out, ldo, out_dtype, M, N, K, waves, s);
    if (mt == 2) return launch_skinny_out<2, 2, kEpiSiluMul>(xp, ldx, wp, ldw, out, ldo, out_dtype, M, N, K, waves, s);
    return launch_skinny_out<4, 2, kEpiSiluMul>(xp, ldx, wp, ldw, out, ldo, out_dtype, M, N, K, waves, s);
  }
  if (mt == 1) return launch_skinny_out<1, 1, kEpiNone>(xp, ldx, wp, ldw, out, ldo, out_dtype, M, N, K, waves, s);
  if (mt == 2) return launch_skinny_out<2, 2, kEpiNone>(xp, ldx, wp, ldw, out, ldo, out_dtype, M, N, K, waves, s);
  return launch_skinny_out<4, 2, kEpiNone>(xp, ldx, wp, ldw, out, ldo, out_dtype, M, N, K, waves, s);
}
