// bfloat16 matrix product for few rows (decode steps and short prompt portions):
//   C[M,N] = X[M,K] . W[N,K]^T,  1 <= M <= 64.
//
// With few rows the product is one pass over W, and HBM bandwidth is the bound.  Reads of X are
// not free either: every workgroup needs the rows of X for the k range it works on, and on
// MI355X bytes that come from the L2 cost about as much as bytes that come from HBM.  So the
// kernel shares X inside a workgroup and makes a workgroup's tile of W wide:
//
//   * a workgroup has WN x WK waves.  Wave (wn, wk) owns 16*NT output columns (rows of W) and
//     every wk-th block of kBlockSteps 32-wide k steps of the workgroup's k slice;
//   * X for one round (WK blocks of k) is staged once through LDS (coalesced 16-byte loads,
//     rows padded by 16 bytes against bank conflicts) and read from there as the B operand of
//     v_mfma_f32_16x16x32_bf16 by all WN waves: X traffic drops by the factor WN;
//   * W goes straight from global memory into the A operand, 16 bytes a lane, one round ahead
//     of its use, so that every wave keeps kBlockSteps * NT kilobyte-sized loads in flight;
//   * the WK partial sums of a column tile are added through LDS in the fixed order wk = 0..WK-1;
//   * gridDim.y splits K further across workgroups when N alone gives too few of them (small
//     workgroups in great number stream best on MI355X).  Each split writes its own float32
//     partial product out[s][M][N]; the kernel that consumes the product (the residual add fused
//     into RMSNorm, the q/k/v preparation) adds the splits in the order s = 0, 1, ..., so results
//     do not depend on timing.  (Adding them here, by the workgroup that arrives last, needs
//     device-scope fences or write-through accesses, and both cost more than they save.)
//
// Operand layout (lane = 16 g + i):  A lane (i, g) = W[n0 + i][32 s + 8 g .. +7],
// B lane (j, g) = X[m0 + j][32 s + 8 g .. +7], C lane (j, g) register r = C[m0 + j][n0 + 4 g + r].
// Rows past M or N are clamped for the loads and skipped at the store; K % 8 == 0.
//
// Epilogue kEpiSiluMul: W holds gate and up rows interleaved in blocks of 16 and the kernel
// writes silu(gate) * up, [M, N/2] (the reference runs an elementwise kernel for this,
// crates/cuda-kernels/csrc/misc/split_qkv.cu:35-52).  Plain product: the reference's
// crates/cuda-kernels/csrc/gemm/gemv.cu:45-,240-330 and cuBLAS for more rows.
#include "common.h"

namespace arle {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x4 __attribute__((ext_vector_type(4)));

constexpr int kEpiNone = 0, kEpiSiluMul = 1;
constexpr int kPad = 8;  // elements of padding per LDS row of X

struct RowsArgs {
  const uint16_t* x;
  int64_t ldx;
  const uint16_t* w;
  int64_t ldw;
  void* out;
  int64_t ldo;
  int M, N, K;
  int rounds_per_split;  // rounds (WK * KBS steps of 32) that one k split covers
  int64_t split_stride;  // elements between the partial products of two k splits
};

template <int MT, int NT, int WN, int WK, int KBS, int EPI, typename TOut>
__global__ __launch_bounds__(WN* WK * 64) void gemm_rows_kernel(const RowsArgs a) {
  constexpr int kThreads = WN * WK * 64;
  constexpr int kRows = MT * 16;
  constexpr int kRoundK = WK * KBS * 32;          // elements of k per round
  constexpr int kPitch = kRoundK + kPad;          // LDS row pitch in elements
  constexpr int kChunksPerRow = kRoundK / 8;      // 16-byte chunks of one row of a round
  constexpr int kChunks = kRows * kChunksPerRow;
  constexpr int kCPT = (kChunks + kThreads - 1) / kThreads;  // chunks each thread stages per round
  static_assert(EPI != kEpiSiluMul || NT == 2, "the fused activation needs the gate and the up tile side by side");
  extern __shared__ __align__(16) uint16_t lds[];  // [2][kRows][kPitch] X, later the partial sums

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wn = wave % WN, wk = wave / WN;
  const int li = lane & 15, g = lane >> 4;
  const int n0 = (blockIdx.x * WN + wn) * (16 * NT);
  const int M = a.M, N = a.N, K = a.K;

  const int steps_total = (K + 31) / 32;
  const int round0 = blockIdx.y * a.rounds_per_split;
  const int rounds = min(a.rounds_per_split, (steps_total + WK * KBS - 1) / (WK * KBS) - round0);

  const uint16_t* wp[NT];
#pragma unroll
  for (int t = 0; t < NT; ++t) wp[t] = a.w + static_cast<int64_t>(min(n0 + 16 * t + li, N - 1)) * a.ldw + 8 * g;

  // staging: chunk c = tid + i * kThreads -> row c / kChunksPerRow, 16-byte column c % kChunksPerRow
  // (threads past the last chunk, when there are more threads than chunks, stage nothing)
  const uint16_t* xsrc[kCPT];
  int xcol[kCPT], xdst[kCPT];
#pragma unroll
  for (int i = 0; i < kCPT; ++i) {
    const int c = tid + i * kThreads;
    const int row = c / kChunksPerRow, col = (c % kChunksPerRow) * 8;
    xsrc[i] = a.x + static_cast<int64_t>(min(row, M - 1)) * a.ldx + col;
    xcol[i] = col;
    xdst[i] = c < kChunks ? row * kPitch + col : -1;
  }

  f32x4 acc[NT][MT];
#pragma unroll
  for (int t = 0; t < NT; ++t)
#pragma unroll
    for (int b = 0; b < MT; ++b) acc[t][b] = f32x4{0.f, 0.f, 0.f, 0.f};

  uint4 xs[kCPT];
  bf16x8 wcur[KBS][NT], wnext[KBS][NT];

  // Loads past K (the last round of a matrix whose K is no multiple of the round) read a clamped,
  // valid address and are zeroed afterwards: the select is on the value, never on the address, so
  // every load stays a plain global load.  K % 8 == 0: a chunk of 8 is inside or outside as a whole.
  auto load_x = [&](int r) {  // global -> registers, round r of this split
    const int k0 = (round0 + r) * kRoundK;
    const bool whole = k0 + kRoundK <= K;
#pragma unroll
    for (int i = 0; i < kCPT; ++i) {
      if (kChunks % kThreads != 0 && xdst[i] < 0) continue;
      if (whole) {
        xs[i] = *reinterpret_cast<const uint4*>(xsrc[i] + k0);
      } else {
        const bool in = k0 + xcol[i] < K;
        const uint4 v = *reinterpret_cast<const uint4*>(xsrc[i] + (in ? k0 : 0) - (in ? 0 : xcol[i]));
        xs[i] = uint4{in ? v.x : 0u, in ? v.y : 0u, in ? v.z : 0u, in ? v.w : 0u};
      }
    }
  };
  auto store_x = [&](int buf) {
#pragma unroll
    for (int i = 0; i < kCPT; ++i)
      if (kChunks % kThreads == 0 || xdst[i] >= 0) *reinterpret_cast<uint4*>(lds + buf * (kRows * kPitch) + xdst[i]) = xs[i];
  };
  auto load_w = [&](int r, bf16x8 (&dst)[KBS][NT]) {
    const int k0 = (round0 + r) * kRoundK + wk * (KBS * 32);
    if (k0 + KBS * 32 <= K) {
#pragma unroll
      for (int u = 0; u < KBS; ++u)
#pragma unroll
        for (int t = 0; t < NT; ++t)
          dst[u][t] = __builtin_bit_cast(bf16x8, *reinterpret_cast<const uint4*>(wp[t] + k0 + 32 * u));
    } else {
#pragma unroll
      for (int u = 0; u < KBS; ++u) {
        const int k = k0 + 32 * u;
        const bool in = k + 8 * g < K;
#pragma unroll
        for (int t = 0; t < NT; ++t) {
          const uint4 v = *reinterpret_cast<const uint4*>(wp[t] + (in ? k : -8 * g));  // row start when outside
          dst[u][t] = __builtin_bit_cast(bf16x8, uint4{in ? v.x : 0u, in ? v.y : 0u, in ? v.z : 0u, in ? v.w : 0u});
        }
      }
    }
  };

  // One round: start the loads of the next round, multiply this round's W registers with X from LDS,
  // park the next round's X in the other LDS buffer.  The two W register sets swap roles from round
  // to round (the loop is unrolled by two), so the loads of round r + 1 stay in flight while round r
  // is computed and nothing is copied.
  auto round_body = [&](int r, bf16x8 (&cur)[KBS][NT], bf16x8 (&nxt)[KBS][NT]) {
    const bool more = r + 1 < rounds;
    if (more) {
      load_x(r + 1);
      load_w(r + 1, nxt);
    }
    const uint16_t* xb = lds + (r & 1) * (kRows * kPitch) + li * kPitch + wk * (KBS * 32) + 8 * g;
#pragma unroll
    for (int u = 0; u < KBS; ++u) {
      bf16x8 xv[MT];
#pragma unroll
      for (int b = 0; b < MT; ++b)
        xv[b] = __builtin_bit_cast(bf16x8, *reinterpret_cast<const uint4*>(xb + b * 16 * kPitch + 32 * u));
#pragma unroll
      for (int t = 0; t < NT; ++t)
#pragma unroll
        for (int b = 0; b < MT; ++b)
          acc[t][b] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(cur[u][t], xv[b], acc[t][b], 0, 0, 0);
    }
    if (more) store_x((r + 1) & 1);
    __syncthreads();
  };

  if (rounds > 0) {
    load_x(0);
    load_w(0, wcur);
    store_x(0);
  }
  __syncthreads();
  for (int r = 0; r < rounds; r += 2) {
    round_body(r, wcur, wnext);
    if (r + 1 < rounds) round_body(r + 1, wnext, wcur);
  }

  // add the WK partial sums of every column tile in the order wk = 0, 1, ...: waves wk > 0 park
  // their registers in LDS (the X buffers are free after the last barrier), waves wk == 0 add
  if constexpr (WK > 1) {
    float* red = reinterpret_cast<float*>(lds);  // [WK-1][WN][NT*MT][64][4]
    if (wk > 0) {
#pragma unroll
      for (int t = 0; t < NT; ++t)
#pragma unroll
        for (int b = 0; b < MT; ++b)
          *reinterpret_cast<f32x4*>(red + ((((wk - 1) * WN + wn) * (NT * MT) + t * MT + b) * 64 + lane) * 4) = acc[t][b];
    }
    __syncthreads();
    if (wk > 0) return;
#pragma unroll
    for (int v = 1; v < WK; ++v)
#pragma unroll
      for (int t = 0; t < NT; ++t)
#pragma unroll
        for (int b = 0; b < MT; ++b) {
          const f32x4 p = *reinterpret_cast<const f32x4*>(red + ((((v - 1) * WN + wn) * (NT * MT) + t * MT + b) * 64 + lane) * 4);
          acc[t][b][0] += p[0];
          acc[t][b][1] += p[1];
          acc[t][b][2] += p[2];
          acc[t][b][3] += p[3];
        }
  }

  // acc[t][b][r] = C[m = 16 b + li][n = n0 + 16 t + 4 g + r]
  TOut* out = static_cast<TOut*>(a.out) + static_cast<int64_t>(blockIdx.y) * a.split_stride;
  if constexpr (EPI == kEpiSiluMul) {
    const int c0 = (n0 / 2) + 4 * g;  // output column of register 0
#pragma unroll
    for (int b = 0; b < MT; ++b) {
      const int mrow = 16 * b + li;
      if (mrow >= M) continue;
      TOut* o = out + static_cast<int64_t>(mrow) * a.ldo + c0;
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        if (n0 + 16 + 4 * g + r >= N) continue;
        const float gate = acc[0][b][r], up = acc[1][b][r];
        o[r] = from_float<TOut>(gate / (1.0f + expf(-gate)) * up);
      }
    }
  } else {
#pragma unroll
    for (int t = 0; t < NT; ++t)
#pragma unroll
      for (int b = 0; b < MT; ++b) {
        const int mrow = 16 * b + li;
        if (mrow >= M) continue;
        const int ncol = n0 + 16 * t + 4 * g;
        TOut* o = out + static_cast<int64_t>(mrow) * a.ldo + ncol;
#pragma unroll
        for (int r = 0; r < 4; ++r)
          if (ncol + r < N) o[r] = from_float<TOut>(acc[t][b][r]);
      }
  }
}

template <int MT, int NT, int WN, int WK, int KBS>
constexpr size_t rows_lds_bytes() {
  const size_t x = 2ull * (MT * 16) * (WK * KBS * 32 + kPad) * sizeof(uint16_t);
  const size_t red = WK > 1 ? static_cast<size_t>(WK - 1) * WN * NT * MT * 64 * 4 * sizeof(float) : 0;
  return x > red ? x : red;
}

template <int MT, int NT, int WN, int WK, int KBS, int EPI, typename TOut>
int launch_rows(const RowsArgs& a, int splits, hipStream_t s) {
  constexpr size_t lds = rows_lds_bytes<MT, NT, WN, WK, KBS>();
  auto kernel = gemm_rows_kernel<MT, NT, WN, WK, KBS, EPI, TOut>;
  if (lds > 64 * 1024) {
    static bool raised = false;  // per instantiation; the attribute belongs to the function, set once
    if (!raised) {
      hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                                         static_cast<int>(lds));
      if (e != hipSuccess) {
        (void)hipGetLastError();  // do not leave the error behind for the next call to find
        return static_cast<int>(e);
      }
      raised = true;
    }
  }
  const int col_groups = (a.N + WN * NT * 16 - 1) / (WN * NT * 16);
  kernel<<<dim3(col_groups, splits), WN * WK * 64, lds, s>>>(a);
  return launch_status();
}

template <int MT, int NT, int WN, int WK, int KBS, int EPI>
int launch_rows_out(const RowsArgs& a, int splits, int out_dtype, hipStream_t s) {
  if (out_dtype == kF32) return launch_rows<MT, NT, WN, WK, KBS, EPI, float>(a, splits, s);
  return launch_rows<MT, NT, WN, WK, KBS, EPI, bf16>(a, splits, s);
}

template <int MT, int NT, int WN, int WK, int KBS>
int dispatch_rows(const RowsArgs& a, int splits, int out_dtype, int epilogue, hipStream_t s) {
  if constexpr (NT == 2) {
    if (epilogue == kEpiSiluMul) return launch_rows_out<MT, NT, WN, WK, KBS, kEpiSiluMul>(a, splits, out_dtype, s);
  }
  return launch_rows_out<MT, NT, WN, WK, KBS, kEpiNone>(a, splits, out_dtype, s);
}

}  // namespace arle

using namespace arle;

// Shapes of a workgroup, by `variant`: (NT, WN, WK, KBS), picked by the caller per matrix shape and row count
// from measurements on MI355X:
//   0  general product                      1  gate/up with the fused activation (two column tiles a wave)
//   2  few output columns, long K           3  very many output columns (an output head)
//   4  few output columns, short K
#define ARLE_ROWS_VARIANTS(X) X(0, 1, 4, 2, 4) X(1, 2, 4, 2, 8) X(2, 1, 2, 4, 4) X(3, 2, 4, 2, 4) X(4, 1, 1, 2, 8)
constexpr int kVariants = 5;

// (k steps of 32 that one round covers) << 20 | (output columns of one workgroup) << 4 | (column tiles a wave);
// -1 for an unknown variant
extern "C" int arle_gemm_rows_geometry(int variant) {
  switch (variant) {
#define X(ID, NT, WN, WK, KBS) \
  case ID:                     \
    return ((WK * KBS) << 20) | ((WN * NT * 16) << 4) | NT;
    ARLE_ROWS_VARIANTS(X)
#undef X
    default:
      return -1;
  }
}

// x [M, K] and w [N, K] bfloat16 with row strides in elements (multiples of 8), 1 <= M <= 64, K % 8 == 0.
// splits == 1: out [M, N] (or [M, N/2] with the fused activation) bfloat16 or float32.
// splits  > 1: out [splits, M, N] float32 partial products, split_stride elements apart, no activation;
//              split s covers rounds [s * rounds_per_split, (s + 1) * rounds_per_split) and none may be empty.
extern "C" int arle_gemm_rows(const void* x, long long ldx, const void* w, long long ldw, void* out, long long ldo,
                              long long split_stride, int out_dtype, int M, int N, int K, int epilogue, int variant,
                              int splits, int rounds_per_split, void* stream) {
  if (M <= 0 || N <= 0) return 0;
  if (M > 64 || K % 8 != 0 || K <= 0 || ldx % 8 != 0 || ldw % 8 != 0 || splits < 1 || splits > 65535 ||
      rounds_per_split < 1 || variant < 0 || variant >= kVariants)
    return static_cast<int>(hipErrorInvalidValue);
  const int round_steps = arle_gemm_rows_geometry(variant) >> 20;
  const int rounds_total = ((K + 31) / 32 + round_steps - 1) / round_steps;
  if (static_cast<long long>(splits - 1) * rounds_per_split >= rounds_total) return static_cast<int>(hipErrorInvalidValue);
  if (splits > 1 && (out_dtype != kF32 || epilogue != kEpiNone)) return static_cast<int>(hipErrorInvalidValue);
  if (epilogue == kEpiSiluMul && (N % 32 != 0 || (arle_gemm_rows_geometry(variant) & 15) != 2))
    return static_cast<int>(hipErrorInvalidValue);
  if (epilogue != kEpiNone && epilogue != kEpiSiluMul) return static_cast<int>(hipErrorInvalidValue);
  hipStream_t s = static_cast<hipStream_t>(stream);
  const RowsArgs a{static_cast<const uint16_t*>(x), ldx, static_cast<const uint16_t*>(w), ldw, out, ldo, M, N, K,
                   rounds_per_split, split_stride};
  switch (variant) {
#define X(ID, NT, WN, WK, KBS)                                                                      \
  case ID:                                                                                          \
    if (M <= 16) return dispatch_rows<1, NT, WN, WK, KBS>(a, splits, out_dtype, epilogue, s);       \
    if (M <= 32) return dispatch_rows<2, NT, WN, WK, KBS>(a, splits, out_dtype, epilogue, s);       \
    return dispatch_rows<4, NT, WN, WK, KBS>(a, splits, out_dtype, epilogue, s);
    ARLE_ROWS_VARIANTS(X)
#undef X
  }
  return static_cast<int>(hipErrorInvalidValue);
}
