// bfloat16 matrix product for few rows (decode steps and short prompt portions):
//   C[M,N] = X[M,K] . W[N,K]^T,  1 <= M <= 64.
//
// With few rows the product is one pass over W, and HBM bandwidth is the bound.  What decides the
// speed on MI355X is how many independent loads of W are in flight on every CU at every moment, so
// the kernel is built around that:
//
//   * many small workgroups of WN x WK waves.  Wave (wn, wk) owns 16 output columns (rows of W: one
//     tile a wave streams better than two) and the wk-th part of the workgroup's k slice;
//   * gridDim.y splits K across workgroups when N alone gives too few of them.  Each split writes its
//     own float32 partial product out[s][M][N]; the kernel that consumes the product (the residual add
//     fused into RMSNorm, the q/k/v preparation) adds the splits in the order s = 0, 1, ..., so results
//     do not depend on timing.  (Adding them here, by the workgroup that arrives last, needs
//     device-scope fences or write-through accesses, and both cost more than they save.)
//   * the rows of X for the workgroup's whole k slice are staged once into LDS (reads of X come from
//     the L2 but cost about as much as reads from HBM, so the WN waves share them).  After that one
//     barrier the waves run free: there is no barrier inside the loop over k;
//   * W goes straight from global memory into the A operand of v_mfma_f32_16x16x32_bf16, 16 bytes a
//     lane, through a ring of PD registers: the load of step s + PD is issued as soon as step s has
//     been multiplied, so every wave keeps PD kilobyte-sized loads in flight.  The X operand comes
//     from LDS through a shorter ring of its own, so that no step waits for an LDS read;
//   * the WK partial sums of a column tile are added through LDS in the fixed order wk = 0..WK-1.
//   * ROUNDS (the fused activation for up to 64 rows): where the X rows of the whole k slice do not fit into LDS,
//     the slice is walked in rounds, each staged, multiplied and left behind a barrier; the sums stay in registers.
//
// Operand layout (lane = 16 g + i):  A lane (i, g) = W[n0 + i][32 s + 8 g .. +7],
// B lane (j, g) = X[m0 + j][32 s + 8 g .. +7], C lane (j, g) register r = C[m0 + j][n0 + 4 g + r].
// Rows past M or N are clamped for the loads and skipped at the store.  K % 8 == 0; where a step of 32
// reaches past K, W is read from a clamped address and meets zeros that the staging put into X.
//
// Epilogue kEpiSiluMul: W holds gate and up rows interleaved in blocks of 16, so even column tiles are
// gate and odd ones the matching up columns.  Neighbouring waves (WN is even) own such a pair; the odd
// wave hands its sums over through LDS and the even one writes silu(gate) * up, [M, N/2] (the reference
// runs an elementwise kernel for this, crates/cuda-kernels/csrc/misc/split_qkv.cu:35-52).  Plain product: the reference's
// crates/cuda-kernels/csrc/gemm/gemv.cu:45-,240-330 and cuBLAS for more rows.
#include "common.h"

namespace arle {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x4 __attribute__((ext_vector_type(4)));

constexpr int kEpiNone = 0, kEpiSiluMul = 1;
constexpr int kPad = 8;  // elements of padding per LDS row of X (16 bytes: rows start in different banks)

struct RowsArgs {
  const uint16_t* x;
  int64_t ldx;
  const uint16_t* w;
  int64_t ldw;
  void* out;
  int64_t ldo;
  int M, N, K;
  int steps_per_split;   // k steps of 32 that one k split covers
  int64_t split_stride;  // elements between the partial products of two k splits
  int tiled;             // w holds operand tiles (see below) instead of rows
  int steps_per_round;   // ROUNDS: k steps of 32 whose X rows are in LDS at one time (the slice is walked in rounds)
};

// W as operand tiles: [ceil(N/16)][ceil(K/32)][64 lanes][8], tile (t, s) lane 16 g + i = W[16 t + i][32 s + 8 g .. +7],
// zeros past N and K.  A wave's load of one k step is then one contiguous kilobyte and its stream through a
// column tile one contiguous run, instead of sixteen 64-byte pieces a row apart: measured 4.5 against 3.6 TB/s
// for the 100 MB gate|up matrix of the Qwen3-4B shape at 8 rows.
__device__ __forceinline__ const uint16_t* tile_base(const RowsArgs& a, int n0, int lane) {
  const int tile = min(n0 / 16, (a.N + 15) / 16 - 1);
  return a.w + static_cast<int64_t>(tile) * ((a.K + 31) / 32) * 512 + lane * 8;
}

// ROUNDS: the k slice of a workgroup is too long for its X rows to fit into LDS at once (more than 27 rows of
// 2,560 columns); it is walked in rounds of steps_per_round steps, each staged, multiplied and left behind a
// barrier, with the sums staying in registers, so that whole sums meet the fused activation for up to 64 rows.
template <int MT, int WN, int WK, int PD, int XD, int EPI, typename TOut, bool ROUNDS = false>
__global__ __launch_bounds__(WN* WK * 64) void gemm_rows_kernel(const RowsArgs a) {
  constexpr int kThreads = WN * WK * 64;
  static_assert(PD % XD == 0, "the X ring must divide the W ring");
  static_assert(EPI != kEpiSiluMul || WN % 2 == 0, "the fused activation pairs neighbouring waves");
  // [M][pitch] X, then [WK-1][WN][MT][64][4] partial sums, then [WN/2][MT][64][4] for the gate/up exchange
  extern __shared__ __align__(16) uint16_t lds[];

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wn = wave % WN, wk = wave / WN;
  const int li = lane & 15, g = lane >> 4;
  const int n0 = (blockIdx.x * WN + wn) * 16;
  const int M = a.M, N = a.N, K = a.K;

  const int steps_total = (K + 31) / 32;
  const int slice_begin = blockIdx.y * a.steps_per_split;
  const int slice_end = min(slice_begin + a.steps_per_split, steps_total);
  const int staged_steps = ROUNDS ? a.steps_per_round : a.steps_per_split;   // steps whose X rows LDS holds at a time
  const int pitch = staged_steps * 32 + kPad;

  f32x4 acc[MT];
#pragma unroll
  for (int b = 0; b < MT; ++b) acc[b] = f32x4{0.f, 0.f, 0.f, 0.f};

  // one round: the steps [s_begin, s_end) of the slice, staged and multiplied (without ROUNDS: the whole slice)
  auto round = [&](const int s_begin, const int s_end) {
    // this wave's steps: the wk-th part of the round
    const int per = (s_end - s_begin + WK - 1) / WK;
    const int w_begin = s_begin + wk * per;
    const int n_steps = max(0, min(w_begin + per, s_end) - w_begin);

    // rows: lane (i, g) reads 16 bytes of row n0 + i; tiles: the wave reads tile s of its column tile, lane by lane
    const uint16_t* wrow = a.tiled ? tile_base(a, n0, lane) : a.w + static_cast<int64_t>(min(n0 + li, N - 1)) * a.ldw;
    const int w_step = a.tiled ? 512 : 32, w_first = a.tiled ? 0 : 8 * g, w_last = a.tiled ? (steps_total - 1) * 512 : K - 8;
    auto load_w = [&](int s) {
      const int e = min(w_step * s + w_first, w_last);  // clamped: always inside the row (the column tile)
      return __builtin_bit_cast(bf16x8, *reinterpret_cast<const uint4*>(wrow + e));
    };

    // the first PD steps of W are on their way before anything else happens; without a condition (a step past
    // the wave's last one is clamped into the row and never used), because a load under a condition is waited
    // for at the end of its branch
    bf16x8 ring[PD];
  #pragma unroll
    for (int u = 0; u < PD; ++u) ring[u] = load_w(w_begin + u);

    // X rows of the slice -> LDS, straight from memory (no registers in between, so every piece of the slice is
    // on its way at once): a wave's 64 lanes fill 1 KB of LDS in lane order from 64 addresses of their own.  A
    // row in LDS is its 16-byte pieces and one piece of padding; padding lanes and lanes past K fetch a piece
    // that exists, and the pieces past K are put to zero afterwards (W is clamped there, X must not count).
    {
      const int cpr = staged_steps * 4;       // pieces of 8 elements per row
      const int cpp = cpr + kPad / 8;         // ... with the padding
      const int total = M * cpp;
      const int k0 = s_begin * 32, k1 = min(s_end * 32, K);
      for (int q0 = wave * 64; q0 < total; q0 += kThreads) {
        const int q = min(q0 + lane, total - 1);
        const int row = q / cpp, cc = q % cpp;
        const int col = k0 + cc * 8;
        const uint16_t* src = a.x + static_cast<int64_t>(row) * a.ldx + ((cc < cpr && col < k1) ? col : k0);
        __builtin_amdgcn_global_load_lds(src, (__attribute__((address_space(3))) void*)(lds + q0 * 8),
                                         16, 0, 0);
      }
      asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
      if (k1 < s_end * 32) {
        __syncthreads();  // the pieces put to zero were fetched by other waves: all of them have to be in first
        const int z0 = (k1 - k0) / 8, nz = (s_end * 32 - k1) / 8;
        for (int i = tid; i < M * nz; i += kThreads)
          *reinterpret_cast<uint4*>(lds + (i / nz) * pitch + (z0 + i % nz) * 8) = uint4{0u, 0u, 0u, 0u};
      }
    }
    __syncthreads();

    const uint16_t* xrow[MT];  // lanes past the last row read the last row; their results are not stored
  #pragma unroll
    for (int b = 0; b < MT; ++b) xrow[b] = lds + min(16 * b + li, M - 1) * pitch + (w_begin - s_begin) * 32 + 8 * g;
    auto load_x = [&](int s, bf16x8 (&dst)[MT]) {
  #pragma unroll
      for (int b = 0; b < MT; ++b) dst[b] = __builtin_bit_cast(bf16x8, *reinterpret_cast<const uint4*>(xrow[b] + 32 * s));
    };
    bf16x8 xring[XD][MT];
  #pragma unroll
    for (int u = 0; u < XD; ++u)
      if (u < n_steps) load_x(u, xring[u]);

    // While a whole round of PD steps and of PD loads ahead is left, the round runs without a condition: only
    // then does each product wait for its own load alone (a load under a condition in a loop makes the next wait
    // a wait for every load).  The last two rounds are written out, not looped over.
    int base = 0;
    for (; base + 2 * PD <= n_steps; base += PD) {
  #pragma unroll
      for (int u = 0; u < PD; ++u) {
        const int s = base + u;  // relative to w_begin
  #pragma unroll
        for (int b = 0; b < MT; ++b)
          acc[b] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ring[u], xring[u % XD][b], acc[b], 0, 0, 0);
        load_x(s + XD, xring[u % XD]);
        ring[u] = load_w(w_begin + s + PD);
        __builtin_amdgcn_sched_barrier(0);  // keep each load right behind its product: PD - 1 stay in flight
      }
    }
    if (base + PD <= n_steps) {  // a whole round of products, fewer than PD loads ahead
  #pragma unroll
      for (int u = 0; u < PD; ++u) {
        const int s = base + u;
  #pragma unroll
        for (int b = 0; b < MT; ++b)
          acc[b] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ring[u], xring[u % XD][b], acc[b], 0, 0, 0);
        if (s + XD < n_steps) load_x(s + XD, xring[u % XD]);
        if (s + PD < n_steps) ring[u] = load_w(w_begin + s + PD);
      }
      base += PD;
    }
    // the last steps, fewer than PD: W is in the ring or on its way, only X is left to fetch
  #pragma unroll
    for (int u = 0; u < PD; ++u) {
      const int s = base + u;
      if (s < n_steps) {
  #pragma unroll
        for (int b = 0; b < MT; ++b)
          acc[b] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ring[u], xring[u % XD][b], acc[b], 0, 0, 0);
        if (s + XD < n_steps) load_x(s + XD, xring[u % XD]);
      }
    }

  };  // round
  if constexpr (ROUNDS) {
    for (int r = slice_begin; r < slice_end; r += staged_steps) {
      if (r > slice_begin) __syncthreads();   // every wave has read the rows of the round before
      round(r, min(r + staged_steps, slice_end));
    }
  } else {
    round(slice_begin, slice_end);
  }

  // add the WK partial sums of every column tile in the order wk = 0, 1, ...: waves wk > 0 park
  // their registers in LDS behind X, waves wk == 0 add
  float* red = reinterpret_cast<float*>(lds + ((M * pitch + 511) / 512) * 512);  // [WK-1][WN][MT][64][4]; X ends on a whole wave's fill
  if constexpr (WK > 1) {
    if (wk > 0) {
#pragma unroll
      for (int b = 0; b < MT; ++b)
        *reinterpret_cast<f32x4*>(red + ((((wk - 1) * WN + wn) * MT + b) * 64 + lane) * 4) = acc[b];
    }
    __syncthreads();
    if (wk > 0) return;
#pragma unroll
    for (int v = 1; v < WK; ++v)
#pragma unroll
      for (int b = 0; b < MT; ++b) {
        const f32x4 p = *reinterpret_cast<const f32x4*>(red + ((((v - 1) * WN + wn) * MT + b) * 64 + lane) * 4);
        acc[b][0] += p[0];
        acc[b][1] += p[1];
        acc[b][2] += p[2];
        acc[b][3] += p[3];
      }
  }

  // acc[b][r] = C[m = 16 b + li][n = n0 + 4 g + r]
  TOut* out = static_cast<TOut*>(a.out) + static_cast<int64_t>(blockIdx.y) * a.split_stride;
  if constexpr (EPI == kEpiSiluMul) {
    float* swap = red + (WK - 1) * WN * MT * 256;  // [WN/2][MT][64][4]: the up sums on their way to the gate wave
    if (wn & 1) {
#pragma unroll
      for (int b = 0; b < MT; ++b) *reinterpret_cast<f32x4*>(swap + (((wn >> 1) * MT + b) * 64 + lane) * 4) = acc[b];
    }
    __syncthreads();  // the waves wk == 0, all that are left
    if (wn & 1) return;
    const int c0 = (n0 / 2) + 4 * g;  // output column of register 0
#pragma unroll
    for (int b = 0; b < MT; ++b) {
      const int mrow = 16 * b + li;
      if (mrow >= M) continue;
      const f32x4 up = *reinterpret_cast<const f32x4*>(swap + (((wn >> 1) * MT + b) * 64 + lane) * 4);
      TOut* o = out + static_cast<int64_t>(mrow) * a.ldo + c0;
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        if (n0 + 16 + 4 * g + r >= N) continue;
        const float gate = acc[b][r];
        o[r] = from_float<TOut>(gate / (1.0f + expf(-gate)) * up[r]);
      }
    }
  } else {
#pragma unroll
    for (int b = 0; b < MT; ++b) {
      const int mrow = 16 * b + li;
      if (mrow >= M) continue;
      const int ncol = n0 + 4 * g;
      TOut* o = out + static_cast<int64_t>(mrow) * a.ldo + ncol;
#pragma unroll
      for (int r = 0; r < 4; ++r)
        if (ncol + r < N) o[r] = from_float<TOut>(acc[b][r]);
    }
  }
}

// ---------------------------------------------------------------------------------------------
// The same product for workgroups that stay: gridDim.x workgroups a k split, each of which stages its X slice
// once and then walks the column groups blockIdx.x, blockIdx.x + gridDim.x, ... with the W ring running on from
// one group into the next.  With more than 16 rows the X slice is large (64 rows of 640 columns are 80 KB), and
// staging it again for every 128 columns, as the kernel above does, costs as much as reading W; here it is
// read once per workgroup, so that W alone is streamed.  Waves: WN, one 16-column tile each; no split of the
// slice inside the workgroup.  The slice is walked in rounds of PD steps; a last round that reaches past the
// slice meets zeros in LDS (the staging puts zeros behind the slice up to a whole round).
template <int MT, int WN, int PD, typename TOut>
__global__ __launch_bounds__(WN * 64) void gemm_stream_kernel(const RowsArgs a) {
  constexpr int kThreads = WN * 64;
  constexpr int XD = 2;
  static_assert(PD % XD == 0, "the X ring must divide the W ring");
  extern __shared__ __align__(16) uint16_t lds[];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int li = lane & 15, g = lane >> 4;
  const int M = a.M, N = a.N, K = a.K;
  const int steps_total = (K + 31) / 32;
  const int s_begin = blockIdx.y * a.steps_per_split;
  const int s_end = min(s_begin + a.steps_per_split, steps_total);
  const int n_steps = s_end - s_begin;
  const int rounds = (n_steps + PD - 1) / PD;
  const int steps_padded = rounds * PD;
  const int pitch = steps_padded * 32 + kPad;
  const int groups_total = (N + WN * 16 - 1) / (WN * 16);
  const int n_mine = (groups_total - static_cast<int>(blockIdx.x) + static_cast<int>(gridDim.x) - 1) / static_cast<int>(gridDim.x);
  if (n_mine <= 0) return;  // the whole workgroup

  auto w_row = [&](int group) {
    const int n0 = (group * WN + wave) * 16;
    return a.tiled ? tile_base(a, n0, lane) : a.w + static_cast<int64_t>(min(n0 + li, N - 1)) * a.ldw;
  };
  const int w_step = a.tiled ? 512 : 32, w_first = a.tiled ? 0 : 8 * g, w_last = a.tiled ? (steps_total - 1) * 512 : K - 8;
  auto load_w = [&](const uint16_t* row, int s) {  // s: step inside the slice (may reach past it, not past K)
    const int e = min(w_step * (s_begin + s) + w_first, w_last);
    return __builtin_bit_cast(bf16x8, *reinterpret_cast<const uint4*>(row + e));
  };
  const uint16_t* wcur = w_row(blockIdx.x);
  bf16x8 ring[PD];
#pragma unroll
  for (int u = 0; u < PD; ++u) ring[u] = load_w(wcur, u);

  {  // X slice -> LDS, as in the kernel above, zeros from the end of the slice to the end of the last round
    const int cpr = steps_padded * 4;
    const int cpp = cpr + kPad / 8;
    const int total = M * cpp;
    const int k0 = s_begin * 32, k1 = min(s_end * 32, K);
    for (int q0 = wave * 64; q0 < total; q0 += kThreads) {
      const int q = min(q0 + lane, total - 1);
      const int row = q / cpp, cc = q % cpp;
      const int col = k0 + cc * 8;
      const uint16_t* src = a.x + static_cast<int64_t>(row) * a.ldx + ((cc < cpr && col < k1) ? col : k0);
      __builtin_amdgcn_global_load_lds(src, (__attribute__((address_space(3))) void*)(lds + q0 * 8), 16, 0, 0);
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    const int z0 = (k1 - k0) / 8, nz = cpr - z0;
    if (nz > 0) {
      __syncthreads();  // the pieces put to zero were fetched by other waves
      for (int i = tid; i < M * nz; i += kThreads)
        *reinterpret_cast<uint4*>(lds + (i / nz) * pitch + (z0 + i % nz) * 8) = uint4{0u, 0u, 0u, 0u};
    }
  }
  __syncthreads();

  const uint16_t* xrow[MT];
#pragma unroll
  for (int b = 0; b < MT; ++b) xrow[b] = lds + min(16 * b + li, M - 1) * pitch + 8 * g;
  auto load_x = [&](int s, bf16x8 (&dst)[MT]) {
#pragma unroll
    for (int b = 0; b < MT; ++b) dst[b] = __builtin_bit_cast(bf16x8, *reinterpret_cast<const uint4*>(xrow[b] + 32 * s));
  };
  bf16x8 xring[XD][MT];
#pragma unroll
  for (int u = 0; u < XD; ++u) load_x(u, xring[u]);  // steps_padded >= PD >= XD

  for (int gi = 0; gi < n_mine; ++gi) {
    const int group = blockIdx.x + gi * gridDim.x;
    // the ring runs on into the workgroup's next group (after the last one: into this one again, unused)
    const uint16_t* wnext_group = w_row(gi + 1 < n_mine ? group + static_cast<int>(gridDim.x) : group);
    f32x4 acc[MT];
#pragma unroll
    for (int b = 0; b < MT; ++b) acc[b] = f32x4{0.f, 0.f, 0.f, 0.f};
    for (int rr = 0; rr < rounds; ++rr) {
      const bool last = rr + 1 == rounds;
      const uint16_t* wnext = last ? wnext_group : wcur;
      const int snext = last ? 0 : (rr + 1) * PD;
#pragma unroll
      for (int u = 0; u < PD; ++u) {
        const int s = rr * PD + u;
#pragma unroll
        for (int b = 0; b < MT; ++b)
          acc[b] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ring[u], xring[u % XD][b], acc[b], 0, 0, 0);
        int sx = s + XD;
        if (sx >= steps_padded) sx -= steps_padded;  // the next group starts at the slice's first step again
        load_x(sx, xring[u % XD]);
        ring[u] = load_w(wnext, snext + u);
        __builtin_amdgcn_sched_barrier(0);  // each load right behind its product
      }
    }
    wcur = wnext_group;
    // acc[b][r] = C[m = 16 b + li][n = n0 + 4 g + r]
    TOut* out = static_cast<TOut*>(a.out) + static_cast<int64_t>(blockIdx.y) * a.split_stride;
    const int ncol = (group * WN + wave) * 16 + 4 * g;
#pragma unroll
    for (int b = 0; b < MT; ++b) {
      const int mrow = 16 * b + li;
      if (mrow >= M) continue;
      TOut* o = out + static_cast<int64_t>(mrow) * a.ldo + ncol;
      if (ncol + 3 < N && (a.ldo & 3) == 0) {
        if constexpr (sizeof(TOut) == 4) {
          *reinterpret_cast<float4*>(o) = float4{acc[b][0], acc[b][1], acc[b][2], acc[b][3]};
        } else {
#pragma unroll
          for (int r = 0; r < 4; ++r) o[r] = from_float<TOut>(acc[b][r]);
        }
      } else {
#pragma unroll
        for (int r = 0; r < 4; ++r)
          if (ncol + r < N) o[r] = from_float<TOut>(acc[b][r]);
      }
    }
  }
}

inline size_t stream_lds_bytes(int M, int steps_per_split, int pd) {
  const int padded = (steps_per_split + pd - 1) / pd * pd;
  return (static_cast<size_t>(M) * (padded * 32 + kPad) + 511) / 512 * 512 * sizeof(uint16_t);
}

// LDS of a launch: the X rows of one k slice and, behind them, the partial sums of the waves wk > 0 and the
// gate/up exchange.
inline size_t rows_lds_bytes(int M, int steps_per_split, int mt, int wn, int wk) {
  const size_t x = (static_cast<size_t>(M) * (steps_per_split * 32 + kPad) + 511) / 512 * 512 * sizeof(uint16_t);
  const size_t red = static_cast<size_t>(wk - 1) * wn * mt * 64 * 4 * sizeof(float);
  const size_t swap = static_cast<size_t>((wn + 1) / 2) * mt * 64 * 4 * sizeof(float);
  return x + red + swap;
}
constexpr size_t kRowsLdsMax = 144 * 1024;  // of the 160 KB of a CU

template <int MT, int WN, int WK, int PD, int XD, int EPI, typename TOut>
int launch_rows(const RowsArgs& a, int splits, hipStream_t s) {
  const size_t lds = rows_lds_bytes(a.M, a.steps_per_split, MT, WN, WK);
  if (lds > kRowsLdsMax) return static_cast<int>(hipErrorInvalidValue);
  auto kernel = gemm_rows_kernel<MT, WN, WK, PD, XD, EPI, TOut>;
  static size_t allowed = 64 * 1024;  // per instantiation: what the function may use so far
  if (lds > allowed) {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                                       static_cast<int>(kRowsLdsMax));
    if (e != hipSuccess) {
      (void)hipGetLastError();  // do not leave the error behind for the next call to find
      return static_cast<int>(e);
    }
    allowed = kRowsLdsMax;
  }
  const int col_groups = (a.N + WN * 16 - 1) / (WN * 16);
  kernel<<<dim3(col_groups, splits), WN * WK * 64, lds, s>>>(a);
  return launch_status();
}

// The fused activation for more rows than LDS holds of all of K at once: one k slice, walked in rounds.
template <int MT, int WN, int WK, int PD, int XD, typename TOut>
int launch_rows_rounds(const RowsArgs& a, hipStream_t s) {
  const size_t lds = rows_lds_bytes(a.M, a.steps_per_round, MT, WN, WK);
  if (lds > kRowsLdsMax) return static_cast<int>(hipErrorInvalidValue);
  auto kernel = gemm_rows_kernel<MT, WN, WK, PD, XD, kEpiSiluMul, TOut, true>;
  static size_t allowed = 64 * 1024;
  if (lds > allowed) {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                                       static_cast<int>(kRowsLdsMax));
    if (e != hipSuccess) {
      (void)hipGetLastError();
      return static_cast<int>(e);
    }
    allowed = kRowsLdsMax;
  }
  const int col_groups = (a.N + WN * 16 - 1) / (WN * 16);
  kernel<<<dim3(col_groups, 1), WN * WK * 64, lds, s>>>(a);
  return launch_status();
}

template <int MT, int WN, int WK, int PD, int XD, int EPI>
int launch_rows_out(const RowsArgs& a, int splits, int out_dtype, hipStream_t s) {
  if (out_dtype == kF32) return launch_rows<MT, WN, WK, PD, XD, EPI, float>(a, splits, s);
  return launch_rows<MT, WN, WK, PD, XD, EPI, bf16>(a, splits, s);
}

template <int MT, int WN, int WK, int PD>
int dispatch_rows(const RowsArgs& a, int splits, int out_dtype, int epilogue, hipStream_t s) {
  constexpr int XD = MT == 1 ? 4 : 2;  // X steps read ahead from LDS (registers: XD * MT * 4)
  if constexpr (WN % 2 == 0) {
    if (epilogue == kEpiSiluMul) return launch_rows_out<MT, WN, WK, PD, XD, kEpiSiluMul>(a, splits, out_dtype, s);
  }
  return launch_rows_out<MT, WN, WK, PD, XD, kEpiNone>(a, splits, out_dtype, s);
}

}  // namespace arle

using namespace arle;

// Shapes of a workgroup, by `variant`: (WN, WK, PD), picked by the caller per matrix shape and row count
// from measurements on MI355X.  The fused activation needs an even WN.
//   0  general product               1  gate/up with the fused activation, a few rows
//   2  few output columns            3  more rows with the fused activation, or very many columns
//   4  general, more columns a workgroup
#define ARLE_ROWS_VARIANTS(X) X(0, 2, 2, 4) X(1, 2, 4, 4) X(2, 1, 4, 4) X(3, 8, 1, 4) X(4, 4, 1, 8)
constexpr int kVariants = 5;

// (waves that share the k slice) << 20 | (output columns of one workgroup) << 4 | (1 if the variant can apply
// the fused activation); -1 for an unknown variant
extern "C" int arle_gemm_rows_geometry(int variant) {
  switch (variant) {
#define X(ID, WN, WK, PD) \
  case ID:                \
    return (WK << 20) | ((WN * 16) << 4) | (WN % 2 == 0 ? 1 : 0);
    ARLE_ROWS_VARIANTS(X)
#undef X
    default:
      return -1;
  }
}

// Bytes of LDS that a launch of `variant` needs for M rows and k slices of steps_per_split steps; the launch
// is refused above arle_gemm_rows_lds_max().
extern "C" long long arle_gemm_rows_lds(int variant, int M, int steps_per_split) {
  const int mt = M <= 16 ? 1 : (M <= 32 ? 2 : 4);
  switch (variant) {
#define X(ID, WN, WK, PD) \
  case ID:                \
    return static_cast<long long>(rows_lds_bytes(M, steps_per_split, mt, WN, WK));
    ARLE_ROWS_VARIANTS(X)
#undef X
    default:
      return -1;
  }
}
extern "C" long long arle_gemm_rows_lds_max() { return static_cast<long long>(kRowsLdsMax); }

// x [M, K] and w [N, K] bfloat16 with row strides in elements (multiples of 8), 1 <= M <= 64, K % 8 == 0.
// splits == 1: out [M, N] (or [M, N/2] with the fused activation) bfloat16 or float32.
// splits  > 1: out [splits, M, N] float32 partial products, split_stride elements apart, no activation;
//              split s covers steps [s * steps_per_split, (s + 1) * steps_per_split) and none may be empty.
// w_tiled: w holds operand tiles (RowsArgs), ldw is not used.
extern "C" int arle_gemm_rows(const void* x, long long ldx, const void* w, long long ldw, int w_tiled, void* out, long long ldo,
                              long long split_stride, int out_dtype, int M, int N, int K, int epilogue, int variant,
                              int splits, int steps_per_split, void* stream) {
  if (M <= 0 || N <= 0) return 0;
  if (M > 64 || K % 8 != 0 || K <= 0 || ldx % 8 != 0 || ldw % 8 != 0 || splits < 1 || splits > 65535 ||
      steps_per_split < 1 || variant < 0 || variant >= kVariants)
    return static_cast<int>(hipErrorInvalidValue);
  const int steps_total = (K + 31) / 32;
  if (static_cast<long long>(splits - 1) * steps_per_split >= steps_total ||
      static_cast<long long>(splits) * steps_per_split < steps_total)
    return static_cast<int>(hipErrorInvalidValue);
  if (splits > 1 && (out_dtype != kF32 || epilogue != kEpiNone)) return static_cast<int>(hipErrorInvalidValue);
  if (epilogue == kEpiSiluMul && (N % 32 != 0 || (arle_gemm_rows_geometry(variant) & 15) != 1))
    return static_cast<int>(hipErrorInvalidValue);
  if (epilogue != kEpiNone && epilogue != kEpiSiluMul) return static_cast<int>(hipErrorInvalidValue);
  hipStream_t s = static_cast<hipStream_t>(stream);
  const RowsArgs a{static_cast<const uint16_t*>(x), ldx, static_cast<const uint16_t*>(w), ldw, out, ldo, M, N, K,
                   steps_per_split, split_stride, w_tiled ? 1 : 0, 0};
  switch (variant) {
#define X(ID, WN, WK, PD)                                                                       \
  case ID:                                                                                      \
    if (M <= 16) return dispatch_rows<1, WN, WK, PD>(a, splits, out_dtype, epilogue, s);        \
    if (M <= 32) return dispatch_rows<2, WN, WK, PD>(a, splits, out_dtype, epilogue, s);        \
    return dispatch_rows<4, WN, WK, PD>(a, splits, out_dtype, epilogue, s);
    ARLE_ROWS_VARIANTS(X)
#undef X
  }
  return static_cast<int>(hipErrorInvalidValue);
}

// gate|up with the fused activation for up to 64 rows: as arle_gemm_rows with epilogue 1, variant 3 (eight waves,
// one column tile each) and one k split, but the X rows of only steps_per_round steps of 32 are in LDS at a time
// (arle_gemm_rows_lds(3, M, steps_per_round) <= arle_gemm_rows_lds_max()); all of K is walked in such rounds.
extern "C" int arle_gemm_rows_rounds(const void* x, long long ldx, const void* w, long long ldw, int w_tiled, void* out,
                                     long long ldo, int out_dtype, int M, int N, int K, int steps_per_round, void* stream) {
  if (M <= 0 || N <= 0) return 0;
  if (M > 64 || K % 8 != 0 || K <= 0 || ldx % 8 != 0 || ldw % 8 != 0 || N % 32 != 0 || steps_per_round < 1)
    return static_cast<int>(hipErrorInvalidValue);
  const int steps_total = (K + 31) / 32;
  hipStream_t s = static_cast<hipStream_t>(stream);
  const RowsArgs a{static_cast<const uint16_t*>(x), ldx, static_cast<const uint16_t*>(w), ldw, out, ldo, M, N, K,
                   steps_total, 0, w_tiled ? 1 : 0, steps_per_round < steps_total ? steps_per_round : steps_total};
  const bool f32 = out_dtype == kF32;
  if (M <= 16) return f32 ? launch_rows_rounds<1, 8, 1, 4, 4, float>(a, s) : launch_rows_rounds<1, 8, 1, 4, 4, bf16>(a, s);
  if (M <= 32) return f32 ? launch_rows_rounds<2, 8, 1, 4, 2, float>(a, s) : launch_rows_rounds<2, 8, 1, 4, 2, bf16>(a, s);
  return f32 ? launch_rows_rounds<4, 8, 1, 4, 2, float>(a, s) : launch_rows_rounds<4, 8, 1, 4, 2, bf16>(a, s);
}

// Shapes of a staying workgroup, by `variant`: (WN, PD).
#define ARLE_STREAM_VARIANTS(X) X(0, 4, 8) X(1, 8, 4) X(2, 8, 8) X(3, 4, 4) X(4, 2, 8)
constexpr int kStreamVariants = 5;

// (output columns of one column group) << 8 | PD; -1 for an unknown variant
extern "C" int arle_gemm_stream_geometry(int variant) {
  switch (variant) {
#define X(ID, WN, PD) \
  case ID:            \
    return ((WN * 16) << 8) | PD;
    ARLE_STREAM_VARIANTS(X)
#undef X
    default:
      return -1;
  }
}

extern "C" long long arle_gemm_stream_lds(int variant, int M, int steps_per_split) {
  const int geometry = arle_gemm_stream_geometry(variant);
  if (geometry < 0) return -1;
  return static_cast<long long>(stream_lds_bytes(M, steps_per_split, geometry & 255));
}

namespace arle {
template <int MT, int WN, int PD, typename TOut>
int launch_stream(const RowsArgs& a, int splits, int workgroups, hipStream_t s) {
  const size_t lds = stream_lds_bytes(a.M, a.steps_per_split, PD);
  if (lds > kRowsLdsMax) return static_cast<int>(hipErrorInvalidValue);
  auto kernel = gemm_stream_kernel<MT, WN, PD, TOut>;
  static size_t allowed = 64 * 1024;
  if (lds > allowed) {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                                       static_cast<int>(kRowsLdsMax));
    if (e != hipSuccess) {
      (void)hipGetLastError();
      return static_cast<int>(e);
    }
    allowed = kRowsLdsMax;
  }
  const int groups = (a.N + WN * 16 - 1) / (WN * 16);
  kernel<<<dim3(min(workgroups, groups), splits), WN * 64, lds, s>>>(a);
  return launch_status();
}

template <int WN, int PD>
int dispatch_stream(const RowsArgs& a, int splits, int workgroups, int out_dtype, hipStream_t s) {
  const bool f32 = out_dtype == kF32;
  if (a.M <= 16)
    return f32 ? launch_stream<1, WN, PD, float>(a, splits, workgroups, s) : launch_stream<1, WN, PD, bf16>(a, splits, workgroups, s);
  if (a.M <= 32)
    return f32 ? launch_stream<2, WN, PD, float>(a, splits, workgroups, s) : launch_stream<2, WN, PD, bf16>(a, splits, workgroups, s);
  return f32 ? launch_stream<4, WN, PD, float>(a, splits, workgroups, s) : launch_stream<4, WN, PD, bf16>(a, splits, workgroups, s);
}
}  // namespace arle

// The product with workgroups that stay (see gemm_stream_kernel): `workgroups` of them for every k split walk
// the column groups.  Operands, splits and the stack of partial products as in arle_gemm_rows; no activation.
extern "C" int arle_gemm_stream(const void* x, long long ldx, const void* w, long long ldw, int w_tiled, void* out, long long ldo,
                                long long split_stride, int out_dtype, int M, int N, int K, int variant, int splits,
                                int steps_per_split, int workgroups, void* stream) {
  if (M <= 0 || N <= 0) return 0;
  if (M > 64 || K % 8 != 0 || K <= 0 || ldx % 8 != 0 || ldw % 8 != 0 || splits < 1 || splits > 65535 ||
      steps_per_split < 1 || workgroups < 1 || variant < 0 || variant >= kStreamVariants)
    return static_cast<int>(hipErrorInvalidValue);
  const int steps_total = (K + 31) / 32;
  if (static_cast<long long>(splits - 1) * steps_per_split >= steps_total ||
      static_cast<long long>(splits) * steps_per_split < steps_total)
    return static_cast<int>(hipErrorInvalidValue);
  if (splits > 1 && out_dtype != kF32) return static_cast<int>(hipErrorInvalidValue);
  hipStream_t s = static_cast<hipStream_t>(stream);
  const RowsArgs a{static_cast<const uint16_t*>(x), ldx, static_cast<const uint16_t*>(w), ldw, out, ldo, M, N, K,
                   steps_per_split, split_stride, w_tiled ? 1 : 0, 0};
  switch (variant) {
#define X(ID, WN, PD) \
  case ID:            \
    return dispatch_stream<WN, PD>(a, splits, workgroups, out_dtype, s);
    ARLE_STREAM_VARIANTS(X)
#undef X
  }
  return static_cast<int>(hipErrorInvalidValue);
}
