// bfloat16 matrix product for many rows (long prompt portions):  C[M,N] = X[M,K] . W[N,K]^T, W given as operand
// tiles (see gemm_rows.hip: [ceil(N/16)][ceil(K/32)][64 lanes][8], zeros past N and K).
//
// With W in that order its operands need no LDS at all: the lanes of a wave read their 16-byte pieces of two
// neighbouring tiles (runs of 512 contiguous bytes) straight into the A operand of v_mfma_f32_32x32x16_bf16, and
// every tile is read by one wave of the workgroup only.  LDS carries X alone.  A workgroup of four waves owns 128
// or 256 rows and 256 columns; wave w owns the columns 64 w .. 64 w + 63 for all rows, so an X operand read from
// LDS meets two W operands.  (32x32x16 and not 16x16x32: one wave a SIMD issues the former at the full rate of
// the matrix cores, 2.4 PFLOP/s measured over the chip, the latter at 1.4.)
//
//   * X goes through registers into LDS in operand order: a lane fetches 16 bytes of a (16 rows x 32 k) piece,
//     four neighbouring lanes the 64 contiguous bytes of a row, and parks them where the lane (row j, half h) of
//     the 32 x 16 operand will read them.  Reads are linear in the lane inside a half; the halves are padded so that
//     the writes of neighbouring lanes meet different banks.  Two stages.
//   * Both streams run ahead of the products through rings of registers (PD and PX steps of 32 k).  Nothing is
//     selected or converted behind a load: a use right behind a load is a wait for that load.
//   * The operand reads of a step are pinned four reads ahead of the products that need them.  PIPE: four LDS
//     stages, the step's barrier in mid-step, and behind it the first operands of the next step are read while
//     the last products of this one run.
//   * bfloat16 results leave through a wave's own part of LDS as whole rows of 128 contiguous bytes.
//   * Workgroups are numbered so that those that an XCD runs at one time are a patch of 8 row blocks x 8 column
//     blocks (up to 8 row blocks: all rows of one column block, so that W is fetched once and X, a few megabytes,
//     stays in every L2): the patch's rows of X and columns of W are what the XCD's L2 has to fetch for it.  Against
//     all row blocks of one column block side by side: 385 instead of 420 us for gate|up at 4,096 rows, 740 instead
//     of 785 at 8,192.
//   * Epilogue kEpiSiluMul (gate and up rows interleaved in blocks of 16): the 32 columns of an accumulator are
//     16 gate and the 16 matching up columns, registers r and r + 8 of the same lane, so silu(gate) * up happens
//     in registers and [M, N/2] is written.
//
// Measured on MI355X, weights cold: gate|up of the Qwen3-4B shape with the activation at 2,048 rows 237-255 us
// against 234-272 us for the library's product and the activation kernel (machines differ); whole prefill steps are
// 0.5 to 4.6 % faster with it at that shape, and 8-9 % slower at hidden sizes of 4,096 and 5,120, so the caller
// takes it for the former only.  The loop without its global loads runs at 930 TFLOP/s on q|k|v at 2,048 rows
// (192 workgroups for 256 compute units), with everything at 760.  Plain products stay with the library, which
// is faster there (q|k|v at 2,048 rows: 60 against 85 us), as the reference
// leaves all of them to cuBLAS (infer/src/ops/linear.rs:921-959) and runs the activation as a kernel of its own
// (crates/cuda-kernels/csrc/misc/split_qkv.cu:35-52).
#include "common.h"

namespace arle {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));  // a plain vector: arrays of HIP's uint4 structs end up in scratch memory

constexpr int kTlWaves = 4;
constexpr int kTlXcds = 8;
constexpr int kEpiNone = 0, kEpiSiluMul = 1;

struct TilesArgs {
  const uint16_t* x;
  int64_t ldx;
  const uint16_t* w;  // operand tiles
  void* out;
  int64_t ldo;
  int M, N, K;
  int m_blocks, n_blocks;
  int patch_rows, patch_cols;  // row blocks x column blocks that run side by side on one XCD
  int steps_per_split;    // steps of 32 k that one workgroup walks: blockIdx.y picks the part of K
  int64_t split_stride;   // elements between the parts' results in `out` (a float32 stack [parts][M][N])
};

// MT: row tiles of 32 that a workgroup owns (4: 128 rows); TN: column tiles of 32 that a wave owns (2: 256
// columns a workgroup; 1: 128, for products with so few rows that they are a matter of streaming W, where more and
// smaller workgroups keep more loads in flight).  gridDim.y parts of K, each leaving a result of its own.
template <int MT, int TN, int PD, int PX, bool PIPE, int EPI, typename TOut>
// (the second figure is waves a SIMD: the registers a wave may have)
__global__ __launch_bounds__(kTlWaves* kWave, MT* TN >= 16 ? 1 : (MT * TN >= 8 || PD >= 8 ? 2 : 3))
void gemm_tiles_kernel(const TilesArgs a) {
  static_assert(!PIPE || TN == 2, "the pipelined loop is written for two column tiles a wave");
  constexpr int kTlCols = 32 * TN * kTlWaves;  // columns a workgroup owns
  static_assert(PD % 2 == 0 && PD % PX == 0, "rounds of PD steps; the LDS stage alternates; the X ring divides the W ring");
  static_assert(MT % 2 == 0, "every wave fetches whole pieces of 16 rows");
  static_assert(!PIPE || PD == 4, "the pipelined loop walks four LDS stages in a round of four steps");
  constexpr int kHalf = 576, kPiece = 2 * kHalf;             // an operand's two halves of 512 bytes, 64 bytes of padding behind each
  constexpr int kRows = 32 * MT, kStage = 2 * MT * kPiece;  // bytes of one LDS stage: the rows' 32 k
  constexpr int XH = 2 * MT / kTlWaves;                    // pieces of 16 rows x 32 k that a wave fetches a step
  constexpr int kOutPitch = 64 * TN + 16;  // bytes of a wave's row of bfloat16 in the epilogue's LDS, padded against bank conflicts
  constexpr int kOutBytes = kTlWaves * 32 * kOutPitch;
  constexpr int kLdsBytes = (PIPE ? 4 : 2) * kStage > kOutBytes ? (PIPE ? 4 : 2) * kStage : kOutBytes;
  __shared__ __align__(16) unsigned char lds[kLdsBytes];
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);  // known to be the same in all lanes
  const int li = lane & 15, g = lane >> 4;   // the lane as (row, 8 k) of a 16 x 32 piece: tiles in memory, fetches of X
  const int j = lane & 31, h = lane >> 5;    // the lane as (row, 8 k) of a 32 x 16 operand

  // workgroup -> (row block, column block): the row blocks of a column block side by side on one XCD
  const int xcd = blockIdx.x % kTlXcds, q = blockIdx.x / kTlXcds;
  const int patch = a.patch_rows * a.patch_cols, in_patch = q % patch, p = q / patch;
  const int row_groups = (a.m_blocks + a.patch_rows - 1) / a.patch_rows;
  const int mb = (p % row_groups) * a.patch_rows + in_patch % a.patch_rows;
  const int nb = ((p / row_groups) * a.patch_cols + in_patch / a.patch_rows) * kTlXcds + xcd;
  if (mb >= a.m_blocks || nb >= a.n_blocks) return;  // the whole workgroup
  const int m0 = mb * kRows, n0 = nb * kTlCols + wave * (32 * TN);
  const int M = a.M, N = a.N, K = a.K;
  const int steps = (K + 31) / 32, n_tiles = (N + 15) / 16;
  const int s_begin = blockIdx.y * a.steps_per_split;                 // this workgroup's part of K
  const int n_steps = min(a.steps_per_split, steps - s_begin);
  const int rounds = n_steps / PD, rest = n_steps % PD;  // whole rounds of the rings, and the steps after them

  // W operand of column tile tn (32 columns), half kk of a step: lane (j, h) takes the piece that lane
  // 16 (2 kk + h) + j % 16 of the 16-column tile 2 tn + j / 16 holds: k = 32 s + 16 kk + 8 h .. + 7
  const uint16_t* wptr[TN];
#pragma unroll
  for (int tn = 0; tn < TN; ++tn)
    wptr[tn] = a.w + static_cast<int64_t>(min(n0 / 16 + 2 * tn + (j >> 4), n_tiles - 1)) * steps * 512 + (16 * h + (j & 15)) * 8;
  auto load_w = [&](int s, bf16x8 (&dst)[TN][2]) {   // s: step inside this workgroup's part
    const int64_t off = static_cast<int64_t>(min(s_begin + s, steps - 1)) * 512;  // a step past K is fetched and never multiplied
#pragma unroll
    for (int tn = 0; tn < TN; ++tn)
#pragma unroll
      for (int kk = 0; kk < 2; ++kk) dst[tn][kk] = *reinterpret_cast<const bf16x8*>(wptr[tn] + off + kk * 256);
  };
  // X: a fetch is 16 rows x 32 k, four lanes a row (64 contiguous bytes), so that four neighbouring lanes ask for one
  // piece of a cache line (the memory pipeline takes the lanes of a load four at a time: with a lane a row it had
  // four times the requests).  Lane 4 r + c holds row r, k 8 c .. + 7 and parks it where lane (j = 16 half + r,
  // h = c % 2) of the operand of half kk = c / 2 reads it.  An operand in LDS is its two halves h of 512 bytes with 64
  // bytes of padding behind each: the four pieces that four neighbouring lanes park (c = 0 .. 3) then fall into
  // different banks, and sixteen lanes in a row of either access never share one.
  // A piece past K is fetched from a place that exists and meets the zeros that the tiles hold there.
  const int fr = lane >> 2, fc = lane & 3;
  const uint16_t* xptr[XH];
#pragma unroll
  for (int p = 0; p < XH; ++p)
    xptr[p] = a.x + static_cast<int64_t>(min(m0 + 16 * (XH * wave + p) + fr, M - 1)) * a.ldx;
  auto load_x = [&](int s, u32x4 (&dst)[XH]) {
    const int col = 32 * (s_begin + s) + 8 * fc;
    const int at = col < K ? col : 0;
#pragma unroll
    for (int p = 0; p < XH; ++p) dst[p] = *reinterpret_cast<const u32x4*>(xptr[p] + at);
  };
  // piece p of the wave is half (XH wave + p) % 2 of row tile (XH wave + p) / 2; XH is even, so p / 2 and p % 2 do
  const int park_at = ((XH / 2 * wave) * 2 + (fc >> 1)) * kPiece + (fc & 1) * kHalf + fr * 16;
  auto park_x = [&](int stage, const u32x4 (&src)[XH]) {
#pragma unroll
    for (int p = 0; p < XH; ++p)
      *reinterpret_cast<u32x4*>(lds + stage * kStage + park_at + (p / 2) * 2 * kPiece + (p % 2) * 256) = src[p];
  };
  const int read_at = h * kHalf + j * 16;   // this lane's place in an operand

  f32x16 acc[MT][TN];
#pragma unroll
  for (int t = 0; t < MT; ++t)
#pragma unroll
    for (int tn = 0; tn < TN; ++tn)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[t][tn][r] = 0.f;

  bf16x8 wring[PD][TN][2];
  u32x4 xring[PX][XH];  // slot u % PX holds step (round * PD + u) + 1: the one parked while step u is multiplied
#pragma unroll
  for (int u = 0; u < PD; ++u) load_w(u, wring[u]);
  {
    u32x4 first[XH];
    load_x(0, first);
#pragma unroll
    for (int u = 0; u < PX; ++u) load_x(u + 1, xring[u]);
    park_x(0, first);
  }
  __syncthreads();

  auto multiply = [&](const bf16x8 (&wt)[TN][2], int stage) {  // the step parked in `stage` with its tiles
    const unsigned char* xs = lds + stage * kStage + read_at;
#pragma unroll
    for (int kk = 0; kk < 2; ++kk)
#pragma unroll
      for (int t = 0; t < MT; ++t) {
        const bf16x8 xop = *reinterpret_cast<const bf16x8*>(xs + (2 * t + kk) * kPiece);
#pragma unroll
        for (int tn = 0; tn < TN; ++tn)
          acc[t][tn] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(wt[tn][kk], xop, acc[t][tn], 0, 0, 0);
      }
    // operand reads run kAhead reads (2 kAhead products) ahead of the products that need them; left to itself the
    // compiler reads two, waits, multiplies four times and reads again
    constexpr int kAhead = 4, kReads = 2 * MT;
    __builtin_amdgcn_sched_group_barrier(0x100, kAhead, 0);
#pragma unroll
    for (int i = 0; i < kReads - kAhead; ++i) {
      __builtin_amdgcn_sched_group_barrier(0x008, TN, 0);
      __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
    }
    __builtin_amdgcn_sched_group_barrier(0x008, TN * kAhead, 0);
  };
  if constexpr (PIPE) {
    // Four stages, so that a step can be parked two steps before anybody reads its stage again, and the barrier of
    // a step can stand in the middle of it: step s + 1 is parked first thing in step s, the barrier comes before
    // the last kA operand reads' worth of products, and behind it the first kA operands of step s + 1 are read
    // while the last products of step s run.  No product waits for an LDS read right behind a barrier.
    constexpr int kA = 4, kR = 2 * MT;
    bf16x8 pre[kA];
#pragma unroll
    for (int i = 0; i < kA; ++i) pre[i] = *reinterpret_cast<const bf16x8*>(lds + 2 * i * kPiece + read_at);  // row tiles 0 .. kA - 1, half 0
    // The step's eight loads go out one at a time between the products, two operand reads and four products
    // apart (sent together they queue in the memory pipeline, and a wave that cannot send a load cannot send the
    // product behind it either): first the halves kk = 1 of the step before, whose registers are free since its
    // last product, then the four pieces of X, then the halves kk = 0 of this step, free after its first half.
    auto load_w1 = [&](int s, bf16x8& dst, int tn, int kk) {
      const int64_t off = static_cast<int64_t>(min(s_begin + s, steps - 1)) * 512;
      dst = *reinterpret_cast<const bf16x8*>(wptr[tn] + off + kk * 256);
    };
    auto load_x1 = [&](int s, u32x4& dst, int p) {
      const int col = 32 * (s_begin + s) + 8 * fc;
      dst = *reinterpret_cast<const u32x4*>(xptr[p] + (col < K ? col : 0));
    };
    static_assert(2 + XH + 2 <= MT, "a load behind every second operand read of a step");
    auto step = [&](bf16x8 (&wt)[2][2], bf16x8 (&wprev)[2][2], u32x4 (&xnext)[XH], int u, int s, bool fetch) {
      park_x((u + 1) & 3, xnext);
      const unsigned char* cur = lds + (u & 3) * kStage + read_at;
      const unsigned char* nxt = lds + ((u + 1) & 3) * kStage + read_at;
      bf16x8 xo[kR];
#pragma unroll
      for (int i = 0; i < kA; ++i) xo[i] = pre[i];
#pragma unroll
      for (int r = 0; r < kR; ++r) {
        if (r == kR - kA) __syncthreads();
        // read r is the operand of row tile r % MT, half r / MT of the step: the two products into one
        // accumulator are 2 MT products apart (a product right behind one into the same accumulator waits for it)
        constexpr auto at = [](int q) { return (2 * (q % MT) + q / MT) * kPiece; };
        if (r + kA < kR)
          xo[r + kA] = *reinterpret_cast<const bf16x8*>(cur + at(r + kA));
        else
          pre[r + kA - kR] = *reinterpret_cast<const bf16x8*>(nxt + at(r + kA - kR));
        if (fetch && (r & 1)) {
          const int q = r >> 1;
          if (q < 2)
            load_w1(s - 1 + PD, wprev[q][1], q, 1);   // in the first step: the same tiles as before the loop, again
          else if (q < 2 + XH)
            load_x1(s + 1 + PX, xnext[q - 2], q - 2);
          else
            load_w1(s + PD, wt[q - 2 - XH][0], q - 2 - XH, 0);
        }
#pragma unroll
        for (int tn = 0; tn < 2; ++tn)
          acc[r % MT][tn] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(wt[tn][r / MT], xo[r], acc[r % MT][tn], 0, 0, 0);
        __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
        if (r & 1) __builtin_amdgcn_sched_group_barrier(0x020, 1, 0);
        __builtin_amdgcn_sched_group_barrier(0x008, 2, 0);
      }
    };
    for (int r = 0; r < rounds; ++r) {
#pragma unroll
      for (int u = 0; u < PD; ++u) step(wring[u], wring[(u + PD - 1) % PD], xring[u % PX], u, r * PD + u, true);
    }
#pragma unroll
    for (int u = 0; u < PD - 1; ++u)
      if (u < rest) step(wring[u], wring[(u + PD - 1) % PD], xring[u % PX], u, rounds * PD + u, false);
  } else {
  for (int r = 0; r < rounds; ++r) {
#pragma unroll
    for (int u = 0; u < PD; ++u) {
      const int s = r * PD + u;
      multiply(wring[u], u & 1);
      load_w(s + PD, wring[u]);
      park_x((u + 1) & 1, xring[u % PX]);
      load_x(s + 1 + PX, xring[u % PX]);
      __syncthreads();
    }
  }
  // the steps after the last whole round: their tiles are in the ring, their X is in the ring or parked
#pragma unroll
  for (int u = 0; u < PD - 1; ++u) {
    if (u < rest) {
      multiply(wring[u], u & 1);
      if (u + 1 < rest) {
        park_x((u + 1) & 1, xring[u % PX]);
        if (u + 1 + PX < rest) load_x(rounds * PD + u + 1 + PX, xring[u % PX]);
        __syncthreads();
      }
    }
  }
  }

  // acc[t][tn][r] = C[m0 + 32 t + j][n0 + 32 tn + 8 (r / 4) + 4 h + r % 4]
  TOut* out = static_cast<TOut*>(a.out) + static_cast<int64_t>(blockIdx.y) * a.split_stride;
  // bfloat16 results whose columns (64 a wave, or 32) all exist: a lane holds pieces of 8 bytes, and stored as they are they
  // would reach memory as 16-byte scraps of a row (a third of the kernel's time at 2,048 x 6,144).  So every
  // row tile goes through a part of LDS that belongs to the wave and leaves as whole rows of 128 (with the
  // activation: 64) contiguous bytes, eight (four) lanes a row.
  constexpr int kOutCols = EPI == kEpiSiluMul ? 16 * TN : 32 * TN;
  if constexpr (sizeof(TOut) == 2) {
    const int c0 = EPI == kEpiSiluMul ? n0 / 2 : n0;          // first output column of the wave
    const int n_out = EPI == kEpiSiluMul ? N / 2 : N;
    __syncthreads();  // every wave is done with the stages (all waves come here, whichever way they store)
    if (c0 + kOutCols <= n_out && (a.ldo & 7) == 0 && (reinterpret_cast<uintptr_t>(a.out) & 15) == 0) {  // the same in all lanes of a wave
      unsigned char* mine = lds + wave * (32 * kOutPitch);
      constexpr int kLanesARow = kOutCols / 8, kRowsAPass = 64 / kLanesARow;
#pragma unroll
      for (int t = 0; t < MT; ++t) {
#pragma unroll
        for (int tn = 0; tn < TN; ++tn) {
          if constexpr (EPI == kEpiSiluMul) {
#pragma unroll
            for (int q4 = 0; q4 < 2; ++q4) {
              float v[4];
#pragma unroll
              for (int e = 0; e < 4; ++e) {
                const float gate = acc[t][tn][4 * q4 + e];
                v[e] = gate / (1.0f + expf(-gate)) * acc[t][tn][4 * q4 + e + 8];
              }
              *reinterpret_cast<uint2*>(mine + j * kOutPitch + (16 * tn + 8 * q4 + 4 * h) * 2) =
                  uint2{pack_bf16x2(v[0], v[1]), pack_bf16x2(v[2], v[3])};
            }
          } else {
#pragma unroll
            for (int q4 = 0; q4 < 4; ++q4)
              *reinterpret_cast<uint2*>(mine + j * kOutPitch + (32 * tn + 8 * q4 + 4 * h) * 2) =
                  uint2{pack_bf16x2(acc[t][tn][4 * q4], acc[t][tn][4 * q4 + 1]),
                        pack_bf16x2(acc[t][tn][4 * q4 + 2], acc[t][tn][4 * q4 + 3])};
          }
        }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
#pragma unroll
        for (int i = 0; i < 32 / kRowsAPass; ++i) {
          const int rr = kRowsAPass * i + lane / kLanesARow, piece = lane % kLanesARow;
          const u32x4 v = *reinterpret_cast<const u32x4*>(mine + rr * kOutPitch + piece * 16);
          const int row = m0 + 32 * t + rr;
          if (row < M)
            *reinterpret_cast<u32x4*>(reinterpret_cast<uint16_t*>(out) + static_cast<int64_t>(row) * a.ldo + c0 + piece * 8) = v;
        }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
      }
      return;
    }
  }
#pragma unroll
  for (int t = 0; t < MT; ++t) {
    const int row = m0 + 32 * t + j;
    if (row >= M) continue;
#pragma unroll
    for (int tn = 0; tn < TN; ++tn) {
      if constexpr (EPI == kEpiSiluMul) {
        // the 32 columns are 16 gate and the 16 matching up columns: registers r and r + 8
#pragma unroll
        for (int q4 = 0; q4 < 2; ++q4) {
          const int col = (n0 + 32 * tn) / 2 + 8 * q4 + 4 * h;
          float v[4];
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            const float gate = acc[t][tn][4 * q4 + e];
            v[e] = gate / (1.0f + expf(-gate)) * acc[t][tn][4 * q4 + e + 8];
          }
          TOut* o = out + static_cast<int64_t>(row) * a.ldo + col;
          if (n0 + 32 * tn + 32 <= N && (a.ldo & 3) == 0) {
            if constexpr (sizeof(TOut) == 2) {
              *reinterpret_cast<uint2*>(o) = uint2{pack_bf16x2(v[0], v[1]), pack_bf16x2(v[2], v[3])};
            } else {
              *reinterpret_cast<float4*>(o) = float4{v[0], v[1], v[2], v[3]};
            }
          } else {
#pragma unroll
            for (int e = 0; e < 4; ++e)
              if (n0 + 32 * tn + 16 + 8 * q4 + 4 * h + e < N) o[e] = from_float<TOut>(v[e]);
          }
        }
      } else {
#pragma unroll
        for (int q4 = 0; q4 < 4; ++q4) {
          const int col = n0 + 32 * tn + 8 * q4 + 4 * h;
          TOut* o = out + static_cast<int64_t>(row) * a.ldo + col;
          const float v[4] = {acc[t][tn][4 * q4], acc[t][tn][4 * q4 + 1], acc[t][tn][4 * q4 + 2], acc[t][tn][4 * q4 + 3]};
          if (col + 3 < N && (a.ldo & 3) == 0) {
            if constexpr (sizeof(TOut) == 2) {
              *reinterpret_cast<uint2*>(o) = uint2{pack_bf16x2(v[0], v[1]), pack_bf16x2(v[2], v[3])};
            } else {
              *reinterpret_cast<float4*>(o) = float4{v[0], v[1], v[2], v[3]};
            }
          } else {
#pragma unroll
            for (int e = 0; e < 4; ++e)
              if (col + e < N) o[e] = from_float<TOut>(v[e]);
          }
        }
      }
    }
  }
}

static int g_patch_rows = 8, g_patch_cols = 8;

template <int MT, int TN, int PD, int PX, bool PIPE, int EPI>
int launch_tiles(TilesArgs a, int splits, int out_dtype, hipStream_t s) {
  a.m_blocks = (a.M + 32 * MT - 1) / (32 * MT);
  a.n_blocks = (a.N + 32 * TN * kTlWaves - 1) / (32 * TN * kTlWaves);
  // The workgroups that an XCD runs at one time (numbered one after the other) are a patch of row blocks x column
  // blocks: what they fetch into the XCD's L2 is the patch's rows of X and columns of W, least for a patch about
  // as tall as wide.  Up to g_patch_rows row blocks the patch is one column block's rows, and W is fetched once.
  a.patch_rows = a.m_blocks < g_patch_rows ? a.m_blocks : g_patch_rows;
  a.patch_cols = a.m_blocks > a.patch_rows ? g_patch_cols : 1;
  const long long cols_an_xcd = (a.n_blocks + kTlXcds - 1) / kTlXcds;
  const long long row_groups = (a.m_blocks + a.patch_rows - 1) / a.patch_rows;
  const long long col_groups = (cols_an_xcd + a.patch_cols - 1) / a.patch_cols;
  const long long grid = row_groups * col_groups * a.patch_rows * a.patch_cols * kTlXcds;
  if (grid > 0x7fffffffLL) return static_cast<int>(hipErrorInvalidValue);
  const dim3 blocks(static_cast<unsigned>(grid), static_cast<unsigned>(splits));
  if (out_dtype == kF32)
    gemm_tiles_kernel<MT, TN, PD, PX, PIPE, EPI, float><<<blocks, kTlWaves * kWave, 0, s>>>(a);
  else
    gemm_tiles_kernel<MT, TN, PD, PX, PIPE, EPI, bf16><<<blocks, kTlWaves * kWave, 0, s>>>(a);
  return launch_status();
}

template <int MT, int TN, int PD, int PX, bool PIPE = false>
int dispatch_tiles(const TilesArgs& a, int splits, int out_dtype, int epilogue, hipStream_t s) {
  return epilogue ? launch_tiles<MT, TN, PD, PX, PIPE, kEpiSiluMul>(a, splits, out_dtype, s)
                  : launch_tiles<MT, TN, PD, PX, PIPE, kEpiNone>(a, splits, out_dtype, s);
}

}  // namespace arle

using namespace arle;

// x [M, K] bfloat16 (row stride ldx, a multiple of 8), w_tiles the operand tiles of W [N, K], K % 8 == 0.
// out [M, N] (epilogue 0) or [M, N/2] (epilogue 1: N % 32 == 0, gate and up rows of W interleaved in blocks of 16),
// bfloat16 or float32, row stride ldo.  row_tiles: row tiles of 32 a workgroup (4 or 8); col_tiles: column tiles of
// 32 a wave (2, or 1 with 4 row tiles); depth: ring depths of W and X as two digits (22, 44, 84), + 100 for the loop
// with the barrier in mid-step (8 row tiles only).  splits > 1: K is cut into parts of steps_per_split steps of 32
// (splits of them cover it), and part p leaves its product at out + p * split_stride as float32, no epilogue.
// The patch of workgroups that an XCD runs at one time (for measurements; rows >= 1, cols >= 1).
extern "C" void arle_gemm_tiles_patch(int rows, int cols) {
  if (rows >= 1 && cols >= 1) g_patch_rows = rows, g_patch_cols = cols;
}

extern "C" int arle_gemm_tiles(const void* x, long long ldx, const void* w_tiles, void* out, long long ldo, int out_dtype,
                               int M, int N, int K, int epilogue, int row_tiles, int col_tiles, int depth, int splits,
                               int steps_per_split, long long split_stride, void* stream) {
  if (M <= 0 || N <= 0) return 0;
  if (K <= 0 || K % 8 != 0 || ldx % 8 != 0 || (epilogue != kEpiNone && epilogue != kEpiSiluMul) ||
      (epilogue == kEpiSiluMul && N % 32 != 0) || splits < 1 || splits > 65535 || steps_per_split < 1)
    return static_cast<int>(hipErrorInvalidValue);
  const int steps = (K + 31) / 32;
  if (static_cast<long long>(splits - 1) * steps_per_split >= steps || static_cast<long long>(splits) * steps_per_split < steps)
    return static_cast<int>(hipErrorInvalidValue);
  if (splits > 1 && (out_dtype != kF32 || epilogue != kEpiNone)) return static_cast<int>(hipErrorInvalidValue);
  const TilesArgs a{static_cast<const uint16_t*>(x), ldx, static_cast<const uint16_t*>(w_tiles), out, ldo, M, N, K,
                    0, 0, 0, 0, steps_per_split, split_stride};
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (col_tiles == 2) {
    if (row_tiles == 4 && depth == 22) return dispatch_tiles<4, 2, 2, 2>(a, splits, out_dtype, epilogue, s);
    if (row_tiles == 4 && depth == 44) return dispatch_tiles<4, 2, 4, 4>(a, splits, out_dtype, epilogue, s);
    if (row_tiles == 8 && depth == 44) return dispatch_tiles<8, 2, 4, 4>(a, splits, out_dtype, epilogue, s);
    if (row_tiles == 8 && depth == 144) return dispatch_tiles<8, 2, 4, 4, true>(a, splits, out_dtype, epilogue, s);
  } else if (col_tiles == 1) {
    if (row_tiles == 4 && depth == 44) return dispatch_tiles<4, 1, 4, 4>(a, splits, out_dtype, epilogue, s);
    if (row_tiles == 4 && depth == 84) return dispatch_tiles<4, 1, 8, 4>(a, splits, out_dtype, epilogue, s);
  }
  return static_cast<int>(hipErrorInvalidValue);
}
