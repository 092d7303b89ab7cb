// Paged causal attention on the matrix cores (bfloat16 storage, 32-bit softmax), one
// kernel for prompt portions and for single decoded tokens, plus the merge of split-KV
// partial results.
//
// Work of one wave (a workgroup is one wave of 64 lanes): one segment of the packed
// step (a request's rows), one kv head, 16*NT "rows" and a range of keys.  A row is a
// (token, q head of the kv head's group) pair, row = token * G + head_in_group, so the
// G = nq/nkv q heads that share a kv head share every key and value that is loaded
// (the reference's decode kernel launches one workgroup per q head and reads the keys
// G times: crates/cuda-kernels/tools/tilelang/batch_decode_paged_hd128.py:112-151).
//
// Everything streams from global memory straight into MFMA operands; nothing is staged
// through LDS:
//   S^T[key][row]  = K[key][:] . Q[row][:]      A = K tile (16 keys x 32 d), B = Q (16 rows x 32 d)
//   O^T[d][row]   += V^T[d][key] P^T[key][row]  A = V^T tile (16 d x 32 keys), B = P (16 rows x 32 keys)
// with v_mfma_f32_16x16x32_bf16.  Lane (i = lane%16, g = lane/16) of an operand holds row i and
// 8 contraction elements chosen by g; the result puts element [4g+r][i] into register r of
// lane (i, g).  So after S^T every lane holds, for its own row i, the scores of keys 4g..4g+3
// of each 16-key tile: exactly the 8 keys (two tiles) it must feed as operand B of the second
// product, if the V^T operand lists the keys in the same order.  The value cache is therefore
// laid out [page][kv head][d][slot in page] (d-major), which makes "4 consecutive keys at one d"
// one 8-byte load, as the key cache [page][kv head][slot][d] makes "8 consecutive d of one key"
// one 16-byte load.  Row statistics (running max m, sum l) live in the lanes of their row.
//
// Keys are walked in blocks of 32 aligned to absolute key index.  With splits > 1 the blocks
// of a row range are dealt to `splits` waves, each writing unnormalised float32 partials
// (o, m, l); attn_merge combines them (FlashDecoding, as the reference's split kernels do:
// batch_decode_paged_hd128.py:239-463).  Scores are scaled by scale*log2(e) and exponentiated
// with exp2; probabilities are narrowed to bfloat16 before the second product, as the
// reference does (batch_prefill_paged_hd128.py:219-225); the sum l uses the 32-bit values.
#include "common.h"
#include "attention_static.h"

#include <cstdio>
#include <mutex>

namespace arle {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

struct AttnArgs {
  const uint16_t* q;
  int64_t q_stride;
  uint16_t* out;
  int64_t o_stride;
  float* ws_o;   // [segment * ws_rows + token of the segment][q head][split][D]   (splits > 1)
  float* ws_ml;  // [segment * ws_rows + token of the segment][q head][split][2]
  const uint16_t* k_pages;  // [page][kv head][slot][D]
  const uint16_t* v_pages;  // [page][kv head][D][slot]
  const int* block_table;
  int table_stride;
  const int* seg_row0;   // [segments + 1] first token row of each segment
  const int* seg_slot;   // [segments]
  const int* seg_start;  // [segments] position of a segment's first token
  int nq, nkv, D, P;
  int p_shift;  // log2(P): page sizes are powers of two, so / and % by P are a shift and a mask
  float scale_log2;
  int window;  // 0: all earlier keys
  int splits;
  int ws_rows;   // token rows that the split-KV workspace holds for a segment
  int portion_splits;  // parts into which the LDS kernel cuts the keys of a row block (1: whole; it writes out)
  float* pws_o;        // [token row][q head][part][D]   (portion_splits > 1)
  float* pws_ml;       // [token row][q head][part][2]
  int rows_max;  // the streaming kernel skips segments with more rows than this (0: takes all)
  long long plan_token;  // names the step for the portions kernels' list of work (0: no name, plan every time)
  // The kernel that prepares q, k and v itself (PREP; steps of single decoded tokens): the fused q|k|v projection
  // comes as a stack of float32 partial products [prep_n][token rows][(nq + 2 nkv) D], q is unused.
  const void* prep_parts;   // float32, or with prep_bf16 the projection itself in bfloat16 (prep_n 1)
  int prep_bf16;
  int prep_n;
  int64_t prep_part_stride, prep_row_stride;  // elements between the parts, and between the rows of a part
  const void* prep_qw;   // per-head norm weights [D] of q and k (null: no norm), float32 if prep_w_f32 else bfloat16
  const void* prep_kw;
  int prep_w_f32;
  const float* prep_cos;  // [positions][prep_rot / 2]
  const float* prep_sin;
  int prep_rot;           // rotated width: 0, or a multiple of 64 up to D
  float prep_eps;
  uint16_t* prep_k_pages;  // the pages again, to write the new token's key and value into
  uint16_t* prep_v_pages;
};

__device__ __forceinline__ bf16x8 load_bf16x8(const uint16_t* p) {
  return __builtin_bit_cast(bf16x8, *reinterpret_cast<const uint4*>(p));
}

__device__ __forceinline__ bf16x8 zero_bf16x8() {
  uint4 z = {0u, 0u, 0u, 0u};
  return __builtin_bit_cast(bf16x8, z);
}

__device__ __forceinline__ float group_max4(float v) {  // over the 4 lanes i, i+16, i+32, i+48
  v = fmaxf(v, __shfl_xor(v, 16, kWave));
  return fmaxf(v, __shfl_xor(v, 32, kWave));
}
__device__ __forceinline__ float group_sum4(float v) {
  v += __shfl_xor(v, 16, kWave);
  return v + __shfl_xor(v, 32, kWave);
}

// EXACT: head_dim == DMAX, known at compile time, so every "is this chunk inside the head" test and
// every multiplication by head_dim folds away; otherwise head_dim is any multiple of 16 up to DMAX.
//
// PREP (steps of single decoded tokens, NT == 1, EXACT): the kernel that prepared q, k and v for this one is folded
// into it.  Every wave adds up its q heads from the stack of partial products of the q|k|v projection, norms and
// rotates them (a lane holds d = 32 c + 8 g .. + 7 of its row, c = 0 .. D / 32 - 1: the rotation partner, rot / 2
// away, is in the same lane when rot is a multiple of 64, and the four lanes of a row add their squares together).
// The one wave of a (segment, kv head) whose keys end with the new token's does the same for its k head, takes the
// v head as it is, writes both into the cache and puts them where the loads of the last block would have brought
// them (the slot in the page still holds what was there before).  A layer of a decode step is one kernel shorter.
//
// WHOLE_IN: the projection comes whole, in bfloat16, instead of as a stack of float32 parts.
//
// INWG (NT == 1, up to four splits): the waves of a (segment, kv head) that share its keys are one workgroup, wave s
// takes split s, and at the end wave 0 takes the others' sums and statistics from LDS and writes the result: no
// partial results in memory and no merge kernel.  For launches with a workgroup for every compute unit without it
// (many requests, few splits); with fewer, one-wave workgroups spread the same waves over more compute units.
constexpr int kInWgWavesMax = 4;
template <int NT, int DMAX, bool EXACT, bool PREP = false, bool INWG = false, bool WHOLE_IN = false>
__global__ __launch_bounds__(INWG ? kInWgWavesMax * kWave : kWave) void attn_mfma_kernel(const AttnArgs a) {
  static_assert(!PREP || (NT == 1 && EXACT), "the folded preparation is written for one row tile and a head_dim known here");
  static_assert(!INWG || NT == 1, "the merge inside the workgroup is written for one row tile");
  constexpr int DCH = DMAX / 32;  // contraction chunks of the first product
  constexpr int DTL = DMAX / 16;  // d tiles of the output
  const int lane = threadIdx.x & (kWave - 1), li = lane & 15, g = lane >> 4;
  const int seg = INWG ? static_cast<int>(blockIdx.z) : static_cast<int>(blockIdx.z) / a.splits;
  const int split = INWG ? __builtin_amdgcn_readfirstlane(static_cast<int>(threadIdx.x) >> 6) : static_cast<int>(blockIdx.z) % a.splits;
  const int kvh = blockIdx.y;
  const int G = a.nq / a.nkv;
  const int row0 = a.seg_row0[seg];
  const int qlen = a.seg_row0[seg + 1] - row0;
  const int rows = qlen * G;
  const int row_begin = blockIdx.x * (16 * NT);
  if (row_begin >= rows) return;  // the whole wave leaves
  if (a.rows_max > 0 && rows > a.rows_max) return;  // long segments belong to the LDS kernel
  const int start = a.seg_start[seg];
  const int* table = a.block_table + static_cast<int64_t>(a.seg_slot[seg]) * a.table_stride;
  const int D = EXACT ? DMAX : a.D, P = a.P;
  const int n_dch = EXACT ? DCH : (D + 31) / 32, n_dt = EXACT ? DTL : D / 16;

  const int tok_min = row_begin / G;
  const int tok_max = (min(row_begin + 16 * NT, rows) - 1) / G;
  const int kv_total = start + qlen;       // keys this request holds after the step
  const int kv_hi = start + tok_max + 1;   // exclusive bound of the keys any row here sees
  const int kv_lo = a.window > 0 ? max(0, start + tok_min - a.window + 1) : 0;
  int b0 = kv_lo / 32, b1 = (kv_hi + 31) / 32;
  if (a.splits > 1) {
    const int per = (b1 - b0 + a.splits - 1) / a.splits;
    b0 = b0 + split * per;
    b1 = min(b0 + per, b1);
  }

  // the lane's own row in each row tile
  int my_pos[NT], my_tok[NT], my_head[NT];
  bool row_ok[NT];
  bf16x8 qreg[NT][DCH];
#pragma unroll
  for (int n = 0; n < NT; ++n) {
    const int row = row_begin + 16 * n + li;
    row_ok[n] = row < rows;
    my_tok[n] = min(row / G, qlen - 1);
    my_head[n] = kvh * G + row % G;
    my_pos[n] = start + my_tok[n];
    if constexpr (PREP) continue;  // q is made below
    const uint16_t* qp = a.q + static_cast<int64_t>(row0 + my_tok[n]) * a.q_stride + my_head[n] * D;
#pragma unroll
    for (int c = 0; c < DCH; ++c) {
      // always a load (from a clamped place) and a choice of the value afterwards: a load under a condition
      // would be waited for on the spot, and would leave registers that are sometimes never written
      const int d = 32 * c + 8 * g;
      const bf16x8 got = load_bf16x8(qp + (EXACT ? d : min(d, D - 8)));
      qreg[n][c] = (EXACT || d < D) ? got : zero_bf16x8();
    }
  }

  f32x4 acc[NT][DTL];
  float m[NT], l[NT];
#pragma unroll
  for (int n = 0; n < NT; ++n) {
    m[n] = -INFINITY;
    l[n] = 0.f;
#pragma unroll
    for (int t = 0; t < DTL; ++t) acc[n][t] = f32x4{0.f, 0.f, 0.f, 0.f};
  }

  const int64_t k_head = static_cast<int64_t>(kvh) * P * D;
  const int64_t page_elems = static_cast<int64_t>(a.nkv) * P * D;

  // Page ids of 64 consecutive logical pages sit in one register across the wave (lane i holds
  // page pg_base + i) and are fetched with a cross-lane read, so that the address of a key or value
  // load does not wait for a block-table load first.  Refilled when the walk leaves the window.
  const int pg_last = (kv_hi - 1) >> a.p_shift;
  int pg_base = 0, pg_reg = 0;
  auto refill_pages = [&](int first_page) {
    pg_base = first_page;
    pg_reg = table[min(first_page + lane, pg_last)];
  };
  const int ps = a.p_shift, pm = P - 1;
  auto page_of = [&](int key) { return __shfl(pg_reg, (key >> ps) - pg_base, kWave); };
  auto clamp_key = [&](int key) { return min(max(key, kv_lo), kv_hi - 1); };
  // the blocks blk and blk + 1 are in use at any time: make sure the register covers both
  auto cover = [&](int blk) {
    const int first = clamp_key(blk * 32) >> ps, last = clamp_key(blk * 32 + 63) >> ps;
    if (first < pg_base || last >= pg_base + kWave) refill_pages(first);
  };

  auto load_k = [&](int blk, bf16x8 (&kreg)[2][DCH]) {
#pragma unroll
    for (int t = 0; t < 2; ++t) {
      const int key = clamp_key(blk * 32 + 16 * t + li);  // a held, written key; out-of-range ones are masked below
      const int page = page_of(key);
      const uint16_t* kp = a.k_pages + page * page_elems + k_head + static_cast<int64_t>(key & pm) * D;
#pragma unroll
      for (int c = 0; c < DCH; ++c) {
        const int d = 32 * c + 8 * g;
        const bf16x8 got = load_bf16x8(kp + (EXACT ? d : min(d, D - 8)));
        kreg[t][c] = (EXACT || d < D) ? got : zero_bf16x8();
      }
    }
  };

  // values of a block: for each 16-key tile the 4 keys 4g..4g+3, at d = 16*dt + li
  auto load_v = [&](int blk, u32x4 (&vreg)[DTL]) {
#pragma unroll
    for (int t = 0; t < 2; ++t) {
      int key4 = blk * 32 + 16 * t + 4 * g;
      key4 = min(max(key4, kv_lo & ~3), (kv_hi - 1) & ~3);
      const int page = page_of(key4);
      const uint16_t* vp = a.v_pages + page * page_elems + k_head + (key4 & pm);
#pragma unroll
      for (int dt = 0; dt < DTL; ++dt) {
        const int drow = EXACT ? 16 * dt + li : min(16 * dt + li, D - 1);  // a tile past head_dim reads its last row
        const u32x2 four = *reinterpret_cast<const u32x2*>(vp + static_cast<int64_t>(drow) * P);
        vreg[dt][2 * t] = four[0];
        vreg[dt][2 * t + 1] = four[1];
      }
    }
  };

  bf16x8 kcur[2][DCH];
  u32x4 vraw[DTL];  // the second product's operand for each d tile: keys 4g..4g+3 of both 16-key tiles
  if (b0 < b1) refill_pages(clamp_key(b0 * 32) >> ps);

  // PREP: q of this lane's row, and in the wave whose keys end with the new token's (`owner`) that token's key as
  // the lanes (any i, g) of a key operand hold it and its value at d = 16 dt + i.  Loads of one kind go out together
  // (a missing part of the stack is fetched from the last one and not added: a load under a condition would be
  // waited for on the spot); the arithmetic of q runs while the first keys and values of
  // the cache and the stack's k and v are on their way.
  [[maybe_unused]] bf16x8 knew[DCH];
  [[maybe_unused]] uint32_t vnew[DTL];
  [[maybe_unused]] const int last_blk = (kv_hi + 31) / 32 - 1;
  [[maybe_unused]] const bool owner = PREP && b0 <= last_blk && last_blk < b1;  // the same in all lanes
  if constexpr (PREP) {
    constexpr int HC = DCH / 2;                 // chunks of 32 columns that half of a head holds
    const int hc = a.prep_rot / 64;             // and that half of the rotated width holds
    // the segment's one token: element `index` of its row (float32 parts, or one bfloat16 row) at spot(index)
    const int elem = WHOLE_IN ? 2 : 4;
    const unsigned char* prow = static_cast<const unsigned char*>(a.prep_parts) + static_cast<int64_t>(row0) * a.prep_row_stride * elem;
    auto spot = [&](int64_t index) { return prow + index * elem; };
    const unsigned char* somewhere = reinterpret_cast<const unsigned char*>(a.k_pages);   // a page: 512 bytes at least
    const int n_parts = a.prep_n;
    // Every load of this prologue is issued without a condition around it (a load under a condition is waited for at
    // the end of its branch, and the loads behind it wait with it): what is not needed is fetched from a place
    // that exists and dropped.
    //
    // The parts of the stack are spread over lanes that would otherwise fetch the same thing, so that a head's parts
    // are all on their way at once: lane i of a q head's row takes the parts i / gp, i / gp + 16 / gp, ... (gp: the
    // group's heads rounded up to a power of two; rows past the group are copies), the lanes i of the k head the
    // parts i % kp, i % kp + kp, ..., the four lanes g of a value the parts g % vp, g % vp + vp, ...  A lane adds
    // its parts in ascending order; the lanes' sums then meet pairwise, the lanes 8, 4, 2, 1 apart in turn (rotations
    // of the 16 lanes i), which leaves every lane that holds the head with the same total: one fixed order, whatever
    // else the step holds.
    // (two loads of 16 bytes a chunk either way: the second one of a bfloat16 row is the first one again; what
    // they brought is only looked at where it is added, so that no load waits for the one before it)
    auto fetch_part = [&](int col0, int u, uint4 (&got)[DCH][2]) {
      const int64_t first = col0 + 8 * g + static_cast<int64_t>(min(u, n_parts - 1)) * a.prep_part_stride;
#pragma unroll
      for (int c = 0; c < DCH; ++c) {
        const unsigned char* at = spot(first + 32 * c);
        got[c][0] = *reinterpret_cast<const uint4*>(at);
        got[c][1] = *reinterpret_cast<const uint4*>(at + (WHOLE_IN ? 0 : 16));
      }
    };
    auto value_of = [&](const uint4 (&got)[DCH][2], int c, int e) {   // c, e are constants where this is called
      const uint32_t wl[4] = {got[c][0].x, got[c][0].y, got[c][0].z, got[c][0].w};
      const uint32_t wh[4] = {got[c][1].x, got[c][1].y, got[c][1].z, got[c][1].w};
      const uint32_t pair = wl[e >> 1];
      const uint32_t narrow = (e & 1) ? pair & 0xffff0000u : pair << 16;
      return __uint_as_float(WHOLE_IN ? narrow : (e < 4 ? wl[e & 3] : wh[e & 3]));
    };
    // one column of the token's row (a value): a load of four bytes either way, sorted out by one_of
    auto fetch_one = [&](int64_t index) {
      return *reinterpret_cast<const uint32_t*>(reinterpret_cast<uintptr_t>(spot(index)) & ~static_cast<uintptr_t>(3));
    };
    auto one_of = [&](uint32_t raw, int64_t index) {
      const uint32_t narrow = (index & 1) ? raw & 0xffff0000u : raw << 16;   // rows begin at multiples of eight elements
      return __uint_as_float(WHOLE_IN ? narrow : raw);
    };
    // x = the lane's parts added up (the first round's loads are `got`); mine, apart: the lane's first part and the
    // distance to its next
    auto add_parts = [&](int col0, int mine, int apart, uint4 (&got)[DCH][2], float (&x)[DCH][8]) {
#pragma unroll
      for (int c = 0; c < DCH; ++c)
#pragma unroll
        for (int e = 0; e < 8; ++e) x[c][e] = 0.f;
      for (int base = 0; base < n_parts; base += apart) {   // the same number of rounds in all lanes
        const int u = base + mine;
        if (base > 0) fetch_part(col0, u, got);
        const bool there = u < n_parts;
#pragma unroll
        for (int c = 0; c < DCH; ++c)
#pragma unroll
          for (int e = 0; e < 8; ++e) x[c][e] += there ? value_of(got, c, e) : 0.f;
      }
    };
    // x += x of the lane `n` to the side in the row of 16 lanes i (a rotation: row_ror)
#define ARLE_MEET(CTRL)                                                                                              \
  _Pragma("unroll") for (int c = 0; c < DCH; ++c) _Pragma("unroll") for (int e = 0; e < 8; ++e)                         \
      x[c][e] += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x[c][e]), CTRL, 0xf, 0xf, false))
    auto meet = [&](float (&x)[DCH][8], int from, int to) {   // the lanes from, from / 2, ..., to apart
      if (from >= 8 && to <= 8) { ARLE_MEET(0x128); }
      if (from >= 4 && to <= 4) { ARLE_MEET(0x124); }
      if (from >= 2 && to <= 2) { ARLE_MEET(0x122); }
      if (from >= 1 && to <= 1) { ARLE_MEET(0x121); }
    };
#undef ARLE_MEET
    // a head's norm weights as this lane holds the head, bfloat16 or float32 in memory: two loads of 16 bytes either
    // way (the second one of bfloat16 weights is the first one again), sorted out afterwards
    auto fetch_weights = [&](const void* w, uint4 (&raw)[DCH][2]) {
      const unsigned char* base = w != nullptr ? static_cast<const unsigned char*>(w) : somewhere;
      const int w_elem = a.prep_w_f32 ? 4 : 2;
#pragma unroll
      for (int c = 0; c < DCH; ++c) {
        const unsigned char* at = base + static_cast<size_t>(32 * c + 8 * g) * w_elem;
        raw[c][0] = *reinterpret_cast<const uint4*>(at);
        raw[c][1] = *reinterpret_cast<const uint4*>(at + (a.prep_w_f32 ? 16 : 0));
      }
    };
    auto weight_of = [&](const uint4 (&raw)[DCH][2], int c, int e) {   // e is a constant where this is called
      const uint32_t lo[4] = {raw[c][0].x, raw[c][0].y, raw[c][0].z, raw[c][0].w};
      const uint32_t hi[4] = {raw[c][1].x, raw[c][1].y, raw[c][1].z, raw[c][1].w};
      const float wide = __uint_as_float(e < 4 ? lo[e & 3] : hi[e & 3]);
      const uint32_t pair = lo[e >> 1];
      const float narrow = __uint_as_float((e & 1) ? pair & 0xffff0000u : pair << 16);
      return a.prep_w_f32 ? wide : narrow;
    };
    // the angles of the token's position, for the chunks of half of the rotated width
    float cs[HC > 0 ? HC : 1][8], sn[HC > 0 ? HC : 1][8];
    {
      const bool turns = hc > 0;
      const float* ct = turns ? a.prep_cos + static_cast<int64_t>(start) * (a.prep_rot / 2) : reinterpret_cast<const float*>(somewhere);
      const float* st = turns ? a.prep_sin + static_cast<int64_t>(start) * (a.prep_rot / 2) : reinterpret_cast<const float*>(somewhere);
#pragma unroll
      for (int c = 0; c < HC; ++c) {
        const int at = 32 * min(c, max(hc - 1, 0)) + 8 * g;
        const float4 c0 = *reinterpret_cast<const float4*>(ct + at), c1 = *reinterpret_cast<const float4*>(ct + at + 4);
        const float4 s0 = *reinterpret_cast<const float4*>(st + at), s1 = *reinterpret_cast<const float4*>(st + at + 4);
        cs[c][0] = c0.x, cs[c][1] = c0.y, cs[c][2] = c0.z, cs[c][3] = c0.w, cs[c][4] = c1.x, cs[c][5] = c1.y, cs[c][6] = c1.z, cs[c][7] = c1.w;
        sn[c][0] = s0.x, sn[c][1] = s0.y, sn[c][2] = s0.z, sn[c][3] = s0.w, sn[c][4] = s1.x, sn[c][5] = s1.y, sn[c][6] = s1.z, sn[c][7] = s1.w;
      }
    }
    // one head as this lane's part of an operand: norm, rotation, bfloat16
    auto finish_head = [&](float (&x)[DCH][8], bool normed, const uint4 (&wraw)[DCH][2], bf16x8 (&dst)[DCH]) {
      if (normed) {
        float ss = 0.f;
#pragma unroll
        for (int c = 0; c < DCH; ++c)
#pragma unroll
          for (int e = 0; e < 8; ++e) ss += x[c][e] * x[c][e];
        ss = group_sum4(ss);
        const float inv = 1.0f / sqrtf(ss / static_cast<float>(DMAX) + a.prep_eps);
#pragma unroll
        for (int c = 0; c < DCH; ++c)
#pragma unroll
          for (int e = 0; e < 8; ++e) x[c][e] = x[c][e] * inv * weight_of(wraw, c, e);
      }
      // d < rot / 2 turns with d + rot / 2, hc chunks up in the same lane.  The chunk numbers are written out for
      // each rotated width that there is (indexed by hc, the arrays would leave the registers).
      auto turn = [&](float (&lo)[8], float (&hi)[8], const float (&c)[8], const float (&s_)[8]) {
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          const float l_ = lo[e], h_ = hi[e];
          lo[e] = l_ * c[e] - h_ * s_[e];
          hi[e] = l_ * s_[e] + h_ * c[e];
        }
      };
      if (hc == HC) {
#pragma unroll
        for (int c = 0; c < HC; ++c) turn(x[c], x[c + HC], cs[c], sn[c]);
      } else if (hc > 0) {
        if constexpr (HC == 2) turn(x[0], x[1], cs[0], sn[0]);   // half of a head of 128 is rotated: hc == 1
      }
#pragma unroll
      for (int c = 0; c < DCH; ++c) {
        uint4 pk;
        pk.x = pack_bf16x2(x[c][0], x[c][1]);
        pk.y = pack_bf16x2(x[c][2], x[c][3]);
        pk.z = pack_bf16x2(x[c][4], x[c][5]);
        pk.w = pack_bf16x2(x[c][6], x[c][7]);
        dst[c] = __builtin_bit_cast(bf16x8, pk);
      }
    };
    int gp = 1;
    while (gp < G) gp <<= 1;                                   // G <= 16
    int kp = 1, vp = 1;                  // lanes i (lanes g) that share the key's (the value's) parts
    while (kp < n_parts && kp < 16) kp <<= 1;
    while (vp < n_parts && vp < 4) vp <<= 1;
    const int q_col = (kvh * G + min(li & (gp - 1), G - 1)) * DMAX;    // live rows (i < G) take their own head
    const int k_col = (a.nq + kvh) * DMAX;
    const int v_mine = g & (vp - 1);
    const int64_t v_col = static_cast<int64_t>(a.nq + a.nkv + kvh) * DMAX + li;
    float xq[DCH][8];
    uint4 gq[DCH][2], wq[DCH][2];
    fetch_weights(a.prep_qw, wq);
    fetch_part(q_col, li / gp, gq);
    if (b0 < b1) {   // the first keys and values of the cache
      load_k(b0, kcur);
      load_v(b0, vraw);
    }
    // the owner's key and value: behind the cache's loads, and waited for behind the arithmetic of q
    [[maybe_unused]] uint4 gk[DCH][2], wk[DCH][2];
    [[maybe_unused]] uint32_t vgot[DTL];
    if (owner) {
      fetch_weights(a.prep_kw, wk);
      fetch_part(k_col, li & (kp - 1), gk);
#pragma unroll
      for (int dt = 0; dt < DTL; ++dt) vgot[dt] = fetch_one(v_col + static_cast<int64_t>(min(v_mine, n_parts - 1)) * a.prep_part_stride + 16 * dt);
    }
    add_parts(q_col, li / gp, 16 / gp, gq, xq);
    if (n_parts > 1) meet(xq, 8, gp);
    finish_head(xq, a.prep_qw != nullptr, wq, qreg[0]);
    if (owner) {
      float xk[DCH][8], vsum[DTL];
      add_parts(k_col, li & (kp - 1), kp, gk, xk);
      meet(xk, kp / 2, 1);
#pragma unroll
      for (int dt = 0; dt < DTL; ++dt) vsum[dt] = v_mine < n_parts ? one_of(vgot[dt], v_col + 16 * dt) : 0.f;
      for (int base = vp; base < n_parts; base += vp) {
        const int u = base + v_mine;
#pragma unroll
        for (int dt = 0; dt < DTL; ++dt) vgot[dt] = fetch_one(v_col + static_cast<int64_t>(min(u, n_parts - 1)) * a.prep_part_stride + 16 * dt);
#pragma unroll
        for (int dt = 0; dt < DTL; ++dt) vsum[dt] += u < n_parts ? one_of(vgot[dt], v_col + 16 * dt) : 0.f;
      }
      if (vp > 1) {
        float far[DTL];
#pragma unroll
        for (int dt = 0; dt < DTL; ++dt) far[dt] = __shfl_xor(vsum[dt], 16, kWave);
#pragma unroll
        for (int dt = 0; dt < DTL; ++dt) vsum[dt] += far[dt];
      }
      if (vp > 2) {
        float far[DTL];
#pragma unroll
        for (int dt = 0; dt < DTL; ++dt) far[dt] = __shfl_xor(vsum[dt], 32, kWave);
#pragma unroll
        for (int dt = 0; dt < DTL; ++dt) vsum[dt] += far[dt];
      }
      finish_head(xk, a.prep_kw != nullptr, wk, knew);
#pragma unroll
      for (int dt = 0; dt < DTL; ++dt) vnew[dt] = f32_to_bf16_bits(vsum[dt]);
    }
  } else if (b0 < b1) {
    load_k(b0, kcur);
    load_v(b0, vraw);
  }

  for (int blk = b0; blk < b1; ++blk) {
    const int key_base = blk * 32;
    const bool more = blk + 1 < b1;
    if (more) cover(blk + 1);
    if constexpr (PREP) {
      if (owner && blk == last_blk && li == (start & 15)) {   // the new token's key, where the load brought the slot's old bits
#pragma unroll
        for (int t = 0; t < 2; ++t)
          if (t == ((start >> 4) & 1)) {
#pragma unroll
            for (int c = 0; c < DCH; ++c) kcur[t][c] = knew[c];
          }
      }
    }

    // scores S^T: s[n][t][r] belongs to key key_base + 16t + 4g + r and row (n, li)
    f32x4 s[NT][2];
#pragma unroll
    for (int n = 0; n < NT; ++n)
#pragma unroll
      for (int t = 0; t < 2; ++t) {
        f32x4 z = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int c = 0; c < DCH; ++c)
          if (EXACT || c < n_dch) z = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kcur[t][c], qreg[n][c], z, 0, 0, 0);
        s[n][t] = z;
      }
    // the key registers are free again: fetch the next block's keys while this block goes on
    if (more) load_k(blk + 1, kcur);

    // a key beyond what the request holds may carry stale bits: its value must be 0, not 0 * garbage
    if (key_base + 32 > kv_total) {
#pragma unroll
      for (int t = 0; t < 2; ++t) {
        const int key4 = key_base + 16 * t + 4 * g;
#pragma unroll
        for (int dt = 0; dt < DTL; ++dt) {
          if (!EXACT && dt >= n_dt) continue;
          if (key4 + 0 >= kv_total) vraw[dt][2 * t] &= 0xffff0000u;
          if (key4 + 1 >= kv_total) vraw[dt][2 * t] &= 0x0000ffffu;
          if (key4 + 2 >= kv_total) vraw[dt][2 * t + 1] &= 0xffff0000u;
          if (key4 + 3 >= kv_total) vraw[dt][2 * t + 1] &= 0x0000ffffu;
        }
      }
    }

    if constexpr (PREP) {
      if (owner && blk == last_blk && g == ((start & 15) >> 2)) {   // and its value, one half of a register
        const int word = 2 * ((start >> 4) & 1) + ((start & 3) >> 1);
        const bool upper = (start & 1) != 0;
#pragma unroll
        for (int dt = 0; dt < DTL; ++dt)
#pragma unroll
          for (int w = 0; w < 4; ++w)
            if (w == word)
              vraw[dt][w] = upper ? (vraw[dt][w] & 0x0000ffffu) | (vnew[dt] << 16) : (vraw[dt][w] & 0xffff0000u) | vnew[dt];
      }
    }

    bf16x8 pb[NT];
#pragma unroll
    for (int n = 0; n < NT; ++n) {
      const int lo = a.window > 0 ? my_pos[n] - a.window + 1 : 0;
      float sv[2][4];
      float bmax = -INFINITY;
#pragma unroll
      for (int t = 0; t < 2; ++t)
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          const int key = key_base + 16 * t + 4 * g + r;
          const bool ok = key >= lo && key <= my_pos[n];
          sv[t][r] = ok ? s[n][t][r] * a.scale_log2 : -INFINITY;
          bmax = fmaxf(bmax, sv[t][r]);
        }
      bmax = group_max4(bmax);
      const float m_new = fmaxf(m[n], bmax);
      const float m_use = m_new == -INFINITY ? 0.f : m_new;  // a row that has seen no key yet
      const float alpha = exp2f(m[n] - m_use);
      float psum = 0.f;
      uint32_t packed[4];
#pragma unroll
      for (int t = 0; t < 2; ++t)
#pragma unroll
        for (int r = 0; r < 4; r += 2) {
          const float p0 = exp2f(sv[t][r] - m_use), p1 = exp2f(sv[t][r + 1] - m_use);
          psum += p0 + p1;
          packed[2 * t + r / 2] = pack_bf16x2(p0, p1);
        }
      psum = group_sum4(psum);
      l[n] = l[n] * alpha + psum;
      m[n] = m_new;
#pragma unroll
      for (int dt = 0; dt < DTL; ++dt) {
        acc[n][dt][0] *= alpha;
        acc[n][dt][1] *= alpha;
        acc[n][dt][2] *= alpha;
        acc[n][dt][3] *= alpha;
      }
      uint4 pk = {packed[0], packed[1], packed[2], packed[3]};
      pb[n] = __builtin_bit_cast(bf16x8, pk);
    }

#pragma unroll
    for (int dt = 0; dt < DTL; ++dt) {
      if (EXACT || dt < n_dt) {
        const bf16x8 vop = __builtin_bit_cast(bf16x8, vraw[dt]);
#pragma unroll
        for (int n = 0; n < NT; ++n)
          acc[n][dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vop, pb[n], acc[n][dt], 0, 0, 0);
      }
    }
    // and the value registers after the second product
    if (more) load_v(blk + 1, vraw);
  }

  if constexpr (PREP) {
    // the new token's key and value go into the cache (their page is among those that the last block had in reach)
    if (owner && a.prep_k_pages != nullptr) {
      const int page = page_of(start);
      const int64_t at = page * page_elems + k_head;
      const int in_page = start & pm;
      if (li == 0) {
#pragma unroll
        for (int c = 0; c < DCH; ++c)
          *reinterpret_cast<uint4*>(a.prep_k_pages + at + static_cast<int64_t>(in_page) * DMAX + 32 * c + 8 * g) =
              __builtin_bit_cast(uint4, knew[c]);
      }
      if (g == 0) {
#pragma unroll
        for (int dt = 0; dt < DTL; ++dt)
          a.prep_v_pages[at + static_cast<int64_t>(16 * dt + li) * P + in_page] = static_cast<uint16_t>(vnew[dt]);
      }
    }
  }

  if constexpr (INWG) {
    // the waves 1 .. splits - 1 hand their sums to wave 0, lane to lane (a lane holds the same rows and columns in
    // every wave): out = sum_s o_s 2^(m_s - m) / sum_s l_s 2^(m_s - m), added in the order of the splits
    constexpr int kPitch = 4 * DTL + 4;   // floats a lane: its sums, m and l, and padding to 16 bytes
    __shared__ __align__(16) float handed[kInWgWavesMax - 1][kWave][kPitch];
    if (split > 0) {
      float* mine = handed[split - 1][lane];
#pragma unroll
      for (int dt = 0; dt < DTL; ++dt)
        *reinterpret_cast<float4*>(mine + 4 * dt) = float4{acc[0][dt][0], acc[0][dt][1], acc[0][dt][2], acc[0][dt][3]};
      *reinterpret_cast<float2*>(mine + 4 * DTL) = float2{m[0], l[0]};
    }
    __syncthreads();
    if (split > 0) return;
    for (int w = 1; w < a.splits; ++w) {
      const float* theirs = handed[w - 1][lane];
      const float2 ml = *reinterpret_cast<const float2*>(theirs + 4 * DTL);
      const float m_all = fmaxf(m[0], ml.x);
      const float m_ref = m_all == -INFINITY ? 0.f : m_all;
      const float f0 = exp2f(m[0] - m_ref), f1 = exp2f(ml.x - m_ref);
      l[0] = l[0] * f0 + ml.y * f1;
      m[0] = m_all;
#pragma unroll
      for (int dt = 0; dt < DTL; ++dt) {
        const float4 v = *reinterpret_cast<const float4*>(theirs + 4 * dt);
        acc[0][dt][0] = acc[0][dt][0] * f0 + v.x * f1;
        acc[0][dt][1] = acc[0][dt][1] * f0 + v.y * f1;
        acc[0][dt][2] = acc[0][dt][2] * f0 + v.z * f1;
        acc[0][dt][3] = acc[0][dt][3] * f0 + v.w * f1;
      }
    }
  }

  // acc[n][dt][r] is O^T[d = 16dt + 4g + r][row (n, li)]
#pragma unroll
  for (int n = 0; n < NT; ++n) {
    if (!row_ok[n]) continue;
    const int64_t tok_row = row0 + my_tok[n];
    if (INWG || a.splits == 1) {
      const float inv_l = l[n] > 0.f ? 1.0f / l[n] : 0.f;
      uint16_t* op = a.out + tok_row * a.o_stride + my_head[n] * D;
#pragma unroll
      for (int dt = 0; dt < DTL; ++dt) {
        if (EXACT || dt < n_dt) {
          uint2 w;
          w.x = static_cast<uint32_t>(f32_to_bf16_bits(acc[n][dt][0] * inv_l)) |
                (static_cast<uint32_t>(f32_to_bf16_bits(acc[n][dt][1] * inv_l)) << 16);
          w.y = static_cast<uint32_t>(f32_to_bf16_bits(acc[n][dt][2] * inv_l)) |
                (static_cast<uint32_t>(f32_to_bf16_bits(acc[n][dt][3] * inv_l)) << 16);
          *reinterpret_cast<uint2*>(op + 16 * dt + 4 * g) = w;
        }
      }
    } else {
      const int64_t ws_row = static_cast<int64_t>(seg) * a.ws_rows + my_tok[n];
      const int64_t slot = (ws_row * a.nq + my_head[n]) * a.splits + split;
      float* wo = a.ws_o + slot * D;
#pragma unroll
      for (int dt = 0; dt < DTL; ++dt) {
        if (EXACT || dt < n_dt) {
          float4 w = {acc[n][dt][0], acc[n][dt][1], acc[n][dt][2], acc[n][dt][3]};
          *reinterpret_cast<float4*>(wo + 16 * dt + 4 * g) = w;
        }
      }
      if (g == 0) {
        a.ws_ml[slot * 2] = m[n];
        a.ws_ml[slot * 2 + 1] = l[n];
      }
    }
  }
}

// out[row][head][:] = sum_s o_s 2^(m_s - m) / sum_s l_s 2^(m_s - m).   One workgroup of four waves
// per (workspace row, head); a workspace row is (segment, token of the segment), and rows past a segment's
// length or of a segment that the streaming kernel left to the LDS kernel are skipped.  Lane s of every wave holds the statistics of split s (splits <= 64) and the
// weights travel by cross-lane reads; wave w adds the splits s = w, w+4, ... with all its loads
// independent of one another, and the four partial sums meet in LDS in wave order.
constexpr int kMergeWaves = 4;
constexpr int kMergeMaxD = 256;
__global__ __launch_bounds__(kMergeWaves* kWave) void attn_merge_kernel(
    const float* __restrict__ ws_o, const float* __restrict__ ws_ml, uint16_t* __restrict__ out,
    int64_t o_stride, const int* __restrict__ seg_row0, int ws_rows, int rows_max, int nq, int nkv, int D,
    int splits) {
  __shared__ float part[kMergeWaves][kMergeMaxD];
  const int head = blockIdx.y;
  const int seg = blockIdx.x / ws_rows, tok = blockIdx.x % ws_rows;
  const int first = seg_row0[seg], qlen = seg_row0[seg + 1] - first;
  if (tok >= qlen || (rows_max > 0 && qlen * (nq / nkv) > rows_max)) return;  // the whole workgroup leaves
  const int row = first + tok;
  const int lane = threadIdx.x % kWave, wave = threadIdx.x / kWave;
  const int64_t base = (static_cast<int64_t>(blockIdx.x) * nq + head) * splits;
  float ms = -INFINITY, ls = 0.f;
  if (lane < splits) {
    const float2 ml = *reinterpret_cast<const float2*>(ws_ml + (base + lane) * 2);
    ms = ml.x;
    ls = ml.y;
  }
  const float mx = wave_max(ms);
  const float wgt = ms > -INFINITY ? exp2f(ms - mx) : 0.f;  // an empty split weighs nothing
  const float denom = wave_sum(ls * wgt);
  const float inv = denom > 0.f ? 1.0f / denom : 0.f;
  // each lane owns d = 4*lane .. 4*lane+3 (D <= 256)
  const int d0 = 4 * lane;
  float4 o = {0.f, 0.f, 0.f, 0.f};
  const bool mine = d0 < D;
  const float* src = ws_o + base * D + (mine ? d0 : 0);
  // rounds of four splits a wave, their loads without a condition (a split past the last one is fetched from the
  // last and weighs nothing): in a loop of single splits every load was waited for before the next one went out
  constexpr int kRound = 4;
  for (int s0 = wave; s0 < splits; s0 += kRound * kMergeWaves) {
    float4 v[kRound];
    float w[kRound];
#pragma unroll
    for (int j = 0; j < kRound; ++j) {
      const int sj = s0 + j * kMergeWaves, sc = min(sj, splits - 1);
      v[j] = *reinterpret_cast<const float4*>(src + static_cast<int64_t>(sc) * D);
      const float got = __shfl(wgt, sc, kWave);  // every lane takes part in the cross-lane read
      w[j] = sj < splits ? got : 0.f;
    }
#pragma unroll
    for (int j = 0; j < kRound; ++j) {
      o.x += v[j].x * w[j];
      o.y += v[j].y * w[j];
      o.z += v[j].z * w[j];
      o.w += v[j].w * w[j];
    }
  }
  if (mine) *reinterpret_cast<float4*>(&part[wave][d0]) = o;
  __syncthreads();
  if (wave == 0 && d0 < D) {
#pragma unroll
    for (int v = 1; v < kMergeWaves; ++v) {
      const float4 p = *reinterpret_cast<const float4*>(&part[v][d0]);
      o.x += p.x;
      o.y += p.y;
      o.z += p.z;
      o.w += p.w;
    }
    uint2 w;
    w.x = static_cast<uint32_t>(f32_to_bf16_bits(o.x * inv)) | (static_cast<uint32_t>(f32_to_bf16_bits(o.y * inv)) << 16);
    w.y = static_cast<uint32_t>(f32_to_bf16_bits(o.z * inv)) | (static_cast<uint32_t>(f32_to_bf16_bits(o.w * inv)) << 16);
    *reinterpret_cast<uint2*>(out + static_cast<int64_t>(row) * o_stride + head * D + d0) = w;
  }
}

// ---------------------------------------------------------------------------------------------
// Prompt portions: the same products, with keys and values staged through LDS.
//
// A workgroup of eight waves owns 128 rows (16 per wave) of one segment and kv head
// and walks the keys in tiles of 64.  All 256 threads fetch a tile with coalesced loads (a key page
// [slot][d] and a value page [d][slot] are contiguous in memory), park it in LDS, and every wave
// reads its MFMA operands from there, so a key or value is read from L2 once per 128 rows instead
// of once per 16.  Two LDS stages: tile i+1 is on its way from memory while tile i is computed.
constexpr int kPfWaves = 8;
constexpr int kPfNT = 1;                          // row tiles of 16 a wave
constexpr int kPfRows = 16 * kPfNT * kPfWaves;    // rows of a workgroup
constexpr int kPfKeys = 64;             // keys of a tile
constexpr int kPfVPad = 4;              // padding of a value row in LDS: 34 dwords a row, so that the 16 rows which
                                        // 16 lanes read or write together (8 bytes each) fall into 16 different bank pairs

// Work is handed out by the item (row block, kv head, segment, part of the keys).  A causal prompt is a triangle:
// the last 128 rows of a segment see 32 times the keys of the first 128, and row blocks assigned to workgroups by
// their number alone leave most of the chip idle while the heaviest ones finish.  So the launch has one or two
// workgroups per CU and the items are listed from the heaviest to the lightest.  Either every workgroup takes the
// next item from a counter until none is left (the counter is a device variable of this module, put to zero by the
// planning kernel and again by the last workgroup that leaves a launch), or, in the kernel that loads tiles straight
// into LDS, the list is dealt out to and fro over the workgroups before the launch (its launcher says when).
// Launches of these kernels on one device must not overlap (they never do on one stream).
//
// The planning kernel (one workgroup) lists the live (row block, segment) pairs in that order: a step
// that mixes a few portions with many decoded tokens has far more pairs that are dead (segments left to the
// other kernel, row blocks past a short segment's end) than live ones, and asking for an item only to drop it
// costs a round trip to the counter each time.  Steps with more pairs than the list holds go without it.
constexpr int kPfPlanMax = 16384;
__device__ unsigned int g_prefill_next_item;
__device__ unsigned int g_prefill_left;               // workgroups of the running launch that have found the list empty
__device__ unsigned int g_prefill_pairs;              // entries of g_prefill_plan
__device__ unsigned int g_prefill_plan[kPfPlanMax];   // (row block << 16) | segment
__device__ int4 g_prefill_seg[kPfPlanMax];            // the entry's segment: first row, rows, first position, table row

__global__ __launch_bounds__(256) void attn_prefill_plan_kernel(const int* __restrict__ seg_row0,
                                                                 const int* __restrict__ seg_start,
                                                                 const int* __restrict__ seg_slot, int segments,
                                                                 int blocks_x, int G, int min_rows, int listed) {
  // The list is ordered by what an entry costs, the tiles of 64 keys that its rows see, heaviest first (a counting
  // sort over that number; entries of one cost in the order their atomics land, which no result depends on):
  // whether the entries are taken from a counter or dealt out to and fro, the heavy ones start first and the
  // light ones fill up.
  constexpr int kBuckets = 2048;  // tiles of 64 keys; longer contexts share the last one
  __shared__ unsigned int bucket[kBuckets];
  __shared__ unsigned int sums[256];
  const int tid = threadIdx.x;
  if (tid == 0) {
    g_prefill_next_item = 0u;
    g_prefill_left = 0u;
  }
  if (!listed) return;  // the whole workgroup
  for (int b = tid; b < kBuckets; b += 256) bucket[b] = 0u;
  __syncthreads();
  const int total = blocks_x * segments;
  auto look = [&](int i, unsigned int& entry, int4& of_seg, int& cost) {
    const int seg = i % segments, rb = blocks_x - 1 - i / segments;
    const int row0 = seg_row0[seg], qlen = seg_row0[seg + 1] - row0;
    const int rows = qlen * G;
    if (rows < min_rows || rb * kPfRows >= rows) return false;
    entry = (static_cast<unsigned int>(rb) << 16) | static_cast<unsigned int>(seg);
    // what a workgroup needs to know of the segment, beside the entry: one load instead of a chain of them
    const int start = seg_start[seg];
    of_seg = int4{row0, qlen, start, seg_slot[seg]};
    const int tok_max = (min((rb + 1) * kPfRows, rows) - 1) / G;
    cost = min((start + tok_max + 1 + 63) / 64, kBuckets - 1);
    return true;
  };
  for (int i = tid; i < total; i += 256) {
    unsigned int entry;
    int4 of_seg;
    int cost;
    if (look(i, entry, of_seg, cost)) atomicAdd(&bucket[kBuckets - 1 - cost], 1u);   // heaviest first
  }
  __syncthreads();
  // where each bucket begins: a thread adds up its eight buckets, thread 0 the 256 sums
  constexpr int kMine = kBuckets / 256;
  unsigned int mine = 0u;
  for (int e = 0; e < kMine; ++e) mine += bucket[tid * kMine + e];
  sums[tid] = mine;
  __syncthreads();
  if (tid == 0) {
    unsigned int run = 0u;
    for (int t = 0; t < 256; ++t) {
      const unsigned int n = sums[t];
      sums[t] = run;
      run += n;
    }
    g_prefill_pairs = run;
  }
  __syncthreads();
  unsigned int at = sums[tid];
  for (int e = 0; e < kMine; ++e) {
    const unsigned int n = bucket[tid * kMine + e];
    bucket[tid * kMine + e] = at;
    at += n;
  }
  __syncthreads();
  for (int i = tid; i < total; i += 256) {
    unsigned int entry;
    int4 of_seg;
    int cost;
    if (look(i, entry, of_seg, cost)) {
      const unsigned int place = atomicAdd(&bucket[kBuckets - 1 - cost], 1u);
      g_prefill_plan[place] = entry;
      g_prefill_seg[place] = of_seg;
    }
  }
}

// One workgroup a CU: two waves on every SIMD, each with the registers it wants (16 rows a wave keep the
// pieces of the next tile in registers beside the accumulators; with 32 rows they are spilled, and a spilled
// load is waited for at once).  The staging registers are plain vector types on purpose: arrays of HIP's
// uint4/uint2 structs went through scratch memory here.
template <int DMAX, bool EXACT>
__global__ __launch_bounds__(kPfWaves* kWave, 1) __attribute__((amdgpu_waves_per_eu(2, 2))) void attn_prefill_lds_kernel(const AttnArgs a, int min_rows,
                                                                                         int blocks_x, int segments, int listed,
                                                                                         int fixed_rounds) {
  constexpr int NT = kPfNT;
  constexpr int DCH = DMAX / 32, DTL = DMAX / 16;
  constexpr int kKPieces = (kPfKeys * (DMAX / 8) + kPfWaves * kWave - 1) / (kPfWaves * kWave);  // 16-byte pieces per thread
  constexpr int kVPieces = (kPfKeys / 4 * DMAX + kPfWaves * kWave - 1) / (kPfWaves * kWave);    // 8-byte pieces per thread
  extern __shared__ __align__(16) unsigned char lds_raw[];
  __shared__ unsigned int item_of_workgroup;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, li = lane & 15, g = lane >> 4;
  const int G = a.nq / a.nkv;
  const unsigned int nkv = static_cast<unsigned int>(a.nkv);
  const unsigned int pairs = listed ? g_prefill_pairs : static_cast<unsigned int>(blocks_x) * segments;
  const unsigned int parts = static_cast<unsigned int>(a.portion_splits);
  const unsigned int items = pairs * nkv * parts;
 // Items dealt out before the launch instead of taken from the counter, as in attn_prefill_dma_kernel (see there):
 // workgroup b takes item b of the first round of gridDim.x items, item gridDim.x - 1 - b of the second, and so on
 // to and fro; an item's list entry is asked for while the item before it runs.
 const bool dealt = fixed_rounds > 0 && listed && items <= static_cast<unsigned long long>(fixed_rounds) * gridDim.x;
 unsigned int round = 0u;
 unsigned int ahead_entry = 0u;
 int4 ahead_seg = {0, 0, 0, 0};
 auto dealt_item = [&](unsigned int r) {
   return r * gridDim.x + ((r & 1u) ? gridDim.x - 1u - blockIdx.x : blockIdx.x);
 };
 if (dealt && blockIdx.x < items) {
   ahead_entry = g_prefill_plan[blockIdx.x / (nkv * parts)];
   ahead_seg = g_prefill_seg[blockIdx.x / (nkv * parts)];
 }
 for (;;) {  // one item per round; every wave of the workgroup leaves at the same round
  unsigned int item;
  if (dealt) {
    if (round > 0u) __syncthreads();  // the item's first tile goes where the last one's tiles were read
    item = dealt_item(round);
    if (item >= items) return;  // every later round lies behind this one
  } else {
    if (tid == 0) item_of_workgroup = atomicAdd(&g_prefill_next_item, 1u);
    __syncthreads();
    item = item_of_workgroup;
    __syncthreads();  // everyone has read it before thread 0 asks for the next
    if (item >= items) {
      // The last workgroup to leave puts the counters back to zero: the layers of a step hand out the same list one
      // after the other, and only the first of them runs the planning kernel.
      if (tid == 0 && atomicAdd(&g_prefill_left, 1u) == gridDim.x - 1) {
        g_prefill_next_item = 0u;
        g_prefill_left = 0u;
      }
      return;
    }
  }
  const unsigned int pair = item / (nkv * parts);
  const int kvh = static_cast<int>((item / parts) % nkv);
  const int part = static_cast<int>(item % parts);
  // the last rows of a segment see the most keys: they are handed out first
  int seg = static_cast<int>(pair % segments), wg_row = (blocks_x - 1 - static_cast<int>(pair / segments)) * kPfRows;
  int row0, qlen, start, slot;
  if (dealt) {
    seg = static_cast<int>(ahead_entry & 0xffffu);
    wg_row = static_cast<int>(ahead_entry >> 16) * kPfRows;
    row0 = ahead_seg.x, qlen = ahead_seg.y, start = ahead_seg.z, slot = ahead_seg.w;
    ++round;
    const unsigned int next = dealt_item(round);
    if (next < items) {
      ahead_entry = g_prefill_plan[next / (nkv * parts)];
      ahead_seg = g_prefill_seg[next / (nkv * parts)];
    }
  } else if (listed) {  // the entry and what the list holds of its segment: two loads side by side
    const unsigned int entry = g_prefill_plan[pair];
    const int4 of_seg = g_prefill_seg[pair];
    seg = static_cast<int>(entry & 0xffffu);
    wg_row = static_cast<int>(entry >> 16) * kPfRows;
    row0 = of_seg.x, qlen = of_seg.y, start = of_seg.z, slot = of_seg.w;
  } else {
    row0 = a.seg_row0[seg];
    qlen = a.seg_row0[seg + 1] - row0;
    start = a.seg_start[seg];
    slot = a.seg_slot[seg];
  }
  const int rows = qlen * G;
  if (rows < min_rows) continue;  // short segments (decoded tokens) belong to the other kernel
  if (wg_row >= rows) continue;
  const int* table = a.block_table + static_cast<int64_t>(slot) * a.table_stride;
  const int D = EXACT ? DMAX : a.D, P = a.P;
  const int n_dch = EXACT ? DCH : (D + 31) / 32, n_dt = EXACT ? DTL : D / 16;

  // LDS: two stages of [64 keys][D + 8] keys and [D][64 + 4] values (bfloat16; rows padded against bank conflicts)
  const int k_pitch = D + 8, v_pitch = kPfKeys + kPfVPad;
  const int stage_elems = kPfKeys * k_pitch + D * v_pitch;
  uint16_t* lds = reinterpret_cast<uint16_t*>(lds_raw);

  // keys this workgroup needs
  const int tok_min = wg_row / G;
  const int tok_max = (min(wg_row + kPfRows, rows) - 1) / G;
  const int kv_total = start + qlen;
  const int kv_hi = start + tok_max + 1;
  const int kv_lo = a.window > 0 ? max(0, start + tok_min - a.window + 1) : 0;
  int t0 = kv_lo / kPfKeys, t1 = (kv_hi + kPfKeys - 1) / kPfKeys;
  if (parts > 1) {  // this workgroup takes one part of the tiles (it may be empty) and leaves partial results
    const int per = (t1 - t0 + static_cast<int>(parts) - 1) / static_cast<int>(parts);
    t0 = t0 + part * per;
    t1 = min(t0 + per, t1);
  }

  // this wave's rows
  const int row_begin = wg_row + 16 * NT * wave;
  const bool wave_has_rows = row_begin < rows;
  const int wave_tok_max = wave_has_rows ? (min(row_begin + 16 * NT, rows) - 1) / G : 0;
  const int wave_kv_hi = start + wave_tok_max + 1;
  const int wave_kv_lo = a.window > 0 ? max(0, start + min(row_begin, rows - 1) / G - a.window + 1) : 0;
  // a tile needs no mask for this wave if it lies at or below its first row's position and at or
  // above its last row's window edge
  const int wave_pos_min = start + min(row_begin, rows - 1) / G;
  const int wave_win_lo = a.window > 0 ? max(0, start + wave_tok_max - a.window + 1) : 0;
  int my_pos[NT], my_tok[NT], my_head[NT];
  bool row_ok[NT];
  bf16x8 qreg[NT][DCH];
#pragma unroll
  for (int n = 0; n < NT; ++n) {
    const int row = row_begin + 16 * n + li;
    row_ok[n] = row < rows;
    my_tok[n] = min(row / G, qlen - 1);
    my_head[n] = kvh * G + row % G;
    my_pos[n] = start + my_tok[n];
    const uint16_t* qp = a.q + static_cast<int64_t>(row0 + my_tok[n]) * a.q_stride + my_head[n] * D;
#pragma unroll
    for (int c = 0; c < DCH; ++c) {
      // always a load (from a clamped place) and a choice of the value afterwards: a load under a condition
      // would be waited for on the spot, and would leave registers that are sometimes never written
      const int d = 32 * c + 8 * g;
      const bf16x8 got = load_bf16x8(qp + (EXACT ? d : min(d, D - 8)));
      qreg[n][c] = (EXACT || d < D) ? got : zero_bf16x8();
    }
  }
  f32x4 acc[NT][DTL];
  float m[NT], l[NT];
#pragma unroll
  for (int n = 0; n < NT; ++n) {
    m[n] = -INFINITY;
    l[n] = 0.f;
#pragma unroll
    for (int t = 0; t < DTL; ++t) acc[n][t] = f32x4{0.f, 0.f, 0.f, 0.f};
  }

  const int64_t head_off = static_cast<int64_t>(kvh) * P * D;
  const int64_t page_elems = static_cast<int64_t>(a.nkv) * P * D;
  // What each thread moves per tile never changes: work the indices out once (they take divisions),
  // leave only "which page" to the loop.
  const int ps = a.p_shift, pm = P - 1;
  const int k_chunks = D / 8;                    // 16-byte pieces of a key row
  const int k_total = kPfKeys * k_chunks;
  const int kp = min(P, kPfKeys);                // keys of one page inside a tile
  const int v_per_row = kp / 4;                  // 8-byte pieces of one d row of a page, inside the tile
  const int v_total = (kPfKeys / 4) * D;
  int k_key[kKPieces], k_col[kKPieces], k_lds[kKPieces];
  int v_d[kVPieces], v_off[kVPieces], v_lds[kVPieces];
#pragma unroll
  for (int j = 0; j < kKPieces; ++j) {
    const int p = tid + j * (kPfWaves * kWave);
    k_key[j] = p < k_total ? p / k_chunks : -1;  // -1: this thread has no such piece
    k_col[j] = (p % k_chunks) * 8;
    k_lds[j] = (p / k_chunks) * k_pitch + k_col[j];
  }
#pragma unroll
  for (int j = 0; j < kVPieces; ++j) {
    // 16 lanes next to each other take 16 consecutive d rows at the same keys (LDS: 16 bank pairs; memory: a
    // wave still covers whole 128-byte lines, because its other lanes take the neighbouring keys)
    const int p = tid + j * (kPfWaves * kWave);
    const int qi = (p / 16) % v_per_row, d = p % 16 + 16 * ((p / (16 * v_per_row)) % (D / 16)), pg = p / (v_per_row * D);
    v_d[j] = p < v_total ? d : -1;
    v_off[j] = pg * kp + 4 * qi;  // first of 4 keys, inside the tile
    v_lds[j] = d * v_pitch + v_off[j];
  }

  // Page ids of 64 consecutive logical pages sit in one register across the wave (lane i: page
  // pg_base + i), so a piece's address needs a cross-lane read, not a block-table load of its own.
  const int pg_last = (kv_hi - 1) >> ps;
  int pg_base = 0, pg_reg = 0;
  auto cover = [&](int tile) {  // make the register hold the pages of this tile
    const int first = min(max(tile * kPfKeys, kv_lo), kv_hi - 1) >> ps;
    const int last = min(max(tile * kPfKeys + kPfKeys - 1, kv_lo), kv_hi - 1) >> ps;
    if (tile == t0 || first < pg_base || last >= pg_base + kWave) {
      pg_base = first;
      pg_reg = table[min(first + lane, pg_last)];
    }
  };

  u32x4 kstage[kKPieces];  // plain vector types: they stay in registers
  u32x2 vstage[kVPieces];
  auto fetch = [&](int tile) {
    const int base = tile * kPfKeys;
    cover(tile);
#pragma unroll
    for (int j = 0; j < kKPieces; ++j) {
      const int key = min(max(base + max(k_key[j], 0), kv_lo), kv_hi - 1);
      const int page = __shfl(pg_reg, (key >> ps) - pg_base, kWave);  // every lane takes part
      if (EXACT || k_key[j] >= 0)
        kstage[j] = *reinterpret_cast<const u32x4*>(a.k_pages + page * page_elems + head_off +
                                                    static_cast<int64_t>(key & pm) * D + k_col[j]);
    }
#pragma unroll
    for (int j = 0; j < kVPieces; ++j) {
      const int off = base + v_off[j];
      const int key4 = min(max(off, kv_lo & ~3), (kv_hi - 1) & ~3);
      const int page = __shfl(pg_reg, (key4 >> ps) - pg_base, kWave);
      if (EXACT || v_d[j] >= 0) {
        // nothing here looks at the loaded value, so no load has to be waited for before the next is issued
        vstage[j] = *reinterpret_cast<const u32x2*>(a.v_pages + page * page_elems + head_off +
                                                    static_cast<int64_t>(v_d[j]) * P + (key4 & pm));
      }
    }
  };
  auto park = [&](int stage, int tile) {  // the pieces of `tile` go from registers to LDS
    uint16_t* ks = lds + stage * stage_elems;
    uint16_t* vs = ks + kPfKeys * k_pitch;
#pragma unroll
    for (int j = 0; j < kKPieces; ++j)
      if (EXACT || k_key[j] >= 0) *reinterpret_cast<u32x4*>(ks + k_lds[j]) = kstage[j];
    const bool unwritten = tile * kPfKeys + kPfKeys > kv_total;  // the request's last tile only
#pragma unroll
    for (int j = 0; j < kVPieces; ++j)
      if (EXACT || v_d[j] >= 0) {
        u32x2 v = vstage[j];
        if (unwritten) {  // slots past the last token may hold anything, also NaN: zero them for the products
          const int off = tile * kPfKeys + v_off[j];
          if (off + 0 >= kv_total) v.x &= 0xffff0000u;
          if (off + 1 >= kv_total) v.x &= 0x0000ffffu;
          if (off + 2 >= kv_total) v.y &= 0xffff0000u;
          if (off + 3 >= kv_total) v.y &= 0x0000ffffu;
        }
        *reinterpret_cast<u32x2*>(vs + v_lds[j]) = v;
      }
  };

  fetch(t0);
  park(0, t0);
  __syncthreads();

  for (int tile = t0; tile < t1; ++tile) {
    const int stage = (tile - t0) & 1;
    const bool more = tile + 1 < t1;
    // the next tile is on its way while this one is computed; its pieces wait in registers (they must not be
    // spilled: a spill has to wait for the loads at once, which is why a wave has 16 rows, not 32)
    if (more) fetch(tile + 1);
    const int key_base = tile * kPfKeys;
    // a wave whose rows see none of this tile's keys only helps with the loads
    const bool computes = wave_has_rows && key_base < wave_kv_hi && key_base + kPfKeys > wave_kv_lo;
    const uint16_t* ks = lds + stage * stage_elems;
    const uint16_t* vs = ks + kPfKeys * k_pitch;
    f32x4 s[NT][4];
    if (computes) {
      // all key operands of the tile are asked for before the first product needs one, so that the
      // LDS latency is paid once, not once per product
      {
        bf16x8 kop[4][DCH];
#pragma unroll
        for (int t = 0; t < 4; ++t)
#pragma unroll
          for (int c = 0; c < DCH; ++c) {
            const int d = 32 * c + 8 * g;
            kop[t][c] = (EXACT || (c < n_dch && d < D))
                            ? __builtin_bit_cast(bf16x8, *reinterpret_cast<const uint4*>(ks + (16 * t + li) * k_pitch + d))
                            : zero_bf16x8();
          }
        // keep the reads above the products: moved in between them, every read's latency shows
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int t = 0; t < 4; ++t) {
          f32x4 z[NT];
#pragma unroll
          for (int n = 0; n < NT; ++n) z[n] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
          for (int c = 0; c < DCH; ++c)
            if (EXACT || c < n_dch) {
#pragma unroll
              for (int n = 0; n < NT; ++n) z[n] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kop[t][c], qreg[n][c], z[n], 0, 0, 0);
            }
#pragma unroll
          for (int n = 0; n < NT; ++n) s[n][t] = z[n];
        }
      }
    }
    if (computes) {
      // Only tiles that touch a row's causal edge or window edge need the mask; the others take
      // the short path.  m is kept in the exponent's domain (score * scale * log2 e).
      const bool masked = key_base + kPfKeys - 1 > wave_pos_min || key_base < wave_win_lo;
      bf16x8 pb[NT][2];
#pragma unroll
      for (int n = 0; n < NT; ++n) {
        if (masked) {
          const int lo = a.window > 0 ? my_pos[n] - a.window + 1 : 0;
#pragma unroll
          for (int t = 0; t < 4; ++t)
#pragma unroll
            for (int r = 0; r < 4; ++r) {
              const int key = key_base + 16 * t + 4 * g + r;
              if (!(key >= lo && key <= my_pos[n])) s[n][t][r] = -INFINITY;
            }
        }
        float bmax = -INFINITY;
#pragma unroll
        for (int t = 0; t < 4; ++t)
#pragma unroll
          for (int r = 0; r < 4; ++r) bmax = fmaxf(bmax, s[n][t][r]);
        bmax = group_max4(bmax) * a.scale_log2;  // scale > 0: the maximum commutes with it
        const float m_new = fmaxf(m[n], bmax);
        const float m_use = m_new == -INFINITY ? 0.f : m_new;  // a row that has seen no key yet
        const float alpha = __builtin_amdgcn_exp2f(m[n] - m_use);
        float psum = 0.f;
        uint32_t packed[8];
#pragma unroll
        for (int t = 0; t < 4; ++t)
#pragma unroll
          for (int r = 0; r < 4; r += 2) {
            const float p0 = __builtin_amdgcn_exp2f(fmaf(s[n][t][r], a.scale_log2, -m_use));
            const float p1 = __builtin_amdgcn_exp2f(fmaf(s[n][t][r + 1], a.scale_log2, -m_use));
            psum += p0 + p1;
            packed[2 * t + r / 2] = pack_bf16x2(p0, p1);
          }
        psum = group_sum4(psum);
        l[n] = l[n] * alpha + psum;
        // the accumulators need the factor only if some row's maximum moved
        if (__builtin_amdgcn_ballot_w64(m_new > m[n]) != 0) {
#pragma unroll
          for (int dt = 0; dt < DTL; ++dt) {
            acc[n][dt][0] *= alpha;
            acc[n][dt][1] *= alpha;
            acc[n][dt][2] *= alpha;
            acc[n][dt][3] *= alpha;
          }
        }
        m[n] = m_new;
        uint4 p01 = {packed[0], packed[1], packed[2], packed[3]};  // keys 4g.. of tiles 0 and 1
        uint4 p23 = {packed[4], packed[5], packed[6], packed[7]};  // ... of tiles 2 and 3
        pb[n][0] = __builtin_bit_cast(bf16x8, p01);
        pb[n][1] = __builtin_bit_cast(bf16x8, p23);
      }

#pragma unroll
      for (int u = 0; u < 2; ++u) {
        // the value operands of 32 keys, all asked for first.  Each is one four-dword vector filled half by
        // half: an operand put together from the scalars of two two-dword vectors just before the product was
        // compiled wrongly in the streaming kernel (the registers of the second pair were handed out again
        // before the product had read them).
        u32x4 vv[DTL];
#pragma unroll
        for (int dt = 0; dt < DTL; ++dt)
          if (EXACT || dt < n_dt) {
            const uint16_t* vrow = vs + (16 * dt + li) * v_pitch + 32 * u + 4 * g;
            const u32x2 va = *reinterpret_cast<const u32x2*>(vrow);
            const u32x2 vb = *reinterpret_cast<const u32x2*>(vrow + 16);
            vv[dt][0] = va[0];
            vv[dt][1] = va[1];
            vv[dt][2] = vb[0];
            vv[dt][3] = vb[1];
          }
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int dt = 0; dt < DTL; ++dt)
          if (EXACT || dt < n_dt) {
            const bf16x8 vop = __builtin_bit_cast(bf16x8, vv[dt]);
#pragma unroll
            for (int n = 0; n < NT; ++n)
              acc[n][dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vop, pb[n][u], acc[n][dt], 0, 0, 0);
          }
      }
    }

    if (more) park(stage ^ 1, tile + 1);  // the other stage was last read before the barrier that ended the previous round
    __syncthreads();
  }

#pragma unroll
  for (int n = 0; n < NT; ++n) {
    if (!row_ok[n]) continue;
    if (parts > 1) {  // unnormalised sums and the statistics of this part, for attn_merge_portions_kernel
      const int64_t slot = ((static_cast<int64_t>(row0 + my_tok[n]) * a.nq + my_head[n]) * parts + part);
      float* wo = a.pws_o + slot * D;
#pragma unroll
      for (int dt = 0; dt < DTL; ++dt)
        if (EXACT || dt < n_dt)
          *reinterpret_cast<float4*>(wo + 16 * dt + 4 * g) = float4{acc[n][dt][0], acc[n][dt][1], acc[n][dt][2], acc[n][dt][3]};
      if (g == 0) {
        a.pws_ml[slot * 2] = m[n];
        a.pws_ml[slot * 2 + 1] = l[n];
      }
      continue;
    }
    const float inv_l = l[n] > 0.f ? 1.0f / l[n] : 0.f;
    uint16_t* op = a.out + static_cast<int64_t>(row0 + my_tok[n]) * a.o_stride + my_head[n] * D;
#pragma unroll
    for (int dt = 0; dt < DTL; ++dt) {
      if (EXACT || dt < n_dt) {
        uint2 w;
        w.x = static_cast<uint32_t>(f32_to_bf16_bits(acc[n][dt][0] * inv_l)) |
              (static_cast<uint32_t>(f32_to_bf16_bits(acc[n][dt][1] * inv_l)) << 16);
        w.y = static_cast<uint32_t>(f32_to_bf16_bits(acc[n][dt][2] * inv_l)) |
              (static_cast<uint32_t>(f32_to_bf16_bits(acc[n][dt][3] * inv_l)) << 16);
        *reinterpret_cast<uint2*>(op + 16 * dt + 4 * g) = w;
      }
    }
  }
 }  // next item
}

// ---------------------------------------------------------------------------------------------
// Prompt portions, head_dim 128: the same work as attn_prefill_lds_kernel, built around three facts that its
// counters showed (no unit busy half the time; a third of the vector instructions spent on moving tiles; every
// wave reading the whole tile from LDS for 16 rows only).
//
//   * A wave owns 32 rows and multiplies with v_mfma_f32_32x32x16_bf16: a key or value operand read from LDS
//     serves twice the rows.  Four waves a workgroup (128 rows, as before), two workgroups a CU.
//   * Tiles go from memory straight to LDS (global_load_lds_dwordx4): no staging registers, no second pass that
//     parks them, and the loads of tile i + 1 are in flight while tile i is computed.
//   * LDS rows carry no padding (a direct load fills 64 consecutive 16-byte pieces); instead piece c of row r
//     lies at position c ^ (r & 7), which a lane gets by fetching the matching piece from memory, so that the
//     operand reads of 32 rows still spread over all banks.
//
// Layouts (lane = 32 h + j):  scores S^T = K . Q^T per 32 keys: A lane (i = j, h) = K[key(i)][16 s + 8 h ..+7],
// B lane (row j, h) = Q[row][16 s + 8 h ..+7], C register r = S^T[i = 8 (r / 4) + 4 h + r % 4][row j], where
// key(i) is i with bits 2 and 3 exchanged: so register r is key 16 (r / 8) + 8 h + r % 8.
// Second product O^T += V^T . P^T in steps of 16 keys: lane (row j, h) offers the eight probabilities that it
// holds anyway, registers 8 u .. 8 u + 7 of a score tile, i.e. keys 16 u + 8 h .. + 7, and the value operand
// of lane (d, h) is the 16-byte piece of row d with those keys.  Nothing moves between lanes.
constexpr int kDmWaves = 4;
constexpr int kDmD = 128;
constexpr int kDmKeys = 64;
constexpr int kDmStageBytes = kDmKeys * kDmD * 2 * 2;  // keys and values of a tile: 32 KB
constexpr float kDmLazyBits = 8.0f;
typedef float f32x16 __attribute__((ext_vector_type(16)));

// Sixteen bytes a lane from memory straight into LDS: the wave's 64 pieces land one after the other from
// lds_base on, which has to be the same in all lanes.  Written as assembly, and not with the compiler's builtin,
// because of what the builtin does to every later wait: while such a load is in flight the compiler takes LDS
// reads to finish in any order and turns each wait for one of them into a wait for all of them, so that no read
// can stay in flight behind a matrix product.  The loads it does not know of only make its own waits for memory
// stricter than needed; that the data has landed before it is read is the caller's business (s_waitcnt vmcnt(0)
// and a barrier).
// A value of lane i and the value of lane i ^ 32, in the same order in both lanes (v_permlane32_swap: one vector
// instruction, where a shuffle is a trip through the LDS unit).
struct HalfPair {
  float lo, hi;
};
__device__ __forceinline__ HalfPair both_halves(float x) {
  const unsigned bits = __float_as_uint(x);
  const auto r = __builtin_amdgcn_permlane32_swap(bits, bits, false, false);
  return {__uint_as_float(r[0]), __uint_as_float(r[1])};
}

#pragma clang diagnostic push
#pragma clang diagnostic ignored "-Winline-asm"  // m0 is a reserved register: naming it as clobbered is the point
__device__ __forceinline__ void load_to_lds_16(const void* src, unsigned char* lds_at) {
  const uint32_t base = __builtin_amdgcn_readfirstlane(
      static_cast<uint32_t>(reinterpret_cast<uintptr_t>((__attribute__((address_space(3))) void*)lds_at)));
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, off" ::"s"(base), "v"(src) : "memory", "m0");
}
// The same with the address as a wave-wide base and a byte offset of the lane.
__device__ __forceinline__ void load_to_lds_16(const void* base_uniform, uint32_t lane_bytes, unsigned char* lds_at) {
  const uint32_t base = __builtin_amdgcn_readfirstlane(
      static_cast<uint32_t>(reinterpret_cast<uintptr_t>((__attribute__((address_space(3))) void*)lds_at)));
  const uint64_t src = reinterpret_cast<uint64_t>(base_uniform);
  // the builtin returns a signed int: widened as it is, a low half with its top bit set would fill the high half
  const uint32_t lo = static_cast<uint32_t>(__builtin_amdgcn_readfirstlane(static_cast<int>(static_cast<uint32_t>(src))));
  const uint32_t hi = static_cast<uint32_t>(__builtin_amdgcn_readfirstlane(static_cast<int>(src >> 32)));
  const uint64_t src_s = (static_cast<uint64_t>(hi) << 32) | lo;
  // s_nop 4: a scalar register written by a vector instruction may not be a memory instruction's address for
  // five cycles, and the compiler does not look into this text for that
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 4\n\tglobal_load_lds_dwordx4 %1, %2" ::"s"(base), "v"(lane_bytes), "s"(src_s)
               : "memory", "m0");
}
#pragma clang diagnostic pop

// WHOLE: the page size is a multiple of the tile's 64 keys, so a tile lies in one page: its address is a
// matter of scalar arithmetic and a lane adds an offset that never changes.  Otherwise a lane looks up the page
// of each of its pieces.
//
// GROUPS == 2: eight waves, two groups of four that take the same 128 rows and every other tile of keys each, with
// tiles of their own in LDS, and put their sums together through LDS at the end.  One such workgroup a CU instead
// of two of four waves: a row block is done in half the time, which is what a launch waits for when it has about
// as many row blocks as the chip has places for them (a causal prompt of 2,048 tokens: 512 row blocks from 1 to 32
// tiles of keys, and the launch lasts as long as the heaviest).
template <bool WHOLE, int GROUPS>
__global__ __launch_bounds__(GROUPS* kDmWaves* kWave, GROUPS == 1 ? 2 : 1) void attn_prefill_dma_kernel(
    const AttnArgs a, int min_rows, int blocks_x, int segments, int listed, int pair_up, int fixed_rounds) {
  constexpr int D = kDmD;
  extern __shared__ __align__(16) unsigned char lds_all[];
  __shared__ unsigned int item_of_workgroup;
  const int tid = threadIdx.x, lane = tid & 63, j = lane & 31, h = lane >> 5;
  const int grp = GROUPS == 1 ? 0 : __builtin_amdgcn_readfirstlane(tid >> 8);   // the group of this wave
  const int wave = __builtin_amdgcn_readfirstlane((tid >> 6) & 3);              // the wave inside its group
  unsigned char* const lds_raw = lds_all + grp * (2 * kDmStageBytes);
  const int G = a.nq / a.nkv;
  const unsigned int nkv = static_cast<unsigned int>(a.nkv);
  const unsigned int pairs = listed ? g_prefill_pairs : static_cast<unsigned int>(blocks_x) * segments;
  const unsigned int parts = static_cast<unsigned int>(a.portion_splits);
  const unsigned int items = pairs * nkv * parts;
  const int P = a.P, ps = a.p_shift, pm = P - 1;
  const uint32_t page_elems32 = static_cast<uint32_t>(a.nkv) * P * D;  // the launcher refuses pages of 2^31 elements
 // With few items a workgroup (up to fixed_rounds) the items are dealt out before the launch instead of taken from
 // the counter: workgroup b takes item b of the first round of gridDim.x items, item gridDim.x - 1 - b of the
 // second, and so on to and fro, so that on a list that runs from heavy to light every workgroup gets about the
 // same, and an item begins without the counter's round trip to memory; its list entry was asked for while the
 // item before it ran.
 const bool dealt = fixed_rounds > 0 && listed && items <= static_cast<unsigned long long>(fixed_rounds) * gridDim.x;
 unsigned int round = 0u;
 unsigned int ahead_entry = 0u;
 int4 ahead_seg = {0, 0, 0, 0};
 auto dealt_item = [&](unsigned int r) {
   return r * gridDim.x + ((r & 1u) ? gridDim.x - 1u - blockIdx.x : blockIdx.x);
 };
 if (dealt && blockIdx.x < items) {
   ahead_entry = g_prefill_plan[blockIdx.x / (nkv * parts)];
   ahead_seg = g_prefill_seg[blockIdx.x / (nkv * parts)];
 }
 for (;;) {
  unsigned int item;
  if (dealt) {
    // two groups: group 0 reads the other's sums from LDS at the end of an item, where its next tiles will land
    if (GROUPS == 2 && round > 0u) __syncthreads();
    item = dealt_item(round);
    if (item >= items) return;  // every later round lies behind this one
  } else {
    if (tid == 0) item_of_workgroup = atomicAdd(&g_prefill_next_item, 1u);
    __syncthreads();
    item = item_of_workgroup;
    __syncthreads();
    if (item >= items) {
      // The last workgroup to leave puts the counters back to zero: the layers of a step hand out the same list one
      // after the other, and only the first of them runs the planning kernel.
      if (tid == 0 && atomicAdd(&g_prefill_left, 1u) == gridDim.x - 1) {
        g_prefill_next_item = 0u;
        g_prefill_left = 0u;
      }
      return;
    }
  }
  unsigned int pair = item / (nkv * parts);
  const int kvh = static_cast<int>((item / parts) % nkv);
  const int part = static_cast<int>(item % parts);
  // The list runs from the heaviest row block to the lightest.  Two workgroups share a CU, and the second
  // half of the first round of workgroups lands beside the first half: so the first pair_up pairs are handed
  // out as they are, the next pair_up from the light end, and then the middle, which gives every CU a heavy
  // and a light item to start with instead of two heavy ones here and two light ones there.
  if (!dealt && pair_up > 0 && pairs >= 2u * pair_up) {
    const unsigned int h = static_cast<unsigned int>(pair_up);
    if (pair >= h) pair = pair < 2u * h ? pairs - 1u - (pair - h) : pair - h;
  }
  int seg = static_cast<int>(pair % segments), wg_row = (blocks_x - 1 - static_cast<int>(pair / segments)) * kPfRows;
  int row0, qlen, start, slot;
  if (dealt) {
    seg = static_cast<int>(ahead_entry & 0xffffu);
    wg_row = static_cast<int>(ahead_entry >> 16) * kPfRows;
    row0 = ahead_seg.x, qlen = ahead_seg.y, start = ahead_seg.z, slot = ahead_seg.w;
    ++round;
    const unsigned int next = dealt_item(round);
    if (next < items) {
      ahead_entry = g_prefill_plan[next / (nkv * parts)];
      ahead_seg = g_prefill_seg[next / (nkv * parts)];
    }
  } else if (listed) {  // the entry and what the list holds of its segment: two loads side by side
    const unsigned int entry = g_prefill_plan[pair];
    const int4 of_seg = g_prefill_seg[pair];
    seg = static_cast<int>(entry & 0xffffu);
    wg_row = static_cast<int>(entry >> 16) * kPfRows;
    row0 = of_seg.x, qlen = of_seg.y, start = of_seg.z, slot = of_seg.w;
  } else {
    row0 = a.seg_row0[seg];
    qlen = a.seg_row0[seg + 1] - row0;
    start = a.seg_start[seg];
    slot = a.seg_slot[seg];
  }
  const int rows = qlen * G;
  if (rows < min_rows) continue;
  if (wg_row >= rows) continue;
  const int* table = a.block_table + static_cast<int64_t>(slot) * a.table_stride;
  const uint32_t head_off32 = static_cast<uint32_t>(kvh) * P * D;

  const int tok_min = wg_row / G;
  const int tok_max = (min(wg_row + kPfRows, rows) - 1) / G;
  const int kv_total = start + qlen;
  const int kv_hi = start + tok_max + 1;
  const int kv_lo = a.window > 0 ? max(0, start + tok_min - a.window + 1) : 0;
  int t0 = kv_lo / kDmKeys, t1 = (kv_hi + kDmKeys - 1) / kDmKeys;
  if (parts > 1) {
    const int per = (t1 - t0 + static_cast<int>(parts) - 1) / static_cast<int>(parts);
    t0 = t0 + part * per;
    t1 = min(t0 + per, t1);
  }

  // this wave's 32 rows; the lane's own row is row_begin + j (both halves h of a row hold the same statistics)
  const int row_begin = wg_row + 32 * wave;
  const bool wave_has_rows = row_begin < rows;
  const int wave_tok_max = wave_has_rows ? (min(row_begin + 32, rows) - 1) / G : 0;
  const int wave_kv_hi = start + wave_tok_max + 1;
  const int wave_pos_min = start + min(row_begin, rows - 1) / G;
  const int wave_kv_lo = a.window > 0 ? max(0, wave_pos_min - a.window + 1) : 0;
  const int wave_win_lo = a.window > 0 ? max(0, start + wave_tok_max - a.window + 1) : 0;
  const int row = row_begin + j;
  const bool row_ok = row < rows;
  const int my_tok = min(row / G, qlen - 1);
  const int my_head = kvh * G + row % G;
  const int my_pos = start + my_tok;
  bf16x8 qreg[D / 16];
  {
    const uint16_t* qp = a.q + static_cast<int64_t>(row0 + my_tok) * a.q_stride + my_head * D + 8 * h;
#pragma unroll
    for (int s = 0; s < D / 16; ++s) qreg[s] = load_bf16x8(qp + 16 * s);
  }
  // Row i of a score tile takes the key whose number has bits 2 and 3 of i exchanged: then the eight scores
  // that a lane holds for a step of the second product belong to eight keys in a row, and the matching values
  // are one 16-byte piece of a d row.
  const int jk = (j & 19) | ((j & 4) << 1) | ((j & 8) >> 1);
  f32x16 o[D / 32];
#pragma unroll
  for (int dt = 0; dt < D / 32; ++dt)
#pragma unroll
    for (int r = 0; r < 16; ++r) o[dt][r] = 0.f;
  float m = -INFINITY, l = 0.f;

  // page ids of 64 consecutive logical pages in one register across the wave (lane i: page pg_base + i)
  const int pg_last = (kv_hi - 1) >> ps;
  int pg_base = 0, pg_reg = 0;
  auto cover = [&](int tile, bool first) {
    const int lo = min(max(tile * kDmKeys, kv_lo), kv_hi - 1) >> ps;
    const int hi = min(max(tile * kDmKeys + kDmKeys - 1, kv_lo), kv_hi - 1) >> ps;
    if (first || lo < pg_base || hi >= pg_base + kWave) {
      pg_base = lo;
      pg_reg = table[min(lo + lane, pg_last)];
    }
  };
  // what a lane fetches for a tile never changes but for the page: four pieces of keys and four of values
  //   keys:   LDS piece q = 64 (4 wave + jj) + lane -> key q / 16 of the tile, position q % 16 in its row
  //   values: LDS piece q                           -> d row q / 8,            position q % 8
  int k_key[4], k_src[4], v_key[4], v_src[4];
#pragma unroll
  for (int jj = 0; jj < 4; ++jj) {
    const int q = 64 * (4 * wave + jj) + lane;
    const int key = q / 16, pos = q % 16;
    k_key[jj] = key;
    k_src[jj] = 8 * (pos ^ (key & 15));              // element offset of the piece inside its key row
    const int d = q / 8, vpos = q % 8;
    v_key[jj] = 8 * (vpos ^ ((d >> 1) & 7));               // first of the piece's eight keys, inside the tile
    v_src[jj] = d * P;                                // element offset of the d row inside a page
  }
  auto fetch = [&](int tile, int stage) {
    const int base = tile * kDmKeys;
    unsigned char* at = lds_raw + stage * kDmStageBytes + (4 * wave) * 1024;
    if constexpr (WHOLE) {
      // keys of the tile that lie outside the request are read as they are (the page is there) and masked
      const int page = __builtin_amdgcn_readlane(pg_reg, __builtin_amdgcn_readfirstlane((base >> ps) - pg_base));
      const uint64_t first = static_cast<uint64_t>(static_cast<uint32_t>(page)) * page_elems32 + head_off32;
      const uint16_t* kb = a.k_pages + first + static_cast<uint32_t>(base & pm) * D;
      const uint16_t* vb = a.v_pages + first + static_cast<uint32_t>(base & pm);
#pragma unroll
      for (int jj = 0; jj < 4; ++jj)
        load_to_lds_16(kb, 2u * static_cast<uint32_t>(k_key[jj] * D + k_src[jj]), at + jj * 1024);
#pragma unroll
      for (int jj = 0; jj < 4; ++jj)
        load_to_lds_16(vb, 2u * static_cast<uint32_t>(v_src[jj] + v_key[jj]), at + kDmKeys * D * 2 + jj * 1024);
      return;
    }
    // Keys: one load takes four keys in a row, which lie in one page (a page holds eight at least), so the page
    // is the wave's and the address scalar arithmetic as above; keys outside the request are read from the
    // nearest page that is there and masked.  Values: a lane's piece holds eight keys of its own, so a lane
    // looks up its own page: the four page ids first (lane exchanges that answer together), then the loads.
    const int wave_u = __builtin_amdgcn_readfirstlane(wave);
    int v_at[4], v_page[4];
#pragma unroll
    for (int jj = 0; jj < 4; ++jj) {
      v_at[jj] = min(max(base + v_key[jj], kv_lo & ~7), (kv_hi - 1) & ~7);
      v_page[jj] = __shfl(pg_reg, (v_at[jj] >> ps) - pg_base, kWave);
    }
#pragma unroll
    for (int jj = 0; jj < 4; ++jj) {
      const int first_key = base + 4 * (4 * wave_u + jj);
      const int page_at = min(max(first_key >> ps, kv_lo >> ps), pg_last) - pg_base;
      const int page = __builtin_amdgcn_readlane(pg_reg, __builtin_amdgcn_readfirstlane(page_at));
      const uint16_t* kb = a.k_pages + static_cast<uint64_t>(static_cast<uint32_t>(page)) * page_elems32 + head_off32 +
                           static_cast<uint32_t>(first_key & pm) * D;
      load_to_lds_16(kb, 2u * static_cast<uint32_t>((lane >> 4) * D + k_src[jj]), at + jj * 1024);
    }
#pragma unroll
    for (int jj = 0; jj < 4; ++jj) {
      const uint16_t* src = a.v_pages + static_cast<uint64_t>(static_cast<uint32_t>(v_page[jj])) * page_elems32 +
                            (head_off32 + v_src[jj] + static_cast<uint32_t>(v_at[jj] & pm));
      load_to_lds_16(src, at + kDmKeys * D * 2 + jj * 1024);
    }
  };
  // Slots past the request's last token may hold anything, also NaN, and 0 * NaN is NaN: in the request's last
  // tile every lane puts the values of such keys to zero in the pieces that it fetched itself.
  auto scrub = [&](int tile, int stage) {
    const int base = tile * kDmKeys;
    if (base + kDmKeys <= kv_total) return;
    unsigned char* at = lds_raw + stage * kDmStageBytes + kDmKeys * D * 2 + (4 * wave) * 1024 + lane * 16;
#pragma unroll
    for (int jj = 0; jj < 4; ++jj) {
      const int key8 = WHOLE ? base + v_key[jj] : min(max(base + v_key[jj], kv_lo & ~7), (kv_hi - 1) & ~7);  // as fetched
      if (key8 + 8 > kv_total) {
        u32x4 v = *reinterpret_cast<u32x4*>(at + jj * 1024);
#pragma unroll
        for (int e = 0; e < 8; ++e)
          if (key8 + e >= kv_total) v[e / 2] &= (e & 1) ? 0x0000ffffu : 0xffff0000u;
        *reinterpret_cast<u32x4*>(at + jj * 1024) = v;
      }
    }
  };

  if (t0 + grp < t1) {
    cover(t0 + grp, true);
    fetch(t0 + grp, 0);
  }
  // The query has to be there before the loop: a wait for it inside the loop would count the tile loads in
  // flight (which the compiler does not know of) and wait for them too.
#pragma unroll
  for (int s = 0; s < D / 16; ++s) asm volatile("" ::"v"(qreg[s]));
  // group g takes the tiles t0 + g, t0 + g + GROUPS, ...; both groups walk the loop as often as group 0 does (the
  // barriers are the workgroup's), a group without a tile in its last round does nothing there
  for (int first = t0; first < t1; first += GROUPS) {
    const int tile = first + grp;
    const int stage = ((first - t0) / GROUPS) & 1;
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // this wave's pieces of the tile have landed
    if (tile < t1) scrub(tile, stage);
    __syncthreads();  // everybody's have; and everybody is done with the other stage
    if (tile + GROUPS < t1) {
      cover(tile + GROUPS, false);
      fetch(tile + GROUPS, stage ^ 1);
    }
    const int key_base = tile * kDmKeys;
    const bool computes = tile < t1 && wave_has_rows && key_base < wave_kv_hi && key_base + kDmKeys > wave_kv_lo;
    if (!computes) continue;
    const unsigned char* ks = lds_raw + stage * kDmStageBytes;
    const unsigned char* vs = ks + kDmKeys * D * 2;

    // scores of 2 x 32 keys: sixteen operand reads and sixteen products, the two halves taking turns, a read
    // issued four products before the product that needs it (the order is pinned below: left to itself the
    // compiler waits for eight reads, multiplies, and waits again)
    f32x16 st[2];
    {
      bf16x8 kop[2][D / 16];
#pragma unroll
      for (int s = 0; s < D / 16; ++s)
#pragma unroll
        for (int t = 0; t < 2; ++t) {
          const int key = 32 * t + jk;
          kop[t][s] = __builtin_bit_cast(
              bf16x8, *reinterpret_cast<const uint4*>(ks + key * (D * 2) + (((2 * s + h) ^ (key & 15)) * 16)));
        }
#pragma unroll
      for (int t = 0; t < 2; ++t)
#pragma unroll
        for (int r = 0; r < 16; ++r) st[t][r] = 0.f;
#pragma unroll
      for (int s = 0; s < D / 16; ++s)
#pragma unroll
        for (int t = 0; t < 2; ++t) st[t] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(kop[t][s], qreg[s], st[t], 0, 0, 0);
      constexpr int kAhead = 4, kOps = 2 * (D / 16);
      __builtin_amdgcn_sched_group_barrier(0x100, kAhead, 0);
#pragma unroll
      for (int i = 0; i < kOps - kAhead; ++i) {
        __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
        __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
      }
      __builtin_amdgcn_sched_group_barrier(0x008, kAhead, 0);
    }
    // st[t][r] belongs to key key_base + 32 t + 16 (r / 8) + 8 h + r % 8 and to this lane's row
    const bool masked = key_base + kDmKeys - 1 > wave_pos_min || key_base < wave_win_lo;
    if (masked) {
      const int lo = a.window > 0 ? my_pos - a.window + 1 : 0;
#pragma unroll
      for (int t = 0; t < 2; ++t)
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const int key = key_base + 32 * t + 16 * (r / 8) + 8 * h + r % 8;
          if (!(key >= lo && key <= my_pos)) st[t][r] = -INFINITY;
        }
    }
    float bmax = -INFINITY;
#pragma unroll
    for (int t = 0; t < 2; ++t)
#pragma unroll
      for (int r = 0; r < 16; ++r) bmax = fmaxf(bmax, st[t][r]);
    {
      const HalfPair both = both_halves(bmax);
      bmax = fmaxf(both.lo, both.hi) * a.scale_log2;  // scale > 0: the maximum commutes with it
    }
    // m is the point that the row's exponentials are taken from, not its exact maximum: it moves only when
    // the maximum has grown by more than kDmLazyBits (exponentials up to 2^8 meanwhile, nothing to a float or
    // a bf16), which after a row's first tiles is rare, so that the 64 sums are rarely multiplied
    const float m_new = bmax > m + kDmLazyBits ? bmax : m;
    const float m_use = m_new == -INFINITY ? 0.f : m_new;  // a row that has seen no key yet
    const float alpha = __builtin_amdgcn_exp2f(m - m_use);
    float psum = 0.f;
    bf16x8 pb[2][2];
#pragma unroll
    for (int t = 0; t < 2; ++t)
#pragma unroll
      for (int u = 0; u < 2; ++u) {
        u32x4 packed;
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          const float p0 = __builtin_amdgcn_exp2f(fmaf(st[t][8 * u + 2 * e], a.scale_log2, -m_use));
          const float p1 = __builtin_amdgcn_exp2f(fmaf(st[t][8 * u + 2 * e + 1], a.scale_log2, -m_use));
          psum += p0 + p1;
          packed[e] = pack_bf16x2(p0, p1);
        }
        pb[t][u] = __builtin_bit_cast(bf16x8, packed);
      }
    {
      const HalfPair both = both_halves(psum);
      psum = both.lo + both.hi;
    }
    l = l * alpha + psum;
    if (__builtin_amdgcn_ballot_w64(m_new > m) != 0) {  // the sums need the factor only if some row's maximum moved
#pragma unroll
      for (int dt = 0; dt < D / 32; ++dt)
#pragma unroll
        for (int r = 0; r < 16; ++r) o[dt][r] *= alpha;
    }
    m = m_new;

    // O^T += V^T . P^T, 16 keys a step; reads and products in turns as above
    {
      u32x4 vop[4][D / 32];
#pragma unroll
      for (int k = 0; k < 4; ++k) {
        const int c = 2 * k + h;  // the piece that holds keys 16 k + 8 h .. + 7 of the tile
#pragma unroll
        for (int dt = 0; dt < D / 32; ++dt) {
          const int d = 32 * dt + j;
          vop[k][dt] = *reinterpret_cast<const u32x4*>(vs + d * (kDmKeys * 2) + ((c ^ ((d >> 1) & 7)) * 16));
        }
      }
#pragma unroll
      for (int k = 0; k < 4; ++k)
#pragma unroll
        for (int dt = 0; dt < D / 32; ++dt)
          o[dt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, vop[k][dt]), pb[k / 2][k % 2], o[dt],
                                                          0, 0, 0);
      constexpr int kAhead = 4, kOps = 4 * (D / 32);
      __builtin_amdgcn_sched_group_barrier(0x100, kAhead, 1);
#pragma unroll
      for (int i = 0; i < kOps - kAhead; ++i) {
        __builtin_amdgcn_sched_group_barrier(0x008, 1, 1);
        __builtin_amdgcn_sched_group_barrier(0x100, 1, 1);
      }
      __builtin_amdgcn_sched_group_barrier(0x008, kAhead, 1);
    }
  }
  __syncthreads();  // the next item's first tile goes into stage 0: everybody has to be done reading

  if constexpr (GROUPS == 2) {
    // group 1 hands its sums to group 0 through LDS (a lane to the same lane of the same wave: 66 floats, laid out
    // so that the 64 lanes of a wave write and read 16 contiguous bytes each): out = o_0 2^(m_0 - m) + o_1 2^(m_1 - m)
    float* mine = reinterpret_cast<float*>(lds_all) + wave * (D / 2 + 2) * kWave;   // [wave][D / 8 + 1 pieces][lane][4]
    if (grp == 1) {
#pragma unroll
      for (int dt = 0; dt < D / 32; ++dt)
#pragma unroll
        for (int q = 0; q < 4; ++q)
          *reinterpret_cast<float4*>(mine + ((4 * dt + q) * kWave + lane) * 4) =
              float4{o[dt][4 * q], o[dt][4 * q + 1], o[dt][4 * q + 2], o[dt][4 * q + 3]};
      *reinterpret_cast<float2*>(mine + (D / 8) * kWave * 4 + lane * 2) = float2{m, l};
    }
    __syncthreads();
    if (grp == 1) continue;  // the barriers at the head of the loop hold it until group 0 has read
    const float2 other = *reinterpret_cast<const float2*>(mine + (D / 8) * kWave * 4 + lane * 2);
    const float m_all = fmaxf(m, other.x);
    const float m_ref = m_all == -INFINITY ? 0.f : m_all;
    const float f0 = __builtin_amdgcn_exp2f(m - m_ref), f1 = __builtin_amdgcn_exp2f(other.x - m_ref);
    l = l * f0 + other.y * f1;
    m = m_all;
#pragma unroll
    for (int dt = 0; dt < D / 32; ++dt)
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const float4 v = *reinterpret_cast<const float4*>(mine + ((4 * dt + q) * kWave + lane) * 4);
        o[dt][4 * q] = o[dt][4 * q] * f0 + v.x * f1;
        o[dt][4 * q + 1] = o[dt][4 * q + 1] * f0 + v.y * f1;
        o[dt][4 * q + 2] = o[dt][4 * q + 2] * f0 + v.z * f1;
        o[dt][4 * q + 3] = o[dt][4 * q + 3] * f0 + v.w * f1;
      }
  }

  // o[dt][r] is O^T[d = 32 dt + 8 (r / 4) + 4 h + r % 4][this lane's row]
  if (row_ok) {
    if (parts > 1) {
      const int64_t slot = ((static_cast<int64_t>(row0 + my_tok) * a.nq + my_head) * parts + part);
      float* wo = a.pws_o + slot * D;
#pragma unroll
      for (int dt = 0; dt < D / 32; ++dt)
#pragma unroll
        for (int q = 0; q < 4; ++q)
          *reinterpret_cast<float4*>(wo + 32 * dt + 8 * q + 4 * h) =
              float4{o[dt][4 * q], o[dt][4 * q + 1], o[dt][4 * q + 2], o[dt][4 * q + 3]};
      if (h == 0) {
        a.pws_ml[slot * 2] = m;
        a.pws_ml[slot * 2 + 1] = l;
      }
    } else {
      const float inv_l = l > 0.f ? 1.0f / l : 0.f;
      uint16_t* op = a.out + static_cast<int64_t>(row0 + my_tok) * a.o_stride + my_head * D;
#pragma unroll
      for (int dt = 0; dt < D / 32; ++dt)
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          uint2 w;
          w.x = pack_bf16x2(o[dt][4 * q] * inv_l, o[dt][4 * q + 1] * inv_l);
          w.y = pack_bf16x2(o[dt][4 * q + 2] * inv_l, o[dt][4 * q + 3] * inv_l);
          *reinterpret_cast<uint2*>(op + 32 * dt + 8 * q + 4 * h) = w;
        }
    }
  }
 }  // next item
}

// The parts of a portion's rows put together: out = sum_p o_p 2^(m_p - m) / sum_p l_p 2^(m_p - m), in the order
// of the parts.  Work items are (listed pair, kv head, eight rows of the row block): a workgroup of eight waves
// takes items blockIdx.x, blockIdx.x + gridDim.x, ... and each wave one row of the item, a lane four columns
// (head_dim <= 256).  No workgroup is launched for nothing, and no wave walks rows one after the other (a row
// is two dependent loads: walking sixteen of them took longer than the attention itself).
constexpr int kPortionPartsMax = 8;
__global__ __launch_bounds__(kPfWaves* kWave) void attn_merge_portions_kernel(const AttnArgs a) {
  const int G = a.nq / a.nkv, D = a.D, parts = a.portion_splits;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int d0 = 4 * lane;
  constexpr int kSubBlocks = kPfRows / kPfWaves;  // items of eight rows in a row block
  const unsigned int items = g_prefill_pairs * a.nkv * kSubBlocks;
  for (unsigned int item = blockIdx.x; item < items; item += gridDim.x) {
    const unsigned int pair = item / (a.nkv * kSubBlocks);
    const int kvh = static_cast<int>((item / kSubBlocks) % a.nkv), sub = static_cast<int>(item % kSubBlocks);
    const unsigned int entry = g_prefill_plan[pair];
    const int seg = static_cast<int>(entry & 0xffffu);
    const int row = static_cast<int>(entry >> 16) * kPfRows + sub * kPfWaves + wave;
    const int row0 = a.seg_row0[seg];
    const int rows = (a.seg_row0[seg + 1] - row0) * G;
    if (row >= rows) continue;  // this wave only
    const int head = kvh * G + row % G;
    const int64_t tok_row = row0 + row / G;
    const int64_t base = (tok_row * a.nq + head) * parts;
    float ms[kPortionPartsMax], ls[kPortionPartsMax];
    float4 os[kPortionPartsMax];
    const float* src = a.pws_o + base * D + (d0 < D ? d0 : 0);
#pragma unroll
    for (int p = 0; p < kPortionPartsMax; ++p) {  // every load first, none under a condition
      const int q = min(p, parts - 1);
      const float2 ml = *reinterpret_cast<const float2*>(a.pws_ml + (base + q) * 2);
      os[p] = *reinterpret_cast<const float4*>(src + static_cast<int64_t>(q) * D);
      ms[p] = p < parts ? ml.x : -INFINITY;
      ls[p] = p < parts ? ml.y : 0.f;
    }
    float mx = -INFINITY;
#pragma unroll
    for (int p = 0; p < kPortionPartsMax; ++p) mx = fmaxf(mx, ms[p]);
    float denom = 0.f;
    float4 o = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int p = 0; p < kPortionPartsMax; ++p) {
      const float w = ms[p] > -INFINITY ? exp2f(ms[p] - mx) : 0.f;  // an empty part weighs nothing
      denom += ls[p] * w;
      o.x += os[p].x * w;
      o.y += os[p].y * w;
      o.z += os[p].z * w;
      o.w += os[p].w * w;
    }
    const float inv = denom > 0.f ? 1.0f / denom : 0.f;
    if (d0 < D) {
      uint2 w;
      w.x = static_cast<uint32_t>(f32_to_bf16_bits(o.x * inv)) | (static_cast<uint32_t>(f32_to_bf16_bits(o.y * inv)) << 16);
      w.y = static_cast<uint32_t>(f32_to_bf16_bits(o.z * inv)) | (static_cast<uint32_t>(f32_to_bf16_bits(o.w * inv)) << 16);
      *reinterpret_cast<uint2*>(a.out + tok_row * a.o_stride + head * D + d0) = w;
    }
  }
}

template <int NT>
int launch_attn(const AttnArgs& a, dim3 grid, hipStream_t s) {
  // head_dim 64 and 128 as compile-time values: no test and no branch around a load, so that the keys and
  // values of the next block stay in flight while this block is computed (a load inside a branch makes the
  // next wait a wait for everything)
  if (a.D == 128)
    attn_mfma_kernel<NT, 128, true><<<grid, kWave, 0, s>>>(a);
  else if (a.D == 64)
    attn_mfma_kernel<NT, 64, true><<<grid, kWave, 0, s>>>(a);
  else if (a.D <= 64)
    attn_mfma_kernel<NT, 64, false><<<grid, kWave, 0, s>>>(a);
  else if (a.D <= 128)
    attn_mfma_kernel<NT, 128, false><<<grid, kWave, 0, s>>>(a);
  else
    attn_mfma_kernel<NT, 256, false><<<grid, kWave, 0, s>>>(a);
  return launch_status();
}

inline size_t prefill_lds_bytes(int D) {
  return 2 * (static_cast<size_t>(kPfKeys) * (D + 8) + static_cast<size_t>(D) * (kPfKeys + kPfVPad)) * sizeof(uint16_t);
}

// The list of live (row block, segment) pairs depends on the step, not on the layer: a caller that names the step
// (plan_token != 0, a number that no other step of the process has) gets the planning kernel for the first launch
// of the step only.  What the list was made from is kept here, on the host, and compared.
struct PlanMade {
  long long token = 0;
  const int* seg_row0 = nullptr;
  const int* seg_start = nullptr;
  const int* seg_slot = nullptr;
  unsigned blocks = 0, segments = 0;
  int group = 0, min_rows = 0, listed = 0;
  void* stream = nullptr;
  int device = -1;
};
static PlanMade g_plan_made;

// The list and its counters are one set of device variables a GPU: a list is current only for the stream and the
// device it was made on (another stream's launches are not ordered behind the planning kernel, another device has
// a list of its own), and for the same step, segments and launch shape.
inline bool plan_is_current(const AttnArgs& a, dim3 grid, int min_rows, int listed, hipStream_t s) {
  int dev = -1;
  if (hipGetDevice(&dev) != hipSuccess) dev = -1;
  const PlanMade now{a.plan_token, a.seg_row0, a.seg_start, a.seg_slot, grid.x, grid.z, a.nq / a.nkv, min_rows, listed,
                     static_cast<void*>(s), dev};
  const bool same = a.plan_token != 0 && dev >= 0 && now.token == g_plan_made.token && now.seg_row0 == g_plan_made.seg_row0 &&
                    now.seg_start == g_plan_made.seg_start && now.seg_slot == g_plan_made.seg_slot &&
                    now.blocks == g_plan_made.blocks && now.segments == g_plan_made.segments &&
                    now.group == g_plan_made.group && now.min_rows == g_plan_made.min_rows && now.listed == g_plan_made.listed &&
                    now.stream == g_plan_made.stream && now.device == g_plan_made.device;
  g_plan_made = now;
  return same;
}

static int g_prefill_pair_up = 1;
static int g_prefill_fixed_rounds = -1;  // items a workgroup up to which they are dealt out before the launch (0: never; -1: by the rule below)
constexpr int kDealtMaxKeys = 4096;      // contexts up to which every launch deals its items out

template <int DMAX, bool EXACT>
int launch_prefill_lds(const AttnArgs& a, dim3 grid, int min_rows, int max_kv_len, hipStream_t s) {
  const size_t lds = prefill_lds_bytes(a.D);
  static size_t allowed = 64 * 1024;  // dynamic LDS above 64 KiB has to be asked for, once per kernel
  if (lds > allowed) {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(&attn_prefill_lds_kernel<DMAX, EXACT>),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(lds));
    if (e != hipSuccess) return static_cast<int>(e);
    allowed = lds;
  }
  static int cus = 0;
  if (cus == 0) {
    int dev = 0, n = 0;
    if (hipGetDevice(&dev) != hipSuccess || hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0)
      n = 256;
    cus = n;
  }
  const long long items = static_cast<long long>(grid.x) * grid.y * grid.z * a.portion_splits;
  const int per_cu = 1;  // eight waves: two on every SIMD, with all the registers they want
  const unsigned workgroups = static_cast<unsigned>(items < static_cast<long long>(per_cu) * cus ? items : per_cu * cus);
  const int listed = static_cast<long long>(grid.x) * grid.z <= kPfPlanMax && grid.x <= 65535 && grid.z <= 65535;
  if (!plan_is_current(a, grid, min_rows, listed, s))
    attn_prefill_plan_kernel<<<1, 256, 0, s>>>(a.seg_row0, a.seg_start, a.seg_slot, static_cast<int>(grid.z),
                                               static_cast<int>(grid.x), a.nq / a.nkv, min_rows, listed);
  if (a.portion_splits > 1 && !listed) return static_cast<int>(hipErrorInvalidValue);  // the merge walks the list
  // dealt out by the rule of launch_prefill_dma_groups (measured there)
  const int fixed_rounds = g_prefill_fixed_rounds >= 0 ? g_prefill_fixed_rounds : (max_kv_len <= kDealtMaxKeys ? 1 << 20 : 2);
  attn_prefill_lds_kernel<DMAX, EXACT><<<workgroups, kPfWaves * kWave, lds, s>>>(a, min_rows, static_cast<int>(grid.x),
                                                                                static_cast<int>(grid.z), listed, fixed_rounds);
  if (a.portion_splits > 1) {
    const long long most = static_cast<long long>(grid.x) * grid.y * grid.z * (kPfRows / kPfWaves);
    attn_merge_portions_kernel<<<static_cast<unsigned>(most < 4LL * cus ? most : 4LL * cus), kPfWaves * kWave, 0, s>>>(a);
  }
  return launch_status();
}


static int g_prefill_groups = -1;  // -1: the launcher decides; 1, 2: forced (measurements and tests)

template <int GROUPS>
int launch_prefill_dma_groups(const AttnArgs& a, dim3 grid, int min_rows, int cus, int max_kv_len, hipStream_t s) {
  const size_t lds = GROUPS * 2 * kDmStageBytes;
  static bool asked = false;  // dynamic LDS of 64 KiB and more has to be asked for, once
  if (!asked) {
    for (const void* kernel : {reinterpret_cast<const void*>(&attn_prefill_dma_kernel<true, GROUPS>),
                               reinterpret_cast<const void*>(&attn_prefill_dma_kernel<false, GROUPS>)}) {
      hipError_t e = hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(lds));
      if (e != hipSuccess) {
        (void)hipGetLastError();
        return static_cast<int>(e);
      }
    }
    asked = true;
  }
  const long long items = static_cast<long long>(grid.x) * grid.y * grid.z * a.portion_splits;
  const long long places = (GROUPS == 1 ? 2LL : 1LL) * cus;  // two workgroups of four waves a CU, or one of eight
  const unsigned workgroups = static_cast<unsigned>(items < places ? items : places);
  const int listed = static_cast<long long>(grid.x) * grid.z <= kPfPlanMax && grid.x <= 65535 && grid.z <= 65535;
  if (a.portion_splits > 1 && !listed) return static_cast<int>(hipErrorInvalidValue);
  if (!plan_is_current(a, grid, min_rows, listed, s))
    attn_prefill_plan_kernel<<<1, 256, 0, s>>>(a.seg_row0, a.seg_start, a.seg_slot, static_cast<int>(grid.z),
                                               static_cast<int>(grid.x), a.nq / a.nkv, min_rows, listed);
  const int pair_up = GROUPS == 1 && g_prefill_pair_up ? static_cast<int>(cus / (static_cast<long long>(a.nkv) * a.portion_splits)) : 0;
  // Items are dealt out before the launch (see the kernel) when none is long, or when a workgroup gets two at most;
  // with long items, several a workgroup, taking them from the counter follows the compute units' differing speeds
  // and the counter's round trip is little beside an item.  Measured on MI355X, dealt against taken, us: a fresh
  // prompt of 2,048 tokens 56.5 against 65.0, of 1,024 30.7 against 34.9, 504 tokens beside 8 decoded ones 32.9
  // against 42.4, four prompts of 2,048 179 against 190, 512 tokens behind 3,584 cached 62.9 against 71.9, segments
  // of 64 to 800 tokens behind 0 to 2,300 372 against 387; a fresh prompt of 8,192 tokens 615 against 598.
  const int fixed_rounds = g_prefill_fixed_rounds >= 0 ? g_prefill_fixed_rounds : (max_kv_len <= kDealtMaxKeys ? 1 << 20 : 2);
  if (a.P % kDmKeys == 0)
    attn_prefill_dma_kernel<true, GROUPS><<<workgroups, GROUPS * kDmWaves * kWave, lds, s>>>(
        a, min_rows, static_cast<int>(grid.x), static_cast<int>(grid.z), listed, pair_up, fixed_rounds);
  else
    attn_prefill_dma_kernel<false, GROUPS><<<workgroups, GROUPS * kDmWaves * kWave, lds, s>>>(
        a, min_rows, static_cast<int>(grid.x), static_cast<int>(grid.z), listed, pair_up, fixed_rounds);
  if (a.portion_splits > 1) {
    const long long most = static_cast<long long>(grid.x) * grid.y * grid.z * (kPfRows / kPfWaves);
    attn_merge_portions_kernel<<<static_cast<unsigned>(most < 4LL * cus ? most : 4LL * cus), kPfWaves * kWave, 0, s>>>(a);
  }
  return launch_status();
}

int launch_prefill_dma(const AttnArgs& a, dim3 grid, int min_rows, int max_qlen, int max_kv_len, hipStream_t s) {
  static int cus = 0;
  if (cus == 0) {
    int dev = 0, n = 0;
    if (hipGetDevice(&dev) != hipSuccess || hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0)
      n = 256;
    cus = n;
  }
  // Every row block goes to two groups of waves where workgroups of four waves would leave the chip part empty:
  // with more than one item for every fourth CU and no more than three for every two (two such workgroups fit a
  // CU), or with up to two a CU when the items are unequal (a fresh prompt, whose last rows see all keys and whose
  // first rows few: the launch lasts as long as its heaviest item).  Items of about one length, two a CU, fill the
  // chip best with four waves each.  Measured on MI355X (32 q heads over 8 kv heads, pages of 16), two groups
  // against one: a fresh prompt of 2,048 tokens 60 against 65 us, of 1,024 tokens 31 against 35, 1,024 tokens
  // behind 3,072 cached 87 against 111; but 512 tokens behind 3,584 (keys in four parts) 79 against 68, eight
  // portions of 256 behind 1,024 each 69 against 62, 8,192 fresh tokens 633 against 604; 512 tokens behind 512
  // cached (one item for every second CU) 27 against 33, a fresh prompt of 128 tokens 12.6 against 11.2.
  const long long items = static_cast<long long>(grid.x) * grid.y * grid.z * a.portion_splits;
  const bool unequal = 2LL * max_qlen > max_kv_len;  // the first rows see less than half of what the last see
  const bool two = g_prefill_groups >= 0 ? g_prefill_groups == 2
                                         : (4 * items > cus && (2 * items <= 3LL * cus || (unequal && items <= 2LL * cus)));
  return two ? launch_prefill_dma_groups<2>(a, grid, min_rows, cus, max_kv_len, s)
             : launch_prefill_dma_groups<1>(a, grid, min_rows, cus, max_kv_len, s);
}

// -1: the launcher decides (below); 1: head_dim 128 portions always run attn_prefill_dma_kernel; 0: always
// attn_prefill_lds_kernel, as every other head_dim does.  For measurements and tests that compare the two.
static int g_prefill_dma = -1;

// The kernel with 32 rows a wave does a tile in two thirds of the time.  Measured inside whole prefill steps of the
// Qwen3-4B shape it is level with the other one for a fresh prompt of 512 tokens and 3 to 5 % of the step ahead
// for portions of 512 behind 512 to 3,584 cached tokens, so it takes every portion that it can.
inline bool prefill_dma_pays(dim3 grid, int max_qlen, int max_kv_len) {
  (void)grid;
  (void)max_qlen;
  (void)max_kv_len;
  if (g_prefill_dma >= 0) return g_prefill_dma != 0;
  return true;
}

}  // namespace arle

using namespace arle;

// A mixed step's decoded tokens beside its portions: the two kinds of segments go to kernels of their own that do
// not depend on each other.  With a side branch the split-KV kernel and its merge are queued on a second stream
// (default priority) between an event that forks it off the caller's stream and one that joins it again, so that
// they run beside the portions kernel; a capture of the caller's stream takes the branch in as parallel nodes.
// Measured on MI355X, 8 decoding requests at 2,048 tokens beside a fresh portion of 504 (Qwen3-4B shape): 8.45
// against 8.80 ms a step, the same bits.
static int g_side_branch = 1;
extern "C" void arle_attn_side_branch(int on) { g_side_branch = on; }

namespace {
struct SideBranch {
  hipStream_t stream = nullptr;
  hipEvent_t fork = nullptr, join = nullptr;
};
SideBranch g_side[64];

// the current device's side stream and events, made at the first call outside a capture (nullptr: there is none:
// making a stream while `s` is being captured would break the capture, so such a call does without the branch)
SideBranch* side_branch(hipStream_t s) {
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return nullptr;
  SideBranch& b = g_side[dev];
  if (b.stream == nullptr) {
    hipStreamCaptureStatus capturing = hipStreamCaptureStatusNone;
    if (hipStreamIsCapturing(s, &capturing) != hipSuccess || capturing != hipStreamCaptureStatusNone) {
      (void)hipGetLastError();
      return nullptr;
    }
    if (hipStreamCreateWithFlags(&b.stream, hipStreamNonBlocking) != hipSuccess ||
        hipEventCreateWithFlags(&b.fork, hipEventDisableTiming) != hipSuccess ||
        hipEventCreateWithFlags(&b.join, hipEventDisableTiming) != hipSuccess) {
      (void)hipGetLastError();
      b = SideBranch{};
      return nullptr;
    }
  }
  return &b;
}
}  // namespace

extern "C" void arle_attn_prefill_variant(int dma) { g_prefill_dma = dma; }
extern "C" void arle_attn_prefill_pair_up(int on) { g_prefill_pair_up = on; }
extern "C" void arle_attn_prefill_fixed_rounds(int rounds) { g_prefill_fixed_rounds = rounds; }
extern "C" void arle_attn_prefill_groups(int groups) { g_prefill_groups = groups; }

// Token rows that the split-KV workspace holds for every segment: the most tokens of a segment whose rows
// (tokens x q heads of a kv head) fit one row tile of 16.
extern "C" int arle_attn_ws_rows(int max_qlen, int nq, int nkv) {
  const int G = nkv > 0 ? nq / nkv : 1;
  return max(1, min(max_qlen, 16 / max(G, 1)));
}

static AttnArgs make_args(const void* q, long long q_stride, void* out, long long o_stride, const void* k_pages,
                          const void* v_pages, const int* block_table, int table_stride, const int* seg_row0,
                          const int* seg_slot, const int* seg_start, int max_qlen, int nq, int nkv, int D,
                          int page_size, float scale, int window, int splits, float* ws_o, float* ws_ml) {
  AttnArgs a;
  a.q = static_cast<const uint16_t*>(q);
  a.q_stride = q_stride;
  a.out = static_cast<uint16_t*>(out);
  a.o_stride = o_stride;
  a.ws_o = ws_o;
  a.ws_ml = ws_ml;
  a.k_pages = static_cast<const uint16_t*>(k_pages);
  a.v_pages = static_cast<const uint16_t*>(v_pages);
  a.block_table = block_table;
  a.table_stride = table_stride;
  a.seg_row0 = seg_row0;
  a.seg_slot = seg_slot;
  a.seg_start = seg_start;
  a.nq = nq;
  a.nkv = nkv;
  a.D = D;
  a.P = page_size;
  a.p_shift = __builtin_ctz(static_cast<unsigned>(page_size));
  a.scale_log2 = scale * 1.4426950408889634f;
  a.window = window;
  a.splits = splits;
  a.ws_rows = arle_attn_ws_rows(max_qlen, nq, nkv);
  a.portion_splits = 1;
  a.plan_token = 0;
  a.pws_o = nullptr;
  a.pws_ml = nullptr;
  a.rows_max = 0;
  a.prep_parts = nullptr;
  a.prep_bf16 = 0;
  a.prep_n = 0;
  a.prep_part_stride = a.prep_row_stride = 0;
  a.prep_qw = a.prep_kw = nullptr;
  a.prep_w_f32 = 0;
  a.prep_cos = a.prep_sin = nullptr;
  a.prep_rot = 0;
  a.prep_eps = 0.f;
  a.prep_k_pages = a.prep_v_pages = nullptr;
  return a;
}

// q, out: bfloat16 [token rows, nq*D] (row strides in elements).  Segments describe the packed
// step: seg_row0[s]..seg_row0[s+1] are the token rows of segment s, whose first token sits at
// position seg_start[s] of the request in block-table row seg_slot[s]; the cache already holds
// the keys and values of these tokens.  max_qlen / min_qlen are the longest and shortest segment, max_kv_len the most
// keys that a segment of more than one token holds after the step (it only steers choices of the portions kernels).  With splits > 1,
// ws_o/ws_ml must hold [segments * ws_rows][nq][splits][D] and [..][2] floats, ws_rows = arle_attn_ws_rows(...),
// and the merge runs after; the split is over the keys of segments of at most 16 rows (decoded tokens and
// portions of a few tokens).  Longer portions go to the LDS kernel; when they have too few row blocks to fill
// the chip, portion_splits > 1 cuts the keys of every row block into that many parts (at most 8), pws_o/pws_ml
// must hold [token rows][nq][portion_splits][D] and [..][2] floats, and a merge of their own runs after.
// plan_token: 0, or a number that names the step (the same for every layer of it, another for every other step of
// the process): the portions kernels then list their work once a step instead of once a call.
// Requires D % 16 == 0, D <= 256, page_size a power of two >= 4.
extern "C" int arle_attn_paged_mfma(const void* q, long long q_stride, void* out, long long o_stride,
                                    const void* k_pages, const void* v_pages, const int* block_table,
                                    int table_stride, const int* seg_row0, const int* seg_slot,
                                    const int* seg_start, int segments, int max_qlen, int min_qlen,
                                    int max_kv_len, int token_rows,
                                    int nq, int nkv, int D, int page_size, float scale, int window,
                                    int splits, float* ws_o, float* ws_ml, int portion_splits, float* pws_o,
                                    float* pws_ml, long long plan_token, void* stream) {
  if (segments == 0 || token_rows == 0) return 0;
  if (D % 16 != 0 || D > 256 || D <= 0 || page_size < 4 || (page_size & (page_size - 1)) != 0 || nq % nkv != 0 ||
      splits < 1 || splits > 64 || portion_splits < 1 || portion_splits > kPortionPartsMax ||
      (portion_splits > 1 && (pws_o == nullptr || pws_ml == nullptr)))
    return static_cast<int>(hipErrorInvalidValue);
  hipStream_t s = static_cast<hipStream_t>(stream);
  AttnArgs a = make_args(q, q_stride, out, o_stride, k_pages, v_pages, block_table, table_stride, seg_row0, seg_slot,
                         seg_start, max_qlen, nq, nkv, D, page_size, scale, window, splits, ws_o, ws_ml);
  a.portion_splits = portion_splits;
  a.pws_o = pws_o;
  a.pws_ml = pws_ml;
  a.plan_token = plan_token;
  const int G = nq / nkv;
  const int max_rows = max_qlen * G, min_rows = min_qlen * G;
  const long long z = static_cast<long long>(segments) * splits;
  if (nkv > 65535 || z > 65535) return static_cast<int>(hipErrorInvalidValue);
  int rc = 0;
  const bool lds_ok = prefill_lds_bytes(D) <= 160 * 1024;
  if (max_rows > 16 && lds_ok) {
    // prompt portions through the LDS kernel; segments of at most 16 rows (decoded tokens of a mixed
    // step) through the streaming kernel
    dim3 grid((max_rows + kPfRows - 1) / kPfRows, nkv, segments);
    SideBranch* side = (min_rows <= 16 && g_side_branch) ? side_branch(s) : nullptr;
    if (side != nullptr) {   // fork: what follows on the side stream waits for what the caller queued so far
      if (hipEventRecord(side->fork, s) != hipSuccess) return static_cast<int>(hipGetLastError());
      if (hipStreamWaitEvent(side->stream, side->fork, 0) != hipSuccess) {
        side = nullptr;      // nothing was queued on the side stream: go on without the branch
        (void)hipGetLastError();
      }
    }
    int side_rc = 0;
    if (side != nullptr) {
      AttnArgs b = a;
      b.rows_max = 16;
      side_rc = launch_attn<1>(b, dim3(1, nkv, static_cast<unsigned>(z)), side->stream);
      if (side_rc == 0 && splits > 1) {
        attn_merge_kernel<<<dim3(segments * b.ws_rows, nq), kMergeWaves * kWave, 0, side->stream>>>(
            ws_o, ws_ml, b.out, o_stride, seg_row0, b.ws_rows, b.rows_max, nq, nkv, D, splits);
        side_rc = launch_status();
      }
    }
    if (side != nullptr && side_rc != 0) {
      // the branch is forked off already: it is joined before the error goes back, so that a capture of `s` does not
      // end with a stream that never came home, and nothing is still writing when the caller goes on
      if (hipEventRecord(side->join, side->stream) == hipSuccess) (void)hipStreamWaitEvent(s, side->join, 0);
      (void)hipGetLastError();
      return side_rc;
    }
    if (D == 64)
      rc = launch_prefill_lds<64, true>(a, grid, 17, max_kv_len, s);
    else if (D == 128 && page_size % 8 == 0 && static_cast<long long>(nkv) * page_size * D < (1LL << 31) &&
             prefill_dma_pays(grid, max_qlen, max_kv_len))
      rc = launch_prefill_dma(a, grid, 17, max_qlen, max_kv_len, s);
    else if (D == 128)
      rc = launch_prefill_lds<128, true>(a, grid, 17, max_kv_len, s);
    else if (D <= 64)
      rc = launch_prefill_lds<64, false>(a, grid, 17, max_kv_len, s);
    else if (D <= 128)
      rc = launch_prefill_lds<128, false>(a, grid, 17, max_kv_len, s);
    else
      rc = launch_prefill_lds<256, false>(a, grid, 17, max_kv_len, s);
    if (side != nullptr) {   // join: the caller's stream goes on when the side branch is done, also after an error
      const bool joined = hipEventRecord(side->join, side->stream) == hipSuccess && hipStreamWaitEvent(s, side->join, 0) == hipSuccess;
      if (!joined) {
        const int e = static_cast<int>(hipGetLastError());
        return rc != 0 ? rc : e;
      }
      return rc;
    }
    if (rc != 0 || min_rows > 16) return rc;
    a.rows_max = 16;
    rc = launch_attn<1>(a, dim3(1, nkv, static_cast<unsigned>(z)), s);
    if (rc != 0 || splits == 1) return rc;
    attn_merge_kernel<<<dim3(segments * a.ws_rows, nq), kMergeWaves * kWave, 0, s>>>(
        ws_o, ws_ml, a.out, o_stride, seg_row0, a.ws_rows, a.rows_max, nq, nkv, D, splits);
    return launch_status();
  }
  if (max_rows > 16 && splits > 1) return static_cast<int>(hipErrorInvalidValue);  // two row tiles: no split
  // one row tile of 16 when a segment's rows fit it (decoded tokens), else two
  const int nt = max_rows <= 16 ? 1 : 2;
  dim3 grid((max_rows + 16 * nt - 1) / (16 * nt), nkv, static_cast<unsigned>(z));
  rc = nt == 1 ? launch_attn<1>(a, grid, s) : launch_attn<2>(a, grid, s);
  if (rc != 0 || splits == 1) return rc;
  attn_merge_kernel<<<dim3(segments * a.ws_rows, nq), kMergeWaves * kWave, 0, s>>>(
      ws_o, ws_ml, a.out, o_stride, seg_row0, a.ws_rows, 0, nq, nkv, D, splits);
  return launch_status();
}

static int g_decode_inwg = -1;   // the splits of a decode step inside one workgroup: -1 by the rule, 0 never, 1 whenever they fit
extern "C" void arle_attn_decode_inwg(int mode) { g_decode_inwg = mode; }

static int compute_units() {
  static int cus = 0;
  if (cus == 0) {
    int dev = 0, n = 0;
    if (hipGetDevice(&dev) != hipSuccess || hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0)
      n = 256;
    cus = n;
  }
  return cus;
}

// A step of single decoded tokens with the preparation of q, k and v folded into the attention: segment s is the
// one token row s.  parts: the fused q|k|v projection of the step as n_parts float32 partial products
// [token rows][(nq + 2 nkv) D] (part_stride elements apart, rows row_stride apart; both multiples of 8, parts
// 16-byte aligned), added in order; or, with parts_bf16, the projection itself in bfloat16 (n_parts 1).  q_w / k_w: per-head norm weights [D] (both or neither; float32 if w_f32, else
// bfloat16; 16-byte aligned), eps inside the root.  cos / sin: float32 [positions][rot / 2], rot 0 (no rotation) or a
// multiple of 64 up to D.  The new token's key and value are written to its slot of the pages (which the block table
// must already hold) and take part in the attention from registers.  D 64 or 128, nq / nkv <= 16; everything else
// as arle_attn_paged_mfma with max_qlen 1.  The same results as arle_qk_prep followed by arle_attn_paged_mfma but
// for the order in which a head's squares are added for its norm.
extern "C" int arle_attn_decode_prep(const void* parts, int parts_bf16, int n_parts, long long part_stride, long long row_stride,
                                     const void* q_w, const void* k_w, int w_f32, const float* cos_t, const float* sin_t,
                                     int rot, float eps, void* out, long long o_stride, void* k_pages, void* v_pages,
                                     const int* block_table, int table_stride, const int* seg_row0, const int* seg_slot,
                                     const int* seg_start, int segments, int nq, int nkv, int D, int page_size,
                                     float scale, int window, int splits, float* ws_o, float* ws_ml, void* stream) {
  if (segments == 0) return 0;
  auto aligned = [](const void* p) { return reinterpret_cast<uintptr_t>(p) % 16 == 0; };
  if ((D != 64 && D != 128) || page_size < 4 || (page_size & (page_size - 1)) != 0 || nkv <= 0 || nq % nkv != 0 ||
      nq / nkv > 16 || splits < 1 || splits > 64 || (splits > 1 && (ws_o == nullptr || ws_ml == nullptr)) ||
      parts == nullptr || n_parts < 1 || (parts_bf16 && n_parts != 1) || part_stride % 8 != 0 || row_stride % 8 != 0 ||
      !aligned(parts) ||
      (q_w == nullptr) != (k_w == nullptr) || !aligned(q_w) || !aligned(k_w) || rot < 0 || rot > D || rot % 64 != 0 ||
      (rot > 0 && (cos_t == nullptr || sin_t == nullptr || !aligned(cos_t) || !aligned(sin_t))) ||
      k_pages == nullptr || v_pages == nullptr || !aligned(k_pages))
    return static_cast<int>(hipErrorInvalidValue);
  const long long z = static_cast<long long>(segments) * splits;
  if (nkv > 65535 || z > 65535) return static_cast<int>(hipErrorInvalidValue);
  hipStream_t s = static_cast<hipStream_t>(stream);
  AttnArgs a = make_args(nullptr, 0, out, o_stride, k_pages, v_pages, block_table, table_stride, seg_row0, seg_slot,
                         seg_start, 1, nq, nkv, D, page_size, scale, window, splits, ws_o, ws_ml);
  a.prep_parts = parts;
  a.prep_bf16 = parts_bf16;
  a.prep_n = n_parts;
  a.prep_part_stride = part_stride;
  a.prep_row_stride = row_stride;
  a.prep_qw = q_w;
  a.prep_kw = k_w;
  a.prep_w_f32 = w_f32;
  a.prep_cos = cos_t;
  a.prep_sin = sin_t;
  a.prep_rot = rot;
  a.prep_eps = eps;
  a.prep_k_pages = static_cast<uint16_t*>(k_pages);
  a.prep_v_pages = static_cast<uint16_t*>(v_pages);
  // two to four splits and a workgroup for every compute unit even so: the splits of a (segment, kv head) share a
  // workgroup and merge in LDS (measured on MI355X at the Qwen3-4B widths, 64 requests at 2,048 tokens in two splits)
  if (splits > 1 && splits <= kInWgWavesMax && g_decode_inwg != 0 &&
      (g_decode_inwg > 0 || static_cast<long long>(segments) * nkv >= compute_units())) {
    const dim3 grid(1, nkv, static_cast<unsigned>(segments));
    if (D == 128 && parts_bf16)
      attn_mfma_kernel<1, 128, true, true, true, true><<<grid, splits * kWave, 0, s>>>(a);
    else if (D == 128)
      attn_mfma_kernel<1, 128, true, true, true, false><<<grid, splits * kWave, 0, s>>>(a);
    else if (parts_bf16)
      attn_mfma_kernel<1, 64, true, true, true, true><<<grid, splits * kWave, 0, s>>>(a);
    else
      attn_mfma_kernel<1, 64, true, true, true, false><<<grid, splits * kWave, 0, s>>>(a);
    return launch_status();
  }
  const dim3 grid(1, nkv, static_cast<unsigned>(z));
  if (D == 128 && parts_bf16)
    attn_mfma_kernel<1, 128, true, true, false, true><<<grid, kWave, 0, s>>>(a);
  else if (D == 128)
    attn_mfma_kernel<1, 128, true, true, false, false><<<grid, kWave, 0, s>>>(a);
  else if (parts_bf16)
    attn_mfma_kernel<1, 64, true, true, false, true><<<grid, kWave, 0, s>>>(a);
  else
    attn_mfma_kernel<1, 64, true, true, false, false><<<grid, kWave, 0, s>>>(a);
  const int rc = launch_status();
  if (rc != 0 || splits == 1) return rc;
  attn_merge_kernel<<<dim3(segments * a.ws_rows, nq), kMergeWaves * kWave, 0, s>>>(
      ws_o, ws_ml, a.out, o_stride, seg_row0, a.ws_rows, 0, nq, nkv, D, splits);
  return launch_status();
}

// ---- the entry point that allocates nothing (attention_static.h) ---------------------------------------------
//
// The split-KV partial results live in this array.  In host code its name is only a handle for
// hipGetSymbolAddress: each GPU holds its own copy at its own address, looked up once per device below, and
// host code uses that address wherever it needs the memory.
static __device__ __align__(256) float scratch[kAttnStaticOFloats + kAttnStaticMlFloats];

namespace {
constexpr int kStaticDevicesMax = 64;
float* g_static_ptr[kStaticDevicesMax];   // per device: where its copy of `scratch` lies
std::mutex g_static_lock;
thread_local char g_static_error[256] = "";

int static_refuse(const char* what, long long got, long long most) {
  std::snprintf(g_static_error, sizeof(g_static_error), "arle_attn_decode_static: %s %lld exceeds the maximum %lld",
                what, got, most);
  return static_cast<int>(hipErrorInvalidValue);
}

// The current device's address of `scratch` (looked up at the first call on that device, with it current).
int static_scratch(float** ptr) {
  int dev = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return static_cast<int>(e);
  if (dev < 0 || dev >= kStaticDevicesMax) return static_cast<int>(hipErrorInvalidDevice);
  std::lock_guard<std::mutex> guard(g_static_lock);
  if (g_static_ptr[dev] == nullptr) {
    void* p = nullptr;
    e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
    if (e != hipSuccess) return static_cast<int>(e);
    if (p == nullptr) return static_cast<int>(hipErrorInvalidSymbol);
    g_static_ptr[dev] = static_cast<float*>(p);
  }
  *ptr = g_static_ptr[dev];
  return 0;
}
}  // namespace

extern "C" const char* arle_attn_decode_static_error() { return g_static_error; }

extern "C" int arle_attn_decode_static(const void* q, long long q_stride, void* out, long long o_stride,
                                       const void* k_pages, const void* v_pages, const int* block_table,
                                       int table_stride, const int* seg_row0, const int* seg_slot,
                                       const int* seg_start, int segments, int max_qlen, int nq, int nkv, int D,
                                       int page_size, float scale, int window, int splits, void* stream) {
  g_static_error[0] = 0;
  if (segments == 0) return 0;
  if (segments < 0 || max_qlen < 1 || nq <= 0 || nkv <= 0 || nq % nkv != 0 || D % 16 != 0 || D > 256 || D <= 0 ||
      page_size < 4 || (page_size & (page_size - 1)) != 0 || splits < 1 || splits > 64) {
    std::snprintf(g_static_error, sizeof(g_static_error),
                  "arle_attn_decode_static: needs head_dim %% 16 == 0 and <= 256, a power-of-two page size >= 4, "
                  "q heads a multiple of kv heads and 1..64 splits");
    return static_cast<int>(hipErrorInvalidValue);
  }
  const int G = nq / nkv;
  if (static_cast<long long>(max_qlen) * G > 16) return static_refuse("rows of a segment (tokens x group)", static_cast<long long>(max_qlen) * G, 16);
  const long long z = static_cast<long long>(segments) * splits;
  if (nkv > 65535) return static_refuse("kv heads", nkv, 65535);
  if (z > 65535) return static_refuse("segments x splits", z, 65535);
  const long long entries = static_cast<long long>(segments) * arle_attn_ws_rows(max_qlen, nq, nkv) * nq * splits;
  float* ws = nullptr;
  if (splits > 1) {
    if (entries * D > kAttnStaticOFloats) return static_refuse("partial outputs (floats)", entries * D, kAttnStaticOFloats);
    if (entries * 2 > kAttnStaticMlFloats) return static_refuse("partial statistics (floats)", entries * 2, kAttnStaticMlFloats);
    const int rc = static_scratch(&ws);
    if (rc != 0) {
      std::snprintf(g_static_error, sizeof(g_static_error),
                    "arle_attn_decode_static: the device address of the scratch array could not be found (HIP error %d)", rc);
      return rc;
    }
  }
  hipStream_t s = static_cast<hipStream_t>(stream);
  float* ws_o = ws;
  float* ws_ml = ws != nullptr ? ws + kAttnStaticOFloats : nullptr;
  AttnArgs a = make_args(q, q_stride, out, o_stride, k_pages, v_pages, block_table, table_stride, seg_row0, seg_slot,
                         seg_start, max_qlen, nq, nkv, D, page_size, scale, window, splits, ws_o, ws_ml);
  int rc = launch_attn<1>(a, dim3(1, nkv, static_cast<unsigned>(z)), s);
  if (rc != 0 || splits == 1) return rc;
  attn_merge_kernel<<<dim3(segments * a.ws_rows, nq), kMergeWaves * kWave, 0, s>>>(
      ws_o, ws_ml, a.out, o_stride, seg_row0, a.ws_rows, 0, nq, nkv, D, splits);
  return launch_status();
}
