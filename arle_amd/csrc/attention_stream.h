// The streaming kernel (single decoded tokens and short portions: operands straight from memory) and the merge of
// its split-KV partial results.  Included by attention_mfma.hip, whose head describes the layouts.
#pragma once
#include "common.h"
#include "attention_args.h"

namespace arle {

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

    // a slot beyond what the request holds may carry stale bits: its value must be 0, not 0 * garbage.  Such slots
    // are fetched in the request's last block only, but not only by the lanes whose own keys they are: with a window
    // of a few keys the lanes of keys in front of it hold the window's first four values instead, which may reach
    // past the last token.  So a lane goes by the keys it fetched.  PREP: the new token's own slot is written behind
    // the loop and stale until then; the lanes that hold it by right get it from registers below.
    const int stale_from = PREP ? start : kv_total;
    if (key_base + 32 > stale_from) {
#pragma unroll
      for (int t = 0; t < 2; ++t) {
        const int key4 = min(max(key_base + 16 * t + 4 * g, kv_lo & ~3), (kv_hi - 1) & ~3);  // as load_v fetched it
#pragma unroll
        for (int dt = 0; dt < DTL; ++dt) {
          if (!EXACT && dt >= n_dt) continue;
          if (key4 + 0 >= stale_from) vraw[dt][2 * t] &= 0xffff0000u;
          if (key4 + 1 >= stale_from) vraw[dt][2 * t] &= 0x0000ffffu;
          if (key4 + 2 >= stale_from) vraw[dt][2 * t + 1] &= 0xffff0000u;
          if (key4 + 3 >= stale_from) vraw[dt][2 * t + 1] &= 0x0000ffffu;
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

}  // namespace arle
