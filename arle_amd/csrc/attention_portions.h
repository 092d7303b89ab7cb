// Prompt portions through LDS: the list of work and its planning kernel, the kernel for any head_dim, and the merge
// of a portion's parts.  Included by attention_mfma.hip behind attention_stream.h.
#pragma once
#include "common.h"
#include "attention_args.h"

namespace arle {

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
          // by the keys that were fetched: in front of a window of a few keys those are the window's first four,
          // which may reach past the last token
          const int off = min(max(tile * kPfKeys + v_off[j], kv_lo & ~3), (kv_hi - 1) & ~3);
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

}  // namespace arle
