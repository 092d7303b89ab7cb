// Prompt portions at head_dim 128: tiles loaded from memory straight into LDS.  Included by attention_mfma.hip
// behind attention_portions.h, whose list of work and constants it uses.
#pragma once
#include "common.h"
#include "attention_portions.h"

namespace arle {

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

}  // namespace arle
