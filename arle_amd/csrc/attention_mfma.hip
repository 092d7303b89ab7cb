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

namespace arle {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x4 __attribute__((ext_vector_type(4)));

struct AttnArgs {
  const uint16_t* q;
  int64_t q_stride;
  uint16_t* out;
  int64_t o_stride;
  float* ws_o;   // [token row][q head][split][D]   (splits > 1)
  float* ws_ml;  // [token row][q head][split][2]
  const uint16_t* k_pages;  // [page][kv head][slot][D]
  const uint16_t* v_pages;  // [page][kv head][D][slot]
  const int* block_table;
  int table_stride;
  const int* seg_row0;   // [segments + 1] first token row of each segment
  const int* seg_slot;   // [segments]
  const int* seg_start;  // [segments] position of a segment's first token
  int nq, nkv, D, P;
  float scale_log2;
  int window;  // 0: all earlier keys
  int splits;
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

template <int NT, int DMAX>
__global__ __launch_bounds__(kWave) void attn_mfma_kernel(const AttnArgs a) {
  constexpr int DCH = DMAX / 32;  // contraction chunks of the first product
  constexpr int DTL = DMAX / 16;  // d tiles of the output
  const int lane = threadIdx.x, li = lane & 15, g = lane >> 4;
  const int seg = blockIdx.z / a.splits, split = blockIdx.z % a.splits;
  const int kvh = blockIdx.y;
  const int G = a.nq / a.nkv;
  const int row0 = a.seg_row0[seg];
  const int qlen = a.seg_row0[seg + 1] - row0;
  const int rows = qlen * G;
  const int row_begin = blockIdx.x * (16 * NT);
  if (row_begin >= rows) return;  // the whole wave leaves
  const int start = a.seg_start[seg];
  const int* table = a.block_table + static_cast<int64_t>(a.seg_slot[seg]) * a.table_stride;
  const int D = a.D, P = a.P;
  const int n_dch = (D + 31) / 32, n_dt = D / 16;

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
    const uint16_t* qp = a.q + static_cast<int64_t>(row0 + my_tok[n]) * a.q_stride + my_head[n] * D;
#pragma unroll
    for (int c = 0; c < DCH; ++c) {
      const int d = 32 * c + 8 * g;
      qreg[n][c] = (c < n_dch && d < D) ? load_bf16x8(qp + d) : zero_bf16x8();
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
  const int pg_last = (kv_hi - 1) / P;
  int pg_base = 0, pg_reg = 0;
  auto refill_pages = [&](int first_page) {
    pg_base = first_page;
    pg_reg = table[min(first_page + lane, pg_last)];
  };
  auto page_of = [&](int key) { return __shfl(pg_reg, key / P - pg_base, kWave); };
  auto clamp_key = [&](int key) { return min(max(key, kv_lo), kv_hi - 1); };
  // the blocks blk and blk + 1 are in use at any time: make sure the register covers both
  auto cover = [&](int blk) {
    const int first = clamp_key(blk * 32) / P, last = clamp_key(blk * 32 + 63) / P;
    if (first < pg_base || last >= pg_base + kWave) refill_pages(first);
  };

  auto load_k = [&](int blk, bf16x8 (&kreg)[2][DCH]) {
#pragma unroll
    for (int t = 0; t < 2; ++t) {
      const int key = clamp_key(blk * 32 + 16 * t + li);  // a held, written key; out-of-range ones are masked below
      const int page = page_of(key);
      const uint16_t* kp = a.k_pages + page * page_elems + k_head + static_cast<int64_t>(key % P) * D;
#pragma unroll
      for (int c = 0; c < DCH; ++c) {
        const int d = 32 * c + 8 * g;
        kreg[t][c] = (c < n_dch && d < D) ? load_bf16x8(kp + d) : zero_bf16x8();
      }
    }
  };

  // values of a block: for each 16-key tile the 4 keys 4g..4g+3, at d = 16*dt + li
  auto load_v = [&](int blk, uint2 (&vreg)[2][DTL]) {
#pragma unroll
    for (int t = 0; t < 2; ++t) {
      int key4 = blk * 32 + 16 * t + 4 * g;
      key4 = min(max(key4, kv_lo & ~3), (kv_hi - 1) & ~3);
      const int page = page_of(key4);
      const uint16_t* vp = a.v_pages + page * page_elems + k_head + (key4 % P);
#pragma unroll
      for (int dt = 0; dt < DTL; ++dt) {
        if (dt < n_dt) vreg[t][dt] = *reinterpret_cast<const uint2*>(vp + static_cast<int64_t>(16 * dt + li) * P);
      }
    }
  };

  bf16x8 kcur[2][DCH];
  uint2 vraw[2][DTL];
  if (b0 < b1) {
    refill_pages(clamp_key(b0 * 32) / P);
    load_k(b0, kcur);
    load_v(b0, vraw);
  }

  for (int blk = b0; blk < b1; ++blk) {
    const int key_base = blk * 32;
    const bool more = blk + 1 < b1;
    if (more) cover(blk + 1);

    // scores S^T: s[n][t][r] belongs to key key_base + 16t + 4g + r and row (n, li)
    f32x4 s[NT][2];
#pragma unroll
    for (int n = 0; n < NT; ++n)
#pragma unroll
      for (int t = 0; t < 2; ++t) {
        f32x4 z = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int c = 0; c < DCH; ++c)
          if (c < n_dch) z = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kcur[t][c], qreg[n][c], z, 0, 0, 0);
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
          if (dt >= n_dt) continue;
          if (key4 + 0 >= kv_total) vraw[t][dt].x &= 0xffff0000u;
          if (key4 + 1 >= kv_total) vraw[t][dt].x &= 0x0000ffffu;
          if (key4 + 2 >= kv_total) vraw[t][dt].y &= 0xffff0000u;
          if (key4 + 3 >= kv_total) vraw[t][dt].y &= 0x0000ffffu;
        }
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
          packed[2 * t + r / 2] = static_cast<uint32_t>(f32_to_bf16_bits(p0)) |
                                  (static_cast<uint32_t>(f32_to_bf16_bits(p1)) << 16);
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
      if (dt < n_dt) {
        uint4 vv = {vraw[0][dt].x, vraw[0][dt].y, vraw[1][dt].x, vraw[1][dt].y};
        const bf16x8 vop = __builtin_bit_cast(bf16x8, vv);
#pragma unroll
        for (int n = 0; n < NT; ++n)
          acc[n][dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vop, pb[n], acc[n][dt], 0, 0, 0);
      }
    }
    // and the value registers after the second product
    if (more) load_v(blk + 1, vraw);
  }

  // acc[n][dt][r] is O^T[d = 16dt + 4g + r][row (n, li)]
#pragma unroll
  for (int n = 0; n < NT; ++n) {
    if (!row_ok[n]) continue;
    const int64_t tok_row = row0 + my_tok[n];
    if (a.splits == 1) {
      const float inv_l = l[n] > 0.f ? 1.0f / l[n] : 0.f;
      uint16_t* op = a.out + tok_row * a.o_stride + my_head[n] * D;
#pragma unroll
      for (int dt = 0; dt < DTL; ++dt) {
        if (dt < n_dt) {
          uint2 w;
          w.x = static_cast<uint32_t>(f32_to_bf16_bits(acc[n][dt][0] * inv_l)) |
                (static_cast<uint32_t>(f32_to_bf16_bits(acc[n][dt][1] * inv_l)) << 16);
          w.y = static_cast<uint32_t>(f32_to_bf16_bits(acc[n][dt][2] * inv_l)) |
                (static_cast<uint32_t>(f32_to_bf16_bits(acc[n][dt][3] * inv_l)) << 16);
          *reinterpret_cast<uint2*>(op + 16 * dt + 4 * g) = w;
        }
      }
    } else {
      const int64_t slot = (tok_row * a.nq + my_head[n]) * a.splits + split;
      float* wo = a.ws_o + slot * D;
#pragma unroll
      for (int dt = 0; dt < DTL; ++dt) {
        if (dt < n_dt) {
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

// out[row][head][:] = sum_s o_s 2^(m_s - m) / sum_s l_s 2^(m_s - m).   One wave per (row, head);
// lane s holds the statistics of split s (splits <= 64), the weights travel by cross-lane reads, and
// the partial outputs are read with independent loads.
__global__ __launch_bounds__(kWave) void attn_merge_kernel(const float* __restrict__ ws_o,
                                                           const float* __restrict__ ws_ml,
                                                           uint16_t* __restrict__ out, int64_t o_stride,
                                                           int nq, int D, int splits) {
  const int row = blockIdx.x, head = blockIdx.y, lane = threadIdx.x;
  const int64_t base = (static_cast<int64_t>(row) * nq + head) * splits;
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
  for (int d = lane; d < D; d += kWave) {
    float o = 0.f;
#pragma unroll 4
    for (int s = 0; s < splits; ++s) o += ws_o[(base + s) * D + d] * __shfl(wgt, s, kWave);
    out[static_cast<int64_t>(row) * o_stride + head * D + d] = f32_to_bf16_bits(o * inv);
  }
}

template <int NT>
int launch_attn(const AttnArgs& a, dim3 grid, hipStream_t s) {
  if (a.D <= 64)
    attn_mfma_kernel<NT, 64><<<grid, kWave, 0, s>>>(a);
  else if (a.D <= 128)
    attn_mfma_kernel<NT, 128><<<grid, kWave, 0, s>>>(a);
  else
    attn_mfma_kernel<NT, 256><<<grid, kWave, 0, s>>>(a);
  return launch_status();
}

}  // namespace arle

using namespace arle;

// q, out: bfloat16 [token rows, nq*D] (row strides in elements).  Segments describe the packed
// step: seg_row0[s]..seg_row0[s+1] are the token rows of segment s, whose first token sits at
// position seg_start[s] of the request in block-table row seg_slot[s]; the cache already holds
// the keys and values of these tokens.  max_qlen is the longest segment.  With splits > 1,
// ws_o/ws_ml must hold [token rows][nq][splits][D] and [..][2] floats and the merge runs after.
// Requires D % 16 == 0, D <= 256, page_size % 4 == 0.
extern "C" int arle_attn_paged_mfma(const void* q, long long q_stride, void* out, long long o_stride,
                                    const void* k_pages, const void* v_pages, const int* block_table,
                                    int table_stride, const int* seg_row0, const int* seg_slot,
                                    const int* seg_start, int segments, int max_qlen, int token_rows,
                                    int nq, int nkv, int D, int page_size, float scale, int window,
                                    int splits, float* ws_o, float* ws_ml, void* stream) {
  if (segments == 0 || token_rows == 0) return 0;
  if (D % 16 != 0 || D > 256 || D <= 0 || page_size % 4 != 0 || nq % nkv != 0 || splits < 1 || splits > 64)
    return static_cast<int>(hipErrorInvalidValue);
  hipStream_t s = static_cast<hipStream_t>(stream);
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
  a.scale_log2 = scale * 1.4426950408889634f;
  a.window = window;
  a.splits = splits;
  const int G = nq / nkv;
  const int max_rows = max_qlen * G;
  // one row tile of 16 when a segment's rows fit it (decoded tokens), else two
  const int nt = max_rows <= 16 ? 1 : 2;
  const long long z = static_cast<long long>(segments) * splits;
  if (nkv > 65535 || z > 65535) return static_cast<int>(hipErrorInvalidValue);
  dim3 grid((max_rows + 16 * nt - 1) / (16 * nt), nkv, static_cast<unsigned>(z));
  int rc = nt == 1 ? launch_attn<1>(a, grid, s) : launch_attn<2>(a, grid, s);
  if (rc != 0 || splits == 1) return rc;
  dim3 mgrid(token_rows, nq);
  attn_merge_kernel<<<mgrid, kWave, 0, s>>>(ws_o, ws_ml, a.out, o_stride, nq, D, splits);
  return launch_status();
}
