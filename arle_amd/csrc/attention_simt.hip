// Paged causal attention, one wave per (token row, q head), 32-bit arithmetic.
//
//   s_c = (q . k_c) / sqrt(D)   for keys  first <= c <= pos   (first = 0, or pos-window+1)
//   o   = sum_c softmax(s)_c v_c
// q head h reads kv head h / (nq/nkv).  Keys and values come from the paged cache
// through the request's block table.  This is the attention of the true 32-bit
// path and the plain counterpart of the MFMA kernels; it is also correct for
// bfloat16 storage (scores, probabilities and sums stay 32-bit).
//
// Keys are walked in tiles of 64 aligned to absolute key index, in ascending
// order, so the sequence of floating-point operations for a row depends only on
// that row's position and window, never on how the prompt was cut into steps,
// on the other rows of the batch, or on which physical pages hold the keys.
// reference counterparts: crates/cuda-kernels/tools/tilelang/batch_prefill_paged_hd128.py:89-232,
// batch_decode_paged_hd128.py:78-236 (scale infer/src/ops/attention.rs:636).
#include "common.h"

namespace arle {

constexpr int kSimtMaxD = 512;

template <typename T>
__global__ __launch_bounds__(kWave) void attn_paged_simt_kernel(
    const T* __restrict__ q, int64_t q_stride, T* __restrict__ out, int64_t o_stride,
    const T* __restrict__ k_pages, const T* __restrict__ v_pages,
    const int* __restrict__ block_table, int table_stride, const int* __restrict__ positions,
    const int* __restrict__ slot_of_token, const int* __restrict__ row_list, int nq, int nkv, int D,
    int page_size, float scale, int window) {
  extern __shared__ float qs[];  // [D]
  const int t = row_list ? row_list[blockIdx.x] : blockIdx.x;
  const int h = blockIdx.y;
  const int lane = threadIdx.x;
  const int kvh = h / (nq / nkv);
  const int pos = positions[t];
  const int* table = block_table + static_cast<int64_t>(slot_of_token[t]) * table_stride;

  const T* qr = q + static_cast<int64_t>(t) * q_stride + h * D;
  for (int d = lane; d < D; d += kWave) qs[d] = to_float(qr[d]);
  __syncthreads();

  const int first = window > 0 ? max(0, pos - window + 1) : 0;
  const int64_t page_elems = static_cast<int64_t>(nkv) * page_size * D;
  const int64_t head_off = static_cast<int64_t>(kvh) * page_size * D;

  float m = -INFINITY, l = 0.f;
  float acc[kSimtMaxD / kWave];
#pragma unroll
  for (int i = 0; i < kSimtMaxD / kWave; ++i) acc[i] = 0.f;

  for (int tile = first / kWave; tile * kWave <= pos; ++tile) {
    const int c = tile * kWave + lane;
    const bool valid = c >= first && c <= pos;
    float s = -INFINITY;
    if (valid) {
      const int page = table[c / page_size];
      const T* kr = k_pages + page * page_elems + head_off + static_cast<int64_t>(c % page_size) * D;
      float dot = 0.f;
      for (int d = 0; d < D; ++d) dot = fmaf(qs[d], to_float(kr[d]), dot);
      s = dot * scale;
    }
    const float m_new = fmaxf(m, wave_max(s));  // the tile holds at least one visible key
    const float alpha = expf(m - m_new);        // 0 on the first tile (m = -inf)
    const float p = valid ? expf(s - m_new) : 0.f;
    l = l * alpha + wave_sum(p);
#pragma unroll
    for (int i = 0; i < kSimtMaxD / kWave; ++i) acc[i] *= alpha;

    const int j_lo = max(first - tile * kWave, 0);
    const int j_hi = min(pos - tile * kWave, kWave - 1);
    for (int j = j_lo; j <= j_hi; ++j) {
      const float pj = __shfl(p, j, kWave);
      const int cj = tile * kWave + j;
      const int page = table[cj / page_size];
      const T* vr = v_pages + page * page_elems + head_off + (cj % page_size);  // [d][slot in page]
#pragma unroll
      for (int i = 0; i < kSimtMaxD / kWave; ++i) {
        const int d = lane + i * kWave;
        if (d < D) acc[i] = fmaf(pj, to_float(vr[static_cast<int64_t>(d) * page_size]), acc[i]);
      }
    }
    m = m_new;
  }

  T* o = out + static_cast<int64_t>(t) * o_stride + h * D;
  const float inv_l = 1.0f / l;
#pragma unroll
  for (int i = 0; i < kSimtMaxD / kWave; ++i) {
    const int d = lane + i * kWave;
    if (d < D) o[d] = from_float<T>(acc[i] * inv_l);
  }
}

}  // namespace arle

using namespace arle;

// q, out: [tokens, nq*D] with row strides in elements.  k_pages [pages, nkv, page_size, D];
// v_pages [pages, nkv, D, page_size].  block_table: [slots, table_stride].  row_list
// (may be null) names the token rows to process; n_rows is its length, or the
// number of tokens when it is null.  window == 0 means all earlier keys.
extern "C" int arle_attn_paged_simt(const void* q, long long q_stride, void* out,
                                    long long o_stride, const void* k_pages, const void* v_pages,
                                    int dtype, const int* block_table, int table_stride,
                                    const int* positions, const int* slot_of_token,
                                    const int* row_list, int n_rows, int nq, int nkv, int D,
                                    int page_size, float scale, int window, void* stream) {
  if (n_rows == 0) return 0;
  if (D > kSimtMaxD || nq % nkv != 0 || nq > 65535) return static_cast<int>(hipErrorInvalidValue);
  hipStream_t s = static_cast<hipStream_t>(stream);
  dim3 grid(n_rows, nq);
  const size_t lds = static_cast<size_t>(D) * sizeof(float);
  if (dtype == kF32) {
    attn_paged_simt_kernel<float><<<grid, kWave, lds, s>>>(
        static_cast<const float*>(q), q_stride, static_cast<float*>(out), o_stride,
        static_cast<const float*>(k_pages), static_cast<const float*>(v_pages), block_table,
        table_stride, positions, slot_of_token, row_list, nq, nkv, D, page_size, scale, window);
  } else {
    attn_paged_simt_kernel<bf16><<<grid, kWave, lds, s>>>(
        static_cast<const bf16*>(q), q_stride, static_cast<bf16*>(out), o_stride,
        static_cast<const bf16*>(k_pages), static_cast<const bf16*>(v_pages), block_table,
        table_stride, positions, slot_of_token, row_list, nq, nkv, D, page_size, scale, window);
  }
  return launch_status();
}
