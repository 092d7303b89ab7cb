// Per-head RMSNorm of q and k, rotary position encoding, and the write of k and v
// into the paged cache, in one pass over the projections of a packed batch.
//
// For every token t and head h (q heads, then k heads, then v heads):
//   x  = head vector [D]
//   x  = x * 1/sqrt(mean(x^2) + eps) * w          (q and k only, if a weight is given)
//   for d < rot/2:  y_d = x_d cos_d - x_{d+rot/2} sin_d ;  y_{d+rot/2} = x_d sin_d + x_{d+rot/2} cos_d
//   (dims >= rot pass through; rot == 0 means no rotation)
//   q -> written back in place; k, v -> cache row of (slot, position), or k in place
//   when no cache is given.
// cos/sin are 32-bit tables [positions, rot/2]; all arithmetic is 32-bit and the
// result is rounded once at the store.
// The projections may also come as a stack of float32 partial products [n_parts][T, (nq + 2 nkv) D]
// (a matrix product whose K was split over workgroups): then every value is the sum of the stack in
// order, q is written to its own buffer and k, v only to the cache.
// reference counterparts: crates/cuda-kernels/csrc/attention/prefill_attention_paged_prep.cu:8-106,
// crates/cuda-kernels/csrc/attention/decode_prep_paged.cu:73-160 (head_dim fixed to 128 there).
//
// Cache layout per layer: keys [page, kv_head, slot_in_page, D]; values [page, kv_head, D, slot_in_page]
// (d-major, so that a matrix-core operand of 4 consecutive keys at one d is one 8-byte load).
#include "common.h"

namespace arle {

constexpr int kPrepWaves = 4;
constexpr int kMaxHeadDim = 512;

template <typename T, typename TW>
__global__ __launch_bounds__(kPrepWaves* kWave) void qk_prep_kernel(
    T* __restrict__ q, int64_t q_stride, T* __restrict__ k, int64_t k_stride,
    const T* __restrict__ v, int64_t v_stride, const TW* __restrict__ q_w,
    const TW* __restrict__ k_w, const float* __restrict__ cos_t, const float* __restrict__ sin_t,
    int rot, const int* __restrict__ positions, const int* __restrict__ slot_of_token,
    const int* __restrict__ block_table, int table_stride, T* __restrict__ k_pages,
    T* __restrict__ v_pages, int nq, int nkv, int D, int page_size, float eps,
    const float* __restrict__ parts, int n_parts, int64_t part_stride, int64_t part_row_stride) {
  extern __shared__ float lds[];  // [kPrepWaves][D]
  const int t = blockIdx.x;
  const int wave = threadIdx.x / kWave;
  const int lane = threadIdx.x % kWave;
  const int head = blockIdx.y * kPrepWaves + wave;  // same for all lanes of a wave
  const bool valid = head < nq + 2 * nkv;
  const bool is_v = valid && head >= nq + nkv;
  const bool is_qk = valid && !is_v;
  const bool is_q = head < nq;
  float* x = lds + wave * D;

  const int pos = positions[t];
  int64_t page_base = 0;  // element offset of the token's page, [page, kv head 0, 0, 0]
  const int in_page = pos % page_size;
  if (valid && !is_q && (k_pages || v_pages)) {
    const int slot = slot_of_token[t];
    const int page = block_table[static_cast<int64_t>(slot) * table_stride + pos / page_size];
    page_base = static_cast<int64_t>(page) * nkv * page_size * D;
  }

  // column `col` of token t's fused [q | k | v] row, summed over the stack of partial products
  const float* part_row = parts ? parts + static_cast<int64_t>(t) * part_row_stride : nullptr;
  // The loads carry no condition (a load under a condition is waited for before the next one is issued):
  // whole rounds of four parts, then one round that fetches the last part again where there is none and
  // does not add it.  The adds are in the order of the parts.
  auto summed = [&](int col) {
    const float* p = part_row + col;
    float acc = 0.f;
    int base = 0;
    for (; base + 4 <= n_parts; base += 4) {
      float e[4];
#pragma unroll
      for (int u = 0; u < 4; ++u) e[u] = p[(base + u) * part_stride];
#pragma unroll
      for (int u = 0; u < 4; ++u) acc += e[u];
    }
    if (base < n_parts) {
      float e[3];
#pragma unroll
      for (int u = 0; u < 3; ++u) e[u] = p[min(base + u, n_parts - 1) * part_stride];
#pragma unroll
      for (int u = 0; u < 3; ++u) acc += base + u < n_parts ? e[u] : 0.f;
    }
    return acc;
  };

  if (is_v && v_pages) {  // v head: copy into the cache, d-major inside the page
    const int kvh = head - nq - nkv;
    const T* vsrc = v + static_cast<int64_t>(t) * v_stride + kvh * D;
    T* vdst = v_pages + page_base + static_cast<int64_t>(kvh) * page_size * D + in_page;
    for (int d = lane; d < D; d += kWave)
      vdst[static_cast<int64_t>(d) * page_size] = parts ? from_float<T>(summed(head * D + d)) : vsrc[d];
  }

  const int local = is_q ? head : head - nq;
  T* src = is_q ? q + static_cast<int64_t>(t) * q_stride + local * D
                : k + static_cast<int64_t>(t) * k_stride + local * D;
  if (is_qk) {
    const TW* w = is_q ? q_w : k_w;
    float ss = 0.f;
    for (int d = lane; d < D; d += kWave) {
      const float val = parts ? summed(head * D + d) : to_float(src[d]);
      x[d] = val;
      ss += val * val;
    }
    if (w) {
      ss = wave_sum(ss);
      const float inv = 1.0f / sqrtf(ss / static_cast<float>(D) + eps);
      for (int d = lane; d < D; d += kWave) x[d] = x[d] * inv * to_float(w[d]);
    }
  }
  __syncthreads();  // every thread of the block arrives: the LDS rows are complete
  if (!is_qk) return;

  T* dst = src;
  if (!is_q && k_pages)
    dst = k_pages + page_base + (static_cast<int64_t>(local) * page_size + in_page) * D;
  const int half = rot / 2;
  const float* cs = cos_t + static_cast<int64_t>(pos) * half;
  const float* sn = sin_t + static_cast<int64_t>(pos) * half;
  for (int d = lane; d < D; d += kWave) {
    float y;
    if (d < half) {
      y = x[d] * cs[d] - x[d + half] * sn[d];
    } else if (d < rot) {
      const int p = d - half;
      y = x[p] * sn[p] + x[d] * cs[p];
    } else {
      y = x[d];
    }
    dst[d] = from_float<T>(y);
  }
}

// bfloat16 with a head_dim that is a power of two >= 64 and a rotated width that is a multiple of 16.
// A workgroup takes one head of TPB = 256 / LPH consecutive tokens; a lane holds eight consecutive
// columns: one 16-byte load and one 16-byte store (q in place, k into its cache row), LPH = head_dim / 8
// lanes a token.  The per-head sum of squares and the rotation partner (the lane rot/16 away) go through
// lane shuffles.  A value head is only moved: its pages keep the head's columns as rows ([D][page_size]),
// so when the workgroup's tokens are one run of consecutive positions of one request that starts at a
// multiple of 16 (the usual case in a prompt portion), the tile is turned in LDS and written as 16-byte
// pieces of eight slots; otherwise every element goes to its slot by itself.
constexpr int kPrepHeads = 4;  // q or k heads of a token that one lane group takes
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

template <int LPH, typename TW>
__global__ __launch_bounds__(256) void qk_prep_bf16x8_kernel(
    uint16_t* __restrict__ q, int64_t q_stride, uint16_t* __restrict__ k, int64_t k_stride,
    const uint16_t* __restrict__ v, int64_t v_stride, const TW* __restrict__ q_w, const TW* __restrict__ k_w,
    const float* __restrict__ cos_t, const float* __restrict__ sin_t, int rot, const int* __restrict__ positions,
    const int* __restrict__ slot_of_token, const int* __restrict__ block_table, int table_stride,
    uint16_t* __restrict__ k_pages, uint16_t* __restrict__ v_pages, int tokens, int nq, int nkv, int page_size,
    float eps) {
  constexpr int D = LPH * 8;
  constexpr int TPB = 256 / LPH;
  constexpr int kPitch = D + 8;  // LDS row of the value tile, in elements
  __shared__ __attribute__((aligned(16))) uint16_t tile[TPB >= 16 ? TPB * kPitch : 8];
  const int tl = threadIdx.x / LPH, d0 = (threadIdx.x % LPH) * 8;
  const int row0 = blockIdx.x * TPB;
  const int t = row0 + tl;
  const bool valid = t < tokens;
  // blockIdx.y: groups of kPrepHeads q heads, then groups of k heads, then the v heads one by one
  const int q_groups = (nq + kPrepHeads - 1) / kPrepHeads, k_groups = (nkv + kPrepHeads - 1) / kPrepHeads;
  const int gy = blockIdx.y;
  const bool is_q = gy < q_groups, is_v = gy >= q_groups + k_groups;
  const int local = is_q ? gy * kPrepHeads : (is_v ? gy - q_groups - k_groups : (gy - q_groups) * kPrepHeads);
  const int pos = valid ? positions[t] : 0;
  const int slot = (valid && !is_q) ? slot_of_token[t] : 0;
  if (is_v) {
    if (v_pages == nullptr) return;
    const uint16_t* src = v + static_cast<int64_t>(t) * v_stride + local * D + d0;
    uint4 raw = {0u, 0u, 0u, 0u};
    if (valid) raw = *reinterpret_cast<const uint4*>(src);
    bool run = false;
    if constexpr (TPB >= 16) {
      const int pos_first = positions[row0], slot_first = slot_of_token[row0];
      const bool fits = valid && pos == pos_first + tl && slot == slot_first && pos_first % 16 == 0 &&
                        page_size % 16 == 0;
      run = __syncthreads_and(fits) != 0;
      if (run) {
        *reinterpret_cast<uint4*>(&tile[tl * kPitch + d0]) = raw;
        __syncthreads();
        constexpr int kPieces = TPB / 8;  // 16-byte pieces of eight slots for each column
        const int d = threadIdx.x / kPieces, first = (threadIdx.x % kPieces) * 8;
        uint32_t wds[4];
#pragma unroll
        for (int e = 0; e < 4; ++e)
          wds[e] = static_cast<uint32_t>(tile[(first + 2 * e) * kPitch + d]) |
                   (static_cast<uint32_t>(tile[(first + 2 * e + 1) * kPitch + d]) << 16);
        const int p = pos_first + first;
        const int page = block_table[static_cast<int64_t>(slot_first) * table_stride + p / page_size];
        uint16_t* dst = v_pages + (static_cast<int64_t>(page) * nkv + local) * D * page_size +
                        static_cast<int64_t>(d) * page_size + p % page_size;
        *reinterpret_cast<uint4*>(dst) = uint4{wds[0], wds[1], wds[2], wds[3]};
      }
    }
    if (!run && valid) {
      const int page = block_table[static_cast<int64_t>(slot) * table_stride + pos / page_size];
      uint16_t* dst = v_pages + (static_cast<int64_t>(page) * nkv + local) * D * page_size +
                      static_cast<int64_t>(d0) * page_size + pos % page_size;
      const uint32_t wds[4] = {raw.x, raw.y, raw.z, raw.w};
#pragma unroll
      for (int e = 0; e < 8; ++e)
        dst[static_cast<int64_t>(e) * page_size] = static_cast<uint16_t>(wds[e / 2] >> (16 * (e & 1)));
    }
    return;
  }
  // q or k: up to kPrepHeads heads of this token, all loads first; the angles and the norm's weight are
  // read once for all of them
  const int count = is_q ? nq : nkv;
  const int n_heads = min(kPrepHeads, count - local);
  uint16_t* base = is_q ? q + static_cast<int64_t>(t) * q_stride + d0 : k + static_cast<int64_t>(t) * k_stride + d0;
  u32x4 raw[kPrepHeads];
#pragma unroll
  for (int h = 0; h < kPrepHeads; ++h) {
    const bool live = valid && h < n_heads;
    const u32x4 got = *reinterpret_cast<const u32x4*>(live ? base + (local + h) * D : (is_q ? q : k));
    raw[h] = live ? got : u32x4{0u, 0u, 0u, 0u};
  }
  const int half = rot / 2;
  const bool low = d0 < half, rotated = d0 < rot;
  const int lane = threadIdx.x % kWave;
  const int from = rotated ? (low ? lane + half / 8 : lane - half / 8) : lane;
  float cs[8], sn[8], wt[8];
  {
    const int cd = low ? d0 : d0 - half;  // column of the cos/sin row
    const float* cp = cos_t + static_cast<int64_t>(pos) * half + cd;
    const float* sp = sin_t + static_cast<int64_t>(pos) * half + cd;
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      cs[e] = (rotated && valid) ? cp[e] : 1.0f;
      sn[e] = (rotated && valid) ? sp[e] : 0.0f;
    }
  }
  const TW* w = is_q ? q_w : k_w;
  if (w != nullptr) {
#pragma unroll
    for (int e = 0; e < 8; ++e) wt[e] = to_float(w[d0 + e]);
  }
  int64_t page_row = -1;
  if (!is_q && k_pages && valid) {
    const int page = block_table[static_cast<int64_t>(slot) * table_stride + pos / page_size];
    page_row = static_cast<int64_t>(page) * nkv * page_size + pos % page_size;
  }
  // every lane takes part in the shuffles below (lanes past the last token or head with zeros)
#pragma unroll
  for (int h = 0; h < kPrepHeads; ++h) {
    float x[8];
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      x[2 * e] = __uint_as_float(raw[h][e] << 16);
      x[2 * e + 1] = __uint_as_float(raw[h][e] & 0xffff0000u);
    }
    if (w != nullptr) {
      float ss = 0.f;
#pragma unroll
      for (int e = 0; e < 8; ++e) ss += x[e] * x[e];
#pragma unroll
      for (int off = LPH / 2; off > 0; off >>= 1) ss += __shfl_xor(ss, off, kWave);
      const float inv = 1.0f / sqrtf(ss / static_cast<float>(D) + eps);
#pragma unroll
      for (int e = 0; e < 8; ++e) x[e] = x[e] * inv * wt[e];
    }
    float y[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const float other = __shfl(x[e], from, kWave);
      y[e] = rotated ? (low ? x[e] * cs[e] - other * sn[e] : other * sn[e] + x[e] * cs[e]) : x[e];
    }
    if (valid && h < n_heads) {
      uint16_t* dst = base + (local + h) * D;
      if (page_row >= 0) dst = k_pages + (page_row + static_cast<int64_t>(local + h) * page_size) * D + d0;
      *reinterpret_cast<u32x4*>(dst) = u32x4{pack_bf16x2(y[0], y[1]), pack_bf16x2(y[2], y[3]),
                                             pack_bf16x2(y[4], y[5]), pack_bf16x2(y[6], y[7])};
    }
  }
}

template <int LPH>
int launch_prep_bf16x8(void* q, long long q_stride, void* k, long long k_stride, const void* v, long long v_stride,
                       const void* q_w, const void* k_w, int w_dtype, const float* cos_t, const float* sin_t, int rot,
                       const int* positions, const int* slot_of_token, const int* block_table, int table_stride,
                       void* k_pages, void* v_pages, int tokens, int nq, int nkv, int page_size, float eps,
                       hipStream_t s) {
  constexpr int TPB = 256 / LPH;
  dim3 grid((tokens + TPB - 1) / TPB, (nq + kPrepHeads - 1) / kPrepHeads + (nkv + kPrepHeads - 1) / kPrepHeads + nkv);
  auto u16 = [](const void* p) { return static_cast<uint16_t*>(const_cast<void*>(p)); };
  if (w_dtype == kF32)
    qk_prep_bf16x8_kernel<LPH, float><<<grid, 256, 0, s>>>(
        u16(q), q_stride, u16(k), k_stride, u16(v), v_stride, static_cast<const float*>(q_w),
        static_cast<const float*>(k_w), cos_t, sin_t, rot, positions, slot_of_token, block_table, table_stride,
        u16(k_pages), u16(v_pages), tokens, nq, nkv, page_size, eps);
  else
    qk_prep_bf16x8_kernel<LPH, bf16><<<grid, 256, 0, s>>>(
        u16(q), q_stride, u16(k), k_stride, u16(v), v_stride, static_cast<const bf16*>(q_w),
        static_cast<const bf16*>(k_w), cos_t, sin_t, rot, positions, slot_of_token, block_table, table_stride,
        u16(k_pages), u16(v_pages), tokens, nq, nkv, page_size, eps);
  return launch_status();
}

template <typename T>
int launch_prep(void* q, long long q_stride, void* k, long long k_stride, const void* v,
                long long v_stride, const void* q_w, const void* k_w, int w_dtype,
                const float* cos_t, const float* sin_t, int rot, const int* positions,
                const int* slot_of_token, const int* block_table, int table_stride, void* k_pages,
                void* v_pages, int tokens, int nq, int nkv, int D, int page_size, float eps,
                const float* parts, int n_parts, long long part_stride, long long part_row_stride,
                hipStream_t s) {
  dim3 grid(tokens, (nq + 2 * nkv + kPrepWaves - 1) / kPrepWaves);
  const size_t lds = static_cast<size_t>(kPrepWaves) * D * sizeof(float);
  if (w_dtype == kF32) {
    qk_prep_kernel<T, float><<<grid, kPrepWaves * kWave, lds, s>>>(
        static_cast<T*>(q), q_stride, static_cast<T*>(k), k_stride, static_cast<const T*>(v),
        v_stride, static_cast<const float*>(q_w), static_cast<const float*>(k_w), cos_t, sin_t, rot,
        positions, slot_of_token, block_table, table_stride, static_cast<T*>(k_pages),
        static_cast<T*>(v_pages), nq, nkv, D, page_size, eps, parts, n_parts, part_stride, part_row_stride);
  } else {
    qk_prep_kernel<T, bf16><<<grid, kPrepWaves * kWave, lds, s>>>(
        static_cast<T*>(q), q_stride, static_cast<T*>(k), k_stride, static_cast<const T*>(v),
        v_stride, static_cast<const bf16*>(q_w), static_cast<const bf16*>(k_w), cos_t, sin_t, rot,
        positions, slot_of_token, block_table, table_stride, static_cast<T*>(k_pages),
        static_cast<T*>(v_pages), nq, nkv, D, page_size, eps, parts, n_parts, part_stride, part_row_stride);
  }
  return launch_status();
}

}  // namespace arle

using namespace arle;

// q [T, nq*D], k [T, nkv*D], v [T, nkv*D] with row strides in elements (so three
// buffers or three column blocks of one fused buffer both fit).  q_w/k_w may be
// null (no per-head norm); rot may be 0 (no rotation; cos/sin unused); k_pages /
// v_pages may be null (no cache write; k is then rewritten in place).
// parts != null: the inputs are n_parts float32 tensors [tokens, (nq + 2 nkv) D] (row stride
// part_row_stride, part_stride elements apart), summed in order; q is only written (a buffer of its
// own), k and v go to the cache only (k_pages and v_pages must be given unless nkv == 0).
extern "C" int arle_qk_prep(void* q, long long q_stride, void* k, long long k_stride, const void* v,
                            long long v_stride, int dtype, const void* q_w, const void* k_w,
                            int w_dtype, const float* cos_t, const float* sin_t, int rot,
                            const int* positions, const int* slot_of_token, const int* block_table,
                            int table_stride, void* k_pages, void* v_pages, int tokens, int nq,
                            int nkv, int D, int page_size, float eps, const float* parts, int n_parts,
                            long long part_stride, long long part_row_stride, void* stream) {
  if (tokens == 0) return 0;
  if (D > kMaxHeadDim || rot > D || (rot & 1)) return static_cast<int>(hipErrorInvalidValue);
  if (parts != nullptr && (n_parts < 1 || (nkv > 0 && (k_pages == nullptr || v_pages == nullptr))))
    return static_cast<int>(hipErrorInvalidValue);
  hipStream_t s = static_cast<hipStream_t>(stream);
  auto aligned = [](const void* p) { return reinterpret_cast<uintptr_t>(p) % 16 == 0; };
  const bool pow2 = D >= 64 && (D & (D - 1)) == 0;
  if (dtype == kBF16 && parts == nullptr && pow2 && rot % 16 == 0 && q_stride % 8 == 0 && k_stride % 8 == 0 &&
      v_stride % 8 == 0 && aligned(q) && aligned(k) && aligned(v) && aligned(k_pages) && aligned(v_pages) &&
      (cos_t == nullptr || (reinterpret_cast<uintptr_t>(cos_t) % 4 == 0))) {
#define ARLE_PREP(LPH)                                                                                          \
  return launch_prep_bf16x8<LPH>(q, q_stride, k, k_stride, v, v_stride, q_w, k_w, w_dtype, cos_t, sin_t, rot,    \
                                 positions, slot_of_token, block_table, table_stride, k_pages, v_pages, tokens, \
                                 nq, nkv, page_size, eps, s)
    if (D == 64) ARLE_PREP(8);
    if (D == 128) ARLE_PREP(16);
    if (D == 256) ARLE_PREP(32);
    if (D == 512) ARLE_PREP(64);
#undef ARLE_PREP
  }
  if (dtype == kF32)
    return launch_prep<float>(q, q_stride, k, k_stride, v, v_stride, q_w, k_w, w_dtype, cos_t, sin_t,
                              rot, positions, slot_of_token, block_table, table_stride, k_pages,
                              v_pages, tokens, nq, nkv, D, page_size, eps, parts, n_parts, part_stride,
                              part_row_stride, s);
  return launch_prep<bf16>(q, q_stride, k, k_stride, v, v_stride, q_w, k_w, w_dtype, cos_t, sin_t,
                           rot, positions, slot_of_token, block_table, table_stride, k_pages,
                           v_pages, tokens, nq, nkv, D, page_size, eps, parts, n_parts, part_stride,
                           part_row_stride, s);
}
