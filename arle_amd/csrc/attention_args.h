// What the attention kernels of attention_mfma.hip share: vector types, the launch's arguments, small helpers.
#pragma once
#include "common.h"

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

}  // namespace arle
