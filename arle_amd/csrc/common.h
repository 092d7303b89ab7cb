// Shared device helpers for the gfx950 kernels: element types, 64-lane wave
// reductions and the launch-status convention of the C entry points.
//
// Every entry point is `extern "C" int arle_<name>(..., void* stream)`; it checks
// nothing about shapes (the Python wrapper does, on the host, before the call),
// launches on the given HIP stream and returns the hipError_t of the launch.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace arle {

constexpr int kWave = 64;

// bfloat16 is carried as its 16 raw bits.
struct bf16 {
  uint16_t bits;
};

__device__ __forceinline__ float to_float(float v) { return v; }
__device__ __forceinline__ float to_float(bf16 v) {
  return __uint_as_float(static_cast<uint32_t>(v.bits) << 16);
}

// Round to nearest, ties to even (the hardware conversion of gfx950, v_cvt_pk_bf16_f32).
__device__ __forceinline__ uint16_t f32_to_bf16_bits(float f) {
  return __builtin_bit_cast(uint16_t, static_cast<__bf16>(f));
}

// Two floats to two bfloat16 in one register: a in the low half, b in the high half.
__device__ __forceinline__ uint32_t pack_bf16x2(float a, float b) {
  typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
  typedef float f32x2_t __attribute__((ext_vector_type(2)));
  const f32x2_t v = {a, b};
  return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, bf16x2_t));
}

template <typename T>
__device__ __forceinline__ T from_float(float v);
template <>
__device__ __forceinline__ float from_float<float>(float v) {
  return v;
}
template <>
__device__ __forceinline__ bf16 from_float<bf16>(float v) {
  bf16 r;
  r.bits = f32_to_bf16_bits(v);
  return r;
}

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int off = kWave / 2; off > 0; off >>= 1) v += __shfl_xor(v, off, kWave);
  return v;
}

__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
  for (int off = kWave / 2; off > 0; off >>= 1) v = fmaxf(v, __shfl_xor(v, off, kWave));
  return v;
}

// Sum over a block of `kWaves` waves; every thread gets the result.  The order
// of additions is fixed (butterfly inside a wave, then waves 0..n-1), so a row's
// reduction never depends on what else is in the launch.
template <int kWaves>
__device__ __forceinline__ float block_sum(float v, float* lds /* [kWaves] */) {
  v = wave_sum(v);
  const int wave = threadIdx.x / kWave;
  if ((threadIdx.x % kWave) == 0) lds[wave] = v;
  __syncthreads();
  float total = 0.f;
#pragma unroll
  for (int i = 0; i < kWaves; ++i) total += lds[i];
  __syncthreads();
  return total;
}

template <int kWaves>
__device__ __forceinline__ float block_max(float v, float* lds /* [kWaves] */) {
  v = wave_max(v);
  const int wave = threadIdx.x / kWave;
  if ((threadIdx.x % kWave) == 0) lds[wave] = v;
  __syncthreads();
  float total = lds[0];
#pragma unroll
  for (int i = 1; i < kWaves; ++i) total = fmaxf(total, lds[i]);
  __syncthreads();
  return total;
}

inline int launch_status() { return static_cast<int>(hipGetLastError()); }

// Element type codes shared with the Python side.
constexpr int kF32 = 0;
constexpr int kBF16 = 1;

}  // namespace arle
