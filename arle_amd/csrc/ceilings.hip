// Two measuring kernels, no part of a model step: what one MI355X gives to a kernel that only reads memory, and
// to one that only multiplies on the matrix cores.  The benchmark reports the engine's kernels against these
// figures beside the published peaks (8 TB/s, 2.5 PFLOP/s bfloat16), which no kernel reaches.
//
//   arle_ceiling_read:  workgroups that stay (one or two a compute unit) read `bytes` in 16-byte pieces a lane,
//                       sixteen loads in flight a lane, each workgroup one contiguous part: the fastest way
//                       found to pull bytes out of HBM3E (6.3 TB/s measured).
//   arle_ceiling_mfma:  every wave issues `iters` rounds of eight independent v_mfma_f32_32x32x16_bf16 (or
//                       sixteen v_mfma_f32_16x16x32_bf16) on registers; 2 * 32 * 32 * 16 flops each.  The operands
//                       are either all the same value near 1.0 or pseudo-random bits with exponents around 1.0:
//                       the chip's clock follows its power, and products of operands whose bits differ draw more
//                       (with all 256 compute units busy 1.65 GHz instead of 2.2 and more, measured), so the second
//                       is the ceiling for real data.
#include "common.h"

namespace arle {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x16 __attribute__((ext_vector_type(16)));

constexpr int kReadUnroll = 16;

__global__ __launch_bounds__(256) void ceiling_read_kernel(const uint4* __restrict__ p, long long n16, float* sink) {
  const long long per_wg = n16 / gridDim.x;  // the host passes a multiple of gridDim.x * 256 * kReadUnroll pieces
  const uint4* mine = p + per_wg * blockIdx.x + threadIdx.x;
  uint32_t acc = 0;
  for (long long i = 0; i < per_wg; i += 256 * kReadUnroll) {
    uint4 v[kReadUnroll];
#pragma unroll
    for (int u = 0; u < kReadUnroll; ++u) v[u] = mine[i + u * 256];
#pragma unroll
    for (int u = 0; u < kReadUnroll; ++u) acc ^= v[u].x ^ v[u].y ^ v[u].z ^ v[u].w;
  }
  if (acc == 0x9e3779b9u) sink[0] = 1.0f;  // keeps the loads alive; memory that holds zeros never writes
}

template <int SHAPE>
__global__ __launch_bounds__(256) void ceiling_mfma_kernel(int iters, int random_operands, float* sink) {
  const uint32_t seed = 0x3f803f80u + threadIdx.x;  // bfloat16 pairs near 1.0
  // random: every 16-bit half keeps a random sign and mantissa and an exponent of 0x30..0x3f or 0xb0..0xbf
  auto bits = [&](uint32_t mul) { return random_operands ? ((seed * mul) & 0xbfffbfffu) | 0x30003000u : seed; };
  const uint4 raw = {bits(2654435761u), bits(40503u), bits(69069u), bits(1664525u)};
  const uint4 raw_b = {bits(22695477u), bits(134775813u), bits(1103515245u), bits(214013u)};
  const bf16x8 a = __builtin_bit_cast(bf16x8, raw), b = __builtin_bit_cast(bf16x8, raw_b);
  float total = 0.f;
  if constexpr (SHAPE == 32) {
    f32x16 acc[8];
#pragma unroll
    for (int u = 0; u < 8; ++u)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[u][r] = 0.f;
    for (int it = 0; it < iters; ++it) {
#pragma unroll
      for (int u = 0; u < 8; ++u) acc[u] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, acc[u], 0, 0, 0);
    }
#pragma unroll
    for (int u = 0; u < 8; ++u) total += acc[u][0] + acc[u][15];
  } else {
    f32x4 acc[16];
#pragma unroll
    for (int u = 0; u < 16; ++u) acc[u] = f32x4{0.f, 0.f, 0.f, 0.f};
    for (int it = 0; it < iters; ++it) {
#pragma unroll
      for (int u = 0; u < 16; ++u) acc[u] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, acc[u], 0, 0, 0);
    }
#pragma unroll
    for (int u = 0; u < 16; ++u) total += acc[u][0] + acc[u][3];
  }
  if (total == 0.123f) sink[0] = total;
}

}  // namespace arle

using namespace arle;

// Reads bytes (rounded down to whole rounds of all workgroups) of p once; returns through *bytes_read how many.
extern "C" int arle_ceiling_read(const void* p, long long bytes, int workgroups, long long* bytes_read, void* sink,
                                 void* stream) {
  if (workgroups < 1 || bytes < 0) return static_cast<int>(hipErrorInvalidValue);
  const long long round = static_cast<long long>(workgroups) * 256 * kReadUnroll * 16;
  const long long whole = bytes / round * round;
  if (bytes_read) *bytes_read = whole;
  if (whole == 0) return 0;
  ceiling_read_kernel<<<workgroups, 256, 0, static_cast<hipStream_t>(stream)>>>(static_cast<const uint4*>(p), whole / 16,
                                                                               static_cast<float*>(sink));
  return launch_status();
}

// shape 32: v_mfma_f32_32x32x16_bf16, eight a round; shape 16: v_mfma_f32_16x16x32_bf16, sixteen a round.  Either
// way a wave does iters * 262144 flops; workgroups of four waves.
extern "C" int arle_ceiling_mfma(int shape, int iters, int workgroups, int random_operands, void* sink, void* stream) {
  if (workgroups < 1 || iters < 1 || (shape != 16 && shape != 32)) return static_cast<int>(hipErrorInvalidValue);
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (shape == 32)
    ceiling_mfma_kernel<32><<<workgroups, 256, 0, s>>>(iters, random_operands, static_cast<float*>(sink));
  else
    ceiling_mfma_kernel<16><<<workgroups, 256, 0, s>>>(iters, random_operands, static_cast<float*>(sink));
  return launch_status();
}
