// Embedding gather and the SiLU-gated product.
//
// embed_gather: out[t, :] = float(table[ids[t], :])      (residual stream is 32-bit)
//   reference counterpart: crates/cuda-kernels/csrc/misc/elementwise_basic.cu:186-211
// silu_mul:     out[t, j] = silu(gate[t, j]) * up[t, j], silu(z) = z / (1 + exp(-z))
//   reference counterpart: crates/cuda-kernels/csrc/misc/elementwise_basic.cu:18-24,34-95
#include "common.h"

namespace arle {

template <typename TT>
__global__ void embed_gather_kernel(const TT* __restrict__ table, const int* __restrict__ ids,
                                    float* __restrict__ out, int hidden) {
  const int t = blockIdx.x;
  const TT* src = table + static_cast<int64_t>(ids[t]) * hidden;
  float* dst = out + static_cast<int64_t>(t) * hidden;
  for (int i = threadIdx.x; i < hidden; i += blockDim.x) dst[i] = to_float(src[i]);
}

// block == 0: gate and up are two [T, width] views.  block > 0: one buffer whose columns alternate
// between `block` gate columns and the `block` matching up columns (gate is its first column).
template <typename T>
__global__ void silu_mul_kernel(const T* __restrict__ gate, const T* __restrict__ up,
                                int64_t in_stride, T* __restrict__ out, int width, int block) {
  const int t = blockIdx.x;
  const int j = blockIdx.y * blockDim.x + threadIdx.x;
  if (j >= width) return;
  const int64_t row = static_cast<int64_t>(t) * in_stride;
  const int64_t gi = block > 0 ? row + (j / block) * 2 * block + j % block : row + j;
  const float g = to_float(gate[gi]);
  const float u = to_float(block > 0 ? gate[gi + block] : up[gi]);
  const float act = g / (1.0f + expf(-g));
  out[static_cast<int64_t>(t) * width + j] = from_float<T>(act * u);
}

// bfloat16, eight columns a thread: two 16-byte loads, one 16-byte store.  width, block (if any) and
// in_stride are multiples of 8 and the pointers 16-byte aligned (the launcher checks).
__global__ void silu_mul_bf16x8_kernel(const uint16_t* __restrict__ gate, const uint16_t* __restrict__ up,
                                       int64_t in_stride, uint16_t* __restrict__ out, int width, int block,
                                       int64_t chunks) {
  const int64_t c = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (c >= chunks) return;
  const int per_row = width / 8;
  const int64_t t = c / per_row;
  const int j = static_cast<int>(c % per_row) * 8;
  const int64_t row = t * in_stride;
  const int64_t gi = block > 0 ? row + (j / block) * 2 * block + j % block : row + j;
  const uint4 g4 = *reinterpret_cast<const uint4*>(gate + gi);
  const uint4 u4 = *reinterpret_cast<const uint4*>(block > 0 ? gate + gi + block : up + gi);
  const uint32_t gw[4] = {g4.x, g4.y, g4.z, g4.w}, uw[4] = {u4.x, u4.y, u4.z, u4.w};
  uint32_t ow[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const float g0 = __uint_as_float(gw[i] << 16), g1 = __uint_as_float(gw[i] & 0xffff0000u);
    const float u0 = __uint_as_float(uw[i] << 16), u1 = __uint_as_float(uw[i] & 0xffff0000u);
    ow[i] = pack_bf16x2(g0 / (1.0f + expf(-g0)) * u0, g1 / (1.0f + expf(-g1)) * u1);
  }
  *reinterpret_cast<uint4*>(out + t * width + j) = uint4{ow[0], ow[1], ow[2], ow[3]};
}

// out[i] = parts[0][i] + parts[1][i] + ..., added in that order: the sum of the float32 partial
// products that a matrix product with K split over workgroups leaves behind.
template <typename TOut>
__global__ void sum_partials_kernel(const float* __restrict__ parts, int n_parts, int64_t stride,
                                    TOut* __restrict__ out, int64_t count) {
  const int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (i >= count) return;
  float v = parts[i];
  for (int sp = 1; sp < n_parts; ++sp) v += parts[sp * stride + i];
  out[i] = from_float<TOut>(v);
}

// Four elements a thread, eight parts in flight at a time (loads without a condition: past the last part the
// last one is fetched again and not added).  count, stride % 4 == 0 and 16-byte aligned pointers.
template <typename TOut>
__global__ __launch_bounds__(256) void sum_partials_x4_kernel(const float* __restrict__ parts, int n_parts, int64_t stride,
                                                              TOut* __restrict__ out, int64_t groups) {
  const int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (i >= groups) return;
  const float* p = parts + 4 * i;
  float4 acc = {0.f, 0.f, 0.f, 0.f};
  for (int base = 0; base < n_parts; base += 8) {
    float4 e[8];
#pragma unroll
    for (int u = 0; u < 8; ++u) e[u] = *reinterpret_cast<const float4*>(p + static_cast<int64_t>(min(base + u, n_parts - 1)) * stride);
#pragma unroll
    for (int u = 0; u < 8; ++u) {
      const bool in = base + u < n_parts;
      acc.x += in ? e[u].x : 0.f;
      acc.y += in ? e[u].y : 0.f;
      acc.z += in ? e[u].z : 0.f;
      acc.w += in ? e[u].w : 0.f;
    }
  }
  if constexpr (sizeof(TOut) == 4) {
    *reinterpret_cast<float4*>(out + 4 * i) = acc;
  } else {
    *reinterpret_cast<uint2*>(out + 4 * i) = uint2{pack_bf16x2(acc.x, acc.y), pack_bf16x2(acc.z, acc.w)};
  }
}

}  // namespace arle

using namespace arle;

extern "C" int arle_embed_gather(const void* table, int table_dtype, const int* ids, float* out,
                                 int tokens, int hidden, void* stream) {
  if (tokens == 0) return 0;
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (table_dtype == kF32) {
    embed_gather_kernel<float><<<tokens, 256, 0, s>>>(static_cast<const float*>(table), ids, out, hidden);
  } else {
    embed_gather_kernel<bf16><<<tokens, 256, 0, s>>>(static_cast<const bf16*>(table), ids, out, hidden);
  }
  return launch_status();
}

// gate and up are two columns blocks of rows with a common row stride (in
// elements), so one fused [T, 2I] buffer and two separate buffers both fit.
extern "C" int arle_silu_mul(const void* gate, const void* up, long long in_stride, void* out,
                             int dtype, int tokens, int width, int block, void* stream) {
  if (tokens == 0 || width == 0) return 0;
  hipStream_t s = static_cast<hipStream_t>(stream);
  auto aligned = [](const void* p) { return reinterpret_cast<uintptr_t>(p) % 16 == 0; };
  if (dtype == kBF16 && width % 8 == 0 && block % 8 == 0 && in_stride % 8 == 0 && aligned(gate) &&
      (block > 0 || aligned(up)) && aligned(out)) {
    const int64_t chunks = static_cast<int64_t>(tokens) * (width / 8);
    silu_mul_bf16x8_kernel<<<static_cast<unsigned>((chunks + 255) / 256), 256, 0, s>>>(
        static_cast<const uint16_t*>(gate), static_cast<const uint16_t*>(up), in_stride,
        static_cast<uint16_t*>(out), width, block, chunks);
    return launch_status();
  }
  dim3 grid(tokens, (width + 255) / 256);
  if (dtype == kF32) {
    silu_mul_kernel<float><<<grid, 256, 0, s>>>(static_cast<const float*>(gate),
                                                static_cast<const float*>(up), in_stride,
                                                static_cast<float*>(out), width, block);
  } else {
    silu_mul_kernel<bf16><<<grid, 256, 0, s>>>(static_cast<const bf16*>(gate),
                                               static_cast<const bf16*>(up), in_stride,
                                               static_cast<bf16*>(out), width, block);
  }
  return launch_status();
}

// parts [n_parts][count] float32 (stride elements apart) -> out [count] float32 or bfloat16.
extern "C" int arle_sum_partials(const float* parts, int n_parts, long long stride, void* out, int out_dtype,
                                 long long count, void* stream) {
  if (count == 0) return 0;
  if (n_parts < 1) return static_cast<int>(hipErrorInvalidValue);
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (count % 4 == 0 && stride % 4 == 0 && reinterpret_cast<uintptr_t>(parts) % 16 == 0 &&
      reinterpret_cast<uintptr_t>(out) % 16 == 0) {
    const int64_t groups = count / 4;
    const unsigned blocks = static_cast<unsigned>((groups + 255) / 256);
    if (out_dtype == kF32)
      sum_partials_x4_kernel<float><<<blocks, 256, 0, s>>>(parts, n_parts, stride, static_cast<float*>(out), groups);
    else
      sum_partials_x4_kernel<bf16><<<blocks, 256, 0, s>>>(parts, n_parts, stride, static_cast<bf16*>(out), groups);
    return launch_status();
  }
  const unsigned blocks = static_cast<unsigned>((count + 255) / 256);
  if (out_dtype == kF32)
    sum_partials_kernel<float><<<blocks, 256, 0, s>>>(parts, n_parts, stride, static_cast<float*>(out), count);
  else
    sum_partials_kernel<bf16><<<blocks, 256, 0, s>>>(parts, n_parts, stride, static_cast<bf16*>(out), count);
  return launch_status();
}
