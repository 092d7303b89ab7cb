// RMSNorm over rows, with and without the residual add fused in.
//
//   inv = 1 / sqrt(mean_j(x_j^2) + eps);   out_j = x_j * inv * w_j     (plain weight)
// reference counterparts: crates/cuda-kernels/csrc/misc/norm.cu:221-359 (rows),
// :462- (add fused in).  Sum of squares, inverse root and products are 32-bit;
// the output is rounded once.
//
// The residual stream is 32-bit in every mode, so the fused form reads and
// updates a float row and adds a delta of the activation type.
#include "common.h"

namespace arle {

constexpr int kNormThreads = 256;
constexpr int kNormWaves = kNormThreads / kWave;

// out[r, :] = norm(x[src(r), :]) with src(r) = rows ? rows[r] : r.
template <typename TIn, typename TOut, typename TW>
__global__ void rmsnorm_kernel(const TIn* __restrict__ x, int64_t x_stride,
                               const TW* __restrict__ w, TOut* __restrict__ out,
                               const int* __restrict__ rows, int width, float eps) {
  __shared__ float lds[kNormWaves];
  const int r = blockIdx.x;
  const int64_t src = rows ? rows[r] : r;
  const TIn* xr = x + src * x_stride;
  float ss = 0.f;
  for (int i = threadIdx.x; i < width; i += kNormThreads) {
    const float v = to_float(xr[i]);
    ss += v * v;
  }
  const float total = block_sum<kNormWaves>(ss, lds);
  const float inv = 1.0f / sqrtf(total / static_cast<float>(width) + eps);
  TOut* o = out + static_cast<int64_t>(r) * width;
  for (int i = threadIdx.x; i < width; i += kNormThreads) {
    o[i] = from_float<TOut>(to_float(xr[i]) * inv * to_float(w[i]));
  }
}

// residual[src(r), :] += delta[src(r), :]; out[r, :] = norm(residual[src(r), :]).
// With `rows` given the sum is not written back: the rows are read for the last
// time (final norm before the output head).
template <typename TD, typename TOut, typename TW>
__global__ void add_rmsnorm_kernel(float* __restrict__ residual, const TD* __restrict__ delta,
                                   const TW* __restrict__ w, TOut* __restrict__ out,
                                   const int* __restrict__ rows, int width, float eps) {
  __shared__ float lds[kNormWaves];
  const int r = blockIdx.x;
  const int64_t src = rows ? rows[r] : r;
  float* res = residual + src * width;
  const TD* d = delta + src * width;
  float ss = 0.f;
  for (int i = threadIdx.x; i < width; i += kNormThreads) {
    const float v = res[i] + to_float(d[i]);
    if (!rows) res[i] = v;
    ss += v * v;
  }
  const float total = block_sum<kNormWaves>(ss, lds);
  const float inv = 1.0f / sqrtf(total / static_cast<float>(width) + eps);
  TOut* o = out + static_cast<int64_t>(r) * width;
  for (int i = threadIdx.x; i < width; i += kNormThreads) {
    const float v = rows ? res[i] + to_float(d[i]) : res[i];
    o[i] = from_float<TOut>(v * inv * to_float(w[i]));
  }
}

// ---- register-resident variants -------------------------------------------------------------
// Rows of up to kVecMax elements (a multiple of 4) are read once with 16-byte loads, kept in
// registers across the reduction and written once.  All loads of a row are issued before anything
// is stored, so that the in-place update of the residual does not serialise them.
constexpr int kVecPerThread = 4;                                   // float4 groups per thread
constexpr int kVecMax = kNormThreads * kVecPerThread * 4;          // 4096 elements

template <typename T>
__device__ __forceinline__ float4 load4(const T* p);
template <>
__device__ __forceinline__ float4 load4<float>(const float* p) {
  return *reinterpret_cast<const float4*>(p);
}
template <>
__device__ __forceinline__ float4 load4<bf16>(const bf16* p) {
  const uint2 raw = *reinterpret_cast<const uint2*>(p);
  return float4{__uint_as_float(raw.x << 16), __uint_as_float(raw.x & 0xffff0000u),
                __uint_as_float(raw.y << 16), __uint_as_float(raw.y & 0xffff0000u)};
}
template <typename T>
__device__ __forceinline__ void store4(T* p, float4 v);
template <>
__device__ __forceinline__ void store4<float>(float* p, float4 v) {
  *reinterpret_cast<float4*>(p) = v;
}
template <>
__device__ __forceinline__ void store4<bf16>(bf16* p, float4 v) {
  uint2 raw;
  raw.x = pack_bf16x2(v.x, v.y);
  raw.y = pack_bf16x2(v.z, v.w);
  *reinterpret_cast<uint2*>(p) = raw;
}

// HAS_DELTA: residual row += delta row first (written back unless `rows` picks rows for the last time).
template <typename TIn, typename TD, typename TOut, typename TW, bool HAS_DELTA>
__global__ __launch_bounds__(kNormThreads) void rmsnorm_vec_kernel(TIn* __restrict__ x, int64_t x_stride,
                                                                   const TD* __restrict__ delta,
                                                                   const TW* __restrict__ w,
                                                                   TOut* __restrict__ out,
                                                                   const int* __restrict__ rows, int width,
                                                                   float eps) {
  __shared__ float lds[kNormWaves];
  const int r = blockIdx.x;
  const int64_t src = rows ? rows[r] : r;
  TIn* xr = x + src * x_stride;
  const TD* dr = HAS_DELTA ? delta + src * static_cast<int64_t>(width) : nullptr;
  float4 v[kVecPerThread], d[kVecPerThread], wv[kVecPerThread];
#pragma unroll
  for (int j = 0; j < kVecPerThread; ++j) {
    const int i = 4 * (threadIdx.x + j * kNormThreads);
    if (i < width) {
      v[j] = load4<TIn>(xr + i);
      if (HAS_DELTA) d[j] = load4<TD>(dr + i);
      wv[j] = load4<TW>(w + i);
    }
  }
  float ss = 0.f;
#pragma unroll
  for (int j = 0; j < kVecPerThread; ++j) {
    const int i = 4 * (threadIdx.x + j * kNormThreads);
    if (i < width) {
      if (HAS_DELTA) {
        v[j].x += d[j].x;
        v[j].y += d[j].y;
        v[j].z += d[j].z;
        v[j].w += d[j].w;
        if (!rows) store4<TIn>(xr + i, v[j]);
      }
      ss += v[j].x * v[j].x + v[j].y * v[j].y + v[j].z * v[j].z + v[j].w * v[j].w;
    }
  }
  const float total = block_sum<kNormWaves>(ss, lds);
  const float inv = 1.0f / sqrtf(total / static_cast<float>(width) + eps);
  TOut* o = out + static_cast<int64_t>(r) * width;
#pragma unroll
  for (int j = 0; j < kVecPerThread; ++j) {
    const int i = 4 * (threadIdx.x + j * kNormThreads);
    if (i < width)
      store4<TOut>(o + i, float4{v[j].x * inv * wv[j].x, v[j].y * inv * wv[j].y, v[j].z * inv * wv[j].z,
                                 v[j].w * inv * wv[j].w});
  }
}

inline bool vec_ok(int width, long long x_stride, const void* a, const void* b, const void* c, const void* d) {
  auto al = [](const void* p) { return p == nullptr || reinterpret_cast<uintptr_t>(p) % 16 == 0; };
  return width % 4 == 0 && width <= kVecMax && x_stride % 4 == 0 && al(a) && al(b) && al(c) && al(d);
}

template <typename TIn, typename TOut>
int launch_rmsnorm(const void* x, long long x_stride, const void* w, int w_dtype, void* out,
                   const int* rows, int n_rows, int width, float eps, hipStream_t s) {
  if (vec_ok(width, x_stride, x, w, out, nullptr)) {
    TIn* xp = const_cast<TIn*>(static_cast<const TIn*>(x));
    if (w_dtype == kF32)
      rmsnorm_vec_kernel<TIn, TIn, TOut, float, false><<<n_rows, kNormThreads, 0, s>>>(
          xp, x_stride, nullptr, static_cast<const float*>(w), static_cast<TOut*>(out), rows, width, eps);
    else
      rmsnorm_vec_kernel<TIn, TIn, TOut, bf16, false><<<n_rows, kNormThreads, 0, s>>>(
          xp, x_stride, nullptr, static_cast<const bf16*>(w), static_cast<TOut*>(out), rows, width, eps);
    return launch_status();
  }
  if (w_dtype == kF32) {
    rmsnorm_kernel<TIn, TOut, float><<<n_rows, kNormThreads, 0, s>>>(
        static_cast<const TIn*>(x), x_stride, static_cast<const float*>(w),
        static_cast<TOut*>(out), rows, width, eps);
  } else {
    rmsnorm_kernel<TIn, TOut, bf16><<<n_rows, kNormThreads, 0, s>>>(
        static_cast<const TIn*>(x), x_stride, static_cast<const bf16*>(w),
        static_cast<TOut*>(out), rows, width, eps);
  }
  return launch_status();
}

template <typename TD, typename TOut>
int launch_add_rmsnorm(float* residual, const void* delta, const void* w, int w_dtype, void* out,
                       const int* rows, int n_rows, int width, float eps, hipStream_t s) {
  if (vec_ok(width, width, residual, delta, w, out)) {
    if (w_dtype == kF32)
      rmsnorm_vec_kernel<float, TD, TOut, float, true><<<n_rows, kNormThreads, 0, s>>>(
          residual, width, static_cast<const TD*>(delta), static_cast<const float*>(w),
          static_cast<TOut*>(out), rows, width, eps);
    else
      rmsnorm_vec_kernel<float, TD, TOut, bf16, true><<<n_rows, kNormThreads, 0, s>>>(
          residual, width, static_cast<const TD*>(delta), static_cast<const bf16*>(w),
          static_cast<TOut*>(out), rows, width, eps);
    return launch_status();
  }
  if (w_dtype == kF32) {
    add_rmsnorm_kernel<TD, TOut, float><<<n_rows, kNormThreads, 0, s>>>(
        residual, static_cast<const TD*>(delta), static_cast<const float*>(w),
        static_cast<TOut*>(out), rows, width, eps);
  } else {
    add_rmsnorm_kernel<TD, TOut, bf16><<<n_rows, kNormThreads, 0, s>>>(
        residual, static_cast<const TD*>(delta), static_cast<const bf16*>(w),
        static_cast<TOut*>(out), rows, width, eps);
  }
  return launch_status();
}

}  // namespace arle

using namespace arle;

// x: [*, width] rows of `in_dtype` with row stride `x_stride` (elements).
extern "C" int arle_rmsnorm(const void* x, int in_dtype, long long x_stride, const void* w,
                            int w_dtype, void* out, int out_dtype, const int* rows, int n_rows,
                            int width, float eps, void* stream) {
  if (n_rows == 0) return 0;
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (in_dtype == kF32 && out_dtype == kF32)
    return launch_rmsnorm<float, float>(x, x_stride, w, w_dtype, out, rows, n_rows, width, eps, s);
  if (in_dtype == kF32 && out_dtype == kBF16)
    return launch_rmsnorm<float, bf16>(x, x_stride, w, w_dtype, out, rows, n_rows, width, eps, s);
  if (in_dtype == kBF16 && out_dtype == kF32)
    return launch_rmsnorm<bf16, float>(x, x_stride, w, w_dtype, out, rows, n_rows, width, eps, s);
  return launch_rmsnorm<bf16, bf16>(x, x_stride, w, w_dtype, out, rows, n_rows, width, eps, s);
}

extern "C" int arle_add_rmsnorm(float* residual, const void* delta, int delta_dtype, const void* w,
                                int w_dtype, void* out, int out_dtype, const int* rows, int n_rows,
                                int width, float eps, void* stream) {
  if (n_rows == 0) return 0;
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (delta_dtype == kF32 && out_dtype == kF32)
    return launch_add_rmsnorm<float, float>(residual, delta, w, w_dtype, out, rows, n_rows, width, eps, s);
  if (delta_dtype == kF32 && out_dtype == kBF16)
    return launch_add_rmsnorm<float, bf16>(residual, delta, w, w_dtype, out, rows, n_rows, width, eps, s);
  if (delta_dtype == kBF16 && out_dtype == kF32)
    return launch_add_rmsnorm<bf16, float>(residual, delta, w, w_dtype, out, rows, n_rows, width, eps, s);
  return launch_add_rmsnorm<bf16, bf16>(residual, delta, w, w_dtype, out, rows, n_rows, width, eps, s);
}
