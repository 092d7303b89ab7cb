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

// residual[src(r), :] += delta[0][src(r), :] + delta[1][src(r), :] + ...; out[r, :] = norm(residual[src(r), :]).
// `delta` is a stack of n_delta tensors delta_stride elements apart (the partial products of a matrix
// product whose K was split over workgroups), added in the order of the stack.
// With `rows` given the sum is not written back: the rows are read for the last
// time (final norm before the output head).
template <typename TD, typename TOut, typename TW>
__global__ void add_rmsnorm_kernel(float* __restrict__ residual, const TD* __restrict__ delta, int n_delta,
                                   int64_t delta_stride, const TW* __restrict__ w, TOut* __restrict__ out,
                                   const int* __restrict__ rows, int width, float eps) {
  __shared__ float lds[kNormWaves];
  const int r = blockIdx.x;
  const int64_t src = rows ? rows[r] : r;
  float* res = residual + src * width;
  const TD* d = delta + src * width;
  auto summed = [&](int i) {  // residual + (delta 0 + delta 1 + ...), as the register-resident kernel adds them
    float dv = to_float(d[i]);
    for (int sp = 1; sp < n_delta; ++sp) dv += to_float(d[sp * delta_stride + i]);
    return res[i] + dv;
  };
  float ss = 0.f;
  for (int i = threadIdx.x; i < width; i += kNormThreads) {
    const float v = summed(i);
    if (!rows) res[i] = v;
    ss += v * v;
  }
  const float total = block_sum<kNormWaves>(ss, lds);
  const float inv = 1.0f / sqrtf(total / static_cast<float>(width) + eps);
  TOut* o = out + static_cast<int64_t>(r) * width;
  for (int i = threadIdx.x; i < width; i += kNormThreads) {
    const float v = rows ? summed(i) : res[i];
    o[i] = from_float<TOut>(v * inv * to_float(w[i]));
  }
}

// ---- register-resident variants -------------------------------------------------------------
// Rows of up to kVecMax elements (a multiple of 4) are read once with 16-byte loads, kept in
// registers across the reduction and written once.  All loads of a row are issued before anything
// is stored, so that the in-place update of the residual does not serialise them.
constexpr int kVecPerThreadMax = 8;                                // float4 groups per thread: 2, 4 or 8 by width
constexpr int kVecMax = kNormThreads * kVecPerThreadMax * 4;       // 8192 elements

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

// HAS_DELTA: residual row += the rows of the delta stack first, in the order of the stack (written back unless
// `rows` picks rows for the last time).  VPT float4 groups a thread (width <= 256 * VPT * 4).  No load stands
// under a condition (a group past the width reads the row's last group again and is left out of the sums and
// stores), so that all of them are in flight together.
template <typename TIn, typename TD, typename TOut, typename TW, bool HAS_DELTA, int VPT>
__global__ __launch_bounds__(kNormThreads) void rmsnorm_vec_kernel(TIn* __restrict__ x, int64_t x_stride,
                                                                   const TD* __restrict__ delta, int n_delta,
                                                                   int64_t delta_stride,
                                                                   const TW* __restrict__ w,
                                                                   TOut* __restrict__ out,
                                                                   const int* __restrict__ rows, int width,
                                                                   float eps) {
  __shared__ float lds[kNormWaves];
  const int r = blockIdx.x;
  const int64_t src = rows ? rows[r] : r;
  TIn* xr = x + src * x_stride;
  const TD* dr = HAS_DELTA ? delta + src * static_cast<int64_t>(width) : nullptr;
  float4 v[VPT], d[VPT], wv[VPT];
  int at[VPT];
  bool in[VPT];
#pragma unroll
  for (int j = 0; j < VPT; ++j) {
    const int i = 4 * (threadIdx.x + j * kNormThreads);
    in[j] = i < width;
    at[j] = in[j] ? i : width - 4;
    v[j] = load4<TIn>(xr + at[j]);
    if (HAS_DELTA) d[j] = load4<TD>(dr + at[j]);
    wv[j] = load4<TW>(w + at[j]);
  }
  if (HAS_DELTA) {  // the rest of the stack, a few rows of loads in flight at a time
#pragma unroll 2
    for (int sp = 1; sp < n_delta; ++sp) {
      float4 e[VPT];
#pragma unroll
      for (int j = 0; j < VPT; ++j) e[j] = load4<TD>(dr + sp * delta_stride + at[j]);
#pragma unroll
      for (int j = 0; j < VPT; ++j) {
        d[j].x += e[j].x;
        d[j].y += e[j].y;
        d[j].z += e[j].z;
        d[j].w += e[j].w;
      }
    }
  }
  float ss = 0.f;
#pragma unroll
  for (int j = 0; j < VPT; ++j) {
    if (HAS_DELTA) {
      v[j].x += d[j].x;
      v[j].y += d[j].y;
      v[j].z += d[j].z;
      v[j].w += d[j].w;
      if (!rows && in[j]) store4<TIn>(xr + at[j], v[j]);
    }
    if (in[j]) ss += v[j].x * v[j].x + v[j].y * v[j].y + v[j].z * v[j].z + v[j].w * v[j].w;
  }
  const float total = block_sum<kNormWaves>(ss, lds);
  const float inv = 1.0f / sqrtf(total / static_cast<float>(width) + eps);
  TOut* o = out + static_cast<int64_t>(r) * width;
#pragma unroll
  for (int j = 0; j < VPT; ++j) {
    if (in[j])
      store4<TOut>(o + at[j], float4{v[j].x * inv * wv[j].x, v[j].y * inv * wv[j].y, v[j].z * inv * wv[j].z,
                                     v[j].w * inv * wv[j].w});
  }
}

// the variant with the fewest groups a thread that covers the width
#define ARLE_NORM_VEC(TIN, TD, TOUT, TW, HAS_DELTA, ...)                                             \
  do {                                                                                               \
    if (width <= kNormThreads * 8)                                                                   \
      rmsnorm_vec_kernel<TIN, TD, TOUT, TW, HAS_DELTA, 2><<<n_rows, kNormThreads, 0, s>>>(__VA_ARGS__); \
    else if (width <= kNormThreads * 16)                                                             \
      rmsnorm_vec_kernel<TIN, TD, TOUT, TW, HAS_DELTA, 4><<<n_rows, kNormThreads, 0, s>>>(__VA_ARGS__); \
    else                                                                                             \
      rmsnorm_vec_kernel<TIN, TD, TOUT, TW, HAS_DELTA, 8><<<n_rows, kNormThreads, 0, s>>>(__VA_ARGS__); \
  } while (0)

// A stack of float32 deltas (the partial products of a matrix product whose K was split over
// workgroups) added into the residual row, then the norm.  Few rows make few workgroups here, so the
// time is the latency of the loads: a workgroup of 1024 threads owns a row, every thread one group of
// four columns, and the loads of the whole stack (up to kStackUnroll at a time) are in flight together.
// Order of addition: residual + (delta 0 + delta 1 + ...), as in the kernels above.
constexpr int kStackThreads = 1024;
constexpr int kStackUnroll = 4;   // parts of the stack that a thread has in flight at a time

template <typename TOut, typename TW>
__global__ __launch_bounds__(kStackThreads) void add_stack_rmsnorm_kernel(
    float* __restrict__ residual, const float* __restrict__ delta, int n_delta, int64_t delta_stride,
    const TW* __restrict__ w, TOut* __restrict__ out, const int* __restrict__ rows, int width, float eps) {
  __shared__ float lds[kStackThreads / kWave];
  const int r = blockIdx.x;
  const int64_t src = rows ? rows[r] : r;
  const int i = 4 * threadIdx.x;
  const bool mine = i < width;
  float* res = residual + src * width;
  const float* dr = delta + src * width;
  const int ic = mine ? i : 0;
  float4 v = load4<float>(res + ic), d = {0.f, 0.f, 0.f, 0.f};
  const float4 wv = load4<TW>(w + ic);
  // The loads of a round carry no condition (a load under a condition is waited for before the next one is
  // issued, and the parts would arrive one after the other): whole rounds of four parts first, then one round
  // whose loads past the last part fetch the last part again and are not added.  Threads past the width read
  // column 0.
  const float* dc = dr + ic;
  int base = 0;
  for (; base + kStackUnroll <= n_delta; base += kStackUnroll) {
    float4 e[kStackUnroll];
#pragma unroll
    for (int u = 0; u < kStackUnroll; ++u) e[u] = load4<float>(dc + (base + u) * delta_stride);
#pragma unroll
    for (int u = 0; u < kStackUnroll; ++u) {
      d.x += e[u].x;
      d.y += e[u].y;
      d.z += e[u].z;
      d.w += e[u].w;
    }
  }
  if (base < n_delta) {
    float4 e[kStackUnroll - 1];
#pragma unroll
    for (int u = 0; u < kStackUnroll - 1; ++u) e[u] = load4<float>(dc + min(base + u, n_delta - 1) * delta_stride);
#pragma unroll
    for (int u = 0; u < kStackUnroll - 1; ++u) {
      const bool in = base + u < n_delta;
      d.x += in ? e[u].x : 0.f;
      d.y += in ? e[u].y : 0.f;
      d.z += in ? e[u].z : 0.f;
      d.w += in ? e[u].w : 0.f;
    }
  }
  v.x += d.x;
  v.y += d.y;
  v.z += d.z;
  v.w += d.w;
  if (mine && !rows) store4<float>(res + i, v);
  const float total =
      block_sum<kStackThreads / kWave>(mine ? v.x * v.x + v.y * v.y + v.z * v.z + v.w * v.w : 0.f, lds);
  const float inv = 1.0f / sqrtf(total / static_cast<float>(width) + eps);
  if (mine)
    store4<TOut>(out + static_cast<int64_t>(r) * width + i,
                 float4{v.x * inv * wv.x, v.y * inv * wv.y, v.z * inv * wv.z, v.w * inv * wv.w});
}

inline bool vec_ok(int width, long long x_stride, const void* a, const void* b, const void* c, const void* d) {
  auto al = [](const void* p) { return p == nullptr || reinterpret_cast<uintptr_t>(p) % 16 == 0; };
  return width % 4 == 0 && width >= 4 && width <= kVecMax && x_stride % 4 == 0 && al(a) && al(b) && al(c) && al(d);
}

template <typename TIn, typename TOut>
int launch_rmsnorm(const void* x, long long x_stride, const void* w, int w_dtype, void* out,
                   const int* rows, int n_rows, int width, float eps, hipStream_t s) {
  if (vec_ok(width, x_stride, x, w, out, nullptr)) {
    TIn* xp = const_cast<TIn*>(static_cast<const TIn*>(x));
    if (w_dtype == kF32)
      ARLE_NORM_VEC(TIn, TIn, TOut, float, false, xp, x_stride, nullptr, 0, 0, static_cast<const float*>(w),
                    static_cast<TOut*>(out), rows, width, eps);
    else
      ARLE_NORM_VEC(TIn, TIn, TOut, bf16, false, xp, x_stride, nullptr, 0, 0, static_cast<const bf16*>(w),
                    static_cast<TOut*>(out), rows, width, eps);
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
int launch_add_rmsnorm(float* residual, const void* delta, int n_delta, long long delta_stride, const void* w,
                       int w_dtype, void* out, const int* rows, int n_rows, int width, float eps, hipStream_t s) {
  if constexpr (sizeof(TD) == 4) {
    if (n_delta > 1 && vec_ok(width, width, residual, delta, w, out) && delta_stride % 4 == 0 &&
        width <= 4 * kStackThreads) {
      if (w_dtype == kF32)
        add_stack_rmsnorm_kernel<TOut, float><<<n_rows, kStackThreads, 0, s>>>(
            residual, static_cast<const float*>(delta), n_delta, delta_stride, static_cast<const float*>(w),
            static_cast<TOut*>(out), rows, width, eps);
      else
        add_stack_rmsnorm_kernel<TOut, bf16><<<n_rows, kStackThreads, 0, s>>>(
            residual, static_cast<const float*>(delta), n_delta, delta_stride, static_cast<const bf16*>(w),
            static_cast<TOut*>(out), rows, width, eps);
      return launch_status();
    }
  }
  if (vec_ok(width, width, residual, delta, w, out) && delta_stride % 4 == 0) {
    if (w_dtype == kF32)
      ARLE_NORM_VEC(float, TD, TOut, float, true, residual, width, static_cast<const TD*>(delta), n_delta,
                    delta_stride, static_cast<const float*>(w), static_cast<TOut*>(out), rows, width, eps);
    else
      ARLE_NORM_VEC(float, TD, TOut, bf16, true, residual, width, static_cast<const TD*>(delta), n_delta,
                    delta_stride, static_cast<const bf16*>(w), static_cast<TOut*>(out), rows, width, eps);
    return launch_status();
  }
  if (w_dtype == kF32) {
    add_rmsnorm_kernel<TD, TOut, float><<<n_rows, kNormThreads, 0, s>>>(
        residual, static_cast<const TD*>(delta), n_delta, delta_stride, static_cast<const float*>(w),
        static_cast<TOut*>(out), rows, width, eps);
  } else {
    add_rmsnorm_kernel<TD, TOut, bf16><<<n_rows, kNormThreads, 0, s>>>(
        residual, static_cast<const TD*>(delta), n_delta, delta_stride, static_cast<const bf16*>(w),
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

// delta: n_delta >= 1 tensors [*, width] of `delta_dtype`, delta_stride elements apart, added in order.
extern "C" int arle_add_rmsnorm(float* residual, const void* delta, int n_delta, long long delta_stride,
                                int delta_dtype, const void* w, int w_dtype, void* out, int out_dtype,
                                const int* rows, int n_rows, int width, float eps, void* stream) {
  if (n_rows == 0) return 0;
  if (n_delta < 1) return static_cast<int>(hipErrorInvalidValue);
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (delta_dtype == kF32 && out_dtype == kF32)
    return launch_add_rmsnorm<float, float>(residual, delta, n_delta, delta_stride, w, w_dtype, out, rows, n_rows, width, eps, s);
  if (delta_dtype == kF32 && out_dtype == kBF16)
    return launch_add_rmsnorm<float, bf16>(residual, delta, n_delta, delta_stride, w, w_dtype, out, rows, n_rows, width, eps, s);
  if (delta_dtype == kBF16 && out_dtype == kF32)
    return launch_add_rmsnorm<bf16, float>(residual, delta, n_delta, delta_stride, w, w_dtype, out, rows, n_rows, width, eps, s);
  return launch_add_rmsnorm<bf16, bf16>(residual, delta, n_delta, delta_stride, w, w_dtype, out, rows, n_rows, width, eps, s);
}
