// Token selection from rows of 32-bit logits: argmax, and temperature sampling
// with min-p / top-k / top-p truncation; plus the repetition / frequency /
// presence penalties applied to logits beforehand.
//
// reference counterparts: crates/cuda-kernels/csrc/misc/sampling.cu:27-87,252-317
// (argmax: first maximum in index order) and :327-596 (temperature -> softmax ->
// top-k -> renormalise -> top-p -> renormalise -> inverse CDF with a uniform u
// drawn on the host); penalties infer/src/sampler.rs:100-140.
//
// Differences kept on purpose: the top-k and top-p thresholds are found exactly, eight
// bits of the bit pattern of the (non-negative) probabilities at a time, from 256-bin
// histograms filled with integer atomics, instead of 32 halvings of a float interval;
// each thread owns a contiguous run of the vocabulary so the inverse CDF walks tokens
// in index order; one launch serves many rows with per-row parameters; and the
// log-probability of a chosen token (the reference has it for greedy rows only,
// sampling.cu:252-317) is a kernel of its own that serves greedy and sampled rows.
#include "common.h"

namespace arle {

constexpr int kSampThreads = 1024;
constexpr int kSampWaves = kSampThreads / kWave;

struct ArgMax {
  float v;
  int i;
};

__device__ __forceinline__ ArgMax better(ArgMax a, ArgMax b) {
  // larger value wins; equal values: smaller index wins
  if (b.v > a.v || (b.v == a.v && b.i < a.i)) return b;
  return a;
}

__device__ __forceinline__ ArgMax block_argmax(ArgMax a, ArgMax* lds /* [kSampWaves] */) {
#pragma unroll
  for (int off = kWave / 2; off > 0; off >>= 1) {
    ArgMax o;
    o.v = __shfl_xor(a.v, off, kWave);
    o.i = __shfl_xor(a.i, off, kWave);
    a = better(a, o);
  }
  const int wave = threadIdx.x / kWave;
  if ((threadIdx.x % kWave) == 0) lds[wave] = a;
  __syncthreads();
  ArgMax r = lds[0];
  for (int i = 1; i < kSampWaves; ++i) r = better(r, lds[i]);
  __syncthreads();
  return r;
}

__device__ __forceinline__ ArgMax row_argmax(const float* x, int n, ArgMax* lds) {
  ArgMax a;
  a.v = -INFINITY;
  a.i = 0x7fffffff;
  for (int i = threadIdx.x; i < n; i += kSampThreads) {
    ArgMax c;
    c.v = x[i];
    c.i = i;
    // NaN never wins a comparison; a row of NaNs yields index 0 below.
    a = better(a, c);
  }
  ArgMax r = block_argmax(a, lds);
  if (r.i == 0x7fffffff) r.i = 0;
  return r;
}

__global__ __launch_bounds__(kSampThreads) void argmax_rows_kernel(const float* __restrict__ logits,
                                                                  int vocab, int* __restrict__ out) {
  __shared__ ArgMax lds[kSampWaves];
  const float* x = logits + static_cast<int64_t>(blockIdx.x) * vocab;
  ArgMax r = row_argmax(x, vocab, lds);
  if (threadIdx.x == 0) out[blockIdx.x] = r.i;
}

// A row cut into gridDim.x chunks, so that a few rows still fill the chip: every workgroup leaves the best
// (value, index) of its chunk in parts[row][chunk], and argmax_merge_kernel picks among them by the same rule.
constexpr int kChunkThreads = 256;

__global__ __launch_bounds__(kChunkThreads) void argmax_chunks_kernel(const float* __restrict__ logits, int vocab,
                                                                     int chunk_len, ArgMax* __restrict__ parts) {
  __shared__ ArgMax lds[kChunkThreads / kWave];
  const int row = blockIdx.y, chunk = blockIdx.x;
  const float* x = logits + static_cast<int64_t>(row) * vocab;
  const int begin = chunk * chunk_len, end = min(vocab, begin + chunk_len);
  ArgMax a;
  a.v = -INFINITY;
  a.i = 0x7fffffff;
  auto take = [&](float v, int i) {
    ArgMax c;
    c.v = v;
    c.i = i;
    a = better(a, c);
  };
  // chunk_len is a multiple of 4: with a 16-byte aligned row, four logits a load
  if (reinterpret_cast<uintptr_t>(x) % 16 == 0) {
    const int whole = begin + (max(end - begin, 0) & ~3);
    for (int i = begin + 4 * static_cast<int>(threadIdx.x); i < whole; i += 4 * kChunkThreads) {
      const float4 v = *reinterpret_cast<const float4*>(x + i);
      take(v.x, i);
      take(v.y, i + 1);
      take(v.z, i + 2);
      take(v.w, i + 3);
    }
    for (int i = whole + static_cast<int>(threadIdx.x); i < end; i += kChunkThreads) take(x[i], i);
  } else {
    for (int i = begin + static_cast<int>(threadIdx.x); i < end; i += kChunkThreads) take(x[i], i);
  }
#pragma unroll
  for (int off = kWave / 2; off > 0; off >>= 1) {
    ArgMax o;
    o.v = __shfl_xor(a.v, off, kWave);
    o.i = __shfl_xor(a.i, off, kWave);
    a = better(a, o);
  }
  if (threadIdx.x % kWave == 0) lds[threadIdx.x / kWave] = a;
  __syncthreads();
  if (threadIdx.x == 0) {
    ArgMax r = lds[0];
    for (int i = 1; i < kChunkThreads / kWave; ++i) r = better(r, lds[i]);
    parts[static_cast<int64_t>(row) * gridDim.x + chunk] = r;
  }
}

__global__ __launch_bounds__(kWave) void argmax_merge_kernel(const ArgMax* __restrict__ parts, int chunks,
                                                             int* __restrict__ out) {
  const ArgMax* p = parts + static_cast<int64_t>(blockIdx.x) * chunks;
  ArgMax a;
  a.v = -INFINITY;
  a.i = 0x7fffffff;
  for (int c = threadIdx.x; c < chunks; c += kWave) a = better(a, p[c]);
#pragma unroll
  for (int off = kWave / 2; off > 0; off >>= 1) {
    ArgMax o;
    o.v = __shfl_xor(a.v, off, kWave);
    o.i = __shfl_xor(a.i, off, kWave);
    a = better(a, o);
  }
  // a row of NaNs (no value ever wins) yields index 0, as in the one-workgroup kernel
  if (threadIdx.x == 0) out[blockIdx.x] = a.i == 0x7fffffff ? 0 : a.i;
}

// ---------------------------------------------------------------------------------------------
// Temperature sampling with min-p, top-k and top-p, many workgroups a row.
//
// e[i] = exp(x[i] / T - max) is kept unnormalised: every filter is "keep e[i] >= some threshold", and since
// e >= 0 the order of the values is the order of their bit patterns.
//   min_p:  e >= min_p                       (the largest e is exp(0) = 1)
//   top_k:  e >= the k-th largest e           (ties of the k-th stay)
//   top_p:  e >= the largest t whose kept mass reaches top_p of the mass kept so far
// The k-th largest value and the mass threshold are found digit by digit, eight bits at a time: a pass over
// the row fills a histogram of 256 bins with the next digit of the elements that match the digits found so
// far; scanning the bins from the top gives the digit in which the count (the mass) is reached.  Counts are
// integers and masses are summed as 64-bit fixed-point numbers (e * 2^40), so the histograms do not depend
// on the order in which workgroups add to them, and every workgroup that reads them finds the same digits.
// The token is then drawn by the inverse CDF in token order: u * (kept mass) falls into a chunk, and inside
// the chunk into a token.
constexpr int kSelThreads = kChunkThreads;
constexpr int kSelWaves = kSelThreads / kWave;
constexpr float kMassScale = 1099511627776.0f;  // 2^40

struct SampleArgs {
  const float* logits;
  float* e;  // [rows, vocab]
  int vocab, chunk_len, chunks;
  const float* temperature;
  const int* top_k;
  const float* top_p;
  const float* min_p;
  const float* u;
  const ArgMax* part_max;          // [rows, chunks]
  unsigned int* hist_k;            // [rows, 4, 256] counts
  unsigned long long* hist_p;      // [rows, 4, 256] masses
  float* chunk_mass;               // [rows, chunks]
  unsigned int* threshold;         // [rows] bits of the final threshold
  int use_top_k, use_top_p;        // 0: no row of this call uses the filter (its passes are not launched)
  int* out;
};

struct RowParams {
  float inv_t, min_p, top_p;
  int k;
  bool greedy, k_active, p_active;
};

__device__ __forceinline__ RowParams row_params(const SampleArgs& a, int row) {
  RowParams r;
  const float temp = a.temperature[row];
  r.k = a.top_k[row];
  r.top_p = a.top_p[row];
  r.min_p = a.min_p[row];
  // Greedy rule of the reference: (T <= 0 or top_k == 1) and no stochastic filter.
  r.greedy = (temp <= 0.f || r.k == 1) && r.top_p >= 1.f && r.min_p <= 0.f;
  r.inv_t = temp > 0.f ? 1.0f / temp : 1.0f;
  r.k_active = a.use_top_k && r.k > 0 && r.k < a.vocab;
  r.p_active = a.use_top_p && r.top_p < 1.f;
  return r;
}

__device__ __forceinline__ unsigned long long shfl_u64(unsigned long long v, int src) {
  const unsigned int lo = __shfl(static_cast<unsigned int>(v), src, kWave);
  const unsigned int hi = __shfl(static_cast<unsigned int>(v >> 32), src, kWave);
  return (static_cast<unsigned long long>(hi) << 32) | lo;
}
__device__ __forceinline__ unsigned int shfl_any(unsigned int v, int src) { return __shfl(v, src, kWave); }
__device__ __forceinline__ unsigned long long shfl_any(unsigned long long v, int src) { return shfl_u64(v, src); }

// Digits of the threshold, most significant first, from `levels` histograms [levels][256] (level l holds the
// elements that match the digits of the levels before it).  need: the rank (the mass) to reach, counted from
// the top, at least 1.  Every thread of the workgroup calls this; bins is LDS [levels * 256], result LDS [4].
// Returns false when the whole row does not reach `need` (then everything is kept).  prefix: the digits found,
// rest: what is left to reach inside the bin of the last digit.
template <typename T>
__device__ bool select_digits(const T* __restrict__ hist, int levels, T need, T* bins, unsigned long long* result,
                              unsigned int& prefix, T& rest) {
  for (int l = 0; l < levels; ++l) bins[l * 256 + threadIdx.x] = hist[l * 256 + threadIdx.x];
  __syncthreads();
  if (threadIdx.x < kWave) {
    const int lane = threadIdx.x;
    unsigned int digits = 0;
    bool ok = true;
    for (int l = 0; l < levels && ok; ++l) {
      T m[4];
#pragma unroll
      for (int j = 0; j < 4; ++j) m[j] = bins[l * 256 + 4 * lane + j];
      const T own = m[0] + m[1] + m[2] + m[3];
      T suffix = own;  // sum over the bins of this lane and of the lanes above it
#pragma unroll
      for (int off = 1; off < kWave; off <<= 1) {
        const T other = shfl_any(suffix, min(lane + off, kWave - 1));
        if (lane + off < kWave) suffix += other;
      }
      const T above_lane = suffix - own;
      const bool here = above_lane < need && suffix >= need;
      unsigned int digit = 0;
      T left = 0;
      if (here) {
        T above = above_lane;
#pragma unroll
        for (int j = 3; j >= 0; --j) {
          if (left == 0 && above + m[j] >= need) {
            digit = 4 * lane + j;
            left = need - above;  // >= 1
          }
          above += m[j];
        }
      }
      const unsigned long long votes = __ballot(here);
      if (votes == 0ull) {
        ok = false;
      } else {
        const int src = __ffsll(static_cast<long long>(votes)) - 1;
        digits = (digits << 8) | shfl_any(digit, src);
        need = shfl_any(left, src);
      }
    }
    if (lane == 0) {
      result[0] = ok ? 1ull : 0ull;
      result[1] = digits;
      result[2] = static_cast<unsigned long long>(need);
    }
  }
  __syncthreads();
  prefix = static_cast<unsigned int>(result[1]);
  rest = static_cast<T>(result[2]);
  const bool ok = result[0] != 0ull;
  __syncthreads();  // bins and result may be used again
  return ok;
}

struct SelectLds {
  unsigned long long bins[4 * 256];
  unsigned long long result[4];
};

// Bits of the top-k threshold of a row (0: keep everything), from the four count histograms.
__device__ unsigned int top_k_bits(const SampleArgs& a, int row, const RowParams& r, SelectLds& lds) {
  if (!r.k_active) return 0u;  // the same for every thread
  unsigned int prefix, rest;
  const bool ok = select_digits<unsigned int>(a.hist_k + static_cast<int64_t>(row) * 1024, 4,
                                              static_cast<unsigned int>(r.k),
                                              reinterpret_cast<unsigned int*>(lds.bins), lds.result, prefix, rest);
  return ok ? prefix : 0u;
}

// The threshold below which min_p and top_k drop a token.
__device__ unsigned int floor_bits(const SampleArgs& a, int row, const RowParams& r, SelectLds& lds) {
  const unsigned int mp = r.min_p > 0.f ? __float_as_uint(r.min_p) : 0u;
  return max(mp, top_k_bits(a, row, r, lds));
}

// What top_p asks of the kept mass, as a fixed-point number (at least 1).
__device__ __forceinline__ unsigned long long top_p_need(float top_p, unsigned long long total) {
  const unsigned long long need = static_cast<unsigned long long>(static_cast<double>(top_p) * static_cast<double>(total));
  return need < 1ull ? 1ull : need;
}

__device__ __forceinline__ float merged_max(const SampleArgs& a, int row, float* lds /* [kSelWaves] */) {
  float v = -INFINITY;
  for (int c = threadIdx.x; c < a.chunks; c += kSelThreads)
    v = fmaxf(v, a.part_max[static_cast<int64_t>(row) * a.chunks + c].v);
  return block_max<kSelWaves>(v, lds);
}

// e = exp(x / T - max) for the chunk, and the first digit's histogram of top_k.
__global__ __launch_bounds__(kSelThreads) void sample_exp_kernel(const SampleArgs a) {
  __shared__ float red[kSelWaves];
  __shared__ unsigned int hist[256];
  const int row = blockIdx.y, chunk = blockIdx.x;
  const RowParams r = row_params(a, row);
  if (r.greedy) return;
  hist[threadIdx.x] = 0u;
  const float mx = merged_max(a, row, red) * r.inv_t;  // the block reduction also orders the LDS writes above
  const float* x = a.logits + static_cast<int64_t>(row) * a.vocab;
  float* e = a.e + static_cast<int64_t>(row) * a.vocab;
  const int begin = chunk * a.chunk_len, end = min(a.vocab, begin + a.chunk_len);
  const unsigned int mp = r.min_p > 0.f ? __float_as_uint(r.min_p) : 0u;
  for (int i = begin + static_cast<int>(threadIdx.x); i < end; i += kSelThreads) {
    const float v = expf(x[i] * r.inv_t - mx);
    e[i] = v;
    const unsigned int bits = __float_as_uint(v);
    if (r.k_active && v >= 0.f && bits >= mp) atomicAdd(&hist[bits >> 24], 1u);
  }
  if (!r.k_active) return;
  __syncthreads();
  const unsigned int n = hist[threadIdx.x];
  if (n) atomicAdd(a.hist_k + static_cast<int64_t>(row) * 1024 + threadIdx.x, n);
}

// Digit `level` (1..3) of the top_k threshold.
__global__ __launch_bounds__(kSelThreads) void sample_top_k_kernel(const SampleArgs a, int level) {
  __shared__ SelectLds sel;
  __shared__ unsigned int hist[256];
  const int row = blockIdx.y, chunk = blockIdx.x;
  const RowParams r = row_params(a, row);
  if (r.greedy || !r.k_active) return;
  unsigned int prefix, rest;
  const bool ok = select_digits<unsigned int>(a.hist_k + static_cast<int64_t>(row) * 1024, level,
                                              static_cast<unsigned int>(r.k),
                                              reinterpret_cast<unsigned int*>(sel.bins), sel.result, prefix, rest);
  if (!ok) return;  // fewer than k tokens are left: all of them stay
  hist[threadIdx.x] = 0u;
  __syncthreads();
  const float* e = a.e + static_cast<int64_t>(row) * a.vocab;
  const int begin = chunk * a.chunk_len, end = min(a.vocab, begin + a.chunk_len);
  const unsigned int mp = r.min_p > 0.f ? __float_as_uint(r.min_p) : 0u;
  const int high = 32 - 8 * level, low = 24 - 8 * level;
  for (int i = begin + static_cast<int>(threadIdx.x); i < end; i += kSelThreads) {
    const float v = e[i];
    const unsigned int bits = __float_as_uint(v);
    if (v >= 0.f && bits >= mp && (bits >> high) == prefix) atomicAdd(&hist[(bits >> low) & 255u], 1u);
  }
  __syncthreads();
  const unsigned int n = hist[threadIdx.x];
  if (n) atomicAdd(a.hist_k + static_cast<int64_t>(row) * 1024 + level * 256 + threadIdx.x, n);
}

// Digit `level` (0..3) of the top_p threshold, over what min_p and top_k have kept.
__global__ __launch_bounds__(kSelThreads) void sample_top_p_kernel(const SampleArgs a, int level) {
  __shared__ SelectLds sel;
  __shared__ unsigned long long hist[256];
  const int row = blockIdx.y, chunk = blockIdx.x;
  const RowParams r = row_params(a, row);
  if (r.greedy || !r.p_active) return;
  const unsigned int floor = floor_bits(a, row, r, sel);
  const unsigned long long* hp = a.hist_p + static_cast<int64_t>(row) * 1024;
  unsigned int prefix = 0u;
  if (level > 0) {
    // the whole kept mass is the sum of the first histogram
    sel.bins[threadIdx.x] = hp[threadIdx.x];
    __syncthreads();
    if (threadIdx.x == 0) {
      unsigned long long total = 0ull;
      for (int b = 0; b < 256; ++b) total += sel.bins[b];
      sel.result[3] = total;
    }
    __syncthreads();
    const unsigned long long need = top_p_need(r.top_p, sel.result[3]);
    __syncthreads();
    unsigned long long rest;
    if (!select_digits<unsigned long long>(hp, level, need, sel.bins, sel.result, prefix, rest)) return;
  }
  hist[threadIdx.x] = 0ull;
  __syncthreads();
  const float* e = a.e + static_cast<int64_t>(row) * a.vocab;
  const int begin = chunk * a.chunk_len, end = min(a.vocab, begin + a.chunk_len);
  const int high = 32 - 8 * level, low = 24 - 8 * level;
  for (int i = begin + static_cast<int>(threadIdx.x); i < end; i += kSelThreads) {
    const float v = e[i];
    const unsigned int bits = __float_as_uint(v);
    if (v >= 0.f && bits >= floor && (level == 0 || (bits >> high) == prefix))
      atomicAdd(&hist[(bits >> low) & 255u], static_cast<unsigned long long>(v * kMassScale));
  }
  __syncthreads();
  const unsigned long long n = hist[threadIdx.x];
  if (n) atomicAdd(const_cast<unsigned long long*>(hp) + level * 256 + threadIdx.x, n);
}

// The final threshold of the row and the kept mass of every chunk.
__global__ __launch_bounds__(kSelThreads) void sample_mass_kernel(const SampleArgs a) {
  __shared__ SelectLds sel;
  __shared__ float red[kSelWaves];
  const int row = blockIdx.y, chunk = blockIdx.x;
  const RowParams r = row_params(a, row);
  if (r.greedy) return;
  unsigned int thr = floor_bits(a, row, r, sel);
  if (r.p_active) {
    const unsigned long long* hp = a.hist_p + static_cast<int64_t>(row) * 1024;
    sel.bins[threadIdx.x] = hp[threadIdx.x];
    __syncthreads();
    if (threadIdx.x == 0) {
      unsigned long long total = 0ull;
      for (int b = 0; b < 256; ++b) total += sel.bins[b];
      sel.result[3] = total;
    }
    __syncthreads();
    const unsigned long long need = top_p_need(r.top_p, sel.result[3]);
    __syncthreads();
    unsigned int prefix;
    unsigned long long rest;
    if (select_digits<unsigned long long>(hp, 4, need, sel.bins, sel.result, prefix, rest)) thr = max(thr, prefix);
  }
  if (chunk == 0 && threadIdx.x == 0) a.threshold[row] = thr;
  const float* e = a.e + static_cast<int64_t>(row) * a.vocab;
  const int begin = chunk * a.chunk_len, end = min(a.vocab, begin + a.chunk_len);
  float mass = 0.f;
  for (int i = begin + static_cast<int>(threadIdx.x); i < end; i += kSelThreads) {
    const float v = e[i];
    if (v >= 0.f && __float_as_uint(v) >= thr) mass += v;
  }
  mass = block_sum<kSelWaves>(mass, red);
  if (threadIdx.x == 0) a.chunk_mass[static_cast<int64_t>(row) * a.chunks + chunk] = mass;
}

// The token: greedy rows take the first maximum; the others the inverse CDF in token order.
__global__ __launch_bounds__(kSelThreads) void sample_pick_kernel(const SampleArgs a) {
  __shared__ ArgMax best[kSelWaves];
  __shared__ float part[kSelThreads];
  __shared__ float chunk_start;
  __shared__ int chunk_of_target, chosen;
  const int row = blockIdx.x;
  const RowParams r = row_params(a, row);
  if (r.greedy) {
    ArgMax m;
    m.v = -INFINITY;
    m.i = 0x7fffffff;
    for (int c = threadIdx.x; c < a.chunks; c += kSelThreads)
      m = better(m, a.part_max[static_cast<int64_t>(row) * a.chunks + c]);
#pragma unroll
    for (int off = kWave / 2; off > 0; off >>= 1) {
      ArgMax o;
      o.v = __shfl_xor(m.v, off, kWave);
      o.i = __shfl_xor(m.i, off, kWave);
      m = better(m, o);
    }
    if (threadIdx.x % kWave == 0) best[threadIdx.x / kWave] = m;
    __syncthreads();
    if (threadIdx.x == 0) {
      ArgMax t = best[0];
      for (int w = 1; w < kSelWaves; ++w) t = better(t, best[w]);
      a.out[row] = t.i == 0x7fffffff ? 0 : t.i;
    }
    return;
  }
  const unsigned int thr = a.threshold[row];
  const float* masses = a.chunk_mass + static_cast<int64_t>(row) * a.chunks;
  if (threadIdx.x == 0) {
    float total = 0.f;
    for (int c = 0; c < a.chunks; ++c) total += masses[c];
    const float target = a.u[row] * total;
    float run = 0.f;
    int at = -1, last = 0;
    float start = 0.f, last_start = 0.f;
    for (int c = 0; c < a.chunks; ++c) {
      const float m = masses[c];
      if (m > 0.f) {
        last = c;
        last_start = run;
      }
      if (at < 0 && target < run + m) {
        at = c;
        start = run;
      }
      run += m;
    }
    chunk_of_target = at >= 0 ? at : last;  // u at or past the whole mass (rounding): the last chunk that holds any
    chunk_start = at >= 0 ? start : last_start;
    part[0] = target;
    chosen = -1;
  }
  __syncthreads();
  const int chunk = chunk_of_target;
  const float target = part[0];
  const float before = chunk_start;
  __syncthreads();
  const float* e = a.e + static_cast<int64_t>(row) * a.vocab;
  const int begin = chunk * a.chunk_len, end = min(a.vocab, begin + a.chunk_len);
  // thread t owns the tokens [lo, hi) of the chunk, in token order
  const int per = (end - begin + kSelThreads - 1) / kSelThreads;
  const int lo = min(begin + static_cast<int>(threadIdx.x) * per, end), hi = min(lo + per, end);
  auto kept = [&](int i) {
    const float v = e[i];
    return (v >= 0.f && __float_as_uint(v) >= thr) ? v : 0.f;
  };
  float mine = 0.f;
  for (int i = lo; i < hi; ++i) mine += kept(i);
  part[threadIdx.x] = mine;
  __syncthreads();
  if (threadIdx.x == 0) {
    float run = before;  // exclusive prefix, serial
    for (int t = 0; t < kSelThreads; ++t) {
      const float c = part[t];
      part[t] = run;
      run += c;
    }
  }
  __syncthreads();
  const float start = part[threadIdx.x];
  if (target >= start && target < start + mine && hi > lo) {
    float run = start;
    int pick = -1;
    for (int i = lo; i < hi; ++i) {
      run += kept(i);
      if (target < run) {
        pick = i;
        break;
      }
    }
    if (pick < 0) {  // rounding left the target past this thread's end: its last kept token
      for (int i = hi - 1; i >= lo; --i)
        if (kept(i) > 0.f) {
          pick = i;
          break;
        }
    }
    if (pick >= 0) atomicMax(&chosen, pick);
  }
  __syncthreads();
  if (chosen < 0) {
    // the target lies outside what the threads found (rounding between the two ways of adding): the last kept
    // token of the chunk, or of the row when the chunk holds none
    int last = -1;
    for (int i = begin + static_cast<int>(threadIdx.x); i < end; i += kSelThreads)
      if (kept(i) > 0.f) last = max(last, i);
    if (last >= 0) atomicMax(&chosen, last);
    __syncthreads();
    if (chosen < 0) {
      for (int i = threadIdx.x; i < a.vocab; i += kSelThreads)
        if (kept(i) > 0.f) last = max(last, i);
      if (last >= 0) atomicMax(&chosen, last);
      __syncthreads();
    }
  }
  if (threadIdx.x == 0) a.out[row] = max(chosen, 0);
}

// logits[row, tok] for each (tok, count) listed for the row:
//   l = l >= 0 ? l / rep : l * rep;   l -= freq * count + presence
__global__ void apply_penalties_kernel(float* __restrict__ logits, int vocab,
                                       const int* __restrict__ indptr, const int* __restrict__ tok,
                                       const int* __restrict__ count, const float* __restrict__ rep,
                                       const float* __restrict__ freq,
                                       const float* __restrict__ pres) {
  const int row = blockIdx.x;
  float* x = logits + static_cast<int64_t>(row) * vocab;
  for (int e = indptr[row] + threadIdx.x; e < indptr[row + 1]; e += blockDim.x) {
    const int id = tok[e];
    const int c = count[e];
    if (id < 0 || id >= vocab || c <= 0) continue;
    float l = x[id];
    const float r = rep[row];
    if (r != 1.0f) l = l >= 0.f ? l / r : l * r;
    x[id] = l - freq[row] * static_cast<float>(c) - pres[row];
  }
}

}  // namespace arle

using namespace arle;

// parts: scratch of arle_argmax_chunks(rows, vocab) * rows pairs of 8 bytes, or null when that count is 1.
extern "C" int arle_argmax_chunks(int rows, int vocab) {
  if (rows <= 0 || vocab < 8192) return 1;
  const int wanted = (2048 + rows - 1) / rows;           // about 2048 workgroups of 256 threads in all
  const int most = vocab / 2048;                         // at least 2048 logits a chunk
  return max(1, min(min(wanted, most), 256));
}

extern "C" int arle_argmax_rows(const float* logits, int rows, int vocab, int* out, void* parts, void* stream) {
  if (rows == 0) return 0;
  hipStream_t s = static_cast<hipStream_t>(stream);
  const int chunks = arle_argmax_chunks(rows, vocab);
  if (chunks == 1) {
    argmax_rows_kernel<<<rows, kSampThreads, 0, s>>>(logits, vocab, out);
    return launch_status();
  }
  if (parts == nullptr) return static_cast<int>(hipErrorInvalidValue);
  const int chunk_len = (((vocab + chunks - 1) / chunks) + 3) & ~3;
  argmax_chunks_kernel<<<dim3(chunks, rows), kChunkThreads, 0, s>>>(logits, vocab, chunk_len,
                                                                    static_cast<ArgMax*>(parts));
  argmax_merge_kernel<<<rows, kWave, 0, s>>>(static_cast<const ArgMax*>(parts), chunks, out);
  return launch_status();
}

// Scratch of a sampling call, in bytes: the histograms (which the caller hands over filled with zeros: the whole
// scratch may simply be zeroed), the chunk maxima and masses, and the thresholds.
static inline size_t sample_hist_p_bytes(int rows) { return static_cast<size_t>(rows) * 1024 * sizeof(unsigned long long); }
static inline size_t sample_hist_k_bytes(int rows) { return static_cast<size_t>(rows) * 1024 * sizeof(unsigned int); }
extern "C" long long arle_sample_scratch_bytes(int rows, int vocab) {
  const size_t chunks = static_cast<size_t>(arle_argmax_chunks(rows, vocab));
  return static_cast<long long>(sample_hist_p_bytes(rows) + sample_hist_k_bytes(rows) +
                                rows * chunks * (sizeof(ArgMax) + sizeof(float)) + rows * sizeof(unsigned int));
}

// One token id per row of logits [rows, vocab] (float32).  probs is scratch [rows, vocab] float32; scratch holds
// arle_sample_scratch_bytes(rows, vocab) zeroed bytes, 8-byte aligned.  use_top_k / use_top_p == 0 promise that
// no row of the call has the filter switched on (top_k in 1..vocab-1, top_p < 1); its passes are then left out.
extern "C" int arle_sample_rows(const float* logits, int rows, int vocab, float* probs,
                                const float* temperature, const int* top_k, const float* top_p,
                                const float* min_p, const float* u, int* out, void* scratch, int use_top_k,
                                int use_top_p, void* stream) {
  if (rows == 0) return 0;
  if (scratch == nullptr || reinterpret_cast<uintptr_t>(scratch) % 8 != 0 || rows > 65535)
    return static_cast<int>(hipErrorInvalidValue);
  hipStream_t s = static_cast<hipStream_t>(stream);
  SampleArgs a;
  a.logits = logits;
  a.e = probs;
  a.vocab = vocab;
  a.chunks = arle_argmax_chunks(rows, vocab);
  a.chunk_len = (((vocab + a.chunks - 1) / a.chunks) + 3) & ~3;
  a.temperature = temperature;
  a.top_k = top_k;
  a.top_p = top_p;
  a.min_p = min_p;
  a.u = u;
  unsigned char* at = static_cast<unsigned char*>(scratch);
  a.hist_p = reinterpret_cast<unsigned long long*>(at);
  at += sample_hist_p_bytes(rows);
  a.hist_k = reinterpret_cast<unsigned int*>(at);
  at += sample_hist_k_bytes(rows);
  ArgMax* part_max = reinterpret_cast<ArgMax*>(at);
  a.part_max = part_max;
  at += static_cast<size_t>(rows) * a.chunks * sizeof(ArgMax);
  a.chunk_mass = reinterpret_cast<float*>(at);
  at += static_cast<size_t>(rows) * a.chunks * sizeof(float);
  a.threshold = reinterpret_cast<unsigned int*>(at);
  a.use_top_k = use_top_k;
  a.use_top_p = use_top_p;
  a.out = out;
  const dim3 grid(a.chunks, rows);
  argmax_chunks_kernel<<<grid, kChunkThreads, 0, s>>>(logits, vocab, a.chunk_len, part_max);
  sample_exp_kernel<<<grid, kSelThreads, 0, s>>>(a);
  if (use_top_k)
    for (int level = 1; level < 4; ++level) sample_top_k_kernel<<<grid, kSelThreads, 0, s>>>(a, level);
  if (use_top_p)
    for (int level = 0; level < 4; ++level) sample_top_p_kernel<<<grid, kSelThreads, 0, s>>>(a, level);
  sample_mass_kernel<<<grid, kSelThreads, 0, s>>>(a);
  sample_pick_kernel<<<rows, kSelThreads, 0, s>>>(a);
  return launch_status();
}

// out[r] = logits[r][token[r]] - logsumexp(logits[r]): the natural-log probability of the chosen token under
// the softmax of the row (for the largest logit this is the reference's -log(sum exp(x - max)),
// crates/cuda-kernels/csrc/misc/sampling.cu:299-316).  One workgroup a row, fixed order of additions.
__global__ __launch_bounds__(kSampThreads) void token_logprob_kernel(const float* __restrict__ logits, int vocab,
                                                                    const int* __restrict__ token,
                                                                    float* __restrict__ out) {
  __shared__ float lds[kSampWaves];
  const float* x = logits + static_cast<int64_t>(blockIdx.x) * vocab;
  float m = -INFINITY;
  for (int i = threadIdx.x; i < vocab; i += kSampThreads) m = fmaxf(m, x[i]);
  m = block_max<kSampWaves>(m, lds);
  float sum = 0.f;
  for (int i = threadIdx.x; i < vocab; i += kSampThreads) sum += expf(x[i] - m);
  sum = block_sum<kSampWaves>(sum, lds);
  if (threadIdx.x == 0) {
    const int t = token[blockIdx.x];
    out[blockIdx.x] = (t >= 0 && t < vocab) ? x[t] - m - logf(sum) : -INFINITY;
  }
}

extern "C" int arle_token_logprobs(const float* logits, int rows, int vocab, const int* token, float* out,
                                   void* stream) {
  if (rows == 0) return 0;
  if (vocab <= 0) return static_cast<int>(hipErrorInvalidValue);
  token_logprob_kernel<<<rows, kSampThreads, 0, static_cast<hipStream_t>(stream)>>>(logits, vocab, token, out);
  return launch_status();
}

extern "C" int arle_apply_penalties(float* logits, int rows, int vocab, const int* indptr,
                                    const int* tok, const int* count, const float* rep,
                                    const float* freq, const float* pres, void* stream) {
  if (rows == 0) return 0;
  apply_penalties_kernel<<<rows, 256, 0, static_cast<hipStream_t>(stream)>>>(
      logits, vocab, indptr, tok, count, rep, freq, pres);
  return launch_status();
}
