// Token selection from rows of 32-bit logits: argmax, and temperature sampling
// with min-p / top-k / top-p truncation; plus the repetition / frequency /
// presence penalties applied to logits beforehand.
//
// reference counterparts: crates/cuda-kernels/csrc/misc/sampling.cu:27-87,252-317
// (argmax: first maximum in index order) and :327-596 (temperature -> softmax ->
// top-k -> renormalise -> top-p -> renormalise -> inverse CDF with a uniform u
// drawn on the host); penalties infer/src/sampler.rs:100-140.
//
// Differences kept on purpose: thresholds are found exactly by bisection on the
// bit pattern of the (non-negative) probabilities instead of 32 halvings of a
// float interval, each thread owns a contiguous run of the vocabulary so the
// inverse CDF walks tokens in index order, and one launch serves many rows with
// per-row parameters.
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

__device__ __forceinline__ float block_sum_f(float v, float* lds) {
  return block_sum<kSampWaves>(v, lds);
}

// Largest threshold bits t such that pred(t) holds, pred being monotone
// (true for small t).  Probabilities are >= 0, so their order as floats is
// their order as unsigned bit patterns.
template <typename Pred>
__device__ __forceinline__ uint32_t bisect_bits(Pred pred) {
  uint32_t t = 0;
  for (int bit = 30; bit >= 0; --bit) {
    const uint32_t cand = t | (1u << bit);
    if (pred(cand)) t = cand;
  }
  return t;
}

__global__ __launch_bounds__(kSampThreads) void sample_rows_kernel(
    const float* __restrict__ logits, int vocab, float* __restrict__ probs /* [rows, vocab] */,
    const float* __restrict__ temperature, const int* __restrict__ top_k,
    const float* __restrict__ top_p, const float* __restrict__ min_p, const float* __restrict__ u,
    int* __restrict__ out) {
  __shared__ ArgMax lds_arg[kSampWaves];
  __shared__ float lds[kSampWaves];
  __shared__ float chunk_sum[kSampThreads];
  __shared__ int chosen;
  const int row = blockIdx.x;
  const float* x = logits + static_cast<int64_t>(row) * vocab;
  float* p = probs + static_cast<int64_t>(row) * vocab;
  const float temp = temperature[row];
  const int k = top_k[row];
  const float tp = top_p[row];
  const float mp = min_p[row];

  // Greedy rule of the reference: (T <= 0 or top_k == 1) and no stochastic filter.
  const bool greedy = (temp <= 0.f || k == 1) && tp >= 1.f && mp <= 0.f;
  if (greedy) {
    ArgMax r = row_argmax(x, vocab, lds_arg);
    if (threadIdx.x == 0) out[row] = r.i;
    return;
  }
  const float inv_t = temp > 0.f ? 1.0f / temp : 1.0f;

  // softmax(x / T)
  float mx = -INFINITY;
  for (int i = threadIdx.x; i < vocab; i += kSampThreads) mx = fmaxf(mx, x[i] * inv_t);
  mx = block_max<kSampWaves>(mx, lds);
  float sum = 0.f;
  for (int i = threadIdx.x; i < vocab; i += kSampThreads) {
    const float e = expf(x[i] * inv_t - mx);
    p[i] = e;
    sum += e;
  }
  sum = block_sum_f(sum, lds);
  float norm = 1.0f / sum;  // pending factor: true probability = p[i] * norm
  float pmax = norm;        // exp(0) * norm

  auto renormalise = [&](float threshold_true) {
    // zero what is below the threshold, fold `norm` in, and renormalise the rest
    float kept = 0.f;
    for (int i = threadIdx.x; i < vocab; i += kSampThreads) {
      float v = p[i] * norm;
      if (v < threshold_true) v = 0.f;
      p[i] = v;
      kept += v;
    }
    kept = block_sum_f(kept, lds);
    norm = 1.0f / kept;
    pmax = pmax * norm;
  };

  if (mp > 0.f) renormalise(mp * pmax);

  if (k > 0 && k < vocab) {
    // fold the pending factor in so that thresholds compare stored values
    for (int i = threadIdx.x; i < vocab; i += kSampThreads) p[i] *= norm;
    norm = 1.0f;
    __syncthreads();
    const uint32_t bits = bisect_bits([&](uint32_t cand) {
      float cnt = 0.f;
      for (int i = threadIdx.x; i < vocab; i += kSampThreads)
        cnt += (__float_as_uint(p[i]) >= cand) ? 1.f : 0.f;
      return block_sum_f(cnt, lds) >= static_cast<float>(k);
    });
    renormalise(__uint_as_float(bits));  // keeps the k largest (and ties of the k-th)
  }

  if (tp < 1.f) {
    for (int i = threadIdx.x; i < vocab; i += kSampThreads) p[i] *= norm;
    norm = 1.0f;
    __syncthreads();
    const uint32_t bits = bisect_bits([&](uint32_t cand) {
      float mass = 0.f;
      for (int i = threadIdx.x; i < vocab; i += kSampThreads)
        mass += (__float_as_uint(p[i]) >= cand) ? p[i] : 0.f;
      return block_sum_f(mass, lds) >= tp;
    });
    renormalise(__uint_as_float(bits));  // smallest top set whose mass reaches top_p
  }
  __syncthreads();

  // inverse CDF in token order: thread i owns tokens [i*chunk, (i+1)*chunk)
  const int chunk = (vocab + kSampThreads - 1) / kSampThreads;
  const int lo = min(static_cast<int>(threadIdx.x) * chunk, vocab);
  const int hi = min(lo + chunk, vocab);
  float mine = 0.f;
  for (int i = lo; i < hi; ++i) mine += p[i] * norm;
  chunk_sum[threadIdx.x] = mine;
  if (threadIdx.x == 0) chosen = -1;
  __syncthreads();
  if (threadIdx.x == 0) {
    float run = 0.f;  // exclusive prefix, serial: 1024 adds
    for (int i = 0; i < kSampThreads; ++i) {
      const float c = chunk_sum[i];
      chunk_sum[i] = run;
      run += c;
    }
  }
  __syncthreads();
  const float target = u[row];
  const float start = chunk_sum[threadIdx.x];
  if (target >= start && target < start + mine && hi > lo) {
    float run = start;
    int pick = -1;
    for (int i = lo; i < hi; ++i) {
      run += p[i] * norm;
      if (target < run) {
        pick = i;
        break;
      }
    }
    if (pick < 0) {  // rounding left the target past the chunk's end: last kept token here
      for (int i = hi - 1; i >= lo; --i)
        if (p[i] > 0.f) {
          pick = i;
          break;
        }
    }
    if (pick >= 0) atomicMax(&chosen, pick);
  }
  __syncthreads();
  if (chosen < 0) {
    // u at or beyond the total mass (rounding): the last token with p > 0
    int last = -1;
    for (int i = threadIdx.x; i < vocab; i += kSampThreads)
      if (p[i] > 0.f) last = max(last, i);
    atomicMax(&chosen, last);
    __syncthreads();
  }
  if (threadIdx.x == 0) out[row] = chosen;
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
  const int wanted = (512 + rows - 1) / rows;            // about 512 workgroups in all
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

// probs is scratch [rows, vocab] 32-bit; each listed token id must appear once per row in
// the penalty lists.
extern "C" int arle_sample_rows(const float* logits, int rows, int vocab, float* probs,
                                const float* temperature, const int* top_k, const float* top_p,
                                const float* min_p, const float* u, int* out, void* stream) {
  if (rows == 0) return 0;
  sample_rows_kernel<<<rows, kSampThreads, 0, static_cast<hipStream_t>(stream)>>>(
      logits, vocab, probs, temperature, top_k, top_p, min_p, u, out);
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
