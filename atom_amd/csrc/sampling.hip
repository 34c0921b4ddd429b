// Sampling from float32 logits, one block per row.
//
//   greedy (temperature 0):  lowest index of the maximum.
//   otherwise:               token = argmax_v softmax(logits / T)_v / (E_v + eps),  E_v ~ Exp(1),
//                            an exponential race, which draws from softmax(logits / T).
//   top-k / top-p:           the race runs only among the kept tokens: the k likeliest, and of the
//                            descending order those whose preceding mass is <= top_p (the likeliest
//                            token always stays).  Both sets are "scaled logit >= threshold" sets, and
//                            each threshold is found by a 32-step search over the bit pattern.
// The noise is either given ([rows, vocab], or one row shared by all with noise_stride 0) or made
// from (seed, counter, token) of the row by an integer mix, so a request's draws do not depend on
// what else is in the batch.
#include "common.h"

constexpr int kSampleThreads = 1024;

__device__ __forceinline__ uint64_t mix64(uint64_t x) {
  x = (x ^ (x >> 30)) * 0xBF58476D1CE4E5B9ull;
  x = (x ^ (x >> 27)) * 0x94D049BB133111EBull;
  return x ^ (x >> 31);
}

__device__ __forceinline__ float exponential_draw(uint64_t seed, uint64_t counter, int token) {
  const uint64_t z = mix64(mix64(seed ^ (counter * 0x9E3779B97F4A7C15ull)) + (uint64_t)(token + 1) * 0xD6E8FEB86659FD93ull);
  const float u = ((float)(z >> 40) + 0.5f) * (1.0f / 16777216.0f);  // in (0, 1)
  return -logf(u);
}

// order-preserving map float -> unsigned
__device__ __forceinline__ uint32_t float_key(float f) {
  const uint32_t u = __float_as_uint(f);
  return (u & 0x80000000u) ? ~u : (u | 0x80000000u);
}

struct MaxIdx {
  float v;
  int i;
};

__device__ __forceinline__ MaxIdx better(MaxIdx a, MaxIdx b) {
  // larger value wins; equal values: lower index
  if (b.v > a.v || (b.v == a.v && b.i < a.i)) return b;
  return a;
}

__device__ MaxIdx block_argmax(MaxIdx m, float* sv, int* si) {
  const int lane = threadIdx.x & (kWave - 1);
  const int wave = threadIdx.x / kWave;
#pragma unroll
  for (int off = kWave / 2; off > 0; off >>= 1) {
    MaxIdx o;
    o.v = __shfl_xor(m.v, off, kWave);
    o.i = __shfl_xor(m.i, off, kWave);
    m = better(m, o);
  }
  __syncthreads();
  if (lane == 0) {
    sv[wave] = m.v;
    si[wave] = m.i;
  }
  __syncthreads();
  MaxIdx r{sv[0], si[0]};
  for (int w = 1; w < (int)(blockDim.x / kWave); ++w) r = better(r, MaxIdx{sv[w], si[w]});
  return r;
}

__global__ void __launch_bounds__(kSampleThreads)
sample_kernel(const float* __restrict__ logits, const float* __restrict__ temperatures,
              const int* __restrict__ top_ks, const float* __restrict__ top_ps,
              const float* __restrict__ noise, long noise_stride, const unsigned long long* __restrict__ seeds,
              const unsigned long long* __restrict__ counters, int* __restrict__ out, int vocab, float eps) {
  __shared__ float sv[16];
  __shared__ int si[16];
  __shared__ float scratch[16];
  const int r = blockIdx.x;
  const int tid = threadIdx.x;
  const float* row = logits + (size_t)r * vocab;
  const float temp = temperatures ? temperatures[r] : 0.f;

  MaxIdx m{-INFINITY, 0x7fffffff};
  for (int v = tid; v < vocab; v += kSampleThreads) m = better(m, MaxIdx{row[v], v});
  m = block_argmax(m, sv, si);
  if (!(temp > 0.f)) {
    if (tid == 0) out[r] = m.i;
    return;
  }
  const float inv_t = 1.f / temp;
  const float top = m.v;
  const int k = top_ks ? top_ks[r] : -1;
  const float p = top_ps ? top_ps[r] : 1.f;
  uint32_t threshold = 0u;  // keep keys >= threshold

  if (k > 0 && k < vocab) {
    // largest key u with count(key >= u) >= k
    uint32_t u = 0u;
    for (int bit = 31; bit >= 0; --bit) {
      const uint32_t cand = u | (1u << bit);
      float cnt = 0.f;
      for (int v = tid; v < vocab; v += kSampleThreads)
        cnt += float_key((row[v] - top) * inv_t) >= cand ? 1.f : 0.f;
      cnt = block_sum(cnt, scratch);
      if (cnt >= (float)k) u = cand;
    }
    threshold = u;
  }
  if (p < 1.f) {
    float z = 0.f;
    for (int v = tid; v < vocab; v += kSampleThreads) z += expf((row[v] - top) * inv_t);
    z = block_sum(z, scratch);
    const float budget = p * z;
    // smallest key u with mass(key > u) <= budget; the predicate is monotone in u
    uint32_t u = 0u;
    for (int bit = 31; bit >= 0; --bit) {
      const uint32_t cand = u | (1u << bit);
      // test cand - 1: if mass above (cand - 1) is still over budget, the answer is >= cand
      float mass = 0.f;
      for (int v = tid; v < vocab; v += kSampleThreads) {
        const float s = (row[v] - top) * inv_t;
        mass += float_key(s) > cand - 1u ? expf(s) : 0.f;
      }
      mass = block_sum(mass, scratch);
      if (mass > budget) u = cand;
    }
    if (u > threshold) threshold = u;
  }

  const float* nrow = noise ? noise + (size_t)r * noise_stride : nullptr;
  const uint64_t seed = seeds ? seeds[r] : 0ull;
  const uint64_t counter = counters ? counters[r] : 0ull;
  MaxIdx best{-INFINITY, 0x7fffffff};
  for (int v = tid; v < vocab; v += kSampleThreads) {
    const float s = (row[v] - top) * inv_t;
    if (float_key(s) < threshold) continue;
    const float e = nrow ? nrow[v] : exponential_draw(seed, counter, v);
    best = better(best, MaxIdx{expf(s) / (e + eps), v});
  }
  best = block_argmax(best, sv, si);
  if (tid == 0) out[r] = best.i;
}

// Greedy rows of a large vocabulary in two steps, so that a few rows still use the whole chip: every
// block finds the maximum of one chunk of one row (lowest index on ties), then one wave per row picks
// among the chunks' maxima, lowest chunk first.
constexpr int kArgmaxChunks = 64;

__global__ void __launch_bounds__(256)
argmax_chunks_kernel(const float* __restrict__ logits, float* __restrict__ ws_vals, int* __restrict__ ws_idx,
                     int vocab) {
  __shared__ float sv[16];
  __shared__ int si[16];
  const int r = blockIdx.y;
  const int chunk = blockIdx.x;
  const int per = (vocab + kArgmaxChunks - 1) / kArgmaxChunks;
  const int lo = chunk * per, hi = min(vocab, lo + per);
  const float* row = logits + (size_t)r * vocab;
  MaxIdx m{-INFINITY, 0x7fffffff};
  for (int v = lo + threadIdx.x; v < hi; v += blockDim.x) m = better(m, MaxIdx{row[v], v});
  m = block_argmax(m, sv, si);
  if (threadIdx.x == 0) {
    ws_vals[r * kArgmaxChunks + chunk] = m.v;
    ws_idx[r * kArgmaxChunks + chunk] = m.i;
  }
}

__global__ void __launch_bounds__(kWave)
argmax_pick_kernel(const float* __restrict__ ws_vals, const int* __restrict__ ws_idx, int* __restrict__ out) {
  const int r = blockIdx.x;
  MaxIdx m{ws_vals[r * kArgmaxChunks + threadIdx.x], ws_idx[r * kArgmaxChunks + threadIdx.x]};
#pragma unroll
  for (int off = kWave / 2; off > 0; off >>= 1) {
    MaxIdx o;
    o.v = __shfl_xor(m.v, off, kWave);
    o.i = __shfl_xor(m.i, off, kWave);
    m = better(m, o);
  }
  if (threadIdx.x == 0) out[r] = m.i;
}

// `ws_vals` / `ws_idx` (rows * 64 elements each, or null) let all-greedy calls take the two-step path.
ATOM_EXPORT int atom_sample(const float* logits, const float* temperatures, const int* top_ks, const float* top_ps,
                            const float* noise, long noise_stride, const unsigned long long* seeds,
                            const unsigned long long* counters, int* out, int rows, int vocab, float eps,
                            float* ws_vals, int* ws_idx, hipStream_t stream) {
  if (rows < 0 || vocab <= 0) return ATOM_BAD_SHAPE;
  if (rows == 0) return ATOM_OK;
  static_assert(kArgmaxChunks == kWave, "the pick kernel holds one chunk per lane");
  if (!temperatures && ws_vals && ws_idx && vocab >= 16384 && rows <= 65535) {
    hipLaunchKernelGGL(argmax_chunks_kernel, dim3(kArgmaxChunks, rows), dim3(256), 0, stream, logits, ws_vals, ws_idx,
                       vocab);
    hipLaunchKernelGGL(argmax_pick_kernel, dim3(rows), dim3(kWave), 0, stream, ws_vals, ws_idx, out);
    return launch_status();
  }
  hipLaunchKernelGGL(sample_kernel, dim3(rows), dim3(kSampleThreads), 0, stream, logits, temperatures, top_ks,
                     top_ps, noise, noise_stride, seeds, counters, out, vocab, eps);
  return launch_status();
}

__global__ void exponential_noise_kernel(float* __restrict__ out, const unsigned long long* __restrict__ seeds,
                                         const unsigned long long* __restrict__ counters, int vocab) {
  const int r = blockIdx.y;
  const int v = blockIdx.x * blockDim.x + threadIdx.x;
  if (v < vocab) out[(size_t)r * vocab + v] = exponential_draw(seeds[r], counters[r], v);
}

ATOM_EXPORT int atom_exponential_noise(float* out, const unsigned long long* seeds,
                                       const unsigned long long* counters, int rows, int vocab,
                                       hipStream_t stream) {
  if (rows < 0 || vocab <= 0 || rows > 65535) return ATOM_BAD_SHAPE;
  if (rows == 0) return ATOM_OK;
  hipLaunchKernelGGL(exponential_noise_kernel, dim3((vocab + 255) / 256, rows), dim3(256), 0, stream, out, seeds,
                     counters, vocab);
  return launch_status();
}
