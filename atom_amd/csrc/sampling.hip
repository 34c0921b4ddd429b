// Sampling from float32 logits: one block per row, or, for large vocabularies (from 16,384 tokens, given
// workspaces), every row spread over 64 blocks (chunk maxima, threshold rounds, the race per chunk, a pick).
//
//   greedy (temperature 0):  lowest index of the maximum.
//   otherwise:               token = argmax_v softmax(logits / T)_v / (E_v + eps),  E_v ~ Exp(1),
//                            an exponential race, which draws from softmax(logits / T).
//   top-k / top-p:           the race runs only among the kept tokens: the k likeliest, and of the
//                            descending order those whose preceding mass is <= top_p (the likeliest
//                            token always stays).  Both sets are "scaled logit >= threshold" sets, and
//                            each threshold is found digit by digit (12, 12 and 8 bits of the logit's
//                            order-preserving bit pattern) from histograms of counts and of mass.
// The noise is either given ([rows, vocab], or one row shared by all with noise_stride 0) or made
// from (seed, counter, token) of the row by an integer mix, so a request's draws do not depend on
// what else is in the batch.
#include "common.h"

constexpr int kSampleThreads = 1024;
constexpr int kDigitBins = 4096;   // bins of the widest digit of the threshold search
constexpr int kArgmaxChunks = 64;  // blocks over which a row of a large vocabulary is spread

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
              const unsigned long long* __restrict__ counters, int* __restrict__ out, int vocab, float eps,
              const float* __restrict__ chunk_vals, const int* __restrict__ chunk_idx) {
  __shared__ float sv[16];
  __shared__ int si[16];
  __shared__ float scratch[16];
  const int r = blockIdx.x;
  const int tid = threadIdx.x;
  const float* row = logits + (size_t)r * vocab;
  const float temp = temperatures ? temperatures[r] : 0.f;

  // the row's maximum: from the chunks' maxima where argmax_chunks_kernel has left them, else a scan
  MaxIdx m{-INFINITY, 0x7fffffff};
  if (chunk_vals) {
    if (tid < kArgmaxChunks) m = MaxIdx{chunk_vals[r * kArgmaxChunks + tid], chunk_idx[r * kArgmaxChunks + tid]};
  } else {
    for (int v = tid; v < vocab; v += kSampleThreads) m = better(m, MaxIdx{row[v], v});
  }
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

  const bool want_k = k > 0 && k < vocab;
  const bool want_p = p < 1.f;
  if (want_k || want_p) {
    // Two thresholds over key = float_key(scaled logit), found together, a digit a pass:
    //   top-k  u_k = the k-th largest key: the largest u with count(key >= u) >= k
    //   top-p  u_p = the smallest u with mass(key > u) <= p * total mass
    // A pass builds, over the keys that share the digits found so far, a histogram of the next digit:
    // counts for u_k, mass (exp of the scaled logit, as a 2^40 fixed-point integer, so that the sums do
    // not depend on the order of the additions) for u_p.  One wave then walks the histogram from the top.
    __shared__ unsigned int hist_cnt[kDigitBins];
    __shared__ unsigned long long hist_mass[kDigitBins];
    __shared__ unsigned int found_k, found_p;          // the digits found so far, as the key's top bits
    __shared__ unsigned int left_k;                    // how many of the k are still to be found below
    __shared__ unsigned long long left_mass;           // how much of the budget is left for what lies below
    if (tid == 0) {
      found_k = found_p = 0u;
      left_k = want_k ? (unsigned int)k : 0u;
      left_mass = 0ull;
    }
    const int shifts[3] = {20, 8, 0};
    const int widths[3] = {12, 12, 8};
    for (int pass = 0; pass < 3; ++pass) {
      const int shift = shifts[pass], bins = 1 << widths[pass];
      for (int b = tid; b < bins; b += kSampleThreads) {
        hist_cnt[b] = 0u;
        hist_mass[b] = 0ull;
      }
      __syncthreads();
      const unsigned int prefix_k = found_k, prefix_p = found_p;
      const int above = shift + widths[pass];      // bits above this digit (32: none)
      for (int v = tid; v < vocab; v += kSampleThreads) {
        const float sl = (row[v] - top) * inv_t;
        const uint32_t key = float_key(sl);
        const uint32_t digit = (key >> shift) & (uint32_t)(bins - 1);
        const uint32_t high = above >= 32 ? 0u : key >> above;
        if (want_k && high == (above >= 32 ? 0u : prefix_k >> above)) atomicAdd(&hist_cnt[digit], 1u);
        if (want_p && high == (above >= 32 ? 0u : prefix_p >> above))
          atomicAdd(&hist_mass[digit], (unsigned long long)(expf(sl) * 1099511627776.f));
      }
      __syncthreads();
      if (tid < kWave) {
        // lane l owns bins [per * l, per * l + per): what lies in higher bins, then a walk down its own
        const int per = bins / kWave;
        unsigned int cnt_own = 0u;
        unsigned long long mass_own = 0ull;
        for (int b = 0; b < per; ++b) {
          cnt_own += hist_cnt[per * tid + b];
          mass_own += hist_mass[per * tid + b];
        }
        unsigned int cnt_above = cnt_own;
        unsigned long long mass_above = mass_own;
#pragma unroll
        for (int off = 1; off < kWave; off <<= 1) {   // inclusive sums over lanes >= this one
          const unsigned int c = __shfl_down(cnt_above, off, kWave);
          const unsigned long long m = __shfl_down(mass_above, off, kWave);
          if (tid + off < kWave) {
            cnt_above += c;
            mass_above += m;
          }
        }
        const unsigned long long total_mass = __shfl(mass_above, 0, kWave);
        cnt_above -= cnt_own;
        mass_above -= mass_own;
        if (want_p && pass == 0 && tid == 0) left_mass = (unsigned long long)((double)p * (double)total_mass);
        // (the budget is read by every lane after this point; it is written by lane 0 of this same wave)
        __builtin_amdgcn_s_waitcnt(0xc07f);
        __builtin_amdgcn_wave_barrier();
        const unsigned int need = left_k;
        const unsigned long long budget = left_mass;
        for (int b = per - 1; b >= 0; --b) {
          const int bin = per * tid + b;
          const unsigned int c = hist_cnt[bin];
          const unsigned long long m = hist_mass[bin];
          if (want_k && cnt_above < need && cnt_above + c >= need) {   // the k-th largest lies in this bin
            found_k = prefix_k | ((unsigned int)bin << shift);
            left_k = need - cnt_above;
          }
          // the lowest bin whose higher bins hold no more than the budget
          if (want_p && mass_above <= budget && (mass_above + m > budget || bin == 0)) {
            found_p = prefix_p | ((unsigned int)bin << shift);
            left_mass = budget - mass_above;
          }
          cnt_above += c;
          mass_above += m;
        }
      }
      __syncthreads();
    }
    if (want_k) threshold = found_k;
    if (want_p && found_p > threshold) threshold = found_p;
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

// The exponential race of rows without top-k / top-p, over chunks: a block runs the race among the tokens of
// one chunk of one row (the row's maximum is the largest of the chunks' maxima that argmax_chunks_kernel
// left), and argmax_pick_kernel picks among the chunks' winners.  A row with temperature 0 hands its chunk's
// maximum on.  Values and tie rule are sample_kernel's, so the token is the same.
__global__ void __launch_bounds__(256)
race_chunks_kernel(const float* __restrict__ logits, const float* __restrict__ temperatures,
                   const float* __restrict__ noise, long noise_stride, const unsigned long long* __restrict__ seeds,
                   const unsigned long long* __restrict__ counters, const float* __restrict__ max_vals,
                   const int* __restrict__ max_idx, float* __restrict__ ws_vals, int* __restrict__ ws_idx, int vocab,
                   float eps, const unsigned int* __restrict__ thresholds) {
  __shared__ float sv[16];
  __shared__ int si[16];
  const int r = blockIdx.y;
  const int chunk = blockIdx.x;
  const uint32_t threshold = thresholds ? thresholds[r] : 0u;   // only keys >= threshold take part
  const float temp = temperatures[r];
  if (!(temp > 0.f)) {
    if (threadIdx.x == 0) {
      ws_vals[r * kArgmaxChunks + chunk] = max_vals[r * kArgmaxChunks + chunk];
      ws_idx[r * kArgmaxChunks + chunk] = max_idx[r * kArgmaxChunks + chunk];
    }
    return;
  }
  float top = max_vals[r * kArgmaxChunks + (threadIdx.x & (kWave - 1))];
#pragma unroll
  for (int off = kWave / 2; off > 0; off >>= 1) top = fmaxf(top, __shfl_xor(top, off, kWave));
  const int per = (vocab + kArgmaxChunks - 1) / kArgmaxChunks;
  const int lo = chunk * per, hi = min(vocab, lo + per);
  const float* row = logits + (size_t)r * vocab;
  const float* nrow = noise ? noise + (size_t)r * noise_stride : nullptr;
  const uint64_t seed = seeds ? seeds[r] : 0ull;
  const uint64_t counter = counters ? counters[r] : 0ull;
  const float inv_t = 1.f / temp;
  MaxIdx best{-INFINITY, 0x7fffffff};
  for (int v = lo + threadIdx.x; v < hi; v += blockDim.x) {
    const float s = (row[v] - top) * inv_t;
    if (float_key(s) < threshold) continue;
    const float e = nrow ? nrow[v] : exponential_draw(seed, counter, v);
    best = better(best, MaxIdx{expf(s) / (e + eps), v});
  }
  best = block_argmax(best, sv, si);
  if (threadIdx.x == 0) {
    ws_vals[r * kArgmaxChunks + chunk] = best.v;
    ws_idx[r * kArgmaxChunks + chunk] = best.i;
  }
}

// ---- top-k / top-p thresholds of rows of a large vocabulary, spread over 64 blocks a row.
//
// The thresholds are those of sample_kernel (u_k: the k-th largest key; u_p: the smallest u with
// mass(key > u) <= p * total mass; mass as a 2^40 fixed-point integer), found digit by digit (12, 12, 8 bits):
// filter_hist_kernel adds a chunk's keys that share the digits found so far to the row's histogram of the next
// digit (counts for u_k, mass for u_p), filter_select_kernel walks the histogram from the top, notes the digit
// and what is left to find below it, and leaves the histogram zeroed for the next pass (and the next call: the
// histograms must be zero when atom_sample is entered, and are when it returns).
// state32[row] = {digits of u_k so far, what is left of k, digits of u_p so far, unused}; state64[row] = what is
// left of the mass budget.
struct FilterPass {
  int shift, width;
};
__device__ __forceinline__ FilterPass filter_pass(int pass) {
  return pass == 0 ? FilterPass{20, 12} : (pass == 1 ? FilterPass{8, 12} : FilterPass{0, 8});
}

template <int PASS>
__global__ void __launch_bounds__(256)
filter_hist_kernel(const float* __restrict__ logits, const float* __restrict__ temperatures,
                   const int* __restrict__ top_ks, const float* __restrict__ top_ps,
                   const float* __restrict__ max_vals, unsigned int* __restrict__ hist_cnt,
                   unsigned long long* __restrict__ hist_mass, const unsigned int* __restrict__ state32, int vocab) {
  const int r = blockIdx.y;
  const int chunk = blockIdx.x;          // of gridDim.x chunks of the row (its own division, not the maxima's)
  const float temp = temperatures[r];
  const int k = top_ks ? top_ks[r] : -1;
  const bool want_k = k > 0 && k < vocab;
  const bool want_p = top_ps && top_ps[r] < 1.f;
  if (!(temp > 0.f) || !(want_k || want_p)) return;
  float top = max_vals[r * kArgmaxChunks + (threadIdx.x & (kWave - 1))];
#pragma unroll
  for (int off = kWave / 2; off > 0; off >>= 1) top = fmaxf(top, __shfl_xor(top, off, kWave));
  const FilterPass fp = filter_pass(PASS);
  const int bins = 1 << fp.width, above = fp.shift + fp.width;
  const uint32_t prefix_k = PASS ? state32[4 * r] >> above : 0u;
  const uint32_t prefix_p = PASS ? state32[4 * r + 2] >> above : 0u;
  const int per = (vocab + (int)gridDim.x - 1) / (int)gridDim.x;
  const int lo = chunk * per, hi = min(vocab, lo + per);
  const float* row = logits + (size_t)r * vocab;
  const float inv_t = 1.f / temp;
  unsigned int* cnt = hist_cnt + (size_t)r * kDigitBins;
  unsigned long long* mass = hist_mass + (size_t)r * kDigitBins;
  if (PASS == 0) {
    // every key takes part: a histogram of the block in LDS first, then its non-empty bins to the row's
    __shared__ unsigned int lcnt[kDigitBins];
    __shared__ unsigned long long lmass[kDigitBins];
    for (int b = threadIdx.x; b < bins; b += blockDim.x) {
      lcnt[b] = 0u;
      lmass[b] = 0ull;
    }
    __syncthreads();
    for (int v = lo + threadIdx.x; v < hi; v += blockDim.x) {
      const float sl = (row[v] - top) * inv_t;
      const uint32_t digit = float_key(sl) >> fp.shift;
      if (want_k) atomicAdd(&lcnt[digit], 1u);
      if (want_p) atomicAdd(&lmass[digit], (unsigned long long)(expf(sl) * 1099511627776.f));
    }
    __syncthreads();
    for (int b = threadIdx.x; b < bins; b += blockDim.x) {
      if (lcnt[b]) atomicAdd(&cnt[b], lcnt[b]);
      if (lmass[b]) atomicAdd(&mass[b], lmass[b]);
    }
  } else {
    for (int v = lo + threadIdx.x; v < hi; v += blockDim.x) {
      const float sl = (row[v] - top) * inv_t;
      const uint32_t key = float_key(sl);
      const uint32_t digit = (key >> fp.shift) & (uint32_t)(bins - 1);
      const uint32_t high = key >> above;
      if (want_k && high == prefix_k) atomicAdd(&cnt[digit], 1u);
      if (want_p && high == prefix_p) atomicAdd(&mass[digit], (unsigned long long)(expf(sl) * 1099511627776.f));
    }
  }
}

constexpr int kSelectThreads = 256;

template <int PASS>
__global__ void __launch_bounds__(kSelectThreads)
filter_select_kernel(const float* __restrict__ temperatures, const int* __restrict__ top_ks,
                     const float* __restrict__ top_ps, unsigned int* __restrict__ hist_cnt,
                     unsigned long long* __restrict__ hist_mass, unsigned int* __restrict__ state32,
                     unsigned long long* __restrict__ state64, unsigned int* __restrict__ thresholds, int vocab) {
  __shared__ unsigned int tot_cnt[kSelectThreads / kWave];
  __shared__ unsigned long long tot_mass[kSelectThreads / kWave];
  __shared__ unsigned int result[2];   // the digits of u_k and u_p found in this pass
  const int r = blockIdx.x;
  const int tid = threadIdx.x;
  const int k = top_ks ? top_ks[r] : -1;
  const float p = top_ps ? top_ps[r] : 1.f;
  const bool want_k = k > 0 && k < vocab;
  const bool want_p = p < 1.f;
  if (!(temperatures[r] > 0.f) || !(want_k || want_p)) {
    if (PASS == 2 && tid == 0) thresholds[r] = 0u;
    return;
  }
  const FilterPass fp = filter_pass(PASS);
  constexpr int BINS = PASS == 2 ? 256 : kDigitBins;
  constexpr int PER = BINS / kSelectThreads;   // thread t owns bins [PER * t, PER * t + PER)
  unsigned int* cnt = hist_cnt + (size_t)r * kDigitBins;
  unsigned long long* mass = hist_mass + (size_t)r * kDigitBins;
  unsigned int c[PER];
  unsigned long long m[PER];
  unsigned int cnt_own = 0u;
  unsigned long long mass_own = 0ull;
#pragma unroll
  for (int b = 0; b < PER; ++b) {
    c[b] = cnt[PER * tid + b];
    m[b] = mass[PER * tid + b];
    cnt[PER * tid + b] = 0u;          // the histogram is left empty for the next pass
    mass[PER * tid + b] = 0ull;
    cnt_own += c[b];
    mass_own += m[b];
  }
  // what lies in the bins above this thread's, and the row's total mass: sums over the higher lanes of the
  // wave by shuffles, over the higher waves through LDS
  const int lane = tid & (kWave - 1), wave = tid / kWave;
  unsigned int cnt_above = cnt_own;
  unsigned long long mass_above = mass_own;
#pragma unroll
  for (int off = 1; off < kWave; off <<= 1) {   // inclusive sums over lanes >= this one
    const unsigned int cc = __shfl_down(cnt_above, off, kWave);
    const unsigned long long mm = __shfl_down(mass_above, off, kWave);
    if (lane + off < kWave) {
      cnt_above += cc;
      mass_above += mm;
    }
  }
  if (lane == 0) {
    tot_cnt[wave] = cnt_above;
    tot_mass[wave] = mass_above;
  }
  if (tid < 2) result[tid] = 0u;
  __syncthreads();
  cnt_above -= cnt_own;
  mass_above -= mass_own;
  unsigned long long total_mass = 0ull;
#pragma unroll
  for (int w = 0; w < kSelectThreads / kWave; ++w) {
    total_mass += tot_mass[w];
    if (w > wave) {
      cnt_above += tot_cnt[w];
      mass_above += tot_mass[w];
    }
  }
  const unsigned int prefix_k = PASS ? state32[4 * r] : 0u;
  const unsigned int prefix_p = PASS ? state32[4 * r + 2] : 0u;
  const unsigned int need = PASS ? state32[4 * r + 1] : (unsigned int)max(k, 0);
  const unsigned long long budget = PASS ? state64[r] : (unsigned long long)((double)p * (double)total_mass);
  __syncthreads();   // every thread has read the state before the finders write it
#pragma unroll
  for (int b = PER - 1; b >= 0; --b) {
    const int bin = PER * tid + b;
    if (want_k && cnt_above < need && cnt_above + c[b] >= need) {   // the k-th largest lies in this bin
      const unsigned int found = prefix_k | ((unsigned int)bin << fp.shift);
      state32[4 * r] = found;
      state32[4 * r + 1] = need - cnt_above;
      result[0] = found;
    }
    // the lowest bin whose higher bins hold no more than the budget
    if (want_p && mass_above <= budget && (mass_above + m[b] > budget || bin == 0)) {
      const unsigned int found = prefix_p | ((unsigned int)bin << fp.shift);
      state32[4 * r + 2] = found;
      state64[r] = budget - mass_above;
      result[1] = found;
    }
    cnt_above += c[b];
    mass_above += m[b];
  }
  if (PASS == 2) {
    __syncthreads();
    if (tid == 0) thresholds[r] = max(result[0], result[1]);   // the race keeps keys >= both thresholds
  }
}

// `ws_vals` / `ws_idx` (rows * 128 elements each, or null) let calls without top-k / top-p spread every row
// of a large vocabulary over 64 blocks.
// `ws_filter` (or null): rows * 4096 * 12 + rows * 32 bytes, 8-byte aligned, all zero on entry (it is zero again
// on return), lets rows with top-k / top-p be spread over 64 blocks too.
ATOM_EXPORT int atom_sample(const float* logits, const float* temperatures, const int* top_ks, const float* top_ps,
                            const float* noise, long noise_stride, const unsigned long long* seeds,
                            const unsigned long long* counters, int* out, int rows, int vocab, float eps,
                            float* ws_vals, int* ws_idx, void* ws_filter, hipStream_t stream) {
  if (rows < 0 || vocab <= 0) return ATOM_BAD_SHAPE;
  if (rows == 0) return ATOM_OK;
  static_assert(kArgmaxChunks == kWave, "the pick kernel holds one chunk per lane");
  if (!top_ks && !top_ps && ws_vals && ws_idx && vocab >= 16384 && rows <= 65535) {
    hipLaunchKernelGGL(argmax_chunks_kernel, dim3(kArgmaxChunks, rows), dim3(256), 0, stream, logits, ws_vals, ws_idx,
                       vocab);
    if (temperatures) {   // the race among each chunk's tokens, into the second half of the workspaces
      float* race_vals = ws_vals + (size_t)rows * kArgmaxChunks;
      int* race_idx = ws_idx + (size_t)rows * kArgmaxChunks;
      hipLaunchKernelGGL(race_chunks_kernel, dim3(kArgmaxChunks, rows), dim3(256), 0, stream, logits, temperatures,
                         noise, noise_stride, seeds, counters, ws_vals, ws_idx, race_vals, race_idx, vocab, eps,
                         (const unsigned int*)nullptr);
      hipLaunchKernelGGL(argmax_pick_kernel, dim3(rows), dim3(kWave), 0, stream, race_vals, race_idx, out);
    } else {
      hipLaunchKernelGGL(argmax_pick_kernel, dim3(rows), dim3(kWave), 0, stream, ws_vals, ws_idx, out);
    }
    return launch_status();
  }
  const bool spread = ws_vals && ws_idx && vocab >= 16384 && rows <= 65535;
  if (spread && ws_filter && temperatures) {
    // chunk maxima; three rounds of (histogram over 64 blocks a row, a walk by one wave a row); the race
    // among the kept tokens of each chunk; the pick among the chunks' winners
    unsigned long long* hist_mass = (unsigned long long*)ws_filter;
    unsigned long long* state64 = hist_mass + (size_t)rows * kDigitBins;
    unsigned int* hist_cnt = (unsigned int*)(state64 + rows);
    unsigned int* state32 = hist_cnt + (size_t)rows * kDigitBins;
    unsigned int* thresholds = state32 + (size_t)rows * 4;   // 4 + 1 words a row: rows * 32 bytes hold them
    const dim3 wide(kArgmaxChunks, rows);
    const dim3 hist_grid = wide;
    hipLaunchKernelGGL(argmax_chunks_kernel, wide, dim3(256), 0, stream, logits, ws_vals, ws_idx, vocab);
#define FILTER_ROUND(P)                                                                                            \
  hipLaunchKernelGGL((filter_hist_kernel<P>), hist_grid, dim3(256), 0, stream, logits, temperatures, top_ks,       \
                     top_ps,                                                                                      \
                     ws_vals, hist_cnt, hist_mass, state32, vocab);                                                \
  hipLaunchKernelGGL((filter_select_kernel<P>), dim3(rows), dim3(kSelectThreads), 0, stream, temperatures, top_ks, \
                     top_ps,                                                                                      \
                     hist_cnt, hist_mass, state32, state64, thresholds, vocab)
    FILTER_ROUND(0);
    FILTER_ROUND(1);
    FILTER_ROUND(2);
#undef FILTER_ROUND
    float* race_vals = ws_vals + (size_t)rows * kArgmaxChunks;
    int* race_idx = ws_idx + (size_t)rows * kArgmaxChunks;
    hipLaunchKernelGGL(race_chunks_kernel, wide, dim3(256), 0, stream, logits, temperatures, noise, noise_stride,
                       seeds, counters, ws_vals, ws_idx, race_vals, race_idx, vocab, eps, thresholds);
    hipLaunchKernelGGL(argmax_pick_kernel, dim3(rows), dim3(kWave), 0, stream, race_vals, race_idx, out);
    return launch_status();
  }
  if (spread)   // the rows' maxima by 64 blocks a row instead of one
    hipLaunchKernelGGL(argmax_chunks_kernel, dim3(kArgmaxChunks, rows), dim3(256), 0, stream, logits, ws_vals, ws_idx,
                       vocab);
  hipLaunchKernelGGL(sample_kernel, dim3(rows), dim3(kSampleThreads), 0, stream, logits, temperatures, top_ks,
                     top_ps, noise, noise_stride, seeds, counters, out, vocab, eps, spread ? ws_vals : nullptr,
                     spread ? ws_idx : nullptr);
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
