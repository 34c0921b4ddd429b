// Paged attention, general form: any head size, any page size, float32 or bfloat16,
// every query token of a mixed batch (prompt portions and single decoded tokens alike).
//
// One block per (query token, query head).  The token's request and absolute position
// are given per token; the keys it sees are positions max(0, p - window + 1) .. p of that
// request, found through the request's block table.  Keys are walked in fixed chunks
// counted from position 0 with a running maximum and sum (all float32), so the result
// for a token depends only on its own keys: not on the batch, not on how the prompt
// was cut into steps, not on which pages hold the keys.
//
// Pages: keys [num_pages, Hkv, page_size, D]; values [num_pages, Hkv, D, page_size].
#include "common.h"

constexpr int kAttnThreads = 128;
constexpr int kAttnChunk = 512;  // keys per pass

template <typename T>
__global__ void __launch_bounds__(kAttnThreads)
paged_attention_generic_kernel(const T* __restrict__ q, const T* __restrict__ k_cache,
                               const T* __restrict__ v_cache, T* __restrict__ out,
                               const int* __restrict__ token_seq, const int* __restrict__ positions,
                               const int* __restrict__ block_tables, int max_blocks, int hq, int hkv,
                               int d, int page_size, float scale, int window) {
  extern __shared__ float smem[];
  float* qs = smem;                  // d
  float* probs = qs + d;             // kAttnChunk
  float* scratch = probs + kAttnChunk;  // 16
  const int t = blockIdx.x;
  const int h = blockIdx.y;
  const int kvh = h / (hq / hkv);
  const int tid = threadIdx.x;
  const int seq = token_seq[t];
  const int pos = positions[t];
  T* dst = out + ((size_t)t * hq + h) * d;
  if (seq < 0) {  // padding row
    for (int i = tid; i < d; i += kAttnThreads) dst[i] = from_f32<T>(0.f);
    return;
  }
  const int* table = block_tables + (size_t)seq * max_blocks;
  const T* qr = q + ((size_t)t * hq + h) * d;
  for (int i = tid; i < d; i += kAttnThreads) qs[i] = to_f32(qr[i]) * scale;
  __syncthreads();

  const int first = (window > 0 && pos - window + 1 > 0) ? pos - window + 1 : 0;
  const int last = pos;  // inclusive
  // each thread owns output dims tid, tid + 128, ... (at most 4 for d <= 512)
  float acc[4] = {0.f, 0.f, 0.f, 0.f};
  float run_max = -INFINITY, run_sum = 0.f;

  // chunks are aligned to multiples of kAttnChunk from position 0, so the grouping of
  // keys does not move with the window start
  for (int base = (first / kAttnChunk) * kAttnChunk; base <= last; base += kAttnChunk) {
    const int lo = base > first ? base : first;
    const int hi = (base + kAttnChunk - 1 < last) ? base + kAttnChunk - 1 : last;
    const int n = hi - lo + 1;
    float local_max = -INFINITY;
    for (int j = tid; j < n; j += kAttnThreads) {
      const int key = lo + j;
      const int page = table[key / page_size];
      const int off = key % page_size;
      const T* kr = k_cache + (((size_t)page * hkv + kvh) * page_size + off) * (size_t)d;
      float s = 0.f;
      for (int i = 0; i < d; ++i) s += qs[i] * to_f32(kr[i]);
      probs[j] = s;
      local_max = fmaxf(local_max, s);
    }
    const float chunk_max = block_max(local_max, scratch);
    const float new_max = fmaxf(run_max, chunk_max);
    const float rescale = (run_max == -INFINITY) ? 0.f : expf(run_max - new_max);
    float local_sum = 0.f;
    for (int j = tid; j < n; j += kAttnThreads) {
      const float p = expf(probs[j] - new_max);
      probs[j] = p;
      local_sum += p;
    }
    const float chunk_sum = block_sum(local_sum, scratch);  // also orders the probs[] writes
    run_sum = run_sum * rescale + chunk_sum;
    run_max = new_max;
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const int i = tid + r * kAttnThreads;
      if (i < d) {
        float a = acc[r] * rescale;
        for (int j = 0; j < n; ++j) {
          const int key = lo + j;
          const int page = table[key / page_size];
          const int off = key % page_size;
          a += probs[j] * to_f32(v_cache[(((size_t)page * hkv + kvh) * d + i) * (size_t)page_size + off]);
        }
        acc[r] = a;
      }
    }
    __syncthreads();  // probs[] is rewritten by the next chunk
  }
  const float inv = 1.f / run_sum;
#pragma unroll
  for (int r = 0; r < 4; ++r) {
    const int i = tid + r * kAttnThreads;
    if (i < d) dst[i] = from_f32<T>(acc[r] * inv);
  }
}

ATOM_EXPORT int atom_paged_attention_generic(const void* q, const void* k_cache, const void* v_cache, void* out,
                                             const int* token_seq, const int* positions,
                                             const int* block_tables, int max_blocks, int dtype, int tokens,
                                             int hq, int hkv, int d, int page_size, float scale, int window,
                                             hipStream_t stream) {
  if (tokens < 0 || hq <= 0 || hkv <= 0 || d <= 0 || page_size <= 0 || max_blocks <= 0) return ATOM_BAD_SHAPE;
  if (hq % hkv) return ATOM_BAD_SHAPE;
  if (d > 4 * kAttnThreads) return ATOM_TOO_LARGE;
  if (hq > 65535) return ATOM_TOO_LARGE;
  if (tokens == 0) return ATOM_OK;
  const size_t smem = (size_t)(d + kAttnChunk + 16) * sizeof(float);
  dim3 grid(tokens, hq), block(kAttnThreads);
  ATOM_DISPATCH_DTYPE(dtype, hipLaunchKernelGGL((paged_attention_generic_kernel<T>), grid, block, smem, stream,
                                                 (const T*)q, (const T*)k_cache, (const T*)v_cache, (T*)out,
                                                 token_seq, positions, block_tables, max_blocks, hq, hkv, d,
                                                 page_size, scale, window));
  return launch_status();
}
