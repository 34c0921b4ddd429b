// Memory-bound kernels of the model step: embedding gather, RMS norm with the
// residual sum, SiLU-gate multiply, and the fused per-head norm + rotation +
// cache write that sits between the QKV product and attention.
//
// All arithmetic is in float32; activations are float32 or bfloat16 (template T),
// the residual stream and norm weights are always float32.
#include "common.h"

// Eight consecutive elements, moved with 16- and 32-byte accesses.
template <typename T>
struct Vec8;
template <>
struct Vec8<float> {
  float4 a, b;
  __device__ __forceinline__ void get(float* f) const {
    f[0] = a.x; f[1] = a.y; f[2] = a.z; f[3] = a.w; f[4] = b.x; f[5] = b.y; f[6] = b.z; f[7] = b.w;
  }
  __device__ __forceinline__ void set(const float* f) {
    a = make_float4(f[0], f[1], f[2], f[3]);
    b = make_float4(f[4], f[5], f[6], f[7]);
  }
};
template <>
struct Vec8<bf16_t> {
  __attribute__((ext_vector_type(8))) __bf16 v;
  __device__ __forceinline__ void get(float* f) const {
#pragma unroll
    for (int i = 0; i < 8; ++i) f[i] = static_cast<float>(v[i]);
  }
  __device__ __forceinline__ void set(const float* f) {
#pragma unroll
    for (int i = 0; i < 8; ++i) v[i] = static_cast<bf16_t>(f[i]);
  }
};

// An input that is still a sum: `splits` float32 slices [rows, width] `stride` elements apart, as the
// skinny matrix product leaves them when it cuts K, plus an optional bias over the width.  Readers
// add the slices in slice order.  `partial == nullptr`: the input is an ordinary tensor.
//
// The readers below issue the loads of several slices (and several elements) before they use any of
// them: a kernel that reads a sum waits for memory once per group of slices, not once per slice.  A
// group is filled up by reading the last slice again (a cache hit) instead of branching.
struct SplitSum {
  const float* partial;
  const float* bias;
  size_t stride;
  int splits;

  // the elements at offset[0..N-1] (bias columns col[0..N-1]); kGroup: slices whose loads are in flight together
  template <int N, int kGroup = 4>
  __device__ __forceinline__ void at_many(const size_t (&offset)[N], const int (&col)[N], float (&out)[N]) const {
#pragma unroll
    for (int n = 0; n < N; ++n) out[n] = 0.f;
    for (int s0 = 0; s0 < splits; s0 += kGroup) {
      float part[N][kGroup];
#pragma unroll
      for (int u = 0; u < kGroup; ++u) {
        const float* slice = partial + (size_t)min(s0 + u, splits - 1) * stride;
#pragma unroll
        for (int n = 0; n < N; ++n) part[n][u] = slice[offset[n]];
      }
#pragma unroll
      for (int u = 0; u < kGroup; ++u) {
        const bool live = s0 + u < splits;
#pragma unroll
        for (int n = 0; n < N; ++n) out[n] += live ? part[n][u] : 0.f;
      }
    }
    if (bias) {
#pragma unroll
      for (int n = 0; n < N; ++n) out[n] += bias[col[n]];
    }
  }

  __device__ __forceinline__ float at(size_t offset, int col) const {
    const size_t offsets[1] = {offset};
    const int cols[1] = {col};
    float out[1];
    at_many<1>(offsets, cols, out);
    return out[0];
  }

  // N runs of eight consecutive elements, each at a 32-byte aligned offset (bias columns col[n] ..)
  template <int N, int kGroup = 4>
  __device__ __forceinline__ void runs_of_8(const size_t (&offset)[N], const int (&col)[N], float (&out)[N][8]) const {
#pragma unroll
    for (int n = 0; n < N; ++n)
#pragma unroll
      for (int e = 0; e < 8; ++e) out[n][e] = 0.f;
    for (int s0 = 0; s0 < splits; s0 += kGroup) {
      Vec8<float> part[N][kGroup];
#pragma unroll
      for (int u = 0; u < kGroup; ++u) {
        const float* slice = partial + (size_t)min(s0 + u, splits - 1) * stride;
#pragma unroll
        for (int n = 0; n < N; ++n) part[n][u] = *reinterpret_cast<const Vec8<float>*>(slice + offset[n]);
      }
#pragma unroll
      for (int u = 0; u < kGroup; ++u) {
        const bool live = s0 + u < splits;
#pragma unroll
        for (int n = 0; n < N; ++n) {
          float v[8];
          part[n][u].get(v);
#pragma unroll
          for (int e = 0; e < 8; ++e) out[n][e] += live ? v[e] : 0.f;
        }
      }
    }
    if (bias) {
#pragma unroll
      for (int n = 0; n < N; ++n) {
        float v[8];
        reinterpret_cast<const Vec8<float>*>(bias + col[n])->get(v);
#pragma unroll
        for (int e = 0; e < 8; ++e) out[n][e] += v[e];
      }
    }
  }
};

// ------------------------------------------------------------------ embedding

template <typename TT, typename TO>
__global__ void embedding_kernel(const TT* __restrict__ table, const int* __restrict__ ids,
                                 TO* __restrict__ out, int hidden, int vocab) {
  const int t = blockIdx.x;
  const int id = ids[t];
  const bool ok = id >= 0 && id < vocab;
  const TT* row = table + (size_t)(ok ? id : 0) * hidden;
  TO* dst = out + (size_t)t * hidden;
  for (int i = threadIdx.x; i < hidden; i += blockDim.x)
    dst[i] = ok ? from_f32<TO>(to_f32(row[i])) : from_f32<TO>(0.f);
}

ATOM_EXPORT int atom_embedding(const void* table, int table_dtype, const int* ids, void* out,
                               int out_dtype, int tokens, int hidden, int vocab, hipStream_t stream) {
  if (tokens < 0 || hidden <= 0 || vocab <= 0) return ATOM_BAD_SHAPE;
  if (tokens == 0) return ATOM_OK;
  dim3 grid(tokens), block(256);
#define LAUNCH(TT, TO) \
  hipLaunchKernelGGL((embedding_kernel<TT, TO>), grid, block, 0, stream, (const TT*)table, ids, (TO*)out, hidden, vocab)
  if (table_dtype == ATOM_F32 && out_dtype == ATOM_F32) LAUNCH(float, float);
  else if (table_dtype == ATOM_BF16 && out_dtype == ATOM_BF16) LAUNCH(bf16_t, bf16_t);
  else if (table_dtype == ATOM_BF16 && out_dtype == ATOM_F32) LAUNCH(bf16_t, float);
  else if (table_dtype == ATOM_F32 && out_dtype == ATOM_BF16) LAUNCH(float, bf16_t);
  else return ATOM_BAD_DTYPE;
#undef LAUNCH
  return launch_status();
}

// ------------------------------------------------------------------ token ids that are still on the device
//
// ids[t] = sampled[source[t]] where source[t] >= 0: a request that decodes takes the token the last step
// sampled for it from the sampler's own output, so that the step can be launched before the host has
// read that token.  Rows with source[t] < 0 keep the id the host wrote.

__global__ void feed_tokens_kernel(int* __restrict__ ids, const int* __restrict__ source,
                                   const int* __restrict__ sampled, int tokens, int num_sampled) {
  const int t = blockIdx.x * blockDim.x + threadIdx.x;
  if (t >= tokens) return;
  const int src = source[t];
  if (src >= 0 && src < num_sampled) ids[t] = sampled[src];
}

ATOM_EXPORT int atom_feed_tokens(int* ids, const int* source, const int* sampled, int tokens, int num_sampled,
                                 hipStream_t stream) {
  if (tokens < 0 || num_sampled < 0) return ATOM_BAD_SHAPE;
  if (tokens == 0) return ATOM_OK;
  hipLaunchKernelGGL(feed_tokens_kernel, dim3((tokens + 255) / 256), dim3(256), 0, stream, ids, source, sampled,
                     tokens, num_sampled);
  return launch_status();
}

// ------------------------------------------------------------------ RMS norm
//
// mode 0: y = norm(x)                                   (residual untouched)
// mode 1: residual = x (as float32); y = norm(residual)  (first layer)
// mode 2: residual += x; y = norm(residual)
// `rows`, when given, names the source row of each output row (x and residual are
// read at rows[r], y is written at r) and the residual is left as it is: the sum
// is formed only for the norm.  Used to norm just the rows whose logits are asked.
// One block per row.

template <typename T>
__global__ void rmsnorm_kernel(const T* __restrict__ x, float* __restrict__ residual,
                               const float* __restrict__ weight, T* __restrict__ y,
                               const int* __restrict__ rows, int width, float eps, int mode, SplitSum xsum) {
  extern __shared__ float smem[];  // width floats + 16 for the reduction
  float* vals = smem;
  float* scratch = smem + width;
  const int r = blockIdx.x;
  const int src = rows ? rows[r] : r;
  const T* xr = x + (size_t)src * width;
  float* rr = residual ? residual + (size_t)src * width : nullptr;
  float ss = 0.f;
  for (int i = threadIdx.x; i < width; i += blockDim.x) {
    float v = xsum.partial ? xsum.at((size_t)src * width + i, i) : to_f32(xr[i]);
    if (mode == 2) v += rr[i];
    vals[i] = v;
    ss += v * v;
  }
  ss = block_sum(ss, scratch);
  const float inv = rsqrtf(ss / (float)width + eps);
  T* yr = y + (size_t)r * width;
  const bool store_residual = mode != 0 && rows == nullptr;
  for (int i = threadIdx.x; i < width; i += blockDim.x) {
    const float v = vals[i];
    if (store_residual) rr[i] = v;
    yr[i] = from_f32<T>(v * inv * weight[i]);
  }
}

// The same for widths that are a multiple of 8: a thread keeps VPT groups of 8 consecutive
// elements in registers, all loads of a row are issued at once (16- and 32-byte accesses) and
// nothing goes through LDS but the reduction.  blockDim.x * 8 * VPT >= width.
template <typename T, int VPT>
__global__ void rmsnorm_vec_kernel(const T* __restrict__ x, float* __restrict__ residual,
                                   const float* __restrict__ weight, T* __restrict__ y,
                                   const int* __restrict__ rows, int width, float eps, int mode, SplitSum xsum) {
  __shared__ float scratch[16];
  const int r = blockIdx.x;
  const int src = rows ? rows[r] : r;
  const T* xr = x + (size_t)src * width;
  float* rr = residual ? residual + (size_t)src * width : nullptr;
  float vals[VPT][8];
  float ss = 0.f;
  Vec8<T> xv[VPT];
  Vec8<float> rv[VPT];
#pragma unroll
  for (int j = 0; j < VPT; ++j) {
    const int i = (threadIdx.x + j * blockDim.x) * 8;
    if (i < width) {
      if (!xsum.partial) xv[j] = *reinterpret_cast<const Vec8<T>*>(xr + i);
      if (mode == 2) rv[j] = *reinterpret_cast<const Vec8<float>*>(rr + i);
    }
  }
  if (xsum.partial) {
    // groups beyond the width read the row's last group again and are not used
    size_t offsets[VPT];
    int cols[VPT];
#pragma unroll
    for (int j = 0; j < VPT; ++j) {
      cols[j] = min((int)(threadIdx.x + j * blockDim.x) * 8, width - 8);
      offsets[j] = (size_t)src * width + cols[j];
    }
    xsum.runs_of_8<VPT, (VPT == 1 ? 8 : 4)>(offsets, cols, vals);
  }
#pragma unroll
  for (int j = 0; j < VPT; ++j) {
    const int i = (threadIdx.x + j * blockDim.x) * 8;
    if (i < width) {
      if (!xsum.partial) xv[j].get(vals[j]);
      if (mode == 2) {
        float add[8];
        rv[j].get(add);
#pragma unroll
        for (int e = 0; e < 8; ++e) vals[j][e] += add[e];
      }
#pragma unroll
      for (int e = 0; e < 8; ++e) ss += vals[j][e] * vals[j][e];
    }
  }
  ss = block_sum(ss, scratch);
  const float inv = rsqrtf(ss / (float)width + eps);
  T* yr = y + (size_t)r * width;
  const bool store_residual = mode != 0 && rows == nullptr;
#pragma unroll
  for (int j = 0; j < VPT; ++j) {
    const int i = (threadIdx.x + j * blockDim.x) * 8;
    if (i < width) {
      if (store_residual) {
        Vec8<float> o;
        o.set(vals[j]);
        *reinterpret_cast<Vec8<float>*>(rr + i) = o;
      }
      Vec8<float> wv = *reinterpret_cast<const Vec8<float>*>(weight + i);
      float w[8], outv[8];
      wv.get(w);
#pragma unroll
      for (int e = 0; e < 8; ++e) outv[e] = vals[j][e] * inv * w[e];
      Vec8<T> o;
      o.set(outv);
      *reinterpret_cast<Vec8<T>*>(yr + i) = o;
    }
  }
}

// `x_partial` (with `x_splits` slices `x_stride` elements apart and an optional `x_bias`) stands for x
// when x is still a sum of slices; x itself is then not read.
ATOM_EXPORT int atom_rmsnorm(const void* x, void* residual, const float* weight, void* y,
                             const int* rows, int dtype, int num_rows, int width, float eps,
                             int mode, const float* x_partial, int x_splits, long x_stride,
                             const float* x_bias, hipStream_t stream) {
  if (num_rows < 0 || width <= 0 || mode < 0 || mode > 2) return ATOM_BAD_SHAPE;
  if (mode != 0 && residual == nullptr) return ATOM_BAD_SHAPE;
  if (x_partial ? (x_splits < 1 || x_stride < 0) : x == nullptr) return ATOM_BAD_SHAPE;
  if (num_rows == 0) return ATOM_OK;
  const SplitSum xsum{x_partial, x_partial ? x_bias : nullptr, (size_t)x_stride, x_splits};
  const bool aligned = (((uintptr_t)x | (uintptr_t)y | (uintptr_t)residual | (uintptr_t)weight |
                         (uintptr_t)x_partial | (uintptr_t)x_bias) & 31) == 0 && (!x_partial || x_stride % 8 == 0);
  if (width % 8 == 0 && width <= 8 * 1024 * 4 && aligned) {
    const int groups = width / 8;
    int threads = groups <= 64 ? 64 : (groups <= 128 ? 128 : (groups <= 256 ? 256 : (groups <= 512 ? 512 : 1024)));
    const int vpt = (groups + threads - 1) / threads;
#define LAUNCH_VEC(V)                                                                                         \
  ATOM_DISPATCH_DTYPE(dtype, hipLaunchKernelGGL((rmsnorm_vec_kernel<T, V>), dim3(num_rows), dim3(threads), 0, \
                                                 stream, (const T*)x, (float*)residual, weight, (T*)y, rows, \
                                                 width, eps, mode, xsum))
    if (vpt == 1) LAUNCH_VEC(1);
    else if (vpt == 2) LAUNCH_VEC(2);
    else LAUNCH_VEC(4);
#undef LAUNCH_VEC
    return launch_status();
  }
  if ((size_t)width * 4 + 64 > 64 * 1024) return ATOM_TOO_LARGE;  // the row is kept in LDS
  const int threads = width >= 2048 ? 512 : (width >= 512 ? 256 : 64);
  const size_t smem = (size_t)width * 4 + 64;
  ATOM_DISPATCH_DTYPE(dtype, hipLaunchKernelGGL((rmsnorm_kernel<T>), dim3(num_rows), dim3(threads), smem,
                                                 stream, (const T*)x, (float*)residual, weight, (T*)y,
                                                 rows, width, eps, mode, xsum));
  return launch_status();
}

// ------------------------------------------------------------------ SiLU(gate) * up

template <typename T>
__global__ void silu_mul_kernel(const T* __restrict__ x, T* __restrict__ y, int inter, size_t total, SplitSum xsum) {
  const size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= total) return;
  const size_t row = idx / inter;
  const int col = (int)(idx - row * inter);
  float g, u;
  if (xsum.partial) {
    const size_t offsets[2] = {row * 2 * inter + col, row * 2 * inter + inter + col};
    const int cols[2] = {col, inter + col};
    float both[2];
    xsum.at_many<2>(offsets, cols, both);
    g = both[0];
    u = both[1];
  } else {
    g = to_f32(x[row * 2 * inter + col]);
    u = to_f32(x[row * 2 * inter + inter + col]);
  }
  y[idx] = from_f32<T>(g / (1.f + expf(-g)) * u);
}

// inter % 8 == 0: a thread handles 8 consecutive columns with 16- or 32-byte accesses
template <typename T>
__global__ void silu_mul_vec_kernel(const T* __restrict__ x, T* __restrict__ y, int inter, size_t groups,
                                    SplitSum xsum) {
  const size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= groups) return;
  const int per_row = inter / 8;
  const size_t row = idx / per_row;
  const int col = (int)(idx - row * per_row) * 8;
  float g[8], u[8], o[8];
  if (xsum.partial) {
    const size_t offsets[2] = {row * 2 * inter + col, row * 2 * inter + inter + col};
    const int cols[2] = {col, inter + col};
    float both[2][8];
    xsum.runs_of_8<2>(offsets, cols, both);
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      g[e] = both[0][e];
      u[e] = both[1][e];
    }
  } else {
    const Vec8<T> gv = *reinterpret_cast<const Vec8<T>*>(x + row * 2 * inter + col);
    const Vec8<T> uv = *reinterpret_cast<const Vec8<T>*>(x + row * 2 * inter + inter + col);
    gv.get(g);
    uv.get(u);
  }
#pragma unroll
  for (int e = 0; e < 8; ++e) o[e] = g[e] / (1.f + expf(-g[e])) * u[e];
  Vec8<T> ov;
  ov.set(o);
  *reinterpret_cast<Vec8<T>*>(y + row * inter + col) = ov;
}

// `x_partial` (slices `x_stride` apart, optional `x_bias`) stands for x when x is still a sum of slices;
// `dtype` is then the type of y.
ATOM_EXPORT int atom_silu_mul(const void* x, void* y, int dtype, int rows, int inter, const float* x_partial,
                              int x_splits, long x_stride, const float* x_bias, hipStream_t stream) {
  if (rows < 0 || inter <= 0) return ATOM_BAD_SHAPE;
  if (x_partial ? (x_splits < 1 || x_stride < 0) : x == nullptr) return ATOM_BAD_SHAPE;
  const size_t total = (size_t)rows * inter;
  if (total == 0) return ATOM_OK;
  const SplitSum xsum{x_partial, x_partial ? x_bias : nullptr, (size_t)x_stride, x_splits};
  const int threads = 256;
  if (inter % 8 == 0 && (((uintptr_t)x | (uintptr_t)y | (uintptr_t)x_partial) & 31) == 0 &&
      (!x_partial || x_stride % 8 == 0)) {
    const size_t groups = total / 8;
    const size_t blocks = (groups + threads - 1) / threads;
    if (blocks > 0x7fffffffu) return ATOM_TOO_LARGE;
    ATOM_DISPATCH_DTYPE(dtype, hipLaunchKernelGGL((silu_mul_vec_kernel<T>), dim3((unsigned)blocks), dim3(threads), 0,
                                                   stream, (const T*)x, (T*)y, inter, groups, xsum));
    return launch_status();
  }
  const size_t blocks = (total + threads - 1) / threads;
  if (blocks > 0x7fffffffu) return ATOM_TOO_LARGE;
  ATOM_DISPATCH_DTYPE(dtype, hipLaunchKernelGGL((silu_mul_kernel<T>), dim3((unsigned)blocks), dim3(threads), 0,
                                                 stream, (const T*)x, (T*)y, inter, total, xsum));
  return launch_status();
}

// ------------------------------------------------------------------ q/k norm + rotation + cache write
//
// Input: the QKV product [tokens, (Hq + 2 Hkv) * D], rows laid out q | k | v.
// One wave per (token, head):
//   q heads:  optional RMS norm over D, rotation, written to q_out [tokens, Hq, D];
//   k heads:  optional RMS norm over D, rotation, written into the key pages;
//   v heads:  written into the value pages as they are.
// Rotation is NeoX style over the first `rotary_dim` elements: pairs (j, j + rotary_dim/2)
// with cos/sin taken from float32 tables [max_pos, rotary_dim/2] at the token's position.
// Pages: keys   [num_pages, Hkv, page_size, D]
//        values [num_pages, Hkv, D, page_size]   (transposed: keys of a page are contiguous per d)
// slot = page * page_size + offset; slot < 0 writes nothing (padding rows).
// `write_kv == 0` skips k and v altogether (a layer that reads another layer's cache).

template <typename T>
__global__ void qk_norm_rope_kv_write_kernel(
    const T* __restrict__ qkv, T* __restrict__ q_out, T* __restrict__ k_cache, T* __restrict__ v_cache,
    const float* __restrict__ q_weight, const float* __restrict__ k_weight, const float* __restrict__ cos_table,
    const float* __restrict__ sin_table, const int* __restrict__ positions, const int* __restrict__ slots,
    int hq, int hkv, int d, int rotary_dim, int page_size, float eps, int write_kv, SplitSum xsum,
    int head_begin) {
  const int t = blockIdx.x;
  const int head = blockIdx.y + head_begin;  // 0..hq-1 q, then hkv k heads, then hkv v heads
  const int lane = threadIdx.x;
  const int row_width = (hq + 2 * hkv) * d;
  const size_t src_off = (size_t)t * row_width + (size_t)head * d;
  const bool is_q = head < hq;
  const bool is_k = !is_q && head < hq + hkv;
  const int kv_head = is_q ? 0 : (is_k ? head - hq : head - hq - hkv);

  if (!is_q && !is_k && write_kv && !xsum.partial && page_size % 8 == 0) {
    // value heads of 8 consecutive tokens whose slots are 8 consecutive, aligned places of one page
    // (the usual case in a prompt portion): the first token's wave writes all 8, 8 keys at a time per
    // d, instead of every token scattering single elements over the transposed page
    const int t0 = t & ~7;
    bool together = t0 + 8 <= (int)gridDim.x;
    int s0 = -1;
    if (together) {
      s0 = slots[t0];
      together = s0 >= 0 && s0 % 8 == 0;
      for (int j = 1; j < 8 && together; ++j) together = slots[t0 + j] == s0 + j;
    }
    if (together) {
      if (t != t0) return;
      const int page0 = s0 / page_size, off0 = s0 - page0 * page_size;
      T* base = v_cache + ((size_t)page0 * hkv + kv_head) * (size_t)d * page_size + off0;
      const T* rows = qkv + (size_t)t0 * row_width + (size_t)head * d;
      for (int i = lane; i < d; i += kWave) {
        float vals[8];
#pragma unroll
        for (int j = 0; j < 8; ++j) vals[j] = to_f32(rows[(size_t)j * row_width + i]);
        Vec8<T> out8;
        out8.set(vals);
        *reinterpret_cast<Vec8<T>*>(base + (size_t)i * page_size) = out8;
      }
      return;
    }
  }

  int slot = -1;
  if (!is_q) {
    if (!write_kv) return;
    slot = slots[t];
    if (slot < 0) return;
  }
  const int page = slot / page_size;
  const int off = slot - page * page_size;

  // The head's d values, read once: where the input is a sum of slices, the loads of four elements and
  // of four slices are in flight together.  They are kept in LDS (the block is this one wave).
  extern __shared__ float head_vals[];   // d floats
  for (int i0 = 0; i0 < d; i0 += 4 * kWave) {
    size_t offsets[4];
    int cols[4];
    float got[4];
#pragma unroll
    for (int n = 0; n < 4; ++n) {
      const int i = min(i0 + n * kWave + lane, d - 1);   // beyond the head: its last element again, not used
      offsets[n] = src_off + i;
      cols[n] = head * d + i;
    }
    if (xsum.partial) {
      xsum.at_many<4>(offsets, cols, got);
    } else {
#pragma unroll
      for (int n = 0; n < 4; ++n) got[n] = to_f32(qkv[offsets[n]]);
    }
#pragma unroll
    for (int n = 0; n < 4; ++n) {
      const int i = i0 + n * kWave + lane;
      if (i < d) head_vals[i] = got[n];
    }
  }
  __syncthreads();

  if (!is_q && !is_k) {  // value head: plain scatter into the transposed page
    T* dst = v_cache + ((size_t)page * hkv + kv_head) * (size_t)d * page_size + off;
    for (int i = lane; i < d; i += kWave) dst[(size_t)i * page_size] = from_f32<T>(head_vals[i]);
    return;
  }

  const float* weight = is_q ? q_weight : k_weight;
  float inv = 1.f;
  if (weight) {
    float ss = 0.f;
    for (int i = lane; i < d; i += kWave) {
      const float v = head_vals[i];
      ss += v * v;
    }
    ss = wave_sum(ss);
    inv = rsqrtf(ss / (float)d + eps);
  }
  T* dst = is_q ? q_out + ((size_t)t * hq + head) * d
                : k_cache + (((size_t)page * hkv + kv_head) * page_size + off) * (size_t)d;
  const int half = rotary_dim / 2;
  // without rotation the three tables may be null: nothing of them is touched then
  const int pos = half > 0 ? positions[t] : 0;
  const float* cs = half > 0 ? cos_table + (size_t)pos * half : nullptr;
  const float* sn = half > 0 ? sin_table + (size_t)pos * half : nullptr;
  for (int j = lane; j < half; j += kWave) {
    float x1 = head_vals[j];
    float x2 = head_vals[j + half];
    if (weight) {
      x1 = x1 * inv * weight[j];
      x2 = x2 * inv * weight[j + half];
    }
    const float c = cs[j], s = sn[j];
    dst[j] = from_f32<T>(x1 * c - x2 * s);
    dst[j + half] = from_f32<T>(x2 * c + x1 * s);
  }
  for (int i = rotary_dim + lane; i < d; i += kWave) {  // the part that is not rotated
    float v = head_vals[i];
    if (weight) v = v * inv * weight[i];
    dst[i] = from_f32<T>(v);
  }
}

// The q and k heads of many tokens, when the whole head is rotated and the input is a tensor: sixteen lanes
// per (token, head), each with D / 16 consecutive elements (vector loads and stores); the rotation partner
// of a lane is 8 lanes away.  256 threads are 16 (token, head) pairs.
template <typename T, int E>
__global__ void __launch_bounds__(256)
qk_norm_rope_vec_kernel(const T* __restrict__ qkv, T* __restrict__ q_out, T* __restrict__ k_cache,
                        const float* __restrict__ q_weight, const float* __restrict__ k_weight,
                        const float* __restrict__ cos_table, const float* __restrict__ sin_table,
                        const int* __restrict__ positions, const int* __restrict__ slots, int tokens, int hq, int hkv,
                        int page_size, float eps, int write_kv, T* __restrict__ v_cache, int qk_blocks) {
  constexpr int D = 16 * E;
  if ((int)blockIdx.x >= qk_blocks) {
    // ---- value heads: half a block (128 threads) takes 8 consecutive tokens of one KV head, lane i of token
    //      j its E elements; the 8 x D tile goes through LDS so that, where the 8 slots are 8 consecutive
    //      aligned places of one page, every d gets its 8 keys in one 16-byte store (value pages are
    //      transposed).  Other groups (a prompt's ragged end, padding) scatter single elements.
    __shared__ T tile[2][8][D];
    const int half = threadIdx.x / 128, within = threadIdx.x % 128;
    const int j = within / 16, vi = within & 15;
    const int groups8 = (tokens + 7) / 8;
    const int vg = ((int)blockIdx.x - qk_blocks) * 2 + half;
    const bool group_live = vg < groups8 * hkv;
    const int g8 = group_live ? vg / hkv : 0, kvh = group_live ? vg - g8 * hkv : 0;
    const int t0 = 8 * g8, tv = t0 + j;
    const size_t v_width = (size_t)(hq + 2 * hkv) * D;
    constexpr int VALIGN = sizeof(T) * E < 16 ? sizeof(T) * E : 16;
    T vals[E];
#pragma unroll
    for (int e = 0; e < E; ++e) vals[e] = from_f32<T>(0.f);
    if (group_live && tv < tokens)
      __builtin_memcpy(vals, __builtin_assume_aligned(qkv + (size_t)tv * v_width + (size_t)(hq + hkv + kvh) * D + E * vi,
                                                      VALIGN), sizeof(vals));
    bool together = group_live && t0 + 8 <= tokens && page_size % 8 == 0;
    int s0 = -1;
    if (together) {
      s0 = slots[t0];
      together = s0 >= 0 && s0 % 8 == 0;
      for (int q = 1; q < 8 && together; ++q) together = slots[t0 + q] == s0 + q;
    }
#pragma unroll
    for (int e = 0; e < E; ++e) tile[half][j][E * vi + e] = vals[e];
    __syncthreads();
    if (!group_live) return;
    if (together) {
      const int page = s0 / page_size, off = s0 - page * page_size;
      T* base = v_cache + ((size_t)page * hkv + kvh) * (size_t)D * page_size + off;
      for (int dd = within; dd < D; dd += 128) {
        T eight[8];
#pragma unroll
        for (int q = 0; q < 8; ++q) eight[q] = tile[half][q][dd];
        __builtin_memcpy(__builtin_assume_aligned(base + (size_t)dd * page_size, sizeof(T) * 8 < 16 ? sizeof(T) * 8 : 16),
                         eight, sizeof(eight));
      }
    } else if (tv < tokens) {
      const int slot = slots[tv];
      if (slot >= 0) {
        const int page = slot / page_size, off = slot - page * page_size;
        T* dst = v_cache + ((size_t)page * hkv + kvh) * (size_t)D * page_size + off;
#pragma unroll
        for (int e = 0; e < E; ++e) dst[(size_t)(E * vi + e) * page_size] = vals[e];
      }
    }
    return;
  }
  const int pair = blockIdx.x * 16 + threadIdx.x / 16;
  const int i = threadIdx.x & 15;
  const int heads = hq + hkv;
  const bool live = pair < tokens * heads;
  const int t = live ? pair / heads : 0;
  const int head = live ? pair - t * heads : 0;
  const bool is_q = head < hq;
  const size_t row_width = (size_t)(hq + 2 * hkv) * D;
  constexpr int ALIGN = sizeof(T) * E < 16 ? sizeof(T) * E : 16;
  T raw[E];
  __builtin_memcpy(raw, __builtin_assume_aligned(qkv + (size_t)t * row_width + (size_t)head * D + E * i, ALIGN),
                   sizeof(raw));
  float x[E];
  float ss = 0.f;
#pragma unroll
  for (int e = 0; e < E; ++e) {
    x[e] = to_f32(raw[e]);
    ss += x[e] * x[e];
  }
  const float* weight = is_q ? q_weight : k_weight;
  if (weight) {
#pragma unroll
    for (int off = 8; off > 0; off >>= 1) ss += __shfl_xor(ss, off, 16);
    const float inv = rsqrtf(ss / (float)D + eps);
#pragma unroll
    for (int e = 0; e < E; ++e) x[e] = x[e] * inv * weight[E * i + e];
  }
  const int pos = positions[t];
  const float* cs = cos_table + (size_t)pos * (D / 2) + E * (i & 7);
  const float* sn = sin_table + (size_t)pos * (D / 2) + E * (i & 7);
  T out[E];
#pragma unroll
  for (int e = 0; e < E; ++e) {
    const float other = __shfl_xor(x[e], 8, 16);
    const float c = cs[e], sv = sn[e];
    out[e] = from_f32<T>(i < 8 ? x[e] * c - other * sv : x[e] * c + other * sv);
  }
  if (!live) return;
  T* dst;
  if (is_q) {
    dst = q_out + ((size_t)t * hq + head) * D + E * i;
  } else {
    if (!write_kv) return;
    const int slot = slots[t];
    if (slot < 0) return;
    const int page = slot / page_size, off = slot - page * page_size;
    dst = k_cache + (((size_t)page * hkv + (head - hq)) * page_size + off) * (size_t)D + E * i;
  }
  __builtin_memcpy(__builtin_assume_aligned(dst, ALIGN), out, sizeof(out));
}

ATOM_EXPORT int atom_qk_norm_rope_kv_write(
    const void* qkv, void* q_out, void* k_cache, void* v_cache, const float* q_weight, const float* k_weight,
    const float* cos_table, const float* sin_table, const int* positions, const int* slots, int dtype,
    int tokens, int hq, int hkv, int d, int rotary_dim, int page_size, float eps, int write_kv,
    const float* x_partial, int x_splits, long x_stride, const float* x_bias, hipStream_t stream) {
  if (tokens < 0 || hq <= 0 || hkv <= 0 || d <= 0 || page_size <= 0) return ATOM_BAD_SHAPE;
  if (x_partial ? (x_splits < 1 || x_stride < 0) : qkv == nullptr) return ATOM_BAD_SHAPE;
  const SplitSum xsum{x_partial, x_partial ? x_bias : nullptr, (size_t)x_stride, x_splits};
  if (rotary_dim < 0 || rotary_dim > d || (rotary_dim & 1)) return ATOM_BAD_SHAPE;
  if (rotary_dim > 0 && (!cos_table || !sin_table || !positions)) return ATOM_BAD_SHAPE;
  if (write_kv && (!k_cache || !v_cache || !slots)) return ATOM_BAD_SHAPE;
  if (hq + 2 * hkv > 65535) return ATOM_TOO_LARGE;
  if (tokens == 0) return ATOM_OK;
  int head_begin = 0;
  const long pairs = (long)tokens * (hq + hkv);
  if (!x_partial && tokens >= 32 && rotary_dim == d && d % 16 == 0 && d <= 256 && (d & (d - 1)) == 0 &&
      pairs / 16 + (long)tokens * hkv < 0x7fffffffL &&
      (((uintptr_t)qkv | (uintptr_t)q_out | (uintptr_t)k_cache | (uintptr_t)v_cache) & 31) == 0) {
    // many tokens: q and k heads and, behind them in the same grid, the value heads through the vector kernel
    const long qk_blocks = (pairs + 15) / 16;
    const long v_blocks = write_kv ? ((long)((tokens + 7) / 8) * hkv + 1) / 2 : 0;
    const dim3 vgrid((unsigned)(qk_blocks + v_blocks)), vblock(256);
#define LAUNCH_ROPE(EE)                                                                                          \
  ATOM_DISPATCH_DTYPE(dtype, hipLaunchKernelGGL((qk_norm_rope_vec_kernel<T, EE>), vgrid, vblock, 0, stream,      \
                                                 (const T*)qkv, (T*)q_out, (T*)k_cache, q_weight, k_weight,      \
                                                 cos_table, sin_table, positions, slots, tokens, hq, hkv,        \
                                                 page_size, eps, write_kv, (T*)v_cache, (int)qk_blocks))
    switch (d / 16) {
      case 1: LAUNCH_ROPE(1); break;
      case 2: LAUNCH_ROPE(2); break;
      case 4: LAUNCH_ROPE(4); break;
      case 8: LAUNCH_ROPE(8); break;
      default: LAUNCH_ROPE(16); break;
    }
#undef LAUNCH_ROPE
    return launch_status();
  }
  dim3 grid(tokens, hq + 2 * hkv - head_begin), block(kWave);
  if ((size_t)d * 4 > 64 * 1024) return ATOM_TOO_LARGE;   // a head's values are kept in LDS
  ATOM_DISPATCH_DTYPE(dtype, hipLaunchKernelGGL((qk_norm_rope_kv_write_kernel<T>), grid, block, (size_t)d * 4, stream,
                                                 (const T*)qkv, (T*)q_out, (T*)k_cache, (T*)v_cache, q_weight,
                                                 k_weight, cos_table, sin_table, positions, slots, hq, hkv, d,
                                                 rotary_dim, page_size, eps, write_kv, xsum, head_begin));
  return launch_status();
}
