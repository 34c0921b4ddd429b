// y[M, N] = x[M, K] * w[N, K]^T (+ bias[N]) in true float32: plain FMA, no matrix
// cores, no reduced-precision mode.  Each output element is one sum over k in
// ascending order, whatever M is, so a row's result does not depend on its batch.
//
// 64 x 64 tiles, 256 threads, each thread a 4 x 4 patch; K is walked 16 at a time
// through LDS.  Any M, N, K (edges are guarded).
#include "common.h"

constexpr int kTile = 64;
constexpr int kStep = 16;

// X and W may be float32 or bfloat16 independently (read, widened, multiplied in float32).
template <typename TX, typename TW, typename TY>
__global__ void __launch_bounds__(256)
gemm_f32_kernel(const TX* __restrict__ x, const TW* __restrict__ w, const float* __restrict__ bias,
                TY* __restrict__ y, int m, int n, int k) {
  __shared__ float xs[kStep][kTile + 4];
  __shared__ float ws[kStep][kTile + 4];
  const int tid = threadIdx.x;
  const int tx = tid % 16;  // column patch
  const int ty = tid / 16;  // row patch
  const int row0 = blockIdx.y * kTile;
  const int col0 = blockIdx.x * kTile;
  float acc[4][4] = {};
  // loading: 64 rows x 16 k = 1024 elements, 4 per thread
  const int lrow = tid / 4;         // 0..63
  const int lk = (tid % 4) * 4;     // 0,4,8,12
  for (int k0 = 0; k0 < k; k0 += kStep) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int kk = k0 + lk + i;
      const int xr = row0 + lrow;
      const int wr = col0 + lrow;
      xs[lk + i][lrow] = (xr < m && kk < k) ? to_f32(x[(size_t)xr * k + kk]) : 0.f;
      ws[lk + i][lrow] = (wr < n && kk < k) ? to_f32(w[(size_t)wr * k + kk]) : 0.f;
    }
    __syncthreads();
#pragma unroll
    for (int kk = 0; kk < kStep; ++kk) {
      float a[4], b[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) a[i] = xs[kk][ty * 4 + i];
#pragma unroll
      for (int j = 0; j < 4; ++j) b[j] = ws[kk][tx * 4 + j];
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = fmaf(a[i], b[j], acc[i][j]);
    }
    __syncthreads();
  }
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int r = row0 + ty * 4 + i;
    if (r >= m) continue;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int c = col0 + tx * 4 + j;
      if (c < n) y[(size_t)r * n + c] = from_f32<TY>(acc[i][j] + (bias ? bias[c] : 0.f));
    }
  }
}

ATOM_EXPORT int atom_gemm_f32(const void* x, int x_dtype, const void* w, int w_dtype, const float* bias, void* y,
                              int y_dtype, int m, int n, int k, hipStream_t stream) {
  if (m < 0 || n <= 0 || k <= 0) return ATOM_BAD_SHAPE;
  if ((unsigned)x_dtype > 1u || (unsigned)w_dtype > 1u || (unsigned)y_dtype > 1u) return ATOM_BAD_DTYPE;
  if (m == 0) return ATOM_OK;
  dim3 grid((n + kTile - 1) / kTile, (m + kTile - 1) / kTile), block(256);
  if (grid.y > 65535) return ATOM_TOO_LARGE;
#define LAUNCH(TX, TW, TY)                                                                          \
  hipLaunchKernelGGL((gemm_f32_kernel<TX, TW, TY>), grid, block, 0, stream, (const TX*)x, (const TW*)w, bias, \
                     (TY*)y, m, n, k)
  const int key = x_dtype * 4 + w_dtype * 2 + y_dtype;
  switch (key) {
    case 0: LAUNCH(float, float, float); break;
    case 1: LAUNCH(float, float, bf16_t); break;
    case 2: LAUNCH(float, bf16_t, float); break;
    case 3: LAUNCH(float, bf16_t, bf16_t); break;
    case 4: LAUNCH(bf16_t, float, float); break;
    case 5: LAUNCH(bf16_t, float, bf16_t); break;
    case 6: LAUNCH(bf16_t, bf16_t, float); break;
    case 7: LAUNCH(bf16_t, bf16_t, bf16_t); break;
    default: return ATOM_BAD_DTYPE;
  }
#undef LAUNCH
  return launch_status();
}
