// y[M, N] = x[M, K] * w[N, K]^T (+ bias) for a few hundred rows, bfloat16 operands, float32 sums on the matrix
// cores (v_mfma_f32_32x32x16_bf16).  This is the product of steps that are neither a handful of decode rows
// (gemm_rows.hip, gemm_skinny.hip stream the weights once and are bound by that stream) nor thousands of prompt
// rows (the BLAS library's large tiles): with 65 to 256 rows a product has too few large tiles to fill 256 CUs,
// and what it costs is the latency of a short kernel.  So the grid here is cut to the chip:
//
//   tile      128 rows of w (output columns) x 64 or 128 rows of x, all of a slice of K; a block of four waves,
//             each with 64 x 32 or 64 x 64 of the tile (w is the A operand, x the B operand, so that a lane ends up
//             with four consecutive columns of one row of y and stores them together);
//   slices    K is cut into 1, 2, 4 or 8 slices so that tiles x slices comes close to the number of CUs without
//             passing it (gemm_tile_plan); a block leaves its float32 partial tile in partial[slice][m][n], and
//             whoever reads the product next adds the slices in slice order, as for the skinny product;
//   order     blocks are numbered so that the tiles and slices that read the same 128 rows of w run side by side
//             on one XCD (blocks go to the eight XCDs in turn, each XCD has an L2 of its own), so those rows come
//             from memory once.
//
// Inside a block: a stage is 64 k of the tile's rows of w and x.  Two register sets take the loads of the stages
// one and two ahead (16-byte loads, eight lanes a row, whole cache lines), two LDS buffers hold the stage being
// multiplied and the next; rows are padded by 16 bytes so that the operand reads (lane (r, h) reads k 8 h .. 8 h + 7
// of row r) spread over the banks.  The loop is written without a branch and with the order of its parts pinned
// (sched_barrier): the compiler counts the loads in flight exactly only in straight-line code, and left to itself
// it reads each operand right before the product that takes it and waits for it there.
//
// Needs K % 64 == 0 (and K a multiple of 64 x slices).  Any M >= 1, any N.
#include "common.h"

typedef __attribute__((ext_vector_type(4))) float f32x4;
typedef __attribute__((ext_vector_type(16))) float f32x16;
typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) __bf16 bf16x4;

constexpr int kTileK = 64;                 // k of a stage
constexpr int kTileRow = kTileK * 2 + 16;  // LDS bytes of a row of a stage
constexpr int kTileN = 128;                // rows of w a tile

struct TileParams {
  const bf16_t* x;     // [m, k]
  const bf16_t* w;     // [n, k]
  const float* bias;   // [n] or null (splits == 1 only)
  void* y;             // splits == 1: [m, n] bfloat16 or float32
  float* partial;      // splits > 1: [splits, m, n]
  int m, n, k, splits, kslice, mtiles, ntiles, out_f32;
};

template <int NT>   // 32-row blocks of x per wave: the tile has 64 NT rows of x
__global__ void __launch_bounds__(256, 2) gemm_tile_kernel(TileParams p) {
  constexpr int BM = 64 * NT;
  constexpr int XL = BM / 32;                    // 16-byte pieces of x a thread brings per stage
  constexpr int WT = kTileN * kTileRow;          // bytes of the w part of a stage
  constexpr int ST = (kTileN + BM) * kTileRow;   // bytes of a stage
  extern __shared__ __attribute__((aligned(16))) char smem[];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int r32 = lane & 31, half = lane >> 5;
  const int wn = wave & 1, wm = wave >> 1;
  const int per_n = p.mtiles * p.splits;
  const int xcd = blockIdx.x & 7, q = blockIdx.x >> 3;
  const int ntile = (q / per_n) * 8 + xcd;
  if (ntile >= p.ntiles) return;   // the grid is rounded up to whole groups of eight column tiles
  const int rest = q % per_n;
  const int mtile = rest / p.splits, split = rest % p.splits;
  const int n0 = ntile * kTileN, m0 = mtile * BM;
  const int k_begin = split * p.kslice;
  const int iters = p.kslice / kTileK;
  const size_t K = p.k;

  // loads: thread t brings 16 bytes: piece t % 8 of row t / 8 + 32 j (rows beyond the matrix: its last row again)
  const int lr = tid >> 3, lc = tid & 7;
  const bf16_t* wp[4];
#pragma unroll
  for (int j = 0; j < 4; ++j) wp[j] = p.w + (size_t)min(n0 + lr + 32 * j, p.n - 1) * K + k_begin + 8 * lc;
  const bf16_t* xp[XL];
#pragma unroll
  for (int j = 0; j < XL; ++j) xp[j] = p.x + (size_t)min(m0 + lr + 32 * j, p.m - 1) * K + k_begin + 8 * lc;
  char* st_w = smem + lr * kTileRow + lc * 16;
  char* st_x = smem + WT + lr * kTileRow + lc * 16;
  const char* rd_w = smem + (64 * wn + r32) * kTileRow + half * 16;
  const char* rd_x = smem + WT + (32 * NT * wm + r32) * kTileRow + half * 16;

  f32x16 acc[2][NT];
#pragma unroll
  for (int a = 0; a < 2; ++a)
#pragma unroll
    for (int b = 0; b < NT; ++b)
#pragma unroll
      for (int i = 0; i < 16; ++i) acc[a][b][i] = 0.f;

  bf16x8 wst[2][4], xst[2][XL];
  auto load_stage = [&](auto set, int kt) {
    const int koff = kt * kTileK;
#pragma unroll
    for (int j = 0; j < 4; ++j) wst[set][j] = *reinterpret_cast<const bf16x8*>(wp[j] + koff);
#pragma unroll
    for (int j = 0; j < XL; ++j) xst[set][j] = *reinterpret_cast<const bf16x8*>(xp[j] + koff);
  };
  auto store_stage = [&](auto set, int buf) {
#pragma unroll
    for (int j = 0; j < 4; ++j) *reinterpret_cast<bf16x8*>(st_w + buf * ST + 32 * j * kTileRow) = wst[set][j];
#pragma unroll
    for (int j = 0; j < XL; ++j) *reinterpret_cast<bf16x8*>(st_x + buf * ST + 32 * j * kTileRow) = xst[set][j];
  };
  bf16x8 af[2][2], bfr[2][NT];
  auto read_operands = [&](auto slot, int buf, int s) {
    const char* wb = rd_w + buf * ST + 32 * s;
    const char* xb = rd_x + buf * ST + 32 * s;
#pragma unroll
    for (int a = 0; a < 2; ++a) af[slot][a] = *reinterpret_cast<const bf16x8*>(wb + 32 * a * kTileRow);
#pragma unroll
    for (int b = 0; b < NT; ++b) bfr[slot][b] = *reinterpret_cast<const bf16x8*>(xb + 32 * b * kTileRow);
  };
  auto multiply = [&](auto slot) {
#pragma unroll
    for (int a = 0; a < 2; ++a)
#pragma unroll
      for (int b = 0; b < NT; ++b)
        acc[a][b] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(af[slot][a], bfr[slot][b], acc[a][b], 0, 0, 0);
  };
  // One step: the stage in `buf` is multiplied while the stage two ahead is loaded into register set `ld` and
  // the stage one ahead goes from register set `st` into the other buffer.  A stage beyond the last is the last
  // one again: loaded and stored, never read.
  auto step = [&](auto ld, auto st, int buf, int kt_load) {
    load_stage(ld, kt_load);
    read_operands(0, buf, 0);
    __builtin_amdgcn_sched_barrier(0);
    read_operands(1, buf, 1);
    __builtin_amdgcn_sched_barrier(0);
    multiply(0);
    __builtin_amdgcn_sched_barrier(0);
    read_operands(0, buf, 2);
    __builtin_amdgcn_sched_barrier(0);
    multiply(1);
    __builtin_amdgcn_sched_barrier(0);
    store_stage(st, buf ^ 1);
    read_operands(1, buf, 3);
    __builtin_amdgcn_sched_barrier(0);
    multiply(0);
    __builtin_amdgcn_sched_barrier(0);
    multiply(1);
    __syncthreads();
  };

  const int last = iters - 1;
  load_stage(0, 0);
  __builtin_amdgcn_sched_barrier(0);
  load_stage(1, min(1, last));
  __builtin_amdgcn_sched_barrier(0);
  store_stage(0, 0);
  __syncthreads();
  const int pairs = iters >> 1;
  for (int pr = 0; pr < pairs; ++pr) {
    const int it = 2 * pr;
    step(0, 1, 0, min(it + 2, last));
    step(1, 0, 1, min(it + 3, last));
  }
  if (iters & 1) step(0, 1, 0, last);

  // the tile transposed: lane holds, for row m = r32 of block b of x, columns n = 8 (i / 4) + 4 half + i % 4 of
  // block a of w
  const bool vec = (p.n & 3) == 0;   // n below is a multiple of 4: the four columns exist together, aligned
#pragma unroll
  for (int b = 0; b < NT; ++b) {
    const int m = m0 + 32 * NT * wm + 32 * b + r32;
    if (m >= p.m) continue;
#pragma unroll
    for (int a = 0; a < 2; ++a)
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        const int n = n0 + 64 * wn + 32 * a + 8 * g + 4 * half;
        if (n >= p.n) continue;
        f32x4 v = {acc[a][b][4 * g], acc[a][b][4 * g + 1], acc[a][b][4 * g + 2], acc[a][b][4 * g + 3]};
        if (p.splits > 1) {
          float* dst = p.partial + ((size_t)split * p.m + m) * p.n + n;
          if (vec) *reinterpret_cast<f32x4*>(dst) = v;
          else
            for (int i = 0; i < 4; ++i)
              if (n + i < p.n) dst[i] = v[i];
          continue;
        }
        if (p.bias)
          for (int i = 0; i < 4; ++i)
            if (n + i < p.n) v[i] += p.bias[n + i];
        if (p.out_f32) {
          float* dst = reinterpret_cast<float*>(p.y) + (size_t)m * p.n + n;
          if (vec) *reinterpret_cast<f32x4*>(dst) = v;
          else
            for (int i = 0; i < 4; ++i)
              if (n + i < p.n) dst[i] = v[i];
        } else {
          bf16_t* dst = reinterpret_cast<bf16_t*>(p.y) + (size_t)m * p.n + n;
          const bf16x4 r = {(bf16_t)v[0], (bf16_t)v[1], (bf16_t)v[2], (bf16_t)v[3]};
          if (vec) *reinterpret_cast<bf16x4*>(dst) = r;
          else
            for (int i = 0; i < 4; ++i)
              if (n + i < p.n) dst[i] = r[i];
        }
      }
  }
}

// 1 if the kernel takes this product.
ATOM_EXPORT int atom_gemm_tile_supports(int m, int n, int k) {
  return m >= 1 && n >= 1 && k >= kTileK && k % kTileK == 0;
}

// Rows of x a tile: 64 up to 64 rows, else 128.
static int tile_rows(int m) { return m <= 64 ? 64 : 128; }

// Into how many slices of K the product is cut on a chip of `num_cus` CUs: the most (1, 2, 4, 8) that keep tiles x
// slices within the CUs, every slice whole stages and at least eight of them.  Measured on an MI355X with the
// products of the 4B, 8B and 32B shapes at 96 to 512 rows: about one block a CU is best (o at 256 rows: 64 tiles, 4
// slices 19.7 us, 2 slices 25.3, 8 slices 22.2; the BLAS library 22.8).
ATOM_EXPORT int atom_gemm_tile_splits(int m, int n, int k, int num_cus) {
  if (!atom_gemm_tile_supports(m, n, k)) return 0;
  const int bm = tile_rows(m);
  const long tiles = (long)((n + kTileN - 1) / kTileN) * ((m + bm - 1) / bm);
  int splits = 1;
  for (int s = 2; s <= 8; s *= 2)
    if (tiles * s <= num_cus && k % (kTileK * s) == 0 && k / s >= 8 * kTileK) splits = s;
  return splits;
}

// splits == 1: y [m, n] bfloat16 or float32 (out_f32), bias [n] float32 or null.
// splits > 1 (a value atom_gemm_tile_splits may return: 2, 4, 8 with k % (64 splits) == 0): partial
// [splits, m, n] float32; y and bias are not used.
ATOM_EXPORT int atom_gemm_tile(const void* x, const void* w, const float* bias, void* y, float* partial, int m, int n,
                               int k, int splits, int out_f32, hipStream_t stream) {
  if (m < 0 || n <= 0 || k <= 0) return ATOM_BAD_SHAPE;
  if (!atom_gemm_tile_supports(m > 0 ? m : 1, n, k)) return ATOM_UNSUPPORTED;
  if (splits != 1 && splits != 2 && splits != 4 && splits != 8) return ATOM_BAD_SHAPE;
  if (k % (kTileK * splits)) return ATOM_BAD_SHAPE;
  if (m == 0) return ATOM_OK;
  if (!x || !w || (splits > 1 ? !partial : !y)) return ATOM_BAD_SHAPE;
  if (((uintptr_t)x | (uintptr_t)w) & 15) return ATOM_BAD_SHAPE;
  if (splits > 1 ? ((uintptr_t)partial & 15) : ((uintptr_t)y & 15)) return ATOM_BAD_SHAPE;
  TileParams p{};
  p.x = (const bf16_t*)x; p.w = (const bf16_t*)w; p.bias = bias; p.y = y; p.partial = partial;
  p.m = m; p.n = n; p.k = k; p.splits = splits; p.kslice = k / splits; p.out_f32 = out_f32;
  const int bm = tile_rows(m);
  p.mtiles = (m + bm - 1) / bm;
  p.ntiles = (n + kTileN - 1) / kTileN;
  const long blocks = (long)((p.ntiles + 7) / 8) * 8 * p.mtiles * splits;
  if (blocks > 0x7fffffffL) return ATOM_TOO_LARGE;
  const dim3 grid((unsigned)blocks), block(256);
  // the two LDS buffers of the larger tile pass the default limit of a block: raised once per kernel
  static bool raised[2] = {false, false};
  const int idx = bm == 64 ? 0 : 1;
  const size_t lds = 2 * (size_t)(kTileN + bm) * kTileRow;
  if (!raised[idx]) {
    const void* fn = idx == 0 ? (const void*)gemm_tile_kernel<1> : (const void*)gemm_tile_kernel<2>;
    if (hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds) != hipSuccess)
      return ATOM_LAUNCH_FAILED;
    raised[idx] = true;
  }
  if (idx == 0) hipLaunchKernelGGL(gemm_tile_kernel<1>, grid, block, lds, stream, p);
  else hipLaunchKernelGGL(gemm_tile_kernel<2>, grid, block, lds, stream, p);
  return launch_status();
}
