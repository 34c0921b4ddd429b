// y = x w^T for up to 8 rows of x (a decode step of few requests), bfloat16 operands, float32 sums on the
// matrix cores, with the step's element-wise work folded in at both ends so that a transformer layer is five
// launches: the RMS norm that precedes a product is applied where the product leaves the matrix cores, and so
// is the residual sum that follows one.
//
// A block owns 16 rows of w (16 output columns; 12 or 8 where the caller asks for narrower tiles, so that a
// width of few tiles spreads over more of the chip's CUs: the matrix cores' tile stays 16 wide and its other
// columns are dropped) and all of K, which is cut into 8 slices (a function of K
// alone); its W waves (4 or 8) each walk 8 / W neighbouring slices, a slice's sum in registers of its own.  A wave streams its part of the 16 rows with the whole-cache-line loads of gemm_skinny.hip
// (non-temporal, 256 contiguous bytes of four rows per load, four quarters of 128 k in flight, each brought
// into the matrix cores' A operand layout through a wave-private LDS area) and the matching 128 k of x, loaded
// together with them, through a second private area, so the waves of a block meet only once: at the end
// they add the slices' partial tiles through LDS in slice order (so the sum does not depend on W either).  No sum ever leaves a block unfinished, so nothing is
// cut into slices that a later kernel would have to add, and what follows the product is done in place:
//
//   norm      x is given as xg[m][k] = bf16(r[m][k] * g[k]), the rows of the residual stream times the norm's
//             weight, with ss[m][i], the sums of squares of ss_parts stretches of row m of r.  The row's factor
//             inv[m] = rsqrt(sum_i ss[m][i] / K + eps) (added in index order) is a scalar of the row, so it is
//             applied to the finished float32 sum instead of to every element before rounding:
//             sum_k bf16(r g)[k] w[n][k] * inv[m].  All of the norm's arithmetic stays float32.
//   epilogue  plain      y[m][n] = sum (+ bias), bfloat16 or float32
//             gate       act[m][c] = silu(sum_gate + b) * (sum_up + b), the block's rows of w being 8 gate
//                        and 8 up rows of the same 8 columns
//             residual   r[m][n] += sum (+ bias) in place (float32); ss_out[m][block] = the sum of squares of
//                        the block's 16 new elements of row m; xg_out[m][n] = bf16(r[m][n] * g_next[n]):
//                        what the product after the next norm takes as its input.
//
// Every row's result is formed in one fixed order whatever else is in the batch.
// Needs K % 8 == 0; any N; 1 <= M <= 8.
#include "common.h"

typedef __attribute__((ext_vector_type(4))) float f32x4;
typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;

struct RowsParams {
  const bf16_t* x;       // [*, k]
  const int* rows;       // row of x (and ss) that is row m of the product, or null for m itself
  const float* ss;       // norm: [*, ss_parts] partial sums of squares of the rows behind x; else null
  const bf16_t* w;       // [n, k]; gate: [2 * inter, k], gate rows first
  const float* bias;     // [n] (gate: [2 * inter]) or null
  void* y;               // plain: [m, n]; gate: [m, inter] bfloat16
  float* res;            // residual: [m, n] float32, added to in place
  float* ss_out;         // residual: [m, tiles]
  bf16_t* xg_out;        // residual: [m, n] or null
  const float* g_next;   // residual: [n], the weight of the norm that follows
  int m, n, k, inter, out_f32, mode, ss_parts, kslice, per_wave, tiles;   // kslice: k of a slice; per_wave: slices a wave
  int cols;              // output columns of a block: 16, 12 or 8 (gate: 8 gate and 8 up rows)
  float eps;
};

enum RowsMode : int { ROWS_PLAIN = 0, ROWS_GATE = 1, ROWS_RESIDUAL = 2 };

constexpr int kRowsQuarter = 128;            // k elements that go through a wave's LDS areas at a time
constexpr int kRowsA = 256 + 16;             // LDS bytes of a row of 128 k, 4 banks of padding
constexpr int kRowsAWave = 16 * kRowsA;      // a wave's layout-change area for w

// MR: rows of x that a wave keeps in LDS (the step's row count rounded up to 1, 2, 4 or 8).
// CG: groups of four rows of w that a block owns (4, or 3 or 2 for tiles of 12 or 8 columns).
template <int MR, int CG>
// (up to 4 rows: 128 registers, so that a CU holds two blocks of 8 waves)
__global__ void __launch_bounds__(512, (MR > 4 ? 3 : 4)) gemm_rows_kernel(RowsParams p) {
  constexpr int COLS = 4 * CG;
  extern __shared__ __attribute__((aligned(16))) char smem[];
  constexpr int AREA = kRowsAWave + MR * kRowsA;
  constexpr int XJ = MR > 4 ? 2 : 1;     // 16-byte pieces of x a lane brings per quarter
  const int tid = threadIdx.x;
  const int lane = tid & (kWave - 1);
  const int wave = __builtin_amdgcn_readfirstlane(tid / kWave);
  const int waves = blockDim.x / kWave;
  char* mine = smem + wave * AREA;
  char* xs = mine + kRowsAWave;
  const int r16 = lane & 15;
  const int g = lane >> 4;
  const int k = p.k;
  const int tile = blockIdx.x;
  const int kb = wave * p.per_wave * p.kslice;
  const int ke = min(k, kb + p.per_wave * p.kslice);
  const int quarters = kb < ke ? (ke - kb + kRowsQuarter - 1) / kRowsQuarter : 0;
  const int slice_quarters = p.kslice / kRowsQuarter;   // a wave has one or two slices: the second starts here

  // row j (0..15) of the block in w
  auto w_row = [&](int j) -> int {
    if (p.mode == ROWS_GATE) return min(tile * 8 + (j & 7), p.inter - 1) + (j >= 8 ? p.inter : 0);
    return min(tile * COLS + j, p.n - 1);
  };
  // a quarter of w: load rg is this lane's 16 bytes of row 4 rg + g at k 8 r16 of the quarter;
  // a quarter of x: piece j is this lane's 16 bytes of row g + 4 j of the batch at the same k
  const bf16_t* wrow[CG];
#pragma unroll
  for (int rg = 0; rg < CG; ++rg) wrow[rg] = p.w + (size_t)w_row(4 * rg + g) * k + 8 * r16;
  const bf16_t* xrow[XJ];
  bool xlive[XJ];
#pragma unroll
  for (int j = 0; j < XJ; ++j) {
    const int m = g + 4 * j;
    xlive[j] = m < MR && m < p.m;
    const int row = min(m, p.m - 1);
    xrow[j] = p.x + (size_t)(p.rows ? p.rows[row] : row) * k + 8 * r16;
  }
  const bf16x8 zero = {0, 0, 0, 0, 0, 0, 0, 0};

  bf16x8 a[4 * CG], xr[4 * XJ];
  auto load_quarter = [&](int q, int slot) {   // quarter q of the wave's range into register slot q % 4
    const int kk = kb + kRowsQuarter * q;
    const bool in = kk + 8 * r16 < ke;
#pragma unroll
    for (int j = 0; j < XJ; ++j)
      xr[XJ * slot + j] = (in && xlive[j]) ? *reinterpret_cast<const bf16x8*>(xrow[j] + kk) : zero;
#pragma unroll
    for (int rg = 0; rg < CG; ++rg)
      a[CG * slot + rg] = in ? __builtin_nontemporal_load(reinterpret_cast<const bf16x8*>(wrow[rg] + kk)) : zero;
  };
  // The norm's factor of every row, from the partial sums of squares in index order: wave v takes rows v and
  // v + waves (there are at least four waves and at most eight rows).  The loads of both rows go out together and
  // ahead of the first quarters of w, so that no wave waits a second time for the cache.
  float* inv_s = reinterpret_cast<float*>(smem + waves * AREA);    // [8], behind the waves' areas
  constexpr int SQ = 8;   // partial sums of squares a lane takes ahead: 512 a row (a width of 6,144 in tiles of 12)
  float sq[2][SQ];
  if (p.ss) {
#pragma unroll
    for (int t = 0; t < 2; ++t) {
      const int m = wave + t * waves;
      const bool live = m < p.m;
      const float* parts = p.ss + (size_t)(p.rows ? p.rows[live ? m : 0] : (live ? m : 0)) * p.ss_parts;
#pragma unroll
      for (int u = 0; u < SQ; ++u) {
        const int i = lane + kWave * u;
        sq[t][u] = (live && i < p.ss_parts) ? parts[i] : 0.f;
      }
    }
  }
#pragma unroll
  for (int s4 = 0; s4 < 4; ++s4)
    if (s4 < quarters) load_quarter(s4, s4);
  if (p.ss) {
#pragma unroll
    for (int t = 0; t < 2; ++t) {
      const int m = wave + t * waves;
      if (m >= p.m) continue;
      float sum = ((sq[t][0] + sq[t][1]) + (sq[t][2] + sq[t][3])) + ((sq[t][4] + sq[t][5]) + (sq[t][6] + sq[t][7]));
      if (p.ss_parts > SQ * kWave) {
        const float* parts = p.ss + (size_t)(p.rows ? p.rows[m] : m) * p.ss_parts;
        for (int i = lane + SQ * kWave; i < p.ss_parts; i += kWave) sum += parts[i];
      }
      sum = wave_sum(sum);
      if (lane == 0) inv_s[m] = rsqrtf(sum / (float)k + p.eps);
    }
  }

  f32x4 acc = {0.f, 0.f, 0.f, 0.f};
  float* part = reinterpret_cast<float*>(smem + waves * AREA + 64) + wave * 2 * 16 * 17;   // [2][16 m][16 c + 1]
  const int xread = min(r16, min(MR, p.m) - 1) * kRowsA + 16 * g;   // rows beyond the batch read its last row; not used
  const int aread = min(r16, COLS - 1) * kRowsA + 16 * g;           // columns beyond the tile read its last; not used

  for (int q0 = 0; q0 < quarters; q0 += 4) {
#pragma unroll
    for (int s4 = 0; s4 < 4; ++s4) {
      const int q = q0 + s4;
      if (q < quarters) {   // the same in all lanes of the wave
        // the quarter into the operand layouts through the wave's own LDS areas
#pragma unroll
        for (int rg = 0; rg < CG; ++rg)
          *reinterpret_cast<bf16x8*>(mine + (4 * rg + g) * kRowsA + r16 * 16) = a[CG * s4 + rg];
#pragma unroll
        for (int j = 0; j < XJ; ++j)
          if (g + 4 * j < MR) *reinterpret_cast<bf16x8*>(xs + (g + 4 * j) * kRowsA + r16 * 16) = xr[XJ * s4 + j];
        if (q + 4 < quarters) load_quarter(q + 4, s4);   // these registers are free again
        __builtin_amdgcn_s_waitcnt(0xc07f);              // lgkmcnt(0): the areas are this wave's alone
        __builtin_amdgcn_wave_barrier();
        if (q == slice_quarters) {   // the wave's second slice starts: the first one's sum is put aside
#pragma unroll
          for (int i = 0; i < 4; ++i) part[r16 * 17 + 4 * g + i] = acc[i];
          acc = f32x4{0.f, 0.f, 0.f, 0.f};
        }
#pragma unroll
        for (int u = 0; u < 4; ++u) {
          const bf16x8 av = *reinterpret_cast<const bf16x8*>(mine + aread + u * 64);
          const bf16x8 bv = *reinterpret_cast<const bf16x8*>(xs + xread + u * 64);
          acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(av, bv, acc, 0, 0, 0);
        }
        __builtin_amdgcn_s_waitcnt(0xc07f);
        __builtin_amdgcn_wave_barrier();
      }
    }
  }

  // ---- the slices' partial tiles, added in slice order: lane (r16, g) holds row m = r16 of x, rows 4 g + i of w
  {
    float* last = part + (quarters > slice_quarters ? 16 * 17 : 0);
#pragma unroll
    for (int i = 0; i < 4; ++i) last[r16 * 17 + 4 * g + i] = acc[i];
    if (p.per_wave == 2 && quarters <= slice_quarters) {   // K ended inside the wave's first slice: the second is empty
#pragma unroll
      for (int i = 0; i < 4; ++i) part[16 * 17 + r16 * 17 + 4 * g + i] = 0.f;
    }
  }
  __syncthreads();
  if (tid >= 256) return;
  const int m = tid >> 4, c = tid & 15;
  float sum = 0.f;
  const float* parts_all = reinterpret_cast<const float*>(smem + waves * AREA + 64);
  for (int wv = 0; wv < waves; ++wv)
    for (int sl = 0; sl < p.per_wave; ++sl) sum += parts_all[(wv * 2 + sl) * 16 * 17 + m * 17 + c];
  const bool live = m < p.m;
  if (p.ss && live) sum *= inv_s[m];

  if (p.mode == ROWS_GATE) {
    // c < 8: the gate value of column tile * 8 + c; its up value is 8 places on
    const float up = __shfl_down(sum, 8, 16);
    const int col = tile * 8 + c;
    if (live && c < 8 && col < p.inter) {
      float gv = sum, uv = up;
      if (p.bias) {
        gv += p.bias[col];
        uv += p.bias[p.inter + col];
      }
      reinterpret_cast<bf16_t*>(p.y)[(size_t)m * p.inter + col] = from_f32<bf16_t>(gv / (1.f + expf(-gv)) * uv);
    }
    return;
  }
  const int col = tile * COLS + c;
  const bool has = live && c < COLS && col < p.n;
  float v = sum + ((has && p.bias) ? p.bias[col] : 0.f);
  if (p.mode == ROWS_RESIDUAL) {
    float sq = 0.f;
    if (has) {
      float* at = p.res + (size_t)m * p.n + col;
      v += *at;
      *at = v;
      sq = v * v;
      if (p.xg_out) p.xg_out[(size_t)m * p.n + col] = from_f32<bf16_t>(v * p.g_next[col]);
    }
#pragma unroll
    for (int off = 8; off > 0; off >>= 1) sq += __shfl_xor(sq, off, 16);
    if (live && c == 0) p.ss_out[(size_t)m * p.tiles + tile] = sq;
    return;
  }
  if (has) {
    if (p.out_f32) reinterpret_cast<float*>(p.y)[(size_t)m * p.n + col] = v;
    else reinterpret_cast<bf16_t*>(p.y)[(size_t)m * p.n + col] = from_f32<bf16_t>(v);
  }
}

static int rows_tiles(int n, int mode, int cols) { return mode == ROWS_GATE ? (n + 7) / 8 : (n + cols - 1) / cols; }
static bool rows_cols_ok(int cols) { return cols == 16 || cols == 12 || cols == 8; }

// Waves a block: enough of them on the chip to keep memory busy, a whole shot of k for each where K allows.
// Measured on an MI355X: eight waves for the narrow products (a block a CU or little more), four where a CU
// holds several blocks anyway (four blocks a CU and more), and from five rows on (two pieces of x a lane and
// quarter) wherever more than one block a CU is there.
static int rows_waves(int m, int tiles, int k) {
  const int shots = (k + 511) / 512;
  const int cus = device_cus();
  int waves = (tiles >= 4 * cus || (m > 4 && tiles > cus)) ? 4 : 8;
  while (waves > 4 && waves > shots) waves >>= 1;
  return waves;
}

// The number of partial sums of squares a row gets from a product of this width in residual mode with
// tiles of ``cols`` columns (16, 12 or 8; 0 for anything else).
ATOM_EXPORT int atom_gemm_rows_parts(int n, int cols) { return rows_cols_ok(cols) ? rows_tiles(n, ROWS_RESIDUAL, cols) : 0; }

// 1 if the kernel takes this product.
ATOM_EXPORT int atom_gemm_rows_supports(int m, int n, int k) {
  return m >= 1 && m <= 8 && n >= 1 && k >= 8 && k % 8 == 0;
}

// mode 0 (plain): y [m, n], bfloat16 or float32 (out_f32).   mode 1 (gate): w is [2 n, k], y [m, n] bfloat16.
// mode 2 (residual): res [m, n] float32 += product, ss_out [m, atom_gemm_rows_parts(n, cols)], and, with g_next [n],
// xg_out [m, n] = bf16(res * g_next).
// cols: output columns a block owns in modes 0 and 2: 16, or 12 or 8 for widths whose 16-column tiles would leave
// CUs without a block or some with one more than others (mode 1 takes 16 only: 8 gate and 8 up rows).
// Input: x [*, k] bfloat16, row rows[i] of it for row i of the product when rows is given; with ss
// [*, ss_parts] x is the rows of a float32 stream times a norm's weight, ss the partial sums of squares of those
// rows, and the product is that of the stream's RMS norm (eps).
ATOM_EXPORT int atom_gemm_rows(const void* x, const int* rows, const float* ss, int ss_parts, float eps, const void* w,
                               const float* bias, void* y, float* res, float* ss_out, void* xg_out,
                               const float* g_next, int m, int n, int k, int mode, int out_f32, int cols,
                               int waves_override, hipStream_t stream) {
  if (m < 0 || n <= 0 || k <= 0 || mode < 0 || mode > 2) return ATOM_BAD_SHAPE;
  if (!rows_cols_ok(cols) || (mode == ROWS_GATE && cols != 16)) return ATOM_UNSUPPORTED;
  if (!atom_gemm_rows_supports(max(m, 1), n, k)) return ATOM_UNSUPPORTED;
  if (m == 0) return ATOM_OK;
  if (!x || !w || (ss && ss_parts < 1)) return ATOM_BAD_SHAPE;
  if (mode == ROWS_RESIDUAL ? (!res || !ss_out || (xg_out && !g_next)) : !y) return ATOM_BAD_SHAPE;
  if (mode == ROWS_GATE && out_f32) return ATOM_UNSUPPORTED;
  if (((uintptr_t)x | (uintptr_t)w) & 15) return ATOM_BAD_SHAPE;
  RowsParams p{};
  p.x = (const bf16_t*)x; p.rows = rows; p.ss = ss; p.w = (const bf16_t*)w; p.bias = bias;
  p.y = y; p.res = res; p.ss_out = ss_out; p.xg_out = (bf16_t*)xg_out; p.g_next = g_next;
  p.m = m; p.k = k; p.out_f32 = out_f32; p.mode = mode; p.ss_parts = ss_parts; p.eps = eps;
  p.n = mode == ROWS_GATE ? 2 * n : n;
  p.inter = mode == ROWS_GATE ? n : 0;
  p.tiles = rows_tiles(n, mode, cols);
  p.cols = cols;
  int waves = rows_waves(m, p.tiles, k);
  if (waves_override == 4 || waves_override == 8) waves = waves_override;
  // 8 slices of K (4 where K is shorter than 8 quarters): the same for every number of rows and of waves
  const int units = (k + kRowsQuarter - 1) / kRowsQuarter;
  const int slices = units >= 8 ? 8 : 4;
  if (waves > slices) waves = slices;
  p.kslice = (units + slices - 1) / slices * kRowsQuarter;
  p.per_wave = slices / waves;
  const int mr = m <= 1 ? 1 : (m <= 2 ? 2 : (m <= 4 ? 4 : 8));
  const size_t lds = (size_t)waves * (kRowsAWave + mr * kRowsA) + 64 + (size_t)waves * 2 * 16 * 17 * 4;
#define GO_ROWS(MRV, CGV) \
  hipLaunchKernelGGL((gemm_rows_kernel<MRV, CGV>), dim3(p.tiles), dim3(64 * waves), lds, stream, p)
#define GO_ROWS_COLS(MRV)              \
  switch (cols) {                      \
    case 8: GO_ROWS(MRV, 2); break;    \
    case 12: GO_ROWS(MRV, 3); break;   \
    default: GO_ROWS(MRV, 4); break;   \
  }
  switch (mr) {
    case 1: GO_ROWS_COLS(1); break;
    case 2: GO_ROWS_COLS(2); break;
    case 4: GO_ROWS_COLS(4); break;
    default: GO_ROWS_COLS(8); break;
  }
#undef GO_ROWS_COLS
#undef GO_ROWS
  return launch_status();
}
