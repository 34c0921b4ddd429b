// y[M, N] = x[M, K] * w[N, K]^T (+ bias) for few rows (M <= 64; narrow products M <= 128), bfloat16 operands,
// float32 accumulation on the matrix cores.  This is the decode-step product: the
// weight matrix is streamed from memory once and the work is bound by that stream.
//
// Two kernels: gemm_skinny_kernel, described here, stages the block's slice of x in LDS and takes up to 16
// rows of x; gemm_mid_kernel, described at its place, streams x beside the weights and takes up to 64 (128).
// takes_mid() says which one runs.
// A block of four waves owns 64 rows of w (64 output columns) and a slice of K; each
// wave owns 16 of the rows and walks its part of the slice in shots of 512 k.  For a shot
// a wave issues all its 16 loads at once, non-temporal, each covering 256 contiguous
// bytes of four rows (whole cache lines: lanes 16 q .. 16 q + 15 read k 128 s .. 128 s + 127
// of row 4 rg + q for load (rg, s)).  The matrix cores want the weights as the A operand of
// v_mfma_f32_16x16x32_bf16 (lane (r, g) holds w[row r][k + 8 g .. k + 8 g + 7]), so each
// quarter of the shot goes through a small wave-private LDS area to change layout.  x is
// the B operand; the block's slice of it is staged in LDS and shared by the four waves, so
// x is read from the cache hierarchy once per 64 rows of w.  Blocks that are neighbours in
// the grid read neighbouring slices of the same rows.
//
// When N / 64 blocks would not fill the chip, K is cut into `splits` slices and every
// block writes its partial tile to partial[split][m][n] (float32).  Whoever reads the
// product next adds the slices in slice order: the norm, the rotation kernel, SiLU-mul,
// or atom_splitk_reduce.  The sum has one fixed order, so a row's result does not
// depend on the rows beside it (to the bit within one of the two kernels; they cut K differently).
//
// Epilogues when K is not cut: plain (bias optional, bfloat16 or float32 out), or
// SiLU-gate: w holds `inter` gate rows then `inter` up rows, a block owns 32 columns of
// each, and writes silu(gate) * up [M, inter].
//
// Needs K % 8 == 0 (16-byte loads).  Any N, any M <= 64; atom_gemm_skinny_supports says which products
// with up to 128 rows it takes.
#include "common.h"
#include "linear_static.h"

#include <mutex>
#include <type_traits>

typedef __attribute__((ext_vector_type(4))) float f32x4;
typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;

struct SkinnyParams {
  const bf16_t* x;     // [m, k]
  const bf16_t* w;     // [n, k]  (gate: [2 * inter, k])
  const float* bias;   // [n] or null (only used when splits == 1)
  void* y;             // splits == 1: [m, n] bfloat16 or float32 (gate: [m, inter] bfloat16)
  float* partial;      // splits > 1: [splits, m, n]
  int m, n, k, inter, out_f32, splits, tiles, kslice, xk;
  int halves, rows_half;   // 65 to 128 rows: two blocks share a tile of w, each with rows_half rows of x
};

struct SkinnyPlan {
  int splits, kslice, xk;
};

constexpr int kSkinnyRows = 64;    // rows of w per block
constexpr int kSkinnyChunk = 512;  // k elements per shot
constexpr int kSkinnyLds = 64 * 1024;
constexpr int kARow = 256 + 16;    // LDS bytes of one row of a quarter shot (128 k), padded by 4 banks
constexpr int kAWave = 16 * kARow; // LDS bytes of a wave's layout-change area

// MT: 16-row tiles of x; launched with one.
template <int MT, bool GATE>
__global__ void __launch_bounds__(256) gemm_skinny_kernel(SkinnyParams p) {
  constexpr int THREADS = 256;
  // [a wave's layout-change area] x 4, then the x slice (later the float32 tile)
  extern __shared__ __attribute__((aligned(16))) char smem_all[];
  char* smem = smem_all + 4 * kAWave;
  const int tid = threadIdx.x;
  const int lane = tid & (kWave - 1);
  const int wave = tid / kWave;          // which 16 of the block's 64 rows
  char* mine = smem_all + wave * kAWave;
  const int r16 = lane & 15;
  const int g = lane >> 4;
  const int k = p.k;
  const int tile = blockIdx.x / p.splits;
  const int split = blockIdx.x - tile * p.splits;
  const int k_begin = split * p.kslice;
  const int k_end = min(k, k_begin + p.kslice);
  const int kw_begin = k_begin, kw_end = k_end;
  const int xrow_bytes = p.xk * 2 + 16;   // 16 bytes of padding: rows start 4 banks apart

  // row j (0..15) of this wave in w
  auto w_row = [&](int j) -> int {
    if (GATE) {
      const int col = tile * 32 + (wave & 1) * 16 + j;
      return min(col, p.inter - 1) + (wave >= 2 ? p.inter : 0);
    }
    return min(tile * kSkinnyRows + wave * 16 + j, p.n - 1);
  };
  // load (rg, s) of a shot: this lane reads 16 bytes of row 4 rg + g at k 128 s + 8 r16
  const bf16_t* wrow[4];
#pragma unroll
  for (int rg = 0; rg < 4; ++rg) wrow[rg] = p.w + (size_t)w_row(4 * rg + g) * k + 8 * r16;
  const bf16x8 zero = {0, 0, 0, 0, 0, 0, 0, 0};

  f32x4 acc[MT];
#pragma unroll
  for (int t = 0; t < MT; ++t) acc[t] = f32x4{0.f, 0.f, 0.f, 0.f};
  int xrow[MT];
#pragma unroll
  for (int t = 0; t < MT; ++t) xrow[t] = min(16 * t + r16, p.m - 1) * xrow_bytes + 16 * g;

  for (int x0 = k_begin; x0 < k_end; x0 += p.xk) {
    const int x1 = min(k_end, x0 + p.xk);
    // this wave's first shot in [x0, x1): its loads go out before x is staged
    int kc = max(x0, kw_begin);
    const int kc_end = min(x1, kw_end);
    bf16x8 a[16];
    auto load_shot = [&](int at) {
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        const int kk = at + 128 * (i >> 2);
        a[i] = (kk + 8 * r16 < k) ? __builtin_nontemporal_load(reinterpret_cast<const bf16x8*>(wrow[i & 3] + kk))
                                  : zero;
      }
    };
    if (kc < kc_end) load_shot(kc);

    const int pieces = (x1 - x0 + 7) / 8;    // 16-byte pieces per row
    if (x0 != k_begin) __syncthreads();      // the previous slice of x has been read
    for (int q = tid; q < p.m * pieces; q += THREADS) {
      const int row = q / pieces, piece = q - row * pieces;
      const int kk = x0 + 8 * piece;
      const bf16x8 v = kk < k ? *reinterpret_cast<const bf16x8*>(p.x + (size_t)row * k + kk) : zero;
      *reinterpret_cast<bf16x8*>(smem + row * xrow_bytes + piece * 16) = v;
    }
    // a shot that reaches beyond K reads pieces the loop above did not write: zero them
    const int padded = ((x1 - x0 + kSkinnyChunk - 1) / kSkinnyChunk) * (kSkinnyChunk / 8);
    for (int q = tid; q < p.m * (padded - pieces); q += THREADS) {
      const int row = q / (padded - pieces), piece = pieces + q - row * (padded - pieces);
      *reinterpret_cast<bf16x8*>(smem + row * xrow_bytes + piece * 16) = zero;
    }
    __syncthreads();

    for (; kc < kc_end; kc += kSkinnyChunk) {
      const char* xb = smem + (kc - x0) * 2;
      const bool more = kc + kSkinnyChunk < kc_end;
#pragma unroll
      for (int s4 = 0; s4 < 4; ++s4) {
        // a quarter of the shot into the operand layout through the wave's own LDS area
#pragma unroll
        for (int rg = 0; rg < 4; ++rg)
          *reinterpret_cast<bf16x8*>(mine + (4 * rg + g) * kARow + r16 * 16) = a[4 * s4 + rg];
        if (more) {   // these four registers are free again: the same quarter of the next shot
#pragma unroll
          for (int rg = 0; rg < 4; ++rg) {
            const int kk = kc + kSkinnyChunk + 128 * s4;
            a[4 * s4 + rg] = (kk + 8 * r16 < k)
                                 ? __builtin_nontemporal_load(reinterpret_cast<const bf16x8*>(wrow[rg] + kk)) : zero;
          }
        }
        __builtin_amdgcn_s_waitcnt(0xc07f);   // lgkmcnt(0): the area is this wave's alone, no block barrier
        __builtin_amdgcn_wave_barrier();
#pragma unroll
        for (int u = 0; u < 4; ++u) {
          const bf16x8 av = *reinterpret_cast<const bf16x8*>(mine + r16 * kARow + u * 64 + g * 16);
#pragma unroll
          for (int t = 0; t < MT; ++t) {
            const bf16x8 bv = *reinterpret_cast<const bf16x8*>(xb + xrow[t] + 64 * (4 * s4 + u));
            acc[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(av, bv, acc[t], 0, 0, 0);
          }
        }
        __builtin_amdgcn_s_waitcnt(0xc07f);
        __builtin_amdgcn_wave_barrier();
      }
    }
  }

  // ---- the block's float32 tile [m][64] through LDS: lane holds rows m = 16 t + r16, columns 16 wave + 4 g + i
  __syncthreads();
  float* tile_f = reinterpret_cast<float*>(smem);   // [m][65]
#pragma unroll
  for (int t = 0; t < MT; ++t) {
    const int m = 16 * t + r16;
    if (m < p.m) {
#pragma unroll
      for (int i = 0; i < 4; ++i) tile_f[m * (kSkinnyRows + 1) + 16 * wave + 4 * g + i] = acc[t][i];
    }
  }
  __syncthreads();

  if (p.splits > 1) {
    float* out_slice = p.partial + (size_t)split * p.m * p.n;
    for (int item = tid; item < p.m * kSkinnyRows; item += THREADS) {
      const int m = item >> 6, c = item & 63;
      int col;
      if (GATE) {
        col = tile * 32 + (c & 31);
        if (col >= p.inter) continue;
        col += (c >= 32 ? p.inter : 0);
      } else {
        col = tile * kSkinnyRows + c;
        if (col >= p.n) continue;
      }
      out_slice[(size_t)m * p.n + col] = tile_f[m * (kSkinnyRows + 1) + c];
    }
    return;
  }
  if (GATE) {
    for (int item = tid; item < p.m * 32; item += THREADS) {
      const int m = item >> 5, c = item & 31;
      const int col = tile * 32 + c;
      if (col >= p.inter) continue;
      float gv = tile_f[m * (kSkinnyRows + 1) + c];
      float uv = tile_f[m * (kSkinnyRows + 1) + 32 + c];
      if (p.bias) {
        gv += p.bias[col];
        uv += p.bias[p.inter + col];
      }
      reinterpret_cast<bf16_t*>(p.y)[(size_t)m * p.inter + col] = from_f32<bf16_t>(gv / (1.f + expf(-gv)) * uv);
    }
  } else {
    for (int item = tid; item < p.m * kSkinnyRows; item += THREADS) {
      const int m = item >> 6, c = item & 63;
      const int col = tile * kSkinnyRows + c;
      if (col >= p.n) continue;
      const float v = tile_f[m * (kSkinnyRows + 1) + c] + (p.bias ? p.bias[col] : 0.f);
      if (p.out_f32) reinterpret_cast<float*>(p.y)[(size_t)m * p.n + col] = v;
      else reinterpret_cast<bf16_t*>(p.y)[(size_t)m * p.n + col] = from_f32<bf16_t>(v);
    }
  }
}

// ---- Up to 64 rows of x (needed from 17 rows on: with that many a useful slice of x no longer fits in LDS
// beside the weights' layout-change areas), x streamed like the weights.  A block of W waves (4 to 8) owns
// 16 W rows of w and a range of K; a chunk is 128 k of those rows and of the rows of x.  Each wave loads
// its own 16 rows of w and a share of the rows of x (the same whole-cache-line loads as above, four
// chunks in flight a wave) and writes them to one of two LDS buffers; after the block's barrier it
// multiplies its rows of w with every 16 rows of x.  The more waves, the fewer times x is read; mid_plan()
// chooses their number and the slices of K.
//
// SiLU-gate: a wave's 16 rows are 8 gate and 8 up rows of the same 8 columns, ordered so that a lane's
// four results are two gate values and the two up values of the same columns.
//
// 65 to 128 rows of x, for products whose blocks of four waves all fit on the chip twice over: every
// block comes twice, side by side in the grid, each with half of the rows of x.  The pair reads its
// rows of w at about the same time, so memory delivers them once.
constexpr int kMidSlice = 1024;   // K is cut in multiples of this
constexpr int kMidAhead = 4;      // chunks in flight a wave (3 and 5 measure the same)

// EXACT: the block's range of K is whole chunks, so no load needs a guard.  TURN: K is not cut, and every
// tile starts its walk through K at another eighth.
template <int MT, bool GATE, bool EXACT, bool TURN>
__global__ void __launch_bounds__(512) gemm_mid_kernel(SkinnyParams p) {
  extern __shared__ __attribute__((aligned(16))) char lds[];   // two chunks of 16 W + 16 MT rows
  const int tid = threadIdx.x;
  const int lane = tid & (kWave - 1);
  const int wave = __builtin_amdgcn_readfirstlane(tid / kWave);
  const int waves = blockDim.x / kWave;
  const int r16 = lane & 15;
  const int g = lane >> 4;
  const int k = p.k;
  // with more than 64 rows of x neighbouring blocks take the same rows of w and a half of x each
  const int unit = blockIdx.x / p.halves;
  const int m_base = (blockIdx.x - unit * p.halves) * p.rows_half;
  const int m_rows = min(p.rows_half, p.m - m_base);
  const int tile = unit / p.splits;
  const int split = unit - tile * p.splits;
  const int k_begin = split * p.kslice;
  const int k_end = min(k, k_begin + p.kslice);
  const int total = (k_end - k_begin + 127) / 128;   // chunks
  const int chunk_bytes = (16 * waves + 16 * MT) * kARow;
  // Blocks that start together would all read the same stretch of their rows, a row's length apart in memory,
  // and so the same few memory channels at any moment: where K is not cut (slices start apart anyway, and
  // measure worse with this) every tile starts its walk through K at another eighth.
  const int first = (TURN && total >= 8) ? (tile & 7) * (total >> 3) : 0;
  auto k_of = [&](int ci) {
    if (!TURN) return k_begin + 128 * ci;
    const int c = ci + first;
    return k_begin + 128 * (c < total ? c : c - total);
  };

  // first column of this wave; row j (0..15) of the wave in w
  const int col0 = GATE ? (tile * waves + wave) * 8 : (tile * waves + wave) * 16;
  auto w_row = [&](int j) -> int {
    if (GATE) return min(col0 + 2 * (j >> 2) + (j & 1), p.inter - 1) + ((j & 2) ? p.inter : 0);
    return min(col0 + j, p.n - 1);
  };
  // load (rg) of a chunk of w: this lane's 16 bytes of row 4 rg + g;  load (q) of x: of row 4 (wave + waves q) + g
  const bf16_t* wrow[4];
  const bf16_t* xrow[4];
  int xat[4];
  bool xmine[4];   // the same in all lanes of a wave
#pragma unroll
  for (int rg = 0; rg < 4; ++rg) {
    wrow[rg] = p.w + (size_t)w_row(4 * rg + g) * k + 8 * r16;
    const int four = wave + waves * rg;   // which four rows of x
    xmine[rg] = four < 4 * MT;
    xat[rg] = (16 * waves + 4 * four + g) * kARow + r16 * 16;
    xrow[rg] = p.x + (size_t)(m_base + min(4 * four + g, m_rows - 1)) * k + 8 * r16;
  }
  const bf16x8 zero = {0, 0, 0, 0, 0, 0, 0, 0};

  f32x4 acc[MT];
#pragma unroll
  for (int t = 0; t < MT; ++t) acc[t] = f32x4{0.f, 0.f, 0.f, 0.f};
  bf16x8 a[4 * kMidAhead], xa[4 * kMidAhead];
  auto load_w = [&](int slot, int ci) {
    const int kk = k_of(ci);
    const bool in = EXACT || kk + 8 * r16 < k_end;
#pragma unroll
    for (int rg = 0; rg < 4; ++rg)
      a[4 * slot + rg] = in ? __builtin_nontemporal_load(reinterpret_cast<const bf16x8*>(wrow[rg] + kk)) : zero;
  };
  auto load_x = [&](int slot, int ci) {
    const int kk = k_of(ci);
    const bool in = EXACT || kk + 8 * r16 < k_end;
#pragma unroll
    for (int rg = 0; rg < 4; ++rg)
      if (xmine[rg]) xa[4 * slot + rg] = in ? *reinterpret_cast<const bf16x8*>(xrow[rg] + kk) : zero;
  };
  // The products of a chunk.  The operands of step u + 1 are read from LDS before the products of step u are
  // issued, and the order is pinned: left to itself the compiler reads each operand right before the product
  // that takes it and waits for it there.
  auto multiply = [&](const char* buf) {
    bf16x8 av[2], bv[2][MT];
    auto operands = [&](int slot, int u) {
      av[slot] = *reinterpret_cast<const bf16x8*>(buf + (16 * wave + r16) * kARow + u * 64 + g * 16);
#pragma unroll
      for (int t = 0; t < MT; ++t)
        bv[slot][t] = *reinterpret_cast<const bf16x8*>(buf + (16 * (waves + t) + r16) * kARow + u * 64 + g * 16);
    };
    operands(0, 0);
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      if (u < 3) operands((u + 1) & 1, u + 1);
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int t = 0; t < MT; ++t)
        acc[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(av[u & 1], bv[u & 1][t], acc[t], 0, 0, 0);
      __builtin_amdgcn_sched_barrier(0);
    }
  };

  // A range of K that is whole chunks and long enough runs its middle without a branch: every wave brings the same
  // number of pieces of x a chunk, XN = ceil(4 MT / waves) (a wave whose piece lies beyond the 4 MT that there are
  // brings one of them again, to the same place), and every chunk's successor exists.  The compiler counts the
  // loads in flight exactly only in straight-line code; with loads inside branches it waits for every one of them
  // once a trip, which empties the queue that the loads ahead are there to keep full.  XN is a constant of the
  // loop, so the loop is there once for each value that this MT can meet.
  int base = 0;
  const int x_each = (4 * MT + waves - 1) / waves;
  auto steady = [&](auto xn) {
    constexpr int XN = decltype(xn)::value;
    const bf16_t* xrow_all[XN];
    int xat_all[XN];
#pragma unroll
    for (int rg = 0; rg < XN; ++rg) {
      const int four = (wave + waves * rg) % (4 * MT);
      xat_all[rg] = (16 * waves + 4 * four + g) * kARow + r16 * 16;
      xrow_all[rg] = p.x + (size_t)(m_base + min(4 * four + g, m_rows - 1)) * k + 8 * r16;
    }
    auto load_both = [&](int slot, int ci) {
      const int kk = k_of(ci);
#pragma unroll
      for (int rg = 0; rg < 4; ++rg)
        a[4 * slot + rg] = __builtin_nontemporal_load(reinterpret_cast<const bf16x8*>(wrow[rg] + kk));
#pragma unroll
      for (int rg = 0; rg < XN; ++rg) xa[4 * slot + rg] = *reinterpret_cast<const bf16x8*>(xrow_all[rg] + kk);
    };
    // (in the order of the chunks, pinned: the loop's waits are counted from the order in which the loads went out,
    // here as in the loop, and the compiler would otherwise send the first chunk's loads last)
#pragma unroll
    for (int slot = 0; slot < kMidAhead; ++slot) {
      load_both(slot, slot);
      __builtin_amdgcn_sched_barrier(0);
    }
    for (; base + 2 * kMidAhead <= total; base += kMidAhead) {
#pragma unroll
      for (int c = 0; c < kMidAhead; ++c) {
        const int ci = base + c;
        char* buf = lds + (ci & 1) * chunk_bytes;
#pragma unroll
        for (int rg = 0; rg < 4; ++rg)
          *reinterpret_cast<bf16x8*>(buf + (16 * wave + 4 * rg + g) * kARow + r16 * 16) = a[4 * c + rg];
#pragma unroll
        for (int rg = 0; rg < XN; ++rg) *reinterpret_cast<bf16x8*>(buf + xat_all[rg]) = xa[4 * c + rg];
        load_both(c, ci + kMidAhead);
        __syncthreads();
        multiply(buf);
      }
    }
  };
  constexpr int XN_MIN = (4 * MT + 7) / 8;   // with eight waves, the most a block has
  bool done = false;
  if (EXACT && total >= 2 * kMidAhead) {
    if (x_each == XN_MIN) { steady(std::integral_constant<int, XN_MIN>{}); done = true; }
    if constexpr (MT >= XN_MIN + 1) {
      if (x_each == XN_MIN + 1) { steady(std::integral_constant<int, XN_MIN + 1>{}); done = true; }
    }
    if constexpr (MT >= XN_MIN + 2) {
      if (x_each == XN_MIN + 2) { steady(std::integral_constant<int, XN_MIN + 2>{}); done = true; }
    }
  }
  if (!done) {
#pragma unroll
    for (int slot = 0; slot < kMidAhead; ++slot)
      if (slot < total) {
        load_w(slot, slot);
        load_x(slot, slot);
      }
  }

  for (; base < total; base += kMidAhead) {
#pragma unroll
    for (int c = 0; c < kMidAhead; ++c) {
      const int ci = base + c;
      if (ci < total) {   // the same in every wave of the block
        char* buf = lds + (ci & 1) * chunk_bytes;
        // the two buffers take turns: a wave that writes chunk ci has passed the barrier of chunk ci - 1,
        // which every wave reaches only after it has read chunk ci - 2
#pragma unroll
        for (int rg = 0; rg < 4; ++rg)
          *reinterpret_cast<bf16x8*>(buf + (16 * wave + 4 * rg + g) * kARow + r16 * 16) = a[4 * c + rg];
#pragma unroll
        for (int rg = 0; rg < 4; ++rg)
          if (xmine[rg]) *reinterpret_cast<bf16x8*>(buf + xat[rg]) = xa[4 * c + rg];
        if (ci + kMidAhead < total) {
          load_w(c, ci + kMidAhead);
          load_x(c, ci + kMidAhead);
        }
        __syncthreads();
        multiply(buf);
      }
    }
  }

  // lane (r16, g) holds, for row 16 t + r16 of the block's rows of x, this wave's rows 4 g .. 4 g + 3 of w
  if (GATE) {
    const int col = col0 + 2 * g;                  // gate columns col, col + 1 in [0], [1]; their up values in [2], [3]
    const bool pair = (p.inter & 1) == 0;          // col is even: both columns exist together, stores are aligned
#pragma unroll
    for (int t = 0; t < MT; ++t) {
      if (16 * t + r16 >= m_rows || col >= p.inter) continue;
      const int m = m_base + 16 * t + r16;
      if (p.splits > 1) {
        float* out_row = p.partial + ((size_t)split * p.m + m) * p.n;
        if (pair) {
          *reinterpret_cast<float2*>(out_row + col) = float2{acc[t][0], acc[t][1]};
          *reinterpret_cast<float2*>(out_row + p.inter + col) = float2{acc[t][2], acc[t][3]};
        } else {
          out_row[col] = acc[t][0];
          out_row[p.inter + col] = acc[t][2];
          if (col + 1 < p.inter) {
            out_row[col + 1] = acc[t][1];
            out_row[p.inter + col + 1] = acc[t][3];
          }
        }
        continue;
      }
      bf16_t r[2];
#pragma unroll
      for (int i = 0; i < 2; ++i) {
        float gv = acc[t][i], uv = acc[t][2 + i];
        if (p.bias && col + i < p.inter) {
          gv += p.bias[col + i];
          uv += p.bias[p.inter + col + i];
        }
        r[i] = from_f32<bf16_t>(gv / (1.f + expf(-gv)) * uv);
      }
      bf16_t* out_row = reinterpret_cast<bf16_t*>(p.y) + (size_t)m * p.inter;
      if (pair) {
        *reinterpret_cast<uint32_t*>(out_row + col) = *reinterpret_cast<const uint32_t*>(r);
      } else {
        out_row[col] = r[0];
        if (col + 1 < p.inter) out_row[col + 1] = r[1];
      }
    }
    return;
  }
  const int col = col0 + 4 * g;
  const bool vec = (p.n & 3) == 0;   // col is a multiple of 4: the four columns exist together, stores are aligned
#pragma unroll
  for (int t = 0; t < MT; ++t) {
    if (16 * t + r16 >= m_rows || col >= p.n) continue;
    const int m = m_base + 16 * t + r16;
    if (p.splits > 1) {
      float* out_row = p.partial + ((size_t)split * p.m + m) * p.n;
      if (vec) {
        *reinterpret_cast<f32x4*>(out_row + col) = acc[t];
      } else {
#pragma unroll
        for (int i = 0; i < 4; ++i)
          if (col + i < p.n) out_row[col + i] = acc[t][i];
      }
      continue;
    }
    f32x4 v = acc[t];
    if (p.bias) {
#pragma unroll
      for (int i = 0; i < 4; ++i)
        if (col + i < p.n) v[i] += p.bias[col + i];
    }
    if (p.out_f32) {
      float* out_row = reinterpret_cast<float*>(p.y) + (size_t)m * p.n;
      if (vec) {
        *reinterpret_cast<f32x4*>(out_row + col) = v;
      } else {
#pragma unroll
        for (int i = 0; i < 4; ++i)
          if (col + i < p.n) out_row[col + i] = v[i];
      }
    } else {
      bf16_t* out_row = reinterpret_cast<bf16_t*>(p.y) + (size_t)m * p.n;
      bf16_t r[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) r[i] = from_f32<bf16_t>(v[i]);
      if (vec) {
        *reinterpret_cast<uint2*>(out_row + col) = *reinterpret_cast<const uint2*>(r);
      } else {
#pragma unroll
        for (int i = 0; i < 4; ++i)
          if (col + i < p.n) out_row[col + i] = r[i];
      }
    }
  }
}

// y[m, n] = sum over splits of partial[s][m][n] (+ bias), in slice order.
template <typename TY>
__global__ void splitk_reduce_kernel(const float* __restrict__ partial, const float* __restrict__ bias,
                                     TY* __restrict__ y, size_t total, int n, int splits) {
  const size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= total) return;
  float s = 0.f;
  for (int sp = 0; sp < splits; ++sp) s += partial[(size_t)sp * total + idx];
  if (bias) s += bias[idx % n];
  y[idx] = from_f32<TY>(s);
}

static int skinny_tiles(int n, int gate) { return gate ? (n + 31) / 32 : (n + kSkinnyRows - 1) / kSkinnyRows; }

// How K is cut between blocks: slices a multiple of 512.  Measured on an MI355X (256 CUs) with the Qwen3-8B
// products: narrow products (fewer row tiles than CUs) run best with about two blocks a CU, wide ones (gate/up,
// head) with four slices.
static SkinnyPlan skinny_plan(int m, int tiles, int k) {
  SkinnyPlan plan{};
  const int units = (k + 511) / 512;
  const int cus = device_cus();
  int s = tiles >= cus ? 4 : (2 * cus + tiles - 1) / tiles;
  s = max(1, min(s, min(units, 32)));
  const int per = (units + s - 1) / s;           // units of 512 per slice
  plan.kslice = per * 512;
  plan.splits = (units + per - 1) / per;
  int cap = (kSkinnyLds - 4 * kAWave - 64) / m / 2 - 8;   // k elements of one row of x that fit
  cap = max(kSkinnyChunk, cap / kSkinnyChunk * kSkinnyChunk);
  plan.xk = min(plan.kslice, cap);
  return plan;
}

// More than 16 rows.  `groups` is the number of 16-row groups of w (8 columns each for SiLU-gate).
// Blocks of 5 to 8 waves run one a CU, blocks of 4 waves two.  Very wide products (three rounds of
// blocks or more whatever the choice) take four waves and K whole: with two blocks a CU one block's
// start and end overlap another's work.  For the others the number of waves and of K slices (multiples
// of 1024) is the one with the least work on the busiest CU: rounds of a block a CU x rows x k a block,
// a little more for fewer waves (x is read once per block), for every round (a block's start and end)
// and for every slice (its partial sums are written and read again).  The choice does not depend on the number of rows of x.
struct MidPlan {
  int waves, tiles, splits, kslice;
};

static MidPlan mid_plan(int groups, int k) {
  MidPlan plan{};
  const int units = (k + kMidSlice - 1) / kMidSlice;
  const int cus = device_cus();
  if ((groups + 7) / 8 > 2 * cus) {
    plan.waves = 4;
    plan.tiles = (groups + 3) / 4;
    plan.splits = 1;
    plan.kslice = units * kMidSlice;
    return plan;
  }
  double best = 1e30;
  for (int s = 1; s <= min(units, 32); ++s) {
    const int per = (units + s - 1) / s;
    const int splits = (units + per - 1) / per;
    if (splits != s) continue;
    for (int w = 8; w >= 4; --w) {
      const long tiles = (groups + w - 1) / w;
      const long rounds = (tiles * splits + cus - 1) / cus;
      const double cost = (double)rounds * w * per * (1. + 1. / w) + 0.5 * rounds + 0.15 * splits * groups / (double)cus;
      if (cost < best - 1e-9) {
        best = cost;
        plan.waves = w;
        plan.tiles = (int)tiles;
        plan.splits = splits;
        plan.kslice = per * kMidSlice;
      }
    }
  }
  return plan;
}

// Which of the two kernels takes a product.  Measured on an MI355X with the Qwen3-8B products: the streaming
// kernel is the faster one from 9 rows on, and for SiLU-gate from the first row (it does not cut K there, so
// the gate is applied in place and no second kernel reads partial sums); with up to 8 rows the kernel that
// stages x is equal or a little faster for the plain products.
static bool takes_mid(int m, int gate) { return gate || m > 8; }
static int mid_groups(int n, int gate) { return gate ? (n + 7) / 8 : (n + 15) / 16; }

// 1 if the skinny kernel takes this product.
ATOM_EXPORT int atom_gemm_skinny_supports(int m, int n, int k) {
  if (m < 1 || n < 1 || k < 8 || k % 8) return 0;
  if (m <= 64) return 1;
  if (m > 128) return 0;
  const MidPlan plan = mid_plan(mid_groups(n, 0), k);   // the same groups with SiLU-gate: n is then twice the columns
  return plan.waves == 4 && plan.tiles * plan.splits <= device_cus();
}

// Into how many slices atom_gemm_skinny cuts K for this product (1: it writes y itself).
ATOM_EXPORT int atom_gemm_skinny_splits(int m, int n, int k, int gate) {
  if (takes_mid(m, gate)) return mid_plan(mid_groups(n, gate), k).splits;
  return skinny_plan(max(m, 1), skinny_tiles(n, gate), k).splits;
}

// gate == 0: x w^T, n columns.  gate == 1: w is [2 n, k] (n gate rows, then n up rows).
// With atom_gemm_skinny_splits(...) == 1 the result goes to y: [m, n] bfloat16 (or float32 with
// out_f32; gate: silu(x wg^T) * (x wu^T), bfloat16), bias added.  Otherwise y is not touched, bias
// is not used and partial[splits][m][columns] receives the slices' products (columns = 2 n for gate).
ATOM_EXPORT int atom_gemm_skinny(const void* x, const void* w, const float* bias, void* y, float* partial,
                                 int m, int n, int k, int out_f32, int gate, hipStream_t stream) {
  if (m < 0 || n <= 0 || k <= 0) return ATOM_BAD_SHAPE;
  if (k % 8 || !atom_gemm_skinny_supports(max(m, 1), gate ? 2 * n : n, k)) return ATOM_UNSUPPORTED;
  if (gate && out_f32) return ATOM_UNSUPPORTED;
  if (m == 0) return ATOM_OK;
  if (((uintptr_t)x | (uintptr_t)w | (uintptr_t)partial) & 15) return ATOM_BAD_SHAPE;
  SkinnyParams p{};
  p.x = (const bf16_t*)x; p.w = (const bf16_t*)w; p.bias = bias; p.y = y; p.partial = partial;
  p.m = m; p.k = k; p.out_f32 = out_f32;
  p.n = gate ? 2 * n : n;
  p.inter = gate ? n : 0;
  p.halves = m > 64 ? 2 : 1;
  p.rows_half = ((m + p.halves - 1) / p.halves + 15) / 16 * 16;
  const int mt = p.rows_half / 16;
  if (takes_mid(m, gate)) {
    if ((uintptr_t)y & 15) return ATOM_BAD_SHAPE;
    const MidPlan plan = mid_plan(mid_groups(n, gate), k);
    p.tiles = plan.tiles; p.splits = plan.splits; p.kslice = plan.kslice;
    if (p.splits > 1 ? partial == nullptr : y == nullptr) return ATOM_BAD_SHAPE;
    const long blocks = (long)p.tiles * p.splits * p.halves;
    if (blocks > 0x7fffffffL) return ATOM_TOO_LARGE;
    const size_t lds = (size_t)2 * (16 * plan.waves + 16 * mt) * kARow;
    // two chunks of LDS are more than a launch gets by default: allow it once per kernel
#define GO_MID(MTV, G, E, T)                                                                                    \
  do {                                                                                                     \
    static bool allowed = false;                                                                           \
    if (!allowed) {                                                                                        \
      if (hipFuncSetAttribute((const void*)gemm_mid_kernel<MTV, G, E, T>,                                        \
                              hipFuncAttributeMaxDynamicSharedMemorySize, 2 * (16 * 8 + 64) * kARow) !=    \
          hipSuccess)                                                                                      \
        return ATOM_LAUNCH_FAILED;                                                                         \
      allowed = true;                                                                                      \
    }                                                                                                      \
    hipLaunchKernelGGL((gemm_mid_kernel<MTV, G, E, T>), dim3(blocks), dim3(64 * plan.waves), lds, stream, p);    \
  } while (0)
#define GO_E(MTV, G, E)                  \
  do {                                   \
    if (turn) GO_MID(MTV, G, E, true);   \
    else GO_MID(MTV, G, E, false);       \
  } while (0)
#define GO(MTV)                               \
  do {                                        \
    if (gate && exact) GO_E(MTV, true, true); \
    else if (gate) GO_E(MTV, true, false);    \
    else if (exact) GO_E(MTV, false, true);   \
    else GO_E(MTV, false, false);             \
  } while (0)
    const bool turn = p.splits == 1;
    const bool exact = k % 128 == 0;   // slices are multiples of 1024
    switch (mt) {
      case 1: GO(1); break;
      case 2: GO(2); break;
      case 3: GO(3); break;
      default: GO(4); break;
    }
#undef GO
#undef GO_E
#undef GO_MID
    return launch_status();
  }
  p.tiles = skinny_tiles(n, gate);
  const SkinnyPlan plan = skinny_plan(m, p.tiles, k);
  p.splits = plan.splits; p.kslice = plan.kslice; p.xk = plan.xk;
  if (p.splits > 1 ? partial == nullptr : y == nullptr) return ATOM_BAD_SHAPE;
  const long blocks = (long)p.tiles * p.splits;
  if (blocks > 0x7fffffffL) return ATOM_TOO_LARGE;
  const size_t lds = (size_t)4 * kAWave + max((size_t)m * (p.xk * 2 + 16), (size_t)m * (kSkinnyRows + 1) * 4);
  // a long slice of x needs more LDS than a launch gets by default: allow it once per kernel
#define GO_ONE(MTV, G)                                                                                   \
  do {                                                                                                   \
    static bool allowed = false;                                                                         \
    if (!allowed) {                                                                                      \
      if (hipFuncSetAttribute((const void*)gemm_skinny_kernel<MTV, G>,                                   \
                              hipFuncAttributeMaxDynamicSharedMemorySize, 96 * 1024) != hipSuccess)      \
        return ATOM_LAUNCH_FAILED;                                                                       \
      allowed = true;                                                                                    \
    }                                                                                                    \
    hipLaunchKernelGGL((gemm_skinny_kernel<MTV, G>), dim3(blocks), dim3(256), lds, stream, p);           \
  } while (0)
#define GO(MTV)                      \
  do {                               \
    if (gate) GO_ONE(MTV, true);     \
    else GO_ONE(MTV, false);         \
  } while (0)
  GO(1);
#undef GO
#undef GO_ONE
  return launch_status();
}

// y[m, n] = sum of partial[s][m][n] over s (+ bias): for readers that cannot add the slices themselves.
ATOM_EXPORT int atom_splitk_reduce(const float* partial, const float* bias, void* y, int m, int n, int splits,
                                   int out_f32, hipStream_t stream) {
  if (m < 0 || n <= 0 || splits < 1) return ATOM_BAD_SHAPE;
  const size_t total = (size_t)m * n;
  if (total == 0) return ATOM_OK;
  const size_t blocks = (total + 255) / 256;
  if (blocks > 0x7fffffffu) return ATOM_TOO_LARGE;
  if (out_f32) hipLaunchKernelGGL(splitk_reduce_kernel<float>, dim3((unsigned)blocks), dim3(256), 0, stream, partial,
                                  bias, (float*)y, total, n, splits);
  else hipLaunchKernelGGL(splitk_reduce_kernel<bf16_t>, dim3((unsigned)blocks), dim3(256), 0, stream, partial, bias,
                          (bf16_t*)y, total, n, splits);
  return launch_status();
}

// ------------------------------------------------------------------ the product that allocates nothing
//
// The slices between the product and the reduction live in this array, one copy on every GPU.  In host
// code its name is only a handle: the address that kernels and copies take is the one that
// hipGetSymbolAddress returns on the device in question, kept per device in static_slices[].
static __device__ __align__(256) float scratch[kLinearStaticFloats];

constexpr int kStaticMaxDevices = 64;
static float* static_slices[kStaticMaxDevices];   // device address of `scratch` on each device, once known
static std::mutex static_slices_lock;

// The current device's copy of the array, or null with `status` set.
static float* static_slices_here(int* status) {
  int device = -1;
  if (hipGetDevice(&device) != hipSuccess || device < 0 || device >= kStaticMaxDevices) {
    *status = ATOM_LAUNCH_FAILED;
    return nullptr;
  }
  std::lock_guard<std::mutex> hold(static_slices_lock);
  if (!static_slices[device]) {
    float* ptr = nullptr;
    if (hipGetSymbolAddress((void**)&ptr, HIP_SYMBOL(scratch)) != hipSuccess || !ptr) {
      (void)hipGetLastError();
      *status = ATOM_LAUNCH_FAILED;
      return nullptr;
    }
    static_slices[device] = ptr;
  }
  *status = ATOM_OK;
  return static_slices[device];
}

ATOM_EXPORT int atom_linear_skinny_static_init(void) {
  int status = ATOM_OK;
  static_slices_here(&status);
  return status;
}

ATOM_EXPORT long atom_linear_skinny_static_limit(void) { return kLinearStaticFloats; }

ATOM_EXPORT int atom_linear_skinny_static(const void* x, const void* w, const float* bias, void* y, int m, int n,
                                          int k, int out_f32, hipStream_t stream) {
  if (m < 0 || n <= 0 || k <= 0 || !x || !w || !y) return ATOM_BAD_SHAPE;
  if (k % 8 || !atom_gemm_skinny_supports(max(m, 1), n, k)) return ATOM_UNSUPPORTED;
  if (m == 0) return ATOM_OK;
  const int splits = atom_gemm_skinny_splits(m, n, k, 0);
  if (splits == 1) return atom_gemm_skinny(x, w, bias, y, nullptr, m, n, k, out_f32, 0, stream);
  if ((long)splits * m * n > kLinearStaticFloats) return ATOM_TOO_LARGE;
  int status = ATOM_OK;
  float* slices = static_slices_here(&status);
  if (!slices) return status;
  status = atom_gemm_skinny(x, w, nullptr, nullptr, slices, m, n, k, 0, 0, stream);
  if (status != ATOM_OK) return status;
  return atom_splitk_reduce(slices, bias, y, m, n, splits, out_f32, stream);
}
