// Paged attention on the matrix cores (bfloat16 in, float32 accumulate), gfx950.
//
// One wave is one work item; it owns up to 16 * RT query rows and walks its keys 16 at a
// time.  Both products are formed transposed so that a lane always holds values of ONE
// query row (row = lane % 16):
//
//     S^T[key][row] = K[key][:] . Q[row][:]        A = K rows (from the key pages),  B = Q
//     O^T[d][row]   = V^T[d][key] . P[row][key]    A = V^T rows (value pages are stored
//                                                  transposed, keys contiguous),     B = P
//
// The first product leaves lane (row, g = lane / 16) with the scores of keys 4g..4g+3 of
// the block, which is exactly the B operand of the second, so probabilities never move
// between lanes, and the running maximum, sum and rescale factor of a row are per-lane
// scalars (the maximum needs two cross-lane exchanges over g).  Softmax is float32, in
// the exp2 domain.
//
// Two modes:
//   decode   a request's single new token: rows are the query heads that share a KV head;
//            the visible keys are split over `parts` waves whose partial results (running
//            maximum, sum, unnormalised output) a second kernel merges.
//   prefill  a tile of consecutive query tokens of one head; causal by absolute position
//            (a portion of a prompt sees the cached keys before it), optional window.
//
// Pages: keys [num_pages, Hkv, page_size, D]; values [num_pages, Hkv, D, page_size];
// page_size a multiple of 4.
#include "common.h"

typedef __attribute__((ext_vector_type(4))) float f32x4;
typedef __attribute__((ext_vector_type(4))) short s16x4;
typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) __bf16 bf16x4;

struct AttnParams {
  const bf16_t* q;        // [tokens, Hq, D]
  const bf16_t* k_cache;
  const bf16_t* v_cache;
  bf16_t* out;            // [tokens, Hq, D]
  const int* cu_q;        // [num_seqs + 1]
  const int* ctx_lens;    // [num_seqs]
  const int* block_tables;  // [num_seqs, max_blocks]
  const int* tiles;       // prefill: [num_tiles, 2] = (request, first row of the tile within its tokens)
  float* ws_o;            // decode: [seqs, Hq, parts, D]
  float* ws_ml;           // decode: [seqs, Hq, parts, 2]
  int max_blocks, hq, hkv, page_size, window, seq_offset, parts, num_tiles;
  int page_shift;         // log2(page_size) where that is a power of two, else -1
  float scale_log2;       // softmax scale * log2(e)
  // decode with the step before attention folded in: q is not read; the float32 QKV product is
  const float* qkv;       // [tokens, (Hq + 2 Hkv) * D], rows q | k | v
  const float* q_weight;  // per-head RMS norm weights [D], or null for no norm
  const float* k_weight;
  const float* cos_table; // [max_pos, D / 2]: the whole head is rotated
  const float* sin_table;
  const int* slots;       // [tokens] cache slot of each token's key and value (-1: none)
  float eps;
  int write_kv;           // 0: the keys and values are another layer's, already written
};

__device__ __forceinline__ s16x4 as_s16x4(bf16x4 v) { return __builtin_bit_cast(s16x4, v); }

// The keys of one part of a decode row: the row's visible keys are cut into steps of ``step`` keys (what a wave
// takes per trip) and the steps are dealt out evenly, the first (steps % parts) parts taking one more.  No part is
// empty unless there are fewer steps than parts, and no two parts differ by more than one step, whatever the
// context length: a rule of "ceil(len / parts) rounded up to whole steps" leaves a third of the parts without
// keys when a part's share is just over two steps.
struct PartKeys {
  int begin, end;   // relative to the first visible key; end may lie past the last key
};
__device__ inline PartKeys part_keys(int len, int parts, int part, int step) {
  const int steps = (len + step - 1) / step;
  const int each = steps / parts, more = steps - each * parts;
  const int first = part * each + min(part, more);
  return PartKeys{first * step, (first + each + (part < more ? 1 : 0)) * step};
}

// Where a key lies: its page's place in the block table and its place in the page.  A power-of-two
// page size (the usual case) makes these a shift and a mask instead of a division per load.
// The choice is made once per group of loads (POW2 is a compile-time constant), never per load: a branch
// between a table look-up and the load that depends on it keeps the loads of a group from being in flight together.
template <bool POW2>
struct PageMath {
  int size, shift;
  __device__ __forceinline__ int index(int key) const { return POW2 ? key >> shift : key / size; }
  __device__ __forceinline__ int within(int key) const { return POW2 ? key & (size - 1) : key % size; }
};
struct Pow2Pages { static constexpr bool value = true; };
struct AnyPages { static constexpr bool value = false; };

// 2^x for x <= 0 (and -inf): the bare instruction.  Results below the smallest normal number become 0,
// which a probability may.
__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }

template <int D, int RT, bool DECODE>
__global__ void __launch_bounds__(kWave) attention_mfma_kernel(AttnParams p) {
  constexpr bool KX32 = (D % 32 == 0);
  constexpr int KCH = KX32 ? D / 32 : D / 16;  // K/Q register chunks
  constexpr int DT = D / 16;                   // output tiles along d
  const int lane = threadIdx.x;
  const int r16 = lane & 15;
  const int g = lane >> 4;
  const int group = p.hq / p.hkv;

  int seq, kvh, head0, nrows, tok0, pos0, part = 0;
  int ctx;
  if (DECODE) {
    seq = blockIdx.z + p.seq_offset;
    kvh = blockIdx.y;
    part = blockIdx.x;
    ctx = p.ctx_lens[seq];
    head0 = kvh * group;
    nrows = group;            // rows are heads head0 .. head0 + group - 1 of one token
    tok0 = p.cu_q[seq];
    pos0 = ctx - 1;
  } else {
    const int tile = blockIdx.x;
    seq = p.tiles[2 * tile];
    if (seq < 0) return;   // an unused entry of a list of fixed length
    const int row_start = p.tiles[2 * tile + 1];
    head0 = blockIdx.y;
    kvh = head0 / group;
    ctx = p.ctx_lens[seq];
    const int q_begin = p.cu_q[seq];
    const int q_len = p.cu_q[seq + 1] - q_begin;
    nrows = min(16 * RT, q_len - row_start);
    tok0 = q_begin + row_start;
    pos0 = ctx - q_len + row_start;   // absolute position of the tile's first row
  }
  const int* table = p.block_tables + (size_t)seq * p.max_blocks;
  const int ps = p.page_size;

  // ---- key range of this work item
  int kb, ke;
  if (DECODE) {
    int vis = 0;
    if (p.window > 0 && ctx - p.window > 0) vis = (ctx - p.window) & ~15;
    const PartKeys mine = part_keys(ctx - vis, p.parts, part, 16);
    kb = vis + mine.begin;
    ke = min(ctx, vis + mine.end);
  } else {
    kb = 0;
    if (p.window > 0 && pos0 - p.window + 1 > 0) kb = (pos0 - p.window + 1) & ~15;
    ke = pos0 + nrows;   // one past the last row's own position
  }

  // ---- per-lane row data
  int row_pos[RT];
  bool row_ok[RT];
  bf16x8 q32[RT][KX32 ? KCH : 1];
  s16x4 q16[RT][KX32 ? 1 : KCH];
#pragma unroll
  for (int rt = 0; rt < RT; ++rt) {
    const int row = rt * 16 + r16;
    row_ok[rt] = row < nrows;
    const bf16_t* qr;
    if (DECODE) {
      row_pos[rt] = pos0;
      qr = p.q + ((size_t)tok0 * p.hq + head0 + row) * D;
    } else {
      row_pos[rt] = pos0 + row;
      qr = p.q + ((size_t)(tok0 + row) * p.hq + head0) * D;
    }
    if (KX32) {
#pragma unroll
      for (int j = 0; j < KCH; ++j) {
        bf16x8 v = {0, 0, 0, 0, 0, 0, 0, 0};
        if (row_ok[rt]) v = *reinterpret_cast<const bf16x8*>(qr + 32 * j + 8 * g);
        q32[rt][j] = v;
      }
    } else {
#pragma unroll
      for (int j = 0; j < KCH; ++j) {
        s16x4 v = {0, 0, 0, 0};
        if (row_ok[rt]) v = *reinterpret_cast<const s16x4*>(qr + 16 * j + 4 * g);
        q16[rt][j] = v;
      }
    }
  }

  f32x4 acc[RT][DT];
  float run_max[RT], run_sum[RT];
#pragma unroll
  for (int rt = 0; rt < RT; ++rt) {
    run_max[rt] = -INFINITY;
    run_sum[rt] = 0.f;
#pragma unroll
    for (int t = 0; t < DT; ++t) acc[rt][t] = f32x4{0.f, 0.f, 0.f, 0.f};
  }

  // One block of 16 keys in registers: the K rows as the first product's A operand, the V^T rows
  // as the second's.  The block after the one being multiplied is loaded ahead of it.
  struct KVBlock {
    bf16x8 k32[KX32 ? KCH : 1];
    s16x4 k16[KX32 ? 1 : KCH];
    s16x4 v[DT];
  };
  // Head sizes whose key rows are a whole number of 16-byte pieces per wave load (32, 64, 128, 256) are
  // read in whole cache lines: piece q = 64 j + lane of the block is 8 elements of key q / (D / 8), and the
  // block then goes through a small LDS area of the wave to reach the operand layout.
  constexpr bool KROWS = KX32 && (D == 32 || D == 64 || D == 128 || D == 256);
  constexpr int KLDS = D * 2 + 16;   // LDS bytes of a key row: rows start 4 banks apart
  __shared__ __attribute__((aligned(16))) char klds[KROWS ? 16 * KLDS : 16];
  auto load_block = [&](int k0, KVBlock& blk) {
    // this lane's key row is k0 + r16 (clamped into the context for addressing)
    const int krow = min(k0 + r16, ke - 1);
    const int kpage = table[krow / ps];
    const bf16_t* kptr = p.k_cache + (((size_t)kpage * p.hkv + kvh) * ps + (krow % ps)) * D;
    if (KROWS) {
#pragma unroll
      for (int j = 0; j < KCH; ++j) {
        const int q = 64 * j + lane;
        const int row = min(k0 + q / (D / 8), ke - 1);
        const int page = table[row / ps];
        blk.k32[j] = __builtin_nontemporal_load(reinterpret_cast<const bf16x8*>(
            p.k_cache + (((size_t)page * p.hkv + kvh) * ps + (row % ps)) * D + (q % (D / 8)) * 8));
      }
    }
    // this lane's V keys are k0 + 4g .. + 3, of output rows d = 16 t + r16
    const int vkey = min(k0 + 4 * g, ((ke - 1) & ~3));
    const int vpage = table[vkey / ps];
    const bf16_t* vptr = p.v_cache + (((size_t)vpage * p.hkv + kvh) * D + r16) * (size_t)ps + (vkey % ps);
    if (KROWS) {
    } else if (KX32) {
#pragma unroll
      for (int j = 0; j < KCH; ++j) blk.k32[j] = *reinterpret_cast<const bf16x8*>(kptr + 32 * j + 8 * g);
    } else {
#pragma unroll
      for (int j = 0; j < KCH; ++j) blk.k16[j] = *reinterpret_cast<const s16x4*>(kptr + 16 * j + 4 * g);
    }
#pragma unroll
    for (int t = 0; t < DT; ++t) blk.v[t] = *reinterpret_cast<const s16x4*>(vptr + (size_t)(16 * t) * ps);
  };

  KVBlock cur, nxt;
  if (kb < ke) load_block(kb, cur);
  for (int k0 = kb; k0 < ke; k0 += 16) {
    if (k0 + 16 < ke) load_block(k0 + 16, nxt);
    f32x4 s[RT];
#pragma unroll
    for (int rt = 0; rt < RT; ++rt) s[rt] = f32x4{0.f, 0.f, 0.f, 0.f};
    if (KROWS) {
#pragma unroll
      for (int j = 0; j < KCH; ++j) {
        const int q = 64 * j + lane;
        *reinterpret_cast<bf16x8*>(klds + (q / (D / 8)) * KLDS + (q % (D / 8)) * 16) = cur.k32[j];
      }
      __builtin_amdgcn_s_waitcnt(0xc07f);   // lgkmcnt(0); the block is one wave
      __builtin_amdgcn_wave_barrier();
#pragma unroll
      for (int j = 0; j < KCH; ++j) {
        const bf16x8 a = *reinterpret_cast<const bf16x8*>(klds + r16 * KLDS + 64 * j + 16 * g);
#pragma unroll
        for (int rt = 0; rt < RT; ++rt) s[rt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, q32[rt][j], s[rt], 0, 0, 0);
      }
      __builtin_amdgcn_s_waitcnt(0xc07f);
      __builtin_amdgcn_wave_barrier();
    } else if (KX32) {
#pragma unroll
      for (int j = 0; j < KCH; ++j)
#pragma unroll
        for (int rt = 0; rt < RT; ++rt)
          s[rt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(cur.k32[j], q32[rt][j], s[rt], 0, 0, 0);
    } else {
#pragma unroll
      for (int j = 0; j < KCH; ++j)
#pragma unroll
        for (int rt = 0; rt < RT; ++rt)
          s[rt] = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(cur.k16[j], q16[rt][j], s[rt], 0, 0, 0);
    }
    s16x4 vreg[DT];
#pragma unroll
    for (int t = 0; t < DT; ++t) vreg[t] = cur.v[t];

    // ---- softmax update per row tile; lane holds keys k0 + 4g + i of row r16.  The maximum is taken over
    //      the raw scores and the scale goes into the exponent's multiply-add; a block of keys that every
    //      row sees whole (all but the last of a decode row's) is not masked.
    const int first_pos = pos0;                                 // the smallest position among the rows
    const int last_pos = DECODE ? pos0 : pos0 + nrows - 1;
    const bool whole = k0 + 15 <= min(first_pos, ke - 1) && (p.window <= 0 || k0 >= last_pos - p.window + 1);
#pragma unroll
    for (int rt = 0; rt < RT; ++rt) {
      float sc[4];
      float mx = -INFINITY;
      if (whole) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          sc[i] = s[rt][i];
          mx = fmaxf(mx, sc[i]);
        }
      } else {
        const int hi = min(row_pos[rt], ke - 1);                        // last visible key
        const int lo = p.window > 0 ? row_pos[rt] - p.window + 1 : 0;   // first visible key
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const int key = k0 + 4 * g + i;
          const bool vis = key <= hi && key >= lo && key >= kb;
          sc[i] = vis ? s[rt][i] : -INFINITY;
          mx = fmaxf(mx, sc[i]);
        }
      }
      mx = rows_max(mx);
      const float new_max = fmaxf(run_max[rt], mx * p.scale_log2);
      const float base = new_max == -INFINITY ? 0.f : new_max;
      const float alpha = fast_exp2(run_max[rt] - base);   // 0 while nothing was seen yet
      float psum = 0.f;
      bf16x4 pb;
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const float pv = fast_exp2(fmaf(sc[i], p.scale_log2, -base));
        psum += pv;
        pb[i] = static_cast<bf16_t>(pv);
      }
      run_sum[rt] = run_sum[rt] * alpha + psum;
      run_max[rt] = new_max;
      const s16x4 pbits = as_s16x4(pb);
#pragma unroll
      for (int t = 0; t < DT; ++t) {
        f32x4 a = acc[rt][t];
        a[0] *= alpha; a[1] *= alpha; a[2] *= alpha; a[3] *= alpha;
        acc[rt][t] = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(vreg[t], pbits, a, 0, 0, 0);
      }
    }
    cur = nxt;
  }

  // ---- write: lane holds O[row r16][d = 16 t + 4 g + i]
#pragma unroll
  for (int rt = 0; rt < RT; ++rt) {
    float total = run_sum[rt];
    total = rows_sum(total);
    if (!row_ok[rt]) continue;
    const int row = rt * 16 + r16;
    if (DECODE && p.parts > 1) {
      const size_t slot = ((size_t)(blockIdx.z * p.hq + head0 + row)) * p.parts + part;
      float* wo = p.ws_o + slot * D;
#pragma unroll
      for (int t = 0; t < DT; ++t) *reinterpret_cast<f32x4*>(wo + 16 * t + 4 * g) = acc[rt][t];
      if (g == 0) {
        p.ws_ml[slot * 2] = run_max[rt];
        p.ws_ml[slot * 2 + 1] = total;
      }
    } else {
      bf16_t* dst = DECODE ? p.out + ((size_t)tok0 * p.hq + head0 + row) * D
                           : p.out + ((size_t)(tok0 + row) * p.hq + head0) * D;
      const float inv = total > 0.f ? 1.f / total : 0.f;
#pragma unroll
      for (int t = 0; t < DT; ++t) {
        bf16x4 o;
#pragma unroll
        for (int i = 0; i < 4; ++i) o[i] = static_cast<bf16_t>(acc[rt][t][i] * inv);
        *reinterpret_cast<bf16x4*>(dst + 16 * t + 4 * g) = o;
      }
    }
  }
}

// Decode for head sizes 32, 64, 128 and 256 with pages of a multiple of 8 keys: the same work items and the
// same two products as above, 32 keys a step, with every load a whole-line, 16-bytes-a-lane, non-temporal
// one.  Key rows reach the first product's A operand through the wave's LDS area as above, but row r of
// the two operand tiles b = 0, 1 is key 8 (r / 4) + 4 b + r % 4 of the step: lane (row, g) is then left
// with the scores of keys 8 g .. 8 g + 7, which is the k order of one v_mfma_f32_16x16x32_bf16 step of the
// second product, and its V^T operand (8 consecutive keys of one d) is one 16-byte load from the value page.
//
// TOGETHER: the parts of a (request, KV head) are the waves of one block (at most 8: two waves a SIMD is what
// the registers allow), which merges their results through LDS and writes the output itself; no second kernel
// and no partial results in memory.  Otherwise a block is one wave and the merge kernel follows.
//
// FUSED: the kernel starts from the float32 QKV product of the step instead of from finished queries.  Every wave
// norms and rotates its query rows itself (a lane's elements of a row and their rotation partners, half a head
// on, are the same lane's, so this costs two exchanges for the sum of squares).  The wave whose keys end with
// the new token (the last part) also norms and rotates that token's key, writes key and value to their page,
// and puts them where the step's loads of that key and value have arrived, in LDS and in registers: the
// loaded ones are whatever the page held before.  No other wave of the grid reads that key.
template <int D, int RT, bool TOGETHER, bool FUSED>
__global__ void __launch_bounds__(TOGETHER ? 8 * kWave : kWave, (D <= 128 ? 2 : 1)) attention_decode32_kernel(AttnParams p) {
  constexpr int KCH = D / 32;      // k steps of the first product
  constexpr int DT = D / 16;       // output tiles along d
  constexpr int KP = D * 32 / 8 / kWave;   // 16-byte pieces of a step's 32 key rows per lane
  constexpr int KLDS = D * 2 + 16;
  constexpr int AREA = 32 * KLDS;  // LDS bytes of a wave: the key rows of a step, later its result
  extern __shared__ __attribute__((aligned(16))) char decode_lds[];
  const int lane = threadIdx.x & (kWave - 1);
  const int wave = threadIdx.x / kWave;
  char* klds = decode_lds + wave * AREA;
  const int r16 = lane & 15;
  const int g = lane >> 4;
  const int group = p.hq / p.hkv;
  const int seq = blockIdx.z + p.seq_offset;
  const int kvh = blockIdx.y;
  const int part = TOGETHER ? wave : blockIdx.x;
  const int ctx = p.ctx_lens[seq];
  const int head0 = kvh * group;
  const int tok0 = p.cu_q[seq];
  const int pos0 = ctx - 1;
  const int* table = p.block_tables + (size_t)seq * p.max_blocks;
  const int ps = p.page_size;

  int vis0 = 0;
  if (p.window > 0 && ctx - p.window > 0) vis0 = (ctx - p.window) & ~31;
  const PartKeys mine = part_keys(ctx - vis0, p.parts, part, 32);
  const int kb = vis0 + mine.begin;
  const int ke = min(ctx, vis0 + mine.end);

  f32x4 acc[RT][DT];
  float run_max[RT], run_sum[RT];
#pragma unroll
  for (int rt = 0; rt < RT; ++rt) {
    run_max[rt] = -INFINITY;
    run_sum[rt] = 0.f;
#pragma unroll
    for (int t = 0; t < DT; ++t) acc[rt][t] = f32x4{0.f, 0.f, 0.f, 0.f};
  }

  struct Step {
    bf16x8 k[KP];
    bf16x8 v[DT];
  };
  const size_t page_elems = (size_t)p.hkv * ps * D;        // elements of a page, all heads
  const int k_head = kvh * ps * D, v_head = kvh * D * ps;
  auto load_step_as = [&](int k0, Step& st, auto kind) {
    const PageMath<decltype(kind)::value> pages{ps, p.page_shift};
#pragma unroll
    for (int j = 0; j < KP; ++j) {
      const int q = kWave * j + lane;                        // piece q: key q / (D / 8), elements (q % (D / 8)) * 8 ..
      const int row = min(k0 + q / (D / 8), ke - 1);
      const int page = table[pages.index(row)];
      st.k[j] = __builtin_nontemporal_load(reinterpret_cast<const bf16x8*>(
          p.k_cache + page * page_elems + (k_head + pages.within(row) * D + (q % (D / 8)) * 8)));
    }
    // this lane's keys of V^T are k0 + 8 g .. + 7 (one page: pages hold a multiple of 8 keys), rows d = 16 t + r16
    const int vkey = min(k0 + 8 * g, (ke - 1) & ~7);
    const int vpage = table[pages.index(vkey)];
    const bf16_t* vptr = p.v_cache + vpage * page_elems + (v_head + r16 * ps + pages.within(vkey));
#pragma unroll
    for (int t = 0; t < DT; ++t)
      st.v[t] = __builtin_nontemporal_load(reinterpret_cast<const bf16x8*>(vptr + (size_t)(16 * t) * ps));
  };
  auto load_step = [&](int k0, Step& st) {
    if (p.page_shift >= 0) load_step_as(k0, st, Pow2Pages{});
    else load_step_as(k0, st, AnyPages{});
  };

  Step cur, nxt;
  if (kb < ke) load_step(kb, cur);
  // (the first step's keys and values are on their way while the queries are made ready)
  bool row_ok[RT];
  bf16x8 q32[RT][KCH];
  // the new token's key and value for the wave that owns them (FUSED): element i of the key at knew[i]
  __shared__ __attribute__((aligned(16))) bf16_t knew_all[FUSED ? (TOGETHER ? 8 : 1) * 2 * D : 8];
  bf16_t* knew = knew_all + (FUSED ? wave * 2 * D : 0);
  bf16_t* vnew = knew + (FUSED ? D : 0);
  const bool owns_new = FUSED && p.write_kv && kb <= pos0 && pos0 < ke;   // the same in all lanes
  if constexpr (FUSED) {
    static_assert(!FUSED || KCH % 2 == 0, "a lane must hold both halves of a rotation pair");
    const size_t row_width = (size_t)(p.hq + 2 * p.hkv) * D;
    const float* base = p.qkv + (size_t)tok0 * row_width;
    const int pos = max(pos0, 0);
    const float* cs = p.cos_table + (size_t)pos * (D / 2);
    const float* sn = p.sin_table + (size_t)pos * (D / 2);
#pragma unroll
    for (int rt = 0; rt < RT; ++rt) {
      const int row = rt * 16 + r16;
      row_ok[rt] = row < group;
      const float* qr = base + (size_t)(head0 + (row_ok[rt] ? row : 0)) * D;
      float x[KCH][8];
      float ss = 0.f;
#pragma unroll
      for (int j = 0; j < KCH; ++j) {
        const f32x4 lo = *reinterpret_cast<const f32x4*>(qr + 32 * j + 8 * g);
        const f32x4 hi = *reinterpret_cast<const f32x4*>(qr + 32 * j + 8 * g + 4);
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          x[j][e] = lo[e];
          x[j][4 + e] = hi[e];
        }
#pragma unroll
        for (int e = 0; e < 8; ++e) ss += x[j][e] * x[j][e];
      }
      if (p.q_weight) {
        ss = rows_sum(ss);
        const float inv = rsqrtf(ss / (float)D + p.eps);
#pragma unroll
        for (int j = 0; j < KCH; ++j)
#pragma unroll
          for (int e = 0; e < 8; ++e) x[j][e] = x[j][e] * inv * p.q_weight[32 * j + 8 * g + e];
      }
#pragma unroll
      for (int j = 0; j < KCH / 2; ++j) {
        bf16x8 first, second;
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          const float c = cs[32 * j + 8 * g + e], sv = sn[32 * j + 8 * g + e];
          const float x1 = x[j][e], x2 = x[j + KCH / 2][e];
          first[e] = static_cast<bf16_t>(row_ok[rt] ? x1 * c - x2 * sv : 0.f);
          second[e] = static_cast<bf16_t>(row_ok[rt] ? x2 * c + x1 * sv : 0.f);
        }
        q32[rt][j] = first;
        q32[rt][j + KCH / 2] = second;
      }
    }
    if (owns_new) {
      // the new key: normed, rotated, to its page and to LDS; the new value: to its page and to LDS
      const float* kr = base + (size_t)(p.hq + kvh) * D;
      const float* vr = base + (size_t)(p.hq + p.hkv + kvh) * D;
      float ss = 0.f;
      for (int i = lane; i < D; i += kWave) ss += kr[i] * kr[i];
      float inv = 1.f;
      if (p.k_weight) inv = rsqrtf(wave_sum(ss) / (float)D + p.eps);
      const int slot = p.slots[tok0];
      const int page = slot / ps, off = slot - page * ps;
      bf16_t* kdst = const_cast<bf16_t*>(p.k_cache) + (((size_t)page * p.hkv + kvh) * ps + off) * (size_t)D;
      bf16_t* vdst = const_cast<bf16_t*>(p.v_cache) + ((size_t)page * p.hkv + kvh) * (size_t)D * ps + off;
      for (int i = lane; i < D / 2; i += kWave) {
        float x1 = kr[i], x2 = kr[i + D / 2];
        if (p.k_weight) {
          x1 = x1 * inv * p.k_weight[i];
          x2 = x2 * inv * p.k_weight[i + D / 2];
        }
        const float c = cs[i], sv = sn[i];
        const bf16_t y1 = static_cast<bf16_t>(x1 * c - x2 * sv), y2 = static_cast<bf16_t>(x2 * c + x1 * sv);
        knew[i] = y1;
        knew[i + D / 2] = y2;
        if (slot >= 0) {
          kdst[i] = y1;
          kdst[i + D / 2] = y2;
        }
      }
      for (int i = lane; i < D; i += kWave) {
        const bf16_t v = static_cast<bf16_t>(vr[i]);
        vnew[i] = v;
        if (slot >= 0) vdst[(size_t)i * ps] = v;
      }
      __builtin_amdgcn_s_waitcnt(0xc07f);
      __builtin_amdgcn_wave_barrier();
    }
  } else {
#pragma unroll
    for (int rt = 0; rt < RT; ++rt) {
      const int row = rt * 16 + r16;
      row_ok[rt] = row < group;
      const bf16_t* qr = p.q + ((size_t)tok0 * p.hq + head0 + row) * D;
#pragma unroll
      for (int j = 0; j < KCH; ++j) {
        bf16x8 v = {0, 0, 0, 0, 0, 0, 0, 0};
        if (row_ok[rt]) v = *reinterpret_cast<const bf16x8*>(qr + 32 * j + 8 * g);
        q32[rt][j] = v;
      }
    }
  }
  for (int k0 = kb; k0 < ke; k0 += 32) {
    if (k0 + 32 < ke) load_step(k0 + 32, nxt);
#pragma unroll
    for (int j = 0; j < KP; ++j) {
      const int q = kWave * j + lane;
      *reinterpret_cast<bf16x8*>(klds + (q / (D / 8)) * KLDS + (q % (D / 8)) * 16) = cur.k[j];
    }
    if (FUSED && owns_new && pos0 < k0 + 32) {
      // this step's loads of the new token's key and value brought what the page held before: put the new ones there
      const int at = pos0 - k0;                       // its place among the step's 32 keys
      if (lane < D / 8)
        *reinterpret_cast<bf16x8*>(klds + at * KLDS + lane * 16) = *reinterpret_cast<const bf16x8*>(knew + 8 * lane);
      if (at >> 3 == g) {
#pragma unroll
        for (int t = 0; t < DT; ++t) {
          const bf16_t v = vnew[16 * t + r16];
#pragma unroll
          for (int e = 0; e < 8; ++e)
            if (e == (at & 7)) cur.v[t][e] = v;
        }
      }
    }
    __builtin_amdgcn_s_waitcnt(0xc07f);   // lgkmcnt(0); the block is one wave
    __builtin_amdgcn_wave_barrier();
    f32x4 s[RT][2];
#pragma unroll
    for (int rt = 0; rt < RT; ++rt) s[rt][0] = s[rt][1] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int b = 0; b < 2; ++b) {
      const char* krow = klds + (8 * (r16 / 4) + 4 * b + (r16 % 4)) * KLDS + 16 * g;
#pragma unroll
      for (int j = 0; j < KCH; ++j) {
        const bf16x8 a = *reinterpret_cast<const bf16x8*>(krow + 64 * j);
#pragma unroll
        for (int rt = 0; rt < RT; ++rt) s[rt][b] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, q32[rt][j], s[rt][b], 0, 0, 0);
      }
    }
    __builtin_amdgcn_s_waitcnt(0xc07f);
    __builtin_amdgcn_wave_barrier();

    // ---- softmax update; lane holds keys k0 + 8 g + 4 b + i of row r16
    const bool whole = k0 + 31 <= ke - 1 && (p.window <= 0 || k0 >= pos0 - p.window + 1);
#pragma unroll
    for (int rt = 0; rt < RT; ++rt) {
      float sc[8];
      float mx = -INFINITY;
      if (whole) {
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          sc[e] = s[rt][e / 4][e % 4];
          mx = fmaxf(mx, sc[e]);
        }
      } else {
        const int lo = p.window > 0 ? pos0 - p.window + 1 : 0;
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          const int key = k0 + 8 * g + e;
          const bool vis = key < ke && key >= lo;
          sc[e] = vis ? s[rt][e / 4][e % 4] : -INFINITY;
          mx = fmaxf(mx, sc[e]);
        }
      }
      mx = rows_max(mx);
      const float new_max = fmaxf(run_max[rt], mx * p.scale_log2);
      const float base = new_max == -INFINITY ? 0.f : new_max;
      const float alpha = fast_exp2(run_max[rt] - base);
      float psum = 0.f;
      bf16x8 pb;
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        const float pv = fast_exp2(fmaf(sc[e], p.scale_log2, -base));
        psum += pv;
        pb[e] = static_cast<bf16_t>(pv);
      }
      run_sum[rt] = run_sum[rt] * alpha + psum;
      run_max[rt] = new_max;
#pragma unroll
      for (int t = 0; t < DT; ++t) {
        f32x4 a = acc[rt][t];
        a[0] *= alpha; a[1] *= alpha; a[2] *= alpha; a[3] *= alpha;
        acc[rt][t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(cur.v[t], pb, a, 0, 0, 0);
      }
    }
    cur = nxt;
  }

  if constexpr (TOGETHER) {
    // ---- every wave leaves its rows' (unnormalised output, maximum, sum) in its LDS area; then all threads
    //      share the elements of the output: parts are added in part order
    constexpr int ROWS = 16 * RT;
    float* mine = reinterpret_cast<float*>(klds);          // [ROWS][D] then [ROWS] maxima then [ROWS] sums
    static_assert(!TOGETHER || (ROWS * D + 2 * ROWS) * 4 <= AREA, "a wave's result must fit where its key rows were");
#pragma unroll
    for (int rt = 0; rt < RT; ++rt) {
      float total = run_sum[rt];
      total = rows_sum(total);
      const int row = rt * 16 + r16;
#pragma unroll
      for (int t = 0; t < DT; ++t) *reinterpret_cast<f32x4*>(mine + row * D + 16 * t + 4 * g) = acc[rt][t];
      if (g == 0) {
        mine[ROWS * D + row] = run_max[rt];
        mine[ROWS * D + ROWS + row] = total;
      }
    }
    __syncthreads();
    const int parts = p.parts;
    for (int item = threadIdx.x; item < group * D; item += blockDim.x) {
      const int row = item / D, dd = item - row * D;
      float top = -INFINITY;
      for (int k = 0; k < parts; ++k)
        top = fmaxf(top, reinterpret_cast<const float*>(decode_lds + k * AREA)[ROWS * D + row]);
      float num = 0.f, den = 0.f;
      for (int k = 0; k < parts; ++k) {
        const float* theirs = reinterpret_cast<const float*>(decode_lds + k * AREA);
        const float m = theirs[ROWS * D + row];
        const float w = m == -INFINITY ? 0.f : fast_exp2(m - top);
        den += w * theirs[ROWS * D + ROWS + row];
        num += w * theirs[row * D + dd];
      }
      p.out[((size_t)tok0 * p.hq + head0 + row) * D + dd] = static_cast<bf16_t>(den > 0.f ? num / den : 0.f);
    }
    return;
  }

  // ---- write: lane holds O[row r16][d = 16 t + 4 g + i]
#pragma unroll
  for (int rt = 0; rt < RT; ++rt) {
    float total = run_sum[rt];
    total = rows_sum(total);
    if (!row_ok[rt]) continue;
    const int row = rt * 16 + r16;
    if (p.parts > 1) {
      const size_t slot = ((size_t)(blockIdx.z * p.hq + head0 + row)) * p.parts + part;
      float* wo = p.ws_o + slot * D;
#pragma unroll
      for (int t = 0; t < DT; ++t) *reinterpret_cast<f32x4*>(wo + 16 * t + 4 * g) = acc[rt][t];
      if (g == 0) {
        p.ws_ml[slot * 2] = run_max[rt];
        p.ws_ml[slot * 2 + 1] = total;
      }
    } else {
      bf16_t* dst = p.out + ((size_t)tok0 * p.hq + head0 + row) * D;
      const float inv = total > 0.f ? 1.f / total : 0.f;
#pragma unroll
      for (int t = 0; t < DT; ++t) {
        bf16x4 o;
#pragma unroll
        for (int i = 0; i < 4; ++i) o[i] = static_cast<bf16_t>(acc[rt][t][i] * inv);
        *reinterpret_cast<bf16x4*>(dst + 16 * t + 4 * g) = o;
      }
    }
  }
}

// Merges the partial results of a decode row: one block of kMergeGroups waves per (request, head).
// Lane k of every wave first holds the weight of part k (parts <= 64).  Wave w then adds the
// parts w, w + kMergeGroups, ... (all their loads are issued together) and the waves' sums are
// added in wave order through LDS.
constexpr int kMergeGroups = 8;

__global__ void __launch_bounds__(kMergeGroups* kWave)
attention_merge_kernel(const float* __restrict__ ws_o, const float* __restrict__ ws_ml,
                       bf16_t* __restrict__ out, const int* __restrict__ cu_q, int seq_offset,
                       int hq, int d, int parts) {
  __shared__ float partial[kMergeGroups][kWave];
  const int seq = blockIdx.y;
  const int head = blockIdx.x;
  const int lane = threadIdx.x & (kWave - 1);
  const int wave = threadIdx.x / kWave;
  const size_t base = ((size_t)seq * hq + head) * parts;
  float m = -INFINITY, l = 0.f;
  if (lane < parts) {
    m = ws_ml[(base + lane) * 2];
    l = ws_ml[(base + lane) * 2 + 1];
  }
  const float top = wave_max(m);
  const float w = (m == -INFINITY) ? 0.f : exp2f(m - top);
  const float den = wave_sum(w * l);
  const float inv = den > 0.f ? 1.f / den : 0.f;
  const int tok = cu_q[seq + seq_offset];
  for (int i0 = 0; i0 < d; i0 += kWave) {
    const int i = i0 + lane;
    float o[kWave / kMergeGroups];
#pragma unroll
    for (int u = 0; u < kWave / kMergeGroups; ++u) {
      const int k = wave + u * kMergeGroups;
      o[u] = (k < parts && i < d) ? ws_o[(base + k) * d + i] : 0.f;
    }
    float num = 0.f;
#pragma unroll
    for (int u = 0; u < kWave / kMergeGroups; ++u) {
      const int k = wave + u * kMergeGroups;
      num += __shfl(w, k & (kWave - 1), kWave) * o[u];
    }
    __syncthreads();   // partial[] of the previous round has been read
    partial[wave][lane] = num;
    __syncthreads();
    if (wave == 0 && i < d) {
      float total = 0.f;
#pragma unroll
      for (int g = 0; g < kMergeGroups; ++g) total += partial[g][lane];
      out[((size_t)tok * hq + head) * d + i] = static_cast<bf16_t>(total * inv);
    }
  }
}

static int page_shift_of(int page_size) {
  if (page_size <= 0 || (page_size & (page_size - 1))) return -1;
  int shift = 0;
  while ((1 << shift) < page_size) ++shift;
  return shift;
}

template <int D, bool FUSED>
static int launch_decode(const AttnParams& p, int seqs, hipStream_t stream) {
  const int group = p.hq / p.hkv;
  dim3 grid(p.parts, p.hkv, seqs), block(kWave);
  constexpr bool LINES = D == 32 || D == 64 || D == 128 || D == 256;
  if (group > 32) return ATOM_UNSUPPORTED;
  if constexpr (LINES) {
    if (p.page_size % 8 == 0) {
      constexpr size_t area = 32 * (D * 2 + 16);   // LDS bytes of a wave
      if (p.parts > 1 && p.parts <= 8 && group <= 16) {
        // the parts of a (request, KV head) as the waves of one block, which merges them itself
        // (up to 16 heads a KV head: their results fit where a wave kept its key rows)
        static bool allowed = false;
        if (!allowed && hipFuncSetAttribute((const void*)attention_decode32_kernel<D, 1, true, FUSED>,
                                            hipFuncAttributeMaxDynamicSharedMemorySize, 8 * area) != hipSuccess)
          return ATOM_LAUNCH_FAILED;
        allowed = true;
        hipLaunchKernelGGL((attention_decode32_kernel<D, 1, true, FUSED>), dim3(1, p.hkv, seqs), dim3(p.parts * kWave),
                           area * p.parts, stream, p);
        return launch_status();
      }
      if (group <= 16) hipLaunchKernelGGL((attention_decode32_kernel<D, 1, false, FUSED>), grid, block, area, stream, p);
      else hipLaunchKernelGGL((attention_decode32_kernel<D, 2, false, FUSED>), grid, block, area, stream, p);
      if (p.parts > 1)
        hipLaunchKernelGGL(attention_merge_kernel, dim3(p.hq, seqs), dim3(kMergeGroups * kWave), 0, stream, p.ws_o,
                           p.ws_ml, p.out, p.cu_q, p.seq_offset, p.hq, D, p.parts);
      return launch_status();
    }
  }
  if constexpr (FUSED) {
    return ATOM_UNSUPPORTED;
  } else {
    if (group <= 16) hipLaunchKernelGGL((attention_mfma_kernel<D, 1, true>), grid, block, 0, stream, p);
    else hipLaunchKernelGGL((attention_mfma_kernel<D, 2, true>), grid, block, 0, stream, p);
    if (p.parts > 1)
      hipLaunchKernelGGL(attention_merge_kernel, dim3(p.hq, seqs), dim3(kMergeGroups * kWave), 0, stream, p.ws_o,
                         p.ws_ml, p.out, p.cu_q, p.seq_offset, p.hq, D, p.parts);
    return launch_status();
  }
}

// ------------------------------------------------------------------ prefill with shared key tiles
//
// A block of four waves owns a tile of query tokens of GH query heads that share a KV head
// (GH = 4, 2 or 1, a divisor of the group size): wave w has head (w % GH) and the 32 tokens
// number (w / GH) of the tile, so a block covers 32 * 4 / GH tokens.  Keys are walked TK (64 or 32) at a
// time; the block loads each K tile (TK keys x D) and V^T tile (D x TK keys) once, through
// registers (the next tile's loads are in flight while this one is multiplied) into LDS, where all
// four waves read them as matrix-core operands.  Products, softmax and layouts are those of the
// kernel above, with both products on v_mfma_f32_16x16x32_bf16: 32 keys of a tile are the k
// dimension of one step of the second product, in the order (4 g + i, 16 + 4 g + i) that the first product
// leaves them in a lane.
//
// With KS = 2 the block has eight waves: the second four are the same heads and tokens again, and the two
// halves take the key tiles in turn (tile 0, 2, 4 .. and 1, 3, 5 ..), each with LDS tiles of its own, and add
// their results at the end through LDS.  A block then keeps two waves on every SIMD for as long as it runs, one
// in its products while the other is in its softmax; a block of four waves only has that while another block
// shares its CU, and the longest blocks of a causal prompt, which decide how long the launch takes, run mostly
// after their shorter neighbours have left.
//
// Needs D % 64 == 0 and page_size % 8 == 0.
constexpr float kLazyMax = 8.f;

template <int D, int GH, int TK, int KS, int RT = 2>
__global__ void __launch_bounds__(256 * KS, (D <= 128 && KS == 1 ? 2 : 1)) attention_prefill_tiled_kernel(AttnParams p) {
  constexpr int KCH = D / 32;
  constexpr int DT = D / 16;
  constexpr int ROWS = 16 * RT;          // query tokens of a wave: 32, or 16 where a launch of 32 would leave CUs idle
  constexpr int SPLIT = 2 / RT;          // blocks that share an entry of the tile list (which names 32 * 4 / GH tokens)
  static_assert(RT == 2 || (RT == 1 && KS > 1), "blocks of 16 tokens a wave come with eight waves only");
  constexpr int KB = TK / 16;            // blocks of 16 keys in a tile
  constexpr int KSTR = D + 8;            // LDS row of a key, in elements: rows start 4 banks apart
  constexpr int VSTR = TK + 8;           // LDS row of V^T (one d), in elements: 16-byte aligned, rows 4 banks apart
  constexpr int PT = D * TK / 8 / 256;   // 16-byte pieces of each tile that a thread moves
#ifndef ATOM_PF_AHEAD
#define ATOM_PF_AHEAD 4
#endif

  constexpr int AHEAD = ATOM_PF_AHEAD;   // operands read from LDS ahead of the product that takes them
  constexpr int TILE_ELEMS = TK * KSTR + D * VSTR;   // a K tile and a V^T tile
  constexpr int NS = RT * DT * 4 + 2 * RT;           // floats a lane hands over when the halves are added
  constexpr int SMEM_TILES = KS * TILE_ELEMS * 2, SMEM_SUMS = KS > 1 ? 4 * NS * kWave * 4 : 0;
  __shared__ __attribute__((aligned(16))) char smem[SMEM_TILES > SMEM_SUMS ? SMEM_TILES : SMEM_SUMS];
  const int part = threadIdx.x / 256;    // which half of the key tiles (always 0 with KS = 1)
  const int tid = threadIdx.x % 256;
  bf16_t* const ks = reinterpret_cast<bf16_t*>(smem) + part * TILE_ELEMS;
  bf16_t* const vs = ks + TK * KSTR;
  const int lane = tid & (kWave - 1);
  const int wave = tid / kWave;
  const int r16 = lane & 15;
  const int g = lane >> 4;
  const int group = p.hq / p.hkv;
  const int ps = p.page_size;

  // The host lists tiles with the most keys first, so tile b and tile n - 1 - b together are about the same
  // work for every b.  Head sizes up to 128 fit two blocks on a CU (256 registers a lane): every block takes
  // one (tile, head group), the grid is one-dimensional, and its first half walks the list from the longest
  // item down while its second half walks it from the shortest up, so that the two blocks that meet on a
  // CU (block b and block b + n / 2, as blocks are handed out in order) are a long and a short one.
  // Larger heads run one block a CU, which takes tile b and then tile n - 1 - b.
  // Blocks of eight waves run one a CU and take the items in the order of the list, longest first.
  constexpr bool TWO = D <= 128;
  for (int pass = 0; pass < 2; ++pass) {
  int tile, ygroup, piece = 0;
  if (KS > 1) {
    if (pass == 1) break;
    const int groups = p.hq / GH;
    const int unit = (int)blockIdx.x / groups;
    tile = unit / SPLIT;
    piece = unit - tile * SPLIT;
    ygroup = (int)blockIdx.x - unit * groups;
  } else if (TWO) {
    if (pass == 1) break;
    const int total = gridDim.x, half = (total + 1) / 2, groups = p.hq / GH;
    const int item = (int)blockIdx.x < half ? (int)blockIdx.x : total - 1 - ((int)blockIdx.x - half);
    tile = item / groups;
    ygroup = item - tile * groups;
  } else {
    tile = pass == 0 ? (int)blockIdx.x : p.num_tiles - 1 - (int)blockIdx.x;
    if (pass == 1 && tile <= (int)blockIdx.x) break;
    ygroup = blockIdx.y;
  }
  const int seq = p.tiles[2 * tile];
  if (seq < 0) continue;   // an unused entry of a list of fixed length (the same for the whole block)
  constexpr int TQ = ROWS * (4 / GH);               // tokens of a block
  const int row_start = p.tiles[2 * tile + 1] + piece * TQ;
  const int head = ygroup * GH + (wave % GH);
  const int kvh = (ygroup * GH) / group;
  const int sub = wave / GH;
  const int ctx = p.ctx_lens[seq];
  const int q_begin = p.cu_q[seq];
  const int q_len = p.cu_q[seq + 1] - q_begin;
  if (row_start >= q_len) continue;                 // the portion ends in the entry's first piece (the whole block)
  const int block_rows = min(TQ, q_len - row_start);
  const int my_row0 = row_start + ROWS * sub;
  const int nrows = max(0, min(ROWS, q_len - my_row0));
  const int pos_block0 = ctx - q_len + row_start;   // position of the block's first token
  const int pos0 = pos_block0 + ROWS * sub;         // of this wave's first token
  const int ke = pos_block0 + block_rows;           // one past the last key any row of the block sees
  const int my_ke = pos0 + nrows;
  int kb = 0;
  if (p.window > 0 && pos_block0 - p.window + 1 > 0) kb = (pos_block0 - p.window + 1) & ~(TK - 1);
  const int* table = p.block_tables + (size_t)seq * p.max_blocks;

  // ---- this wave's queries
  int row_pos[RT];
  bool row_ok[RT];
  bf16x8 q32[RT][KCH];
#pragma unroll
  for (int rt = 0; rt < RT; ++rt) {
    const int row = rt * 16 + r16;
    row_ok[rt] = row < nrows;
    row_pos[rt] = pos0 + row;
    const bf16_t* qr = p.q + ((size_t)(q_begin + my_row0 + row) * p.hq + head) * D;
#pragma unroll
    for (int j = 0; j < KCH; ++j) {
      bf16x8 v = {0, 0, 0, 0, 0, 0, 0, 0};
      if (row_ok[rt]) v = *reinterpret_cast<const bf16x8*>(qr + 32 * j + 8 * g);
      q32[rt][j] = v;
    }
  }
  f32x4 acc[RT][DT];
  float run_max[RT], run_sum[RT];
#pragma unroll
  for (int rt = 0; rt < RT; ++rt) {
    run_max[rt] = -INFINITY;
    run_sum[rt] = 0.f;
#pragma unroll
    for (int t = 0; t < DT; ++t) acc[rt][t] = f32x4{0.f, 0.f, 0.f, 0.f};
  }

  // ---- moving a tile: piece q of K is (key q / (D/8), 8 elements at (q % (D/8)) * 8);
  //      piece q of V^T is (d = q / (TK/8), the 8 keys at (q % (TK/8)) * 8)
  bf16x8 kreg[PT], vreg[PT];
  const uint32_t page_elems = (uint32_t)p.hkv * ps * D;    // elements of a page, all heads
  const int k_head = kvh * ps * D, v_head = kvh * D * ps;  // this KV head's part of a key page and of a value page
  // The pages of a tile are looked up a tile before its loads go out (`pages_of`), so that no load waits for a
  // table entry; a thread's pieces of V^T all lie in one page (256 is a multiple of the pieces per row).
  static_assert(256 % (TK / 8) == 0, "a thread's V^T pieces must share their keys");
  int kpage[PT], vpage = 0;
  auto pages_of_as = [&](int k0, auto kind) {
    const PageMath<decltype(kind)::value> pages{ps, p.page_shift};
#pragma unroll
    for (int j = 0; j < PT; ++j) {
      const int key = min(k0 + (tid + 256 * j) / (D / 8), ke - 1);
      kpage[j] = table[pages.index(key)];
    }
    const int vkey = min(k0 + (tid % (TK / 8)) * 8, (ke - 1) & ~7);
    vpage = table[pages.index(vkey)];
  };
  auto pages_of = [&](int k0) {
    if (p.page_shift >= 0) pages_of_as(k0, Pow2Pages{});
    else pages_of_as(k0, AnyPages{});
  };
  auto load_tile_as = [&](int k0, auto kind) {
    const PageMath<decltype(kind)::value> pages{ps, p.page_shift};
    const int vkey = min(k0 + (tid % (TK / 8)) * 8, (ke - 1) & ~7);
    const bf16_t* vbase = p.v_cache + (uint64_t)(uint32_t)vpage * page_elems + (v_head + pages.within(vkey));
#pragma unroll
    for (int j = 0; j < PT; ++j) {
      const int q = tid + 256 * j;
      const int key = min(k0 + q / (D / 8), ke - 1);
      kreg[j] = *reinterpret_cast<const bf16x8*>(p.k_cache + (uint64_t)(uint32_t)kpage[j] * page_elems +
                                                 (k_head + pages.within(key) * D + (q % (D / 8)) * 8));
      vreg[j] = *reinterpret_cast<const bf16x8*>(vbase + (q / (TK / 8)) * ps);
    }
  };
  auto load_tile = [&](int k0) {
    if (p.page_shift >= 0) load_tile_as(k0, Pow2Pages{});
    else load_tile_as(k0, AnyPages{});
  };
  auto store_tile = [&]() {
#pragma unroll
    for (int j = 0; j < PT; ++j) {
      const int q = tid + 256 * j;
      *reinterpret_cast<bf16x8*>(ks + (q / (D / 8)) * KSTR + (q % (D / 8)) * 8) = kreg[j];
      // Within every 32 keys of a V^T row the keys are laid in the order in which the second product
      // takes them: lane group g holds keys 4 g .. 4 g + 3 and 16 + 4 g .. 16 + 4 g + 3 (what the first
      // product left it), so these eight lie together at 8 g: key c goes to 8 ((c % 16) / 4) + 4 (c / 16) + c % 4.
      const bf16x4 lo = {vreg[j][0], vreg[j][1], vreg[j][2], vreg[j][3]};
      const bf16x4 hi = {vreg[j][4], vreg[j][5], vreg[j][6], vreg[j][7]};
      const int c0 = (q % (TK / 8)) * 8;              // first key of the piece within the tile
      const int in32 = c0 % 32;
      const int at_lo = 8 * ((in32 % 16) / 4) + 4 * (in32 / 16);
      bf16_t* dst = vs + (q / (TK / 8)) * VSTR + (c0 - in32);
      *reinterpret_cast<bf16x4*>(dst + at_lo) = lo;
      *reinterpret_cast<bf16x4*>(dst + at_lo + 8) = hi;   // keys c0 + 4 ..: the next lane group
    }
  };

  constexpr int STEP = KS * TK;          // keys the block walks at a time
  if (kb + part * TK < ke) {
    pages_of(kb + part * TK);
    load_tile(kb + part * TK);
    if (kb + part * TK + STEP < ke) pages_of(kb + part * TK + STEP);
  }
  for (int kk = kb; kk < ke; kk += STEP) {
    const int k0 = kk + part * TK;       // this half's tile
    __syncthreads();   // the previous tile has been read by every wave
    if (k0 < ke) store_tile();
    __syncthreads();
    if (k0 + STEP < ke) {
      load_tile(k0 + STEP);
      if (k0 + 2 * STEP < ke) pages_of(k0 + 2 * STEP);
    }
    if (nrows == 0 || k0 >= my_ke) continue;   // the whole wave: nothing of this tile is visible to it

    // ---- S^T for the blocks of 16 keys
    f32x4 s[RT][KB];
#pragma unroll
    for (int rt = 0; rt < RT; ++rt)
#pragma unroll
      for (int b = 0; b < KB; ++b) s[rt][b] = f32x4{0.f, 0.f, 0.f, 0.f};
    // (the head-size chunks outermost: successive products go to different accumulators).  The operand of
    // product i + AHEAD is read from LDS while product i runs: the order is pinned, because left to itself the
    // compiler reads every operand just before its product and waits for it.
    {
      constexpr int NQK = KCH * KB;
      auto k_operand = [&](int i) {
        return *reinterpret_cast<const bf16x8*>(ks + (16 * (i % KB) + r16) * KSTR + 32 * (i / KB) + 8 * g);
      };
      bf16x8 kf[AHEAD];
#pragma unroll
      for (int i = 0; i < AHEAD; ++i) kf[i] = k_operand(i);
#pragma unroll
      for (int i = 0; i < NQK; ++i) {
        __builtin_amdgcn_sched_barrier(0);
        const bf16x8 a = kf[i % AHEAD];
#pragma unroll
        for (int rt = 0; rt < RT; ++rt)
          s[rt][i % KB] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, q32[rt][i / KB], s[rt][i % KB], 0, 0, 0);
        if (i + AHEAD < NQK) kf[i % AHEAD] = k_operand(i + AHEAD);
      }
      __builtin_amdgcn_sched_barrier(0);
    }
    constexpr int NPV = (KB / 2) * DT;
    auto v_operand = [&](int i) {
      return *reinterpret_cast<const bf16x8*>(vs + (16 * (i % DT) + r16) * VSTR + 32 * (i / DT) + 8 * g);
    };
    bf16x8 vf[AHEAD];

    // ---- softmax update; lane holds keys k0 + 16 b + 4 g + i of row r16.  The maximum is taken over the
    //      raw scores and the scale goes into the exponent's multiply-add.  A tile that every row of the
    //      wave sees whole (all but the last one or two of a causal prompt) needs no masking.
    bf16x8 pb[RT][KB / 2];
    float alpha[RT];
    bool rescale = false;
    const bool whole = k0 + TK - 1 <= min(pos0, ke - 1) && (p.window <= 0 || k0 >= pos0 + nrows - p.window);
#pragma unroll
    for (int rt = 0; rt < RT; ++rt) {
      float sc[4 * KB];
      float mx = -INFINITY;
      if (whole) {
#pragma unroll
        for (int b = 0; b < KB; ++b)
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            sc[4 * b + i] = s[rt][b][i];
            mx = fmaxf(mx, sc[4 * b + i]);
          }
      } else {
        // the visible keys, counted from this lane's first key of the tile: 16 b + i is compared with constants
        const int first = k0 + 4 * g;
        const int hi = min(row_pos[rt], ke - 1) - first;
        const int lo = (p.window > 0 ? row_pos[rt] - p.window + 1 : 0) - first;
#pragma unroll
        for (int b = 0; b < KB; ++b)
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            const bool vis = 16 * b + i <= hi && 16 * b + i >= lo;
            sc[4 * b + i] = vis ? s[rt][b][i] : -INFINITY;
            mx = fmaxf(mx, sc[4 * b + i]);
          }
      }
      mx = rows_max(mx);
      // The running maximum follows the tile's only when that is larger by more than kLazyMax (in powers of two):
      // the weights of a tile are then at most 2^kLazyMax instead of 1, which float32 sums and bfloat16 weights hold
      // as well, and after a row's first tiles nothing has to be scaled again.
      const float tile_max = mx * p.scale_log2;
      const float new_max = tile_max > run_max[rt] + kLazyMax ? tile_max : run_max[rt];
      const float base = new_max == -INFINITY ? 0.f : new_max;
      alpha[rt] = fast_exp2(run_max[rt] - base);
      rescale = rescale || alpha[rt] != 1.f;
      float psum = 0.f;
#pragma unroll
      for (int e = 0; e < 4 * KB; ++e) {
        const float pv = fast_exp2(fmaf(sc[e], p.scale_log2, -base));
        psum += pv;
        pb[rt][e / 8][e % 8] = static_cast<bf16_t>(pv);
      }
      run_sum[rt] = run_sum[rt] * alpha[rt] + psum;
      run_max[rt] = new_max;
    }
    // the running maxima of most tiles after the first few do not move: skip the rescaling then
    if (__any(rescale)) {
#pragma unroll
      for (int rt = 0; rt < RT; ++rt)
#pragma unroll
        for (int t = 0; t < DT; ++t) {
          acc[rt][t][0] *= alpha[rt]; acc[rt][t][1] *= alpha[rt];
          acc[rt][t][2] *= alpha[rt]; acc[rt][t][3] *= alpha[rt];
        }
    }

    // ---- O^T += V^T P^T, 32 keys a step
    {
#pragma unroll
      for (int i = 0; i < AHEAD; ++i) vf[i] = v_operand(i);
#pragma unroll
      for (int i = 0; i < NPV; ++i) {
        __builtin_amdgcn_sched_barrier(0);
        const bf16x8 a = vf[i % AHEAD];
#pragma unroll
        for (int rt = 0; rt < RT; ++rt)
          acc[rt][i % DT] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, pb[rt][i / DT], acc[rt][i % DT], 0, 0, 0);
        if (i + AHEAD < NPV) vf[i % AHEAD] = v_operand(i + AHEAD);
      }
      __builtin_amdgcn_sched_barrier(0);
    }
  }

  // ---- the two halves of the key tiles are added: the second hands its sums, maxima and accumulators over
  //      through LDS, lane by lane (both halves hold the same rows and columns in the same lanes)
  if constexpr (KS > 1) {
    if (kb + TK < ke) {      // the same for the whole block: the second half had a tile at all
      __syncthreads();       // every wave has read its last tiles
      float* area = reinterpret_cast<float*>(smem) + (size_t)wave * NS * kWave + lane;
      if (part == 1) {
#pragma unroll
        for (int rt = 0; rt < RT; ++rt) {
#pragma unroll
          for (int t = 0; t < DT; ++t)
#pragma unroll
            for (int i = 0; i < 4; ++i) area[((rt * DT + t) * 4 + i) * kWave] = acc[rt][t][i];
          area[(RT * DT * 4 + rt) * kWave] = run_max[rt];
          area[(RT * DT * 4 + RT + rt) * kWave] = run_sum[rt];
        }
      }
      __syncthreads();
      if (part == 0) {
#pragma unroll
        for (int rt = 0; rt < RT; ++rt) {
          const float other_max = area[(RT * DT * 4 + rt) * kWave];
          const float other_sum = area[(RT * DT * 4 + RT + rt) * kWave];
          const float top = fmaxf(run_max[rt], other_max);
          const float base = top == -INFINITY ? 0.f : top;
          const float mine = fast_exp2(run_max[rt] - base), theirs = fast_exp2(other_max - base);
          run_sum[rt] = run_sum[rt] * mine + other_sum * theirs;
#pragma unroll
          for (int t = 0; t < DT; ++t)
#pragma unroll
            for (int i = 0; i < 4; ++i)
              acc[rt][t][i] = acc[rt][t][i] * mine + area[((rt * DT + t) * 4 + i) * kWave] * theirs;
        }
      }
    }
    if (part != 0) return;   // nothing follows but the first half's writes
  }

  // ---- write: lane holds O[row r16][d = 16 t + 4 g + i]
#pragma unroll
  for (int rt = 0; rt < RT; ++rt) {
    float total = run_sum[rt];
    total = rows_sum(total);
    if (!row_ok[rt]) continue;
    const int row = rt * 16 + r16;
    bf16_t* dst = p.out + ((size_t)(q_begin + my_row0 + row) * p.hq + head) * D;
    const float inv = total > 0.f ? 1.f / total : 0.f;
#pragma unroll
    for (int t = 0; t < DT; ++t) {
      bf16x4 o;
#pragma unroll
      for (int i = 0; i < 4; ++i) o[i] = static_cast<bf16_t>(acc[rt][t][i] * inv);
      *reinterpret_cast<bf16x4*>(dst + 16 * t + 4 * g) = o;
    }
  }
  }   // the two tiles of the block
}

// Query tokens per block of the tiled prefill kernel for this head size, page size and group, or 0
// if it does not take them.
ATOM_EXPORT int atom_attention_prefill_tile_rows(int d, int page_size, int group) {
  if (d % 64 || d > 256 || page_size % 8 || group < 1) return 0;
  const int gh = group % 4 == 0 ? 4 : (group % 2 == 0 ? 2 : 1);
  return 32 * (4 / gh);
}

template <int D>
static int launch_prefill_tiled(const AttnParams& p, int num_tiles, int rows_per_tile, bool halves, bool low,
                                hipStream_t stream) {
  const int group = p.hq / p.hkv;
  const int gh = group % 4 == 0 ? 4 : (group % 2 == 0 ? 2 : 1);
  if (rows_per_tile != 32 * (4 / gh)) return ATOM_BAD_SHAPE;
  dim3 grid((num_tiles + 1) / 2, p.hq / gh), block(256);
  if (D <= 128) grid = dim3(num_tiles * (p.hq / gh), 1);
  constexpr int TK = D <= 128 ? 64 : 32;
  if constexpr (D <= 128) {
    if (halves && low) {   // ... and 16 tokens a wave: two blocks for every entry of the list
      block = dim3(512);
      grid = dim3(2 * num_tiles * (p.hq / gh), 1);
      if (gh == 4) hipLaunchKernelGGL((attention_prefill_tiled_kernel<D, 4, TK, 2, 1>), grid, block, 0, stream, p);
      else if (gh == 2) hipLaunchKernelGGL((attention_prefill_tiled_kernel<D, 2, TK, 2, 1>), grid, block, 0, stream, p);
      else hipLaunchKernelGGL((attention_prefill_tiled_kernel<D, 1, TK, 2, 1>), grid, block, 0, stream, p);
      return launch_status();
    }
    if (halves) {   // eight waves a block, the key tiles taken in turn by its two halves
      block = dim3(512);
      if (gh == 4) hipLaunchKernelGGL((attention_prefill_tiled_kernel<D, 4, TK, 2>), grid, block, 0, stream, p);
      else if (gh == 2) hipLaunchKernelGGL((attention_prefill_tiled_kernel<D, 2, TK, 2>), grid, block, 0, stream, p);
      else hipLaunchKernelGGL((attention_prefill_tiled_kernel<D, 1, TK, 2>), grid, block, 0, stream, p);
      return launch_status();
    }
  }
  if (gh == 4) hipLaunchKernelGGL((attention_prefill_tiled_kernel<D, 4, TK, 1>), grid, block, 0, stream, p);
  else if (gh == 2) hipLaunchKernelGGL((attention_prefill_tiled_kernel<D, 2, TK, 1>), grid, block, 0, stream, p);
  else hipLaunchKernelGGL((attention_prefill_tiled_kernel<D, 1, TK, 1>), grid, block, 0, stream, p);
  return launch_status();
}

template <int D>
static int launch_prefill(const AttnParams& p, int num_tiles, int rows_per_tile, hipStream_t stream) {
  dim3 grid(num_tiles, p.hq), block(kWave);
  if (rows_per_tile == 16) hipLaunchKernelGGL((attention_mfma_kernel<D, 1, false>), grid, block, 0, stream, p);
  else if (rows_per_tile == 32) hipLaunchKernelGGL((attention_mfma_kernel<D, 2, false>), grid, block, 0, stream, p);
  else return ATOM_BAD_SHAPE;
  return launch_status();
}

#define ATOM_FOR_HEAD_DIM(d, CALL)        \
  switch (d) {                            \
    case 16: CALL(16); break;             \
    case 32: CALL(32); break;             \
    case 64: CALL(64); break;             \
    case 96: CALL(96); break;             \
    case 128: CALL(128); break;           \
    case 256: CALL(256); break;           \
    default: return ATOM_UNSUPPORTED;     \
  }

// 1 if this head size has a matrix-core kernel.
ATOM_EXPORT int atom_attention_mfma_supports(int d, int page_size, int group) {
  if (page_size % 4 || group > 32) return 0;
  return d == 16 || d == 32 || d == 64 || d == 96 || d == 128 || d == 256;
}

static int check_common(int hq, int hkv, int d, int page_size, int max_blocks) {
  if (hq <= 0 || hkv <= 0 || hq % hkv || d <= 0 || page_size <= 0 || page_size % 4 || max_blocks <= 0)
    return ATOM_BAD_SHAPE;
  if (hq > 65535) return ATOM_TOO_LARGE;
  return ATOM_OK;
}

// Decode: requests seq_offset .. seq_offset + seqs - 1 each bring one new token (row cu_q[seq]).
// ws_o needs seqs * hq * parts * d floats, ws_ml seqs * hq * parts * 2 (unused when parts == 1).
ATOM_EXPORT int atom_attention_decode(const void* q, const void* k_cache, const void* v_cache, void* out,
                                      const int* cu_q, const int* ctx_lens, const int* block_tables, int max_blocks,
                                      int seq_offset, int seqs, int hq, int hkv, int d, int page_size, float scale,
                                      int window, int parts, float* ws_o, float* ws_ml, hipStream_t stream) {
  if (int st = check_common(hq, hkv, d, page_size, max_blocks)) return st;
  if (seqs < 0 || parts < 1 || seq_offset < 0) return ATOM_BAD_SHAPE;
  if (parts > kWave) return ATOM_TOO_LARGE;   // the merge keeps one part per lane
  if (parts > 1 && (!ws_o || !ws_ml)) return ATOM_BAD_SHAPE;
  if (seqs > 65535 || hkv > 65535) return ATOM_TOO_LARGE;
  if (seqs == 0) return ATOM_OK;
  AttnParams p{};
  p.q = (const bf16_t*)q; p.k_cache = (const bf16_t*)k_cache; p.v_cache = (const bf16_t*)v_cache;
  p.out = (bf16_t*)out; p.cu_q = cu_q; p.ctx_lens = ctx_lens; p.block_tables = block_tables; p.tiles = nullptr;
  p.ws_o = ws_o; p.ws_ml = ws_ml; p.max_blocks = max_blocks; p.hq = hq; p.hkv = hkv; p.page_size = page_size;
  p.window = window; p.seq_offset = seq_offset; p.parts = parts; p.scale_log2 = scale * 1.4426950408889634f;
  p.page_shift = page_shift_of(page_size);
#define CALL(DD) return launch_decode<DD, false>(p, seqs, stream)
  ATOM_FOR_HEAD_DIM(d, CALL)
#undef CALL
  return ATOM_OK;
}

// 1 if atom_attention_decode_fused takes this head size, page size and group: the head sizes whose rotation
// pairs lie in one lane, pages of a multiple of 8 keys.
ATOM_EXPORT int atom_attention_decode_fused_supports(int d, int page_size, int group) {
  return (d == 64 || d == 128 || d == 256) && page_size > 0 && page_size % 8 == 0 && group >= 1 && group <= 32;
}

// Decode attention that starts from the step's float32 QKV product [tokens, (Hq + 2 Hkv) * D]: per-head RMS norm
// of q and k (weights may be null), rotation of the whole head by the tables at each request's last position,
// the new key and value written at slots[token] (write_kv), attention over the pages.  Otherwise as
// atom_attention_decode.
ATOM_EXPORT int atom_attention_decode_fused(const float* qkv, const float* q_weight, const float* k_weight,
                                            const float* cos_table, const float* sin_table, const int* slots,
                                            float eps, int write_kv, void* k_cache, void* v_cache, void* out,
                                            const int* cu_q, const int* ctx_lens, const int* block_tables,
                                            int max_blocks, int seq_offset, int seqs, int hq, int hkv, int d,
                                            int page_size, float scale, int window, int parts, float* ws_o,
                                            float* ws_ml, hipStream_t stream) {
  if (int st = check_common(hq, hkv, d, page_size, max_blocks)) return st;
  if (!atom_attention_decode_fused_supports(d, page_size, hq / hkv)) return ATOM_UNSUPPORTED;
  if (seqs < 0 || parts < 1 || seq_offset < 0 || !qkv || !cos_table || !sin_table) return ATOM_BAD_SHAPE;
  if (write_kv && (!slots || !k_cache || !v_cache)) return ATOM_BAD_SHAPE;
  if (parts > kWave) return ATOM_TOO_LARGE;
  if (parts > 1 && (!ws_o || !ws_ml)) return ATOM_BAD_SHAPE;
  if (seqs > 65535 || hkv > 65535) return ATOM_TOO_LARGE;
  if (((uintptr_t)qkv) & 15) return ATOM_BAD_SHAPE;
  if (seqs == 0) return ATOM_OK;
  AttnParams p{};
  p.q = nullptr; p.k_cache = (const bf16_t*)k_cache; p.v_cache = (const bf16_t*)v_cache;
  p.out = (bf16_t*)out; p.cu_q = cu_q; p.ctx_lens = ctx_lens; p.block_tables = block_tables; p.tiles = nullptr;
  p.ws_o = ws_o; p.ws_ml = ws_ml; p.max_blocks = max_blocks; p.hq = hq; p.hkv = hkv; p.page_size = page_size;
  p.window = window; p.seq_offset = seq_offset; p.parts = parts; p.scale_log2 = scale * 1.4426950408889634f;
  p.page_shift = page_shift_of(page_size);
  p.qkv = qkv; p.q_weight = q_weight; p.k_weight = k_weight; p.cos_table = cos_table; p.sin_table = sin_table;
  p.slots = slots; p.eps = eps; p.write_kv = write_kv;
  switch (d) {
    case 64: return launch_decode<64, true>(p, seqs, stream);
    case 128: return launch_decode<128, true>(p, seqs, stream);
    case 256: return launch_decode<256, true>(p, seqs, stream);
    default: return ATOM_UNSUPPORTED;
  }
}

// Prefill: `tiles` lists (request, first row) for every tile of `rows_per_tile` query tokens: 16 or 32 for
// the kernel in which every wave loads its own keys, atom_attention_prefill_tile_rows() with `tiled` (1: blocks of
// four waves; 2: of eight waves whose halves take the key tiles in turn; 3: the same with 16 tokens a wave, two
// blocks for every entry of the list).
ATOM_EXPORT int atom_attention_prefill(const void* q, const void* k_cache, const void* v_cache, void* out,
                                       const int* cu_q, const int* ctx_lens, const int* block_tables, int max_blocks,
                                       const int* tiles, int num_tiles, int rows_per_tile, int tiled, int hq, int hkv,
                                       int d, int page_size, float scale, int window, hipStream_t stream) {
  if (int st = check_common(hq, hkv, d, page_size, max_blocks)) return st;
  if (num_tiles < 0 || !tiles) return ATOM_BAD_SHAPE;
  if (num_tiles == 0) return ATOM_OK;
  AttnParams p{};
  p.q = (const bf16_t*)q; p.k_cache = (const bf16_t*)k_cache; p.v_cache = (const bf16_t*)v_cache;
  p.out = (bf16_t*)out; p.cu_q = cu_q; p.ctx_lens = ctx_lens; p.block_tables = block_tables; p.tiles = tiles;
  p.ws_o = nullptr; p.ws_ml = nullptr; p.max_blocks = max_blocks; p.hq = hq; p.hkv = hkv; p.page_size = page_size;
  p.window = window; p.seq_offset = 0; p.parts = 1; p.scale_log2 = scale * 1.4426950408889634f;
  p.page_shift = page_shift_of(page_size);
  p.num_tiles = num_tiles;
  if (tiled) {   // tiles of atom_attention_prefill_tile_rows() tokens for the kernel with shared key tiles
    if (!atom_attention_prefill_tile_rows(d, page_size, hq / hkv)) return ATOM_UNSUPPORTED;
    switch (d) {
      case 64: return launch_prefill_tiled<64>(p, num_tiles, rows_per_tile, tiled > 1, tiled > 2, stream);
      case 128: return launch_prefill_tiled<128>(p, num_tiles, rows_per_tile, tiled > 1, tiled > 2, stream);
      case 192: return launch_prefill_tiled<192>(p, num_tiles, rows_per_tile, tiled > 1, tiled > 2, stream);
      case 256: return launch_prefill_tiled<256>(p, num_tiles, rows_per_tile, tiled > 1, tiled > 2, stream);
      default: return ATOM_UNSUPPORTED;
    }
  }
#define CALL(DD) return launch_prefill<DD>(p, num_tiles, rows_per_tile, stream)
  ATOM_FOR_HEAD_DIM(d, CALL)
#undef CALL
  return ATOM_OK;
}
