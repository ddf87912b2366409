// Paged attention on MFMA for bfloat16, one head size per build (QRT_HEAD_DIM,
// a multiple of 16). Serves prompt portions, single decoded tokens and batches
// that mix both, with optional splitting of the keys across blocks.
//
// Rows. For one sequence and one key/value head the work is a matrix of
// q_len * g rows, row = token * g + (query head within the group): all g query
// heads that share a key head sit in the same tile, so a decoded token fills g
// rows and a prompt portion fills tiles of 16 rows per wave. The host passes a
// list of tiles (sequence, first row); the grid walks it, one block per tile and key head.
//
// Products. Scores are formed transposed, S^T = K Q^T, with the 16x16x32 MFMA:
// the A operand is 16 keys x 32 head elements read straight from the key page,
// the B operand 32 head elements x 16 rows of Q held in registers (a head size
// with a 16-wide remainder pads that step with zeros). The 16 key
// rows of the two MFMAs that cover a block of 32 keys are permuted (row
// 4 quad + r of sub-block kb holds key 8 quad + 4 kb + r) so that each lane ends
// up with the scores of 8 consecutive keys for its row: exactly the B operand
// (P^T) of the second product O^T = V^T P^T, whose A operand is then 8
// consecutive keys of one head element: one 16-byte read from the value page,
// which stores values transposed ([page, head, D, offset]). No data crosses
// lanes except the row maximum and sum.
//
// Softmax is online, float32, in base 2 (scale * log2 e is folded into the
// exponent's argument); probabilities are rounded to bfloat16 for the second
// product, accumulation is float32. Key j is visible to the row at position p
// iff j <= p and (no window or j > p - window).
#include "common.h"
#include <math.h>

#ifndef QRT_HEAD_DIM
#error "build with -DQRT_HEAD_DIM=<multiple of 16>"
#endif
#if QRT_HEAD_DIM % 16 != 0 || QRT_HEAD_DIM < 16 || QRT_HEAD_DIM > 512
#error "QRT_HEAD_DIM must be a multiple of 16 between 16 and 512"
#endif


// 8 head elements from ``p`` for the quads that hold real data, zeros for the others: a head
// size with a 16-wide remainder runs the 32-wide MFMA with the upper half of the step empty.
// (A 16x16x16 MFMA chained onto the 16x16x32 ones for that remainder gave results that
// differed from run to run; one MFMA shape per accumulator chain does not.)
__device__ __forceinline__ bf16x8_t load_tail(const bf16_t* p, int quad) {
  bf16x8_t v;
#pragma unroll
  for (int e = 0; e < 8; ++e) v[e] = (bf16_t)0.0f;
  if (quad < 2) v = *(const bf16x8_t*)(p + 8 * quad);
  return v;
}

struct AttnTileArgs {
  const bf16_t* q;        // [T, nq * D]
  bf16_t* out;            // [T, nq * D]
  const bf16_t* k_cache;  // [pages, nkv, page_size, D]
  const bf16_t* v_cache;  // [pages, nkv, D, page_size]
  const int* cu_q;        // [S + 1]
  const int* kv_lens;     // [S]
  const int* block_table; // [S, table_width]
  const int* tile_seq;    // [num_tiles]
  const int* tile_row0;   // [num_tiles]
  float* part_o;          // [T, nq, num_splits, D]   (num_splits > 1)
  float* part_lse;        // [T, nq, num_splits]      base-2 log of the split's sum, -inf if empty
  int table_width, num_tiles, nq, nkv, page_size, window, num_splits, waves;
  float scale_log2;
  int row_tiles;  // tiles of 16 rows per wave (general kernel): 1, 2 or 4
  int use_lds;    // long portions: share keys and values of a block of waves through LDS (1), and
                  // cut the blocks of keys between two groups of four waves in one block (2)
  // a launch that covers only some of the step's sequences (the others go to another kernel):
  // the tokens whose rows the merge of key splits may write; null: all rows
  const int* merge_tokens;
  int num_merge_tokens;
  // Decoding with the step's own keys and values still in the product that made them (one
  // token per sequence; qkv non-null): the kernel normalises and rotates the token's query and
  // key heads itself, attends over the cache up to the token before, adds the token's own key
  // and value from registers, and stores them into the cache for the steps to come. `q` is
  // then unused.
  const bf16_t* qkv;       // [T, qkv_stride]: nq query heads, nkv key heads, nkv value heads of D
  long qkv_stride;
  const float* q_weight;   // [D] or null: no norm
  const float* k_weight;
  const float* rope;       // [T, D]: cosines of the D / 2 angles, then their sines; null: no rotation
  const int* slots;        // [T]: place of the token in the cache, page * page_size + offset
  float eps;
  // Decoding over sequences of very different lengths: instead of num_splits equal parts of every
  // sequence, pieces of split_blocks 32-key blocks, as many as a sequence has (at most num_splits),
  // listed in `items` as (sequence, piece), whole pieces first and the sequences' last, shorter
  // pieces after them, then (-1, 0) up to max_items. The launch is (key head, item): blocks of
  // equal work, the heavy ones next to each other in launch order, which spreads them evenly over
  // the compute units. qrt_attention_work_list fills the list from the step's lengths.
  int split_blocks, max_items;
  int* items;              // [max_items][2] or null
};

constexpr int D = QRT_HEAD_DIM;
constexpr int KFULL = D / 32;        // 32-wide steps of the first product
constexpr bool KTAIL = (D % 32) != 0;  // one 16-wide step more
constexpr int DB = D / 16;           // 16-wide blocks of the head dimension

// One tile of 16 rows meets one block of 32 keys: sc holds the raw scores (this lane: its row,
// keys base + 8 quad + e), vv the block's values as MFMA operands. Online softmax in base 2;
// the running maximum m is kept in scaled units (score * scale * log2 e). masked = false is for
// blocks every row of the tile sees in full, the common case away from the diagonal: no compare,
// no select. The rescale of the accumulator is skipped when no row's maximum moved.
// The scale is positive (checked on the host), so the maximum may be taken before scaling.
// Position -> (page of the block table, offset in the page). Division by a run-time number
// costs some thirty instructions per use; page sizes are powers of two in practice, so the
// kernels are built twice: P2 = true shifts and masks, P2 = false divides.
template <bool P2> __device__ __forceinline__ int page_div(int x, int ps, int shift) { return P2 ? x >> shift : x / ps; }
template <bool P2> __device__ __forceinline__ int page_mod(int x, int ps) { return P2 ? x & (ps - 1) : x % ps; }

// The first ``n`` of the 8 values of ``v`` (n <= 0: none, n >= 8: all), zeros for the others:
// four masks made once per group of keys and four ANDs per operand. A group of 8 keys that
// straddles the last key any row of the block of waves sees holds, after it, places nobody has
// written since the page's last holder: their probabilities are zero, but 0 x NaN is NaN, so
// the values themselves become zeros, key by key.
__device__ __forceinline__ bf16x8_t keep_first(bf16x8_t v, int n) {
  typedef unsigned int u32x4_t __attribute__((ext_vector_type(4)));
  u32x4_t bits = __builtin_bit_cast(u32x4_t, v);
#pragma unroll
  for (int j = 0; j < 4; ++j) bits[j] &= n >= 2 * j + 2 ? 0xffffffffu : (n == 2 * j + 1 ? 0x0000ffffu : 0u);
  return __builtin_bit_cast(bf16x8_t, bits);
}

// The larger of two, a NaN if either is one (IEEE 754-2019 maximum): one instruction, where
// fmaxf first quiets every operand whose origin the compiler cannot see (three for one).
__device__ __forceinline__ float max2(float a, float b) { return __builtin_elementwise_maximum(a, b); }

// max over the four lanes that hold one row (lane, lane ^ 16, lane ^ 32, lane ^ 48): two swaps of
// register halves between rows of 16 lanes, no LDS traffic and no address arithmetic
__device__ __forceinline__ float row_max4(float x) {
  typedef unsigned int u32x2_t __attribute__((ext_vector_type(2)));
  const unsigned int u = __float_as_uint(x);
  const u32x2_t a = __builtin_amdgcn_permlane16_swap(u, u, false, false);
  const float y = max2(__uint_as_float(a[0]), __uint_as_float(a[1]));
  const unsigned int v = __float_as_uint(y);
  const u32x2_t b = __builtin_amdgcn_permlane32_swap(v, v, false, false);
  return max2(__uint_as_float(b[0]), __uint_as_float(b[1]));
}

__device__ __forceinline__ void tile_update(const f32x4_t sc[2], const bf16x8_t* vv, bool masked, int base,
                                            int quad, bool row_valid, int qpos, int window, float scale_log2,
                                            float& m, float& l, f32x4_t* o) {
  float s[8];
#pragma unroll
  for (int e = 0; e < 8; ++e) s[e] = sc[e >> 2][e & 3];
  if (masked) {  // the same for the whole wave
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const int key = base + 8 * quad + e;
      const bool vis = row_valid && key <= qpos && (window == 0 || key > qpos - window);
      s[e] = vis ? s[e] : -INFINITY;
    }
  }
  float mx = -INFINITY;
#pragma unroll
  for (int e = 0; e < 8; ++e) mx = max2(mx, s[e]);
  mx = row_max4(mx);
  const float m_new = max2(m, mx * scale_log2);
  const float m_use = m_new == -INFINITY ? 0.f : m_new;  // a row that has seen no key yet
  // v_exp_f32 directly: results below the normal range may flush to zero, which is what they are worth here
  const float corr = __builtin_amdgcn_exp2f(m - m_use);
  float psum = 0.f;
  bf16x8_t pb;
#pragma unroll
  for (int e = 0; e < 8; ++e) {
    const float pe = __builtin_amdgcn_exp2f(fmaf(s[e], scale_log2, -m_use));
    psum += pe;
    pb[e] = (bf16_t)pe;
  }
  m = m_new;
  if (__any(corr != 1.0f)) {
    l *= corr;
#pragma unroll
    for (int i = 0; i < DB; ++i) o[i] *= corr;
  }
  l += psum;
#pragma unroll
  for (int i = 0; i < DB; ++i) o[i] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vv[i], pb, o[i], 0, 0, 0);
}

// The same for RT tiles of a wave at once, step by step across the tiles instead of tile by
// tile: the tiles' chains (scores -> maximum -> exponentials -> second product) do not depend
// on each other, and written side by side in one stretch of code without branches between them
// the exponentials of one tile can issue while the matrix pipe works on another's products.
template <int RT>
__device__ __forceinline__ void tiles_update(const f32x4_t (*sc)[2], const bf16x8_t* vv, unsigned whole, int base,
                                             int quad, const bool* row_valid, const int* qpos, int window,
                                             float scale_log2, float* m, float* l, f32x4_t (*o)[DB]) {
  // whole: bit t says that every row of tile t sees all 32 keys (one scalar for the wave: an
  // array of flags went through vector registers, a dozen instructions per block of keys)
  float s[RT][8];
#pragma unroll
  for (int t = 0; t < RT; ++t)
#pragma unroll
    for (int e = 0; e < 8; ++e) s[t][e] = sc[t][e >> 2][e & 3];
  if (whole != (1u << RT) - 1) {  // the same for the whole wave
#pragma unroll
    for (int t = 0; t < RT; ++t)
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        const int key = base + 8 * quad + e;
        const bool vis = ((whole >> t) & 1) || (row_valid[t] && key <= qpos[t] && (window == 0 || key > qpos[t] - window));
        s[t][e] = vis ? s[t][e] : -INFINITY;
      }
  }
  float m_use[RT], corr[RT];
  bool moved = false;
#pragma unroll
  for (int t = 0; t < RT; ++t) {
    float mx = -INFINITY;
#pragma unroll
    for (int e = 0; e < 8; ++e) mx = max2(mx, s[t][e]);
    mx = row_max4(mx);
    const float m_new = max2(m[t], mx * scale_log2);
    m_use[t] = m_new == -INFINITY ? 0.f : m_new;
    corr[t] = __builtin_amdgcn_exp2f(m[t] - m_use[t]);
    m[t] = m_new;
    moved |= corr[t] != 1.0f;
  }
  bf16x8_t pb[RT];
#pragma unroll
  for (int t = 0; t < RT; ++t) {
    float psum = 0.f;
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const float pe = __builtin_amdgcn_exp2f(fmaf(s[t][e], scale_log2, -m_use[t]));
      psum += pe;
      pb[t][e] = (bf16_t)pe;
    }
    l[t] = l[t] * corr[t] + psum;
  }
  if (__any(moved)) {
#pragma unroll
    for (int t = 0; t < RT; ++t)
#pragma unroll
      for (int i = 0; i < DB; ++i) o[t][i] *= corr[t];
  }
#pragma unroll
  for (int i = 0; i < DB; ++i)
#pragma unroll
    for (int t = 0; t < RT; ++t) o[t][i] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vv[i], pb[t], o[t][i], 0, 0, 0);
}

// ------------------------------------------------ keys and values straight from the pages
struct KvBlock {  // the keys and values of one block of 32 keys, as MFMA operands
  bf16x8_t k[2][KFULL > 0 ? KFULL : 1];
  bf16x8_t kt[2];
  bf16x8_t v[DB];
};

// Every load is unconditional: positions are clamped into [lo, pos_max], which lies in pages
// the sequence holds; what was read from a clamped place is masked (keys) or zeroed (values)
// before use. Loads under branches would make the compiler wait for all loads in flight
// wherever it can no longer count them.
template <bool P2>
__device__ __forceinline__ void block_pages(const int* __restrict__ table, int base, int lo, int pos_max, int ps,
                                            int r16, int quad, int pg[3]) {
  const int psh = __builtin_ctz(ps);
#pragma unroll
  for (int kb = 0; kb < 2; ++kb) {
    const int kidx = min(max(base + 8 * (r16 >> 2) + 4 * kb + (r16 & 3), lo), pos_max);
    pg[kb] = table[page_div<P2>(kidx, ps, psh)];
  }
  const int kv0 = min(max(base + 8 * quad, lo & ~7), pos_max & ~7);
  pg[2] = table[page_div<P2>(kv0, ps, psh)];
}

// ONCE: the block is the only reader of these keys and values in the step (decoding: one block
// per sequence and key head serves the whole group of query heads), so they are loaded
// non-temporally and leave the caches alone.
// live = false (uniform over the wave): a load past the wave's last block, issued only so that
// the loop has one shape; every lane then reads the cache's first bytes, a few lines for the
// whole wave, instead of a block of keys and values that nobody uses.
template <bool P2, bool ONCE = false>
__device__ __forceinline__ void block_load(const AttnTileArgs& a, int kvh, int base, int lo, int pos_max, int r16,
                                           int quad, const int pg[3], KvBlock& blk, bool live = true) {
  const int ps = a.page_size;
#pragma unroll
  for (int kb = 0; kb < 2; ++kb) {
    const int kidx = min(max(base + 8 * (r16 >> 2) + 4 * kb + (r16 & 3), lo), pos_max);
    const bf16_t* kp = live ? a.k_cache + (((size_t)pg[kb] * a.nkv + kvh) * ps + page_mod<P2>(kidx, ps)) * D : a.k_cache;
#pragma unroll
    for (int i = 0; i < KFULL; ++i)
      blk.k[kb][i] = ONCE ? load_once8(kp + 32 * i + 8 * quad) : *(const bf16x8_t*)(kp + 32 * i + 8 * quad);
    if (KTAIL) blk.kt[kb] = load_tail(kp + 32 * KFULL, quad);
  }
  const int kv0 = min(max(base + 8 * quad, lo & ~7), pos_max & ~7);
  const bf16_t* vp = live ? a.v_cache + (((size_t)pg[2] * a.nkv + kvh) * D + r16) * ps + page_mod<P2>(kv0, ps) : a.v_cache;
#pragma unroll
  for (int i = 0; i < DB; ++i)
    blk.v[i] = ONCE ? load_once8(vp + (size_t)16 * i * ps) : *(const bf16x8_t*)(vp + (size_t)16 * i * ps);
}

// General kernel (prompt portions and mixed batches). A wave owns RT tiles of 16
// rows each, 16 * RT consecutive rows of the sequence's row matrix; a block is
// four waves, 64 * RT rows. The keys and values of a block of 32 keys are read
// once into registers and multiplied with all RT tiles, which divides the
// operand traffic per MFMA by RT.
template <int RT, bool P2>
__global__ __launch_bounds__(256, RT <= 2 ? 2 : 1) void attention_bf16_kernel(AttnTileArgs a) {
  const int lane = threadIdx.x & 63, wave = uniform_wave_number();
  const int r16 = lane & 15, quad = lane >> 4;
  // blocks of one tile are neighbours in the launch order, one per key head: with as many key
  // heads as XCDs, a head's keys and values stay in one XCD's L2
  const int tile = blockIdx.x / a.nkv, kvh = blockIdx.x - tile * a.nkv, split = blockIdx.z;
  const int seq = a.tile_seq[tile];
  const int g = a.nq / a.nkv;
  const int q_begin = a.cu_q[seq];
  const int q_len = a.cu_q[seq + 1] - q_begin;
  const int kv_len = a.kv_lens[seq];
  const int n_rows = q_len * g;
  const int row0 = a.tile_row0[tile] + 16 * RT * wave;
  if (row0 >= n_rows) return;
  const int first_pos = kv_len - q_len;
  const int ps = a.page_size, psh = __builtin_ctz(ps);
  const int* table = a.block_table + (size_t)seq * a.table_width;

  // per tile: this lane's row, its token's position, and Q as B operands kept for the whole loop
  bool row_valid[RT];
  int qpos[RT], tile_pos_min[RT], tile_pos_max[RT];  // this lane's position; the tile's range of positions
  size_t row_index[RT];
  bf16x8_t qreg[RT][KFULL > 0 ? KFULL : 1];
  bf16x8_t qtail[RT];
#pragma unroll
  for (int t = 0; t < RT; ++t) {
    const int my_row = row0 + 16 * t + r16;
    row_valid[t] = my_row < n_rows;
    const int row_c = row_valid[t] ? my_row : n_rows - 1;
    const int tok = row_c / g, hg = row_c - tok * g;
    qpos[t] = first_pos + tok;
    // the same for every lane: kept in scalar registers so that the choice below is a plain branch
    tile_pos_min[t] = __builtin_amdgcn_readfirstlane(first_pos + min(row0 + 16 * t, n_rows - 1) / g);
    tile_pos_max[t] = __builtin_amdgcn_readfirstlane(first_pos + min(row0 + 16 * t + 15, n_rows - 1) / g);
    row_index[t] = (size_t)(q_begin + tok) * a.nq + kvh * g + hg;
    const bf16_t* qp = a.q + row_index[t] * D;
#pragma unroll
    for (int i = 0; i < KFULL; ++i) qreg[t][i] = *(const bf16x8_t*)(qp + 32 * i + 8 * quad);
    qtail[t] = load_tail(qp, 2);  // zeros
    if (KTAIL) qtail[t] = load_tail(qp + 32 * KFULL, quad);
  }

  // keys this wave may need: [lo, pos_max]
  const int row_last = min(row0 + 16 * RT - 1, n_rows - 1);
  const int pos_min = first_pos + row0 / g, pos_max = first_pos + row_last / g;
  const int lo = a.window > 0 ? max(0, pos_min - a.window + 1) : 0;
  const int blk_begin = lo >> 5, blk_end = (pos_max >> 5) + 1;
  const int per = (blk_end - blk_begin + a.num_splits - 1) / a.num_splits;
  const int b0 = blk_begin + split * per;
  const int b1 = min(blk_end, b0 + per);

  f32x4_t o[RT][DB];
  float m[RT], l[RT];
#pragma unroll
  for (int t = 0; t < RT; ++t) {
    m[t] = -INFINITY;
    l[t] = 0.f;
#pragma unroll
    for (int i = 0; i < DB; ++i) o[t][i] = (f32x4_t){0.f, 0.f, 0.f, 0.f};
  }

  // page numbers are looked up one block ahead of the loads that need them; all loads are
  // unconditional (clamped), see block_pages / block_load
  if (b0 < b1) {
    int pg[3], pg_next[3];
    block_pages<P2>(table, b0 << 5, lo, pos_max, ps, r16, quad, pg);
    for (int b = b0; b < b1; ++b) {
      const int base = b << 5;
      KvBlock blk;
      block_load<P2>(a, kvh, base, lo, pos_max, r16, quad, pg, blk);
      block_pages<P2>(table, min(b + 1, b1 - 1) << 5, lo, pos_max, ps, r16, quad, pg_next);
      // values of keys outside [lo, pos_max] came from a clamped place, or from places after the
      // sequence's last key in its last page, and may be anything
      const int kv0 = base + 8 * quad;
      if (base < lo || base + 31 > pos_max) {  // the same for the whole wave
        const int keep = kv0 + 7 >= lo ? pos_max - kv0 + 1 : 0;
#pragma unroll
        for (int i = 0; i < DB; ++i) blk.v[i] = keep_first(blk.v[i], keep);
      }
#pragma unroll
      for (int t = 0; t < RT; ++t) {
        f32x4_t s[2];
#pragma unroll
        for (int kb = 0; kb < 2; ++kb) {
          f32x4_t acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
          for (int i = 0; i < KFULL; ++i)
            acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(blk.k[kb][i], qreg[t][i], acc, 0, 0, 0);
          if (KTAIL) acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(blk.kt[kb], qtail[t], acc, 0, 0, 0);
          s[kb] = acc;
        }
        // every row of the tile sees the whole block unless it touches the diagonal or the window's edge
        const bool whole = base + 31 <= tile_pos_min[t] && (a.window == 0 || base > tile_pos_max[t] - a.window);
        tile_update(s, blk.v, !whole, base, quad, row_valid[t], qpos[t], a.window, a.scale_log2, m[t], l[t], o[t]);
      }
#pragma unroll
      for (int i = 0; i < 3; ++i) pg[i] = pg_next[i];
    }
  }

#pragma unroll
  for (int t = 0; t < RT; ++t) {
    float lt = l[t];
    lt += __shfl_xor(lt, 16, 64);
    lt += __shfl_xor(lt, 32, 64);
    if (!row_valid[t]) continue;
    const float inv = lt > 0.f ? 1.0f / lt : 0.f;
    if (a.num_splits == 1) {
      bf16_t* op = a.out + row_index[t] * D;
#pragma unroll
      for (int i = 0; i < DB; ++i) {
        bf16x4_t w;
#pragma unroll
        for (int r = 0; r < 4; ++r) w[r] = (bf16_t)(o[t][i][r] * inv);
        *(bf16x4_t*)(op + 16 * i + 4 * quad) = w;
      }
    } else {
      float* op = a.part_o + (row_index[t] * a.num_splits + split) * D;
#pragma unroll
      for (int i = 0; i < DB; ++i) {
        f32x4_t w = o[t][i] * inv;
        *(f32x4_t*)(op + 16 * i + 4 * quad) = w;
      }
      if (quad == 0) a.part_lse[row_index[t] * a.num_splits + split] = lt > 0.f ? m[t] + log2f(lt) : -INFINITY;
    }
  }
}

// Long portions: the same tiling (a wave owns RT tiles of 16 rows, a block four waves), but the
// keys and values of a block of 32 keys are brought into LDS once per block of waves instead
// of once per wave, and the next block's loads are in flight while the current one is
// multiplied: 256 threads each fetch a few 16-byte pieces into registers, the waves multiply
// from the other LDS stage, then the registers are stored and one barrier ends the round.
// LDS rows are padded to strides of 32 bytes modulo 64. Measured on the device with
// ds_read_b128, lane 16 q + r reading row r at 16 q bytes (an MFMA operand): such rows are
// read at 220 B/clk per compute unit, the full rate, rows of 16 bytes modulo 64 (D + 8
// elements at D = 128; 40 elements) at half of it. (All patterns tried fit this: in one cycle
// the LDS serves lanes 0-7 together with lanes 24-31, and so on, 64 banks of 4 bytes. The
// kernel's time did not change with it: it is not bound by LDS reads.)
constexpr int KROW = D % 32 == 0 ? D + 16 : D;  // elements per key row in LDS
// Two tiles of a wave meet a block of 32 keys, with the rows' reference maxima moved lazily.
// The exponentials are taken against a reference m that may lie below the row's true maximum by
// up to LAZY (in units of the scaled scores, base 2): probabilities then reach 2^LAZY at most,
// which bfloat16 and the float32 sums hold as well as values below one, and the quotient of
// accumulator and sum does not change. As long as no score of the wave rises above its row's
// reference by more than that, and no tile touches the diagonal or a window's edge, a round is
// two stretches of code without a branch: products and lane-local maxima, then exponentials and
// second products, which the compiler can place side by side. No maximum across the four lanes
// of a row, no factor for the accumulator, no test whether it moved. Otherwise (the first block
// of keys, the blocks at the diagonal, a row whose scores jump) the reference is set to the true
// maximum and the accumulator shrunk as in tiles_update.
constexpr float LAZY = 8.0f;

__device__ __forceinline__ void tile_mask(f32x4_t sc[2], int base, int quad, bool row_valid, int qpos, int window) {
#pragma unroll
  for (int e = 0; e < 8; ++e) {
    const int key = base + 8 * quad + e;
    const bool vis = row_valid && key <= qpos && (window == 0 || key > qpos - window);
    sc[e >> 2][e & 3] = vis ? sc[e >> 2][e & 3] : -INFINITY;
  }
}

__device__ __forceinline__ float lane_max(const f32x4_t sc[2]) {
  float mx = -INFINITY;
#pragma unroll
  for (int e = 0; e < 8; ++e) mx = max2(mx, sc[e >> 2][e & 3]);
  return mx;
}

// the slow part: reference to the true maximum, sum and accumulator shrunk to it
__device__ __forceinline__ void tile_move_reference(float lane_mx, float scale_log2, float& m, float& l, f32x4_t* o) {
  const float m_new = max2(m, row_max4(lane_mx) * scale_log2);
  const float m_use = m_new == -INFINITY ? 0.f : m_new;  // a row that has seen no key yet
  const float corr = __builtin_amdgcn_exp2f(m - m_use);
  m = m_new;
  l *= corr;
#pragma unroll
  for (int i = 0; i < DB; ++i) o[i] *= corr;
}

__device__ __forceinline__ void tile_probabilities(const f32x4_t sc[2], float scale_log2, float m, float& l,
                                                   bf16x8_t& pb) {
  const float m_use = m == -INFINITY ? 0.f : m;
  float psum = 0.f;
#pragma unroll
  for (int e = 0; e < 8; ++e) {
    const float pe = __builtin_amdgcn_exp2f(fmaf(sc[e >> 2][e & 3], scale_log2, -m_use));
    psum += pe;
    pb[e] = (bf16_t)pe;
  }
  l += psum;
}

constexpr int VROW = 48;                        // elements per value row (one head element, 32 keys) in LDS
constexpr int STAGE_ELEMS = 32 * KROW + D * VROW;

//
// G = 2: eight waves, two groups of four that both own the block's rows and take the blocks of
// keys in turn (group 0 the even ones of the block's range, group 1 the odd ones), each with LDS
// stages, running maxima, sums and accumulators of its own; at the end group 1 hands its sums
// over through LDS and group 0 joins them. A causal prompt without history is a triangle: the row
// tile at its end walks 64 blocks of keys at 2,048 tokens, the one at its start one, and a wave's
// round is a chain (products, maxima, exponentials, products) that another wave on the SIMD
// hides only in part: a block alone on its compute unit walked a round in 0.78 of the time it
// takes beside a second block. So the longest tile alone set the kernel's time (64 rounds; 72 us
// where an even spread of the rounds over the compute units would take 48). Cut this way the
// longest chain is half as long, a compute unit holds one block of eight waves at a time, and
// the blocks, longest first, are dealt out as compute units fall free.
template <int RT, bool P2, int G>
__global__ __launch_bounds__(256 * G, G == 1 ? 2 : 1) void attention_bf16_prefill_kernel(AttnTileArgs a) {
  extern __shared__ bf16_t lds_kv[];  // [G][2][STAGE_ELEMS]
  const int lane = threadIdx.x & 63, wave_of_block = uniform_wave_number();
  const int grp = G == 1 ? 0 : wave_of_block >> 2, wave = G == 1 ? wave_of_block : wave_of_block & 3;
  const int r16 = lane & 15, quad = lane >> 4;
  const int tile = blockIdx.x / a.nkv, kvh = blockIdx.x - tile * a.nkv, split = blockIdx.z;
  const int seq = a.tile_seq[tile];
  const int g = a.nq / a.nkv;
  const int q_begin = a.cu_q[seq];
  const int q_len = a.cu_q[seq + 1] - q_begin;
  const int kv_len = a.kv_lens[seq];
  const int n_rows = q_len * g;
  const int tile_row0 = a.tile_row0[tile];  // first row of the block of waves; < n_rows
  const int row0 = tile_row0 + 16 * RT * wave;
  const bool wave_has_rows = row0 < n_rows;
  const int first_pos = kv_len - q_len;
  const int ps = a.page_size, psh = __builtin_ctz(ps);
  const int* table = a.block_table + (size_t)seq * a.table_width;

  bool row_valid[RT];
  int qpos[RT], tile_pos_min[RT], tile_pos_max[RT];  // this lane's position; the tile's range of positions
  size_t row_index[RT];
  bf16x8_t qreg[RT][KFULL > 0 ? KFULL : 1];
  bf16x8_t qtail[RT];
#pragma unroll
  for (int t = 0; t < RT; ++t) {
    const int my_row = row0 + 16 * t + r16;
    row_valid[t] = my_row < n_rows;
    const int row_c = min(my_row, n_rows - 1);
    const int tok = row_c / g, hg = row_c - tok * g;
    qpos[t] = first_pos + tok;
    // the same for every lane: kept in scalar registers so that the choice below is a plain branch
    tile_pos_min[t] = __builtin_amdgcn_readfirstlane(first_pos + min(row0 + 16 * t, n_rows - 1) / g);
    tile_pos_max[t] = __builtin_amdgcn_readfirstlane(first_pos + min(row0 + 16 * t + 15, n_rows - 1) / g);
    row_index[t] = (size_t)(q_begin + tok) * a.nq + kvh * g + hg;
    const bf16_t* qp = a.q + row_index[t] * D;
#pragma unroll
    for (int i = 0; i < KFULL; ++i) qreg[t][i] = *(const bf16x8_t*)(qp + 32 * i + 8 * quad);
    qtail[t] = load_tail(qp, 2);  // zeros
    if (KTAIL) qtail[t] = load_tail(qp + 32 * KFULL, quad);
  }

  // keys the block of waves needs, and the part of them this wave needs
  const int blk_last_row = min(tile_row0 + 64 * RT - 1, n_rows - 1);
  const int blk_pos_min = first_pos + tile_row0 / g, blk_pos_max = first_pos + blk_last_row / g;
  const int lo = a.window > 0 ? max(0, blk_pos_min - a.window + 1) : 0;
  // the blocks of keys of this block of waves, and of them the part of this split
  const int all_b0 = lo >> 5, all_b1 = (blk_pos_max >> 5) + 1;
  const int per = (all_b1 - all_b0 + a.num_splits - 1) / a.num_splits;
  const int b0 = all_b0 + split * per, b1 = min(all_b1, b0 + per);
  int wb0 = b1, wb1 = b0;  // this wave's blocks: none unless it has rows
  if (wave_has_rows) {
    const int row_last = min(row0 + 16 * RT - 1, n_rows - 1);
    const int pos_min = first_pos + row0 / g, pos_max = first_pos + row_last / g;
    wb0 = (a.window > 0 ? max(0, pos_min - a.window + 1) : 0) >> 5;
    wb1 = min((pos_max >> 5) + 1, b1);  // not into the next split's blocks
  }

  f32x4_t o[RT][DB];
  float m[RT], l[RT];
#pragma unroll
  for (int t = 0; t < RT; ++t) {
    m[t] = -INFINITY;
    l[t] = 0.f;
#pragma unroll
    for (int i = 0; i < DB; ++i) o[t][i] = (f32x4_t){0.f, 0.f, 0.f, 0.f};
  }

  // Who fetches what. A block of 32 keys is four groups of 8 consecutive keys, one per wave.
  // Pages hold a multiple of 8 keys, so a group lies in one page: the wave needs ONE block-table
  // entry per block, found with scalar instructions, for its keys (8 rows of D elements, one
  // contiguous piece of memory) and for the same 8 keys of the transposed values (one 16-byte
  // piece per head element). Entries are looked up one round before the loads that need them:
  // lookup(b + 2) and fetch(b + 1) are in flight while block b is multiplied. Every load is
  // unconditional (the group's first key is clamped into pages the sequence holds; what lies
  // outside is masked with the scores or zeroed by a select): with loads under branches the
  // compiler can no longer count which are in flight and waits for all of them in the middle of
  // the products.
  const size_t page_stride = (size_t)a.nkv * ps * D;  // elements per page, keys and values alike
  const bf16_t* k_head = a.k_cache + (size_t)kvh * ps * D;
  const bf16_t* v_head = a.v_cache + (size_t)kvh * D * ps;
  const int w8 = 8 * wave;  // this wave's group within a block
  constexpr int LANE_PIECES = (D + 63) / 64;   // 16-byte pieces per lane, of keys and of values
  constexpr bool ALL_LANES = D % 64 == 0;
  struct Pieces { bf16x8_t k[LANE_PIECES], v[LANE_PIECES]; };
  Pieces set_a, set_b;  // two blocks of keys on their way: one asked for a round ago, one just now
  auto group_start = [&](int b) { return min(max((b << 5) + w8, lo & ~7), blk_pos_max & ~7); };
  auto lookup = [&](int b) { return table[page_div<P2>(group_start(b), ps, psh)]; };
  auto fetch = [&](int b, int page, Pieces& in) {  // global -> registers
    const int off = page_mod<P2>(group_start(b), ps);
    const bf16_t* kp = k_head + (size_t)page * page_stride + (size_t)off * D;  // 8 keys: 8 D elements in a row
    const bf16_t* vp = v_head + (size_t)page * page_stride + off;
#pragma unroll
    for (int i = 0; i < LANE_PIECES; ++i) {
      const int c = lane + 64 * i;
      if (ALL_LANES || c < D) {
        in.k[i] = *(const bf16x8_t*)(kp + 8 * c);
        in.v[i] = *(const bf16x8_t*)(vp + (size_t)c * ps);
      }
    }
  };
  auto stash = [&](int b, int stage, const Pieces& in) {  // registers -> LDS: block b into its stage
    bf16_t* kb = lds_kv + (2 * grp + stage) * STAGE_ELEMS;
    bf16_t* vb = kb + 32 * KROW;
    // values of keys no row of the block sees were read from a clamped place, or lie after the
    // sequence's last key in its last page: they may be anything, and 0 * NaN is NaN, so they
    // become zeros
    const int g0 = (b << 5) + w8;
    const int keep = g0 + 7 >= lo ? blk_pos_max - g0 + 1 : 0;
#pragma unroll
    for (int i = 0; i < LANE_PIECES; ++i) {
      const int c = lane + 64 * i;
      if (ALL_LANES || c < D) {
        // keys: piece c of the group is key c / (D / 8) of it, elements 8 (c % (D / 8)) onward; row
        // 16 s2 + r16 of the stage holds the key that lane r16 of sub-block s2 multiplies (key
        // 8 q + 4 s2 + r of the block sits in row 16 s2 + 4 q + r), so that the 16 lanes of an
        // operand read 16 consecutive padded rows, all in different banks
        const int kl = c / (D / 8), part = c - kl * (D / 8);
        const int row = 16 * (kl >> 2) + (w8 >> 1) + (kl & 3);
        *(bf16x8_t*)(kb + row * KROW + 8 * part) = in.k[i];
        *(bf16x8_t*)(vb + c * VROW + w8) = keep_first(in.v[i], keep);
      }
    }
  };

  // The first block is fetched and stored on every path, also by a split that is left without
  // blocks (it takes the sequence's last block and never looks at it): the wait for these
  // loads then also settles, for the compiler, that the queries have arrived. Were it under a
  // branch, the waits it places for the queries inside the loop would also wait for the loads
  // of the block after next, in the middle of the products.
  // Keys and values are asked for two rounds before they are multiplied (a round takes about as
  // long as a load that hits in L2: with one round of lead the store to LDS sometimes waited for
  // it; measured 2 to 7 % off the kernel's time). Set A carries the blocks of even rounds, set B
  // those of odd rounds; a set is free again once its block has been stored.
  // A group's blocks are b0 + grp, b0 + grp + G, ...; every group runs the rounds of the one
  // with the most blocks (the barriers are the whole block's), the last of them idle if need be.
  const int b_first = min(b0 + grp, all_b1 - 1);
  const int b_last = max(b1 - 1, b_first);  // loads past the end repeat the last block and are not used
  auto multiply = [&](int b, int stage) {
    if (b >= wb0 && b < wb1) {  // uniform over the wave
      const int base = b << 5;
      const bf16_t* kb = lds_kv + (2 * grp + stage) * STAGE_ELEMS;
      const bf16_t* vb = kb + 32 * KROW;
      bf16x8_t kk[2][KFULL > 0 ? KFULL : 1], kt[2];
#pragma unroll
      for (int s2 = 0; s2 < 2; ++s2) {
        const bf16_t* kp = kb + (16 * s2 + r16) * KROW;
#pragma unroll
        for (int i = 0; i < KFULL; ++i) kk[s2][i] = *(const bf16x8_t*)(kp + 32 * i + 8 * quad);
        if (KTAIL) {
          kt[s2] = load_tail(kp, 2);
          if (quad < 2) kt[s2] = *(const bf16x8_t*)(kp + 32 * KFULL + 8 * quad);
        }
      }
      bf16x8_t vv[DB];
#pragma unroll
      for (int i = 0; i < DB; ++i) vv[i] = *(const bf16x8_t*)(vb + (16 * i + r16) * VROW + 8 * quad);

      auto scores = [&](int t, f32x4_t sc[2]) {
#pragma unroll
        for (int s2 = 0; s2 < 2; ++s2) {
          f32x4_t acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
          for (int i = 0; i < KFULL; ++i)
            acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kk[s2][i], qreg[t][i], acc, 0, 0, 0);
          if (KTAIL) acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kt[s2], qtail[t], acc, 0, 0, 0);
          sc[s2] = acc;
        }
      };
      // every row of the tile sees the whole block unless it touches the diagonal or the window's edge
      auto sees_all = [&](int t) {
        return (base + 31 <= tile_pos_min[t]) & ((a.window == 0) | (base > tile_pos_max[t] - a.window));
      };
      if constexpr (RT == 2) {
        f32x4_t sc0[2], sc1[2];
        bf16x8_t pb0, pb1;
        scores(0, sc0);
        scores(1, sc1);
        const bool edge = !(sees_all(0) & sees_all(1));  // the same for the whole wave
        float mx0 = lane_max(sc0), mx1 = lane_max(sc1);
        const bool jumps = mx0 * a.scale_log2 > m[0] + LAZY || mx1 * a.scale_log2 > m[1] + LAZY;
        if (edge || __any(jumps)) {
          if (!sees_all(0)) {
            tile_mask(sc0, base, quad, row_valid[0], qpos[0], a.window);
            mx0 = lane_max(sc0);
          }
          if (!sees_all(1)) {
            tile_mask(sc1, base, quad, row_valid[1], qpos[1], a.window);
            mx1 = lane_max(sc1);
          }
          tile_move_reference(mx0, a.scale_log2, m[0], l[0], o[0]);
          tile_move_reference(mx1, a.scale_log2, m[1], l[1], o[1]);
        }
        tile_probabilities(sc0, a.scale_log2, m[0], l[0], pb0);
        tile_probabilities(sc1, a.scale_log2, m[1], l[1], pb1);
#pragma unroll
        for (int i = 0; i < DB; ++i) o[0][i] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vv[i], pb0, o[0][i], 0, 0, 0);
#pragma unroll
        for (int i = 0; i < DB; ++i) o[1][i] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vv[i], pb1, o[1][i], 0, 0, 0);
      } else {
        f32x4_t sc[RT][2];
        unsigned whole = 0;
#pragma unroll
        for (int t = 0; t < RT; ++t) {
          scores(t, sc[t]);
          whole |= (unsigned)sees_all(t) << t;
        }
        tiles_update<RT>(sc, vv, whole, base, quad, row_valid, qpos, a.window, a.scale_log2, m, l, o);
      }
    }
  };
  int page = lookup(b_first);
  fetch(b_first, page, set_a);
  page = lookup(min(b0 + grp + G, b_last));
  stash(b_first, 0, set_a);
  fetch(min(b0 + grp + G, b_last), page, set_b);
  page = lookup(min(b0 + grp + 2 * G, b_last));
  __syncthreads();
  for (int round = b0; round < b1; round += 2 * G) {
    const int b = round + grp;  // this group's block of the even round; b + G the odd round's
    // even round: set A is free, set B holds block b + G
    fetch(min(b + 2 * G, b_last), page, set_a);
    page = lookup(min(b + 3 * G, b_last));
    multiply(b, 0);
    stash(min(b + G, b_last), 1, set_b);
    __syncthreads();
    // odd round: set B is free, set A holds block b + 2 G. With an odd number of blocks the last
    // odd round has nothing to multiply (b + G >= b1 lies outside every wave's range) and only
    // fetches and stores the last block once more. Leaving the loop here instead gave the
    // compiler a path back to the loop's head with set A's loads in flight, and made it wait
    // for every load at the head of every round.
    fetch(min(b + 3 * G, b_last), page, set_b);
    page = lookup(min(b + 4 * G, b_last));
    multiply(b + G, 1);
    stash(min(b + 2 * G, b_last), 0, set_a);
    __syncthreads();
  }

  if constexpr (G == 2) {
    // Group 1 hands its reference maxima, sums and accumulators to group 0, lane to lane (the two
    // hold the same rows in the same lanes), through the LDS the stages no longer need (the loop's
    // last barrier lies behind every read of them). Both references are lazy ones, below the
    // rows' maxima by 2^LAZY at most; the join takes the larger and shrinks the other side.
    f32x4_t* xo = (f32x4_t*)lds_kv;                                 // [4 waves][RT][DB][64 lanes]
    float* xm = (float*)(xo + 4 * RT * DB * 64);                    // [4 waves][RT][2][64 lanes]
    if (grp == 1) {
#pragma unroll
      for (int t = 0; t < RT; ++t) {
#pragma unroll
        for (int i = 0; i < DB; ++i) xo[((wave * RT + t) * DB + i) * 64 + lane] = o[t][i];
        xm[((wave * RT + t) * 2 + 0) * 64 + lane] = m[t];
        xm[((wave * RT + t) * 2 + 1) * 64 + lane] = l[t];
      }
    }
    __syncthreads();
    if (grp == 0) {
#pragma unroll
      for (int t = 0; t < RT; ++t) {
        const float m1 = xm[((wave * RT + t) * 2 + 0) * 64 + lane], l1 = xm[((wave * RT + t) * 2 + 1) * 64 + lane];
        const float m_new = max2(m[t], m1);
        const float m_use = m_new == -INFINITY ? 0.f : m_new;
        const float f0 = __builtin_amdgcn_exp2f(m[t] - m_use), f1 = __builtin_amdgcn_exp2f(m1 - m_use);
        m[t] = m_new;
        l[t] = l[t] * f0 + l1 * f1;
#pragma unroll
        for (int i = 0; i < DB; ++i) o[t][i] = o[t][i] * f0 + xo[((wave * RT + t) * DB + i) * 64 + lane] * f1;
      }
    }
  }

#pragma unroll
  for (int t = 0; t < RT; ++t) {
    float lt = l[t];
    lt += __shfl_xor(lt, 16, 64);
    lt += __shfl_xor(lt, 32, 64);
    if (!row_valid[t] || !wave_has_rows || grp != 0) continue;
    const float inv = lt > 0.f ? 1.0f / lt : 0.f;
    if (a.num_splits == 1) {
      bf16_t* op = a.out + row_index[t] * D;
#pragma unroll
      for (int i = 0; i < DB; ++i) {
        bf16x4_t w;
#pragma unroll
        for (int r = 0; r < 4; ++r) w[r] = (bf16_t)(o[t][i][r] * inv);
        *(bf16x4_t*)(op + 16 * i + 4 * quad) = w;
      }
    } else {
      float* op = a.part_o + (row_index[t] * a.num_splits + split) * D;
#pragma unroll
      for (int i = 0; i < DB; ++i) {
        f32x4_t w = o[t][i] * inv;
        *(f32x4_t*)(op + 16 * i + 4 * quad) = w;
      }
      if (quad == 0) a.part_lse[row_index[t] * a.num_splits + split] = lt > 0.f ? m[t] + log2f(lt) : -INFINITY;
    }
  }
}

// Few splits: every load is asked for before the first is used (clamped indices, so none stands
// under a branch), one trip to memory instead of two; the sums are those of the kernel's loop.
// A thread takes elements threadIdx.x and threadIdx.x + blockDim.x of the row.
template <int MAX>
__device__ __forceinline__ void merge_few(const float* __restrict__ part_o, const float* __restrict__ lse,
                                          bf16_t* __restrict__ out, int num_splits, size_t row) {
  float ls[MAX], pv[2][MAX];
  const int d0 = min((int)threadIdx.x, D - 1), d1 = min((int)(threadIdx.x + blockDim.x), D - 1);
#pragma unroll
  for (int s = 0; s < MAX; ++s) {
    const int sc = min(s, num_splits - 1);
    ls[s] = lse[sc];
    pv[0][s] = part_o[(row * num_splits + sc) * D + d0];
    pv[1][s] = part_o[(row * num_splits + sc) * D + d1];
  }
  float mx = -INFINITY;
#pragma unroll
  for (int s = 0; s < MAX; ++s) mx = fmaxf(mx, ls[s]);
  float acc[2] = {0.f, 0.f}, wsum = 0.f;
  if (mx != -INFINITY) {
#pragma unroll
    for (int s = 0; s < MAX; ++s) {
      if (s < num_splits) {
        const float w = exp2f(ls[s] - mx);
        wsum += w;
        if (w > 0.f) {  // the part of an empty split was never written
          acc[0] += w * pv[0][s];
          acc[1] += w * pv[1][s];
        }
      }
    }
  }
  if ((int)threadIdx.x < D) out[row * D + threadIdx.x] = (bf16_t)(wsum > 0.f ? acc[0] / wsum : 0.f);
  if ((int)(threadIdx.x + blockDim.x) < D)
    out[row * D + threadIdx.x + blockDim.x] = (bf16_t)(wsum > 0.f ? acc[1] / wsum : 0.f);
}

// out[row] = sum_s 2^(lse_s - M) O_s / sum_s 2^(lse_s - M); empty splits weigh 0
__global__ void attention_merge_kernel(const float* __restrict__ part_o, const float* __restrict__ part_lse,
                                       bf16_t* __restrict__ out, int num_splits, const int* __restrict__ tokens,
                                       int nq) {
  // rows are (token, query head); with a token list the grid walks the listed tokens' rows only
  const size_t row = tokens ? (size_t)tokens[blockIdx.x / nq] * nq + blockIdx.x % nq : blockIdx.x;
  const float* lse = part_lse + row * num_splits;
  if (num_splits <= 64 && D <= 2 * (int)blockDim.x) {
    if (num_splits <= 8) merge_few<8>(part_o, lse, out, num_splits, row);
    else if (num_splits <= 16) merge_few<16>(part_o, lse, out, num_splits, row);
    else if (num_splits <= 32) merge_few<32>(part_o, lse, out, num_splits, row);
    else merge_few<64>(part_o, lse, out, num_splits, row);
    return;
  }
  float mx = -INFINITY;
  for (int s = 0; s < num_splits; ++s) mx = fmaxf(mx, lse[s]);
  for (int d = threadIdx.x; d < D; d += blockDim.x) {
    float acc = 0.f, wsum = 0.f;
    if (mx != -INFINITY) {
      const float* po = part_o + row * num_splits * D + d;
#pragma unroll 8
      for (int s = 0; s < num_splits; ++s) {
        const float w = exp2f(lse[s] - mx);
        wsum += w;
        if (w > 0.f) acc += w * po[(size_t)s * D];
      }
    }
    out[row * D + d] = (bf16_t)(wsum > 0.f ? acc / wsum : 0.f);
  }
}

// ------------------------------------------------------------------ decoding
// Tiles of at most 16 rows (a decoded token's g query heads, or a very short
// portion): one block of DW waves per (tile, key head, split). The waves take the
// block's 32-key blocks round-robin, each with its own running maximum, sum and
// accumulator; the keys and values of the next two blocks are on their way while
// one is multiplied, and page numbers are fetched two blocks further ahead, so that
// no load waits for another. The waves' results meet in LDS. With several splits each
// block writes its normalised part and the base-2 log of its sum, and a second
// small kernel merges them. (Merging in the block that arrives last at a counter
// needs a device-scope fence in every block; with one L2 per XCD that fence costs
// more than the second launch: measured 355 us against 98 us at 64 sequences. With
// write-through atomic stores in place of the fence it costs what the second launch
// costs.)
constexpr int DW = 4;

// The 32-key blocks of the cache that a tile of the decode kernel walks: [begin, end). `fused`:
// the cache holds the keys before the tile's one token (which the kernel adds from registers).
__device__ __forceinline__ void decode_key_blocks(int kv_len, int q_len, int window, bool fused, int& begin, int& end) {
  const int own = fused ? 1 : 0;
  const int first_pos = kv_len - q_len;
  const int pos_max = first_pos + max(q_len, 1) - 1 - own;
  const int lo = window > 0 ? max(0, first_pos - window + 1) : 0;
  const bool any_cached = !fused || (pos_max >= lo && window != 1);
  begin = lo >> 5;
  end = any_cached ? (pos_max >> 5) + 1 : begin;
}

// The work list of a decode launch in pieces (AttnTileArgs::items). One block; up to LIST_TILES
// sequences. Every sequence has at least one piece (its last piece also takes the token's own key
// in the fused form), at most ceil(blocks / split_blocks).
constexpr int LIST_TILES = 1024;
__global__ __launch_bounds__(256) void attention_work_list_kernel(AttnTileArgs a, int fused) {
  __shared__ int whole[LIST_TILES + 1], rest[LIST_TILES + 1];  // pieces of each tile, then where they begin
  for (int t = threadIdx.x; t < a.num_tiles; t += blockDim.x) {
    const int seq = a.tile_seq ? a.tile_seq[t] : t;
    int begin, end;
    decode_key_blocks(a.kv_lens[seq], a.cu_q[seq + 1] - a.cu_q[seq], a.window, fused != 0, begin, end);
    const int blocks = end - begin;
    whole[t] = blocks / a.split_blocks;
    rest[t] = blocks % a.split_blocks != 0 || blocks == 0 ? 1 : 0;
  }
  __syncthreads();
  if (threadIdx.x == 0) {
    int at = 0;
    for (int t = 0; t < a.num_tiles; ++t) { const int n = whole[t]; whole[t] = at; at += n; }
    whole[a.num_tiles] = at;
    for (int t = 0; t < a.num_tiles; ++t) { const int n = rest[t]; rest[t] = at; at += n; }
    rest[a.num_tiles] = at;
  }
  __syncthreads();
  for (int t = threadIdx.x; t < a.num_tiles; t += blockDim.x) {
    const int seq = a.tile_seq ? a.tile_seq[t] : t;
    const int n_whole = whole[t + 1] - whole[t];
    for (int p = 0; p < n_whole; ++p) {
      const int at = whole[t] + p;
      if (at < a.max_items) { a.items[2 * at] = seq; a.items[2 * at + 1] = p; }
    }
    if (rest[t + 1] > rest[t] && rest[t] < a.max_items) { a.items[2 * rest[t]] = seq; a.items[2 * rest[t] + 1] = n_whole; }
  }
  for (int i = rest[a.num_tiles] + threadIdx.x; i < a.max_items; i += blockDim.x) { a.items[2 * i] = -1; a.items[2 * i + 1] = 0; }
}

__device__ __forceinline__ void block_compute(KvBlock& blk, const bf16x8_t* qreg, bf16x8_t qtail, int base, int lo,
                                              int pos_min, int pos_max, int quad, bool row_valid, int qpos,
                                              int window, float scale_log2, float& m, float& l, f32x4_t* o) {
  f32x4_t s[2];
#pragma unroll
  for (int kb = 0; kb < 2; ++kb) {
    f32x4_t acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int i = 0; i < KFULL; ++i) acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(blk.k[kb][i], qreg[i], acc, 0, 0, 0);
    if (KTAIL) acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(blk.kt[kb], qtail, acc, 0, 0, 0);
    s[kb] = acc;
  }
  // the same for the whole wave: does every row see all 32 keys?
  const bool whole = base + 31 <= pos_min && (window == 0 || base > pos_max - window);
  if (!whole) {
    // values of keys outside [lo, pos_max] came from a clamped place, or from places after the
    // sequence's last key in its last page, and may be anything
    const int kv0 = base + 8 * quad;
    const int keep = kv0 + 7 >= lo ? pos_max - kv0 + 1 : 0;
#pragma unroll
    for (int i = 0; i < DB; ++i) blk.v[i] = keep_first(blk.v[i], keep);
  }
  tile_update(s, blk.v, !whole, base, quad, row_valid, qpos, window, scale_log2, m, l, o);
}

// One head of a token's product (x, D elements, D a multiple of 64) as an MFMA operand: RMSNorm
// over the head in float32 (weight after the normalisation), NeoX rotation pairing element j
// with j + D / 2 by the angles of `rope`, rounded to bfloat16 last, as the kernel that writes
// queries and keys to memory does. A lane holds elements 32 i + 8 quad .. + 7 of k-step i, so a
// pair lies in one lane (k-steps i and i + KFULL / 2) and the head's sum of squares in the four
// lanes of a row.
__device__ __forceinline__ void head_as_operand(const bf16_t* __restrict__ x, const float* __restrict__ w,
                                                const float* __restrict__ rope, float eps, int quad,
                                                bf16x8_t* out) {
  constexpr int KF = KFULL > 0 ? KFULL : 1, HALF_STEPS = KF / 2;
  float v[KF][8];
  float ss = 0.f;
#pragma unroll
  for (int i = 0; i < KF; ++i) {
    const bf16x8_t r = *(const bf16x8_t*)(x + 32 * i + 8 * quad);
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      v[i][e] = (float)r[e];
      ss += v[i][e] * v[i][e];
    }
  }
  if (w) {
    ss += __shfl_xor(ss, 16, 64);
    ss += __shfl_xor(ss, 32, 64);
    const float inv = rsqrtf(ss / (float)D + eps);
#pragma unroll
    for (int i = 0; i < KF; ++i)
#pragma unroll
      for (int e = 0; e < 8; ++e) v[i][e] = v[i][e] * inv * w[32 * i + 8 * quad + e];
  }
  if (rope) {
#pragma unroll
    for (int i = 0; i < HALF_STEPS; ++i)
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        const int j = 32 * i + 8 * quad + e;
        const float cs = rope[j], sn = rope[D / 2 + j];
        const float x1 = v[i][e], x2 = v[i + HALF_STEPS][e];
        v[i][e] = x1 * cs - x2 * sn;
        v[i + HALF_STEPS][e] = x2 * cs + x1 * sn;
      }
  }
#pragma unroll
  for (int i = 0; i < KF; ++i)
#pragma unroll
    for (int e = 0; e < 8; ++e) out[i][e] = (bf16_t)v[i][e];
}

constexpr bool DECODE_ONCE = true;  // measured: 2 % off a decode step at batch 1 and at batch 64, level at batch 8

template <bool P2, bool FUSED = false>
__global__ __launch_bounds__(64 * DW, D <= 128 ? 2 : 1) void attention_bf16_decode_kernel(AttnTileArgs a) {
  // per wave: maximum and sum per row, unnormalised accumulator [16][D]
  extern __shared__ float lds[];
  float* lds_m = lds;                 // [DW][16]
  float* lds_l = lds + DW * 16;       // [DW][16]
  float* lds_o = lds + 2 * DW * 16;   // [DW][16][D]

  const int lane = threadIdx.x & 63, wave = uniform_wave_number();
  const int r16 = lane & 15, quad = lane >> 4;
  // every sequence is one tile here, so without a list the block's number is the sequence's: one
  // dependent load less before the first key arrives. A list names the sequences of a launch
  // that covers only some of the step's.
  int seq, kvh, split;
  if (a.items) {  // pieces from the work list: (key head, item)
    seq = a.items[2 * blockIdx.y];
    if (seq < 0) return;  // past the end of the list
    split = a.items[2 * blockIdx.y + 1];
    kvh = blockIdx.x;
  } else {
    seq = a.tile_seq ? a.tile_seq[blockIdx.x] : blockIdx.x;
    kvh = blockIdx.y;
    split = blockIdx.z;
  }
  const int g = a.nq / a.nkv;
  const int q_begin = a.cu_q[seq];
  const int q_len = a.cu_q[seq + 1] - q_begin;
  const int kv_len = a.kv_lens[seq];
  const int n_rows = q_len * g;  // <= 16 by the launch condition
  const int first_pos = kv_len - q_len;
  const bool row_valid = r16 < n_rows;
  const int row_c = row_valid ? r16 : max(n_rows - 1, 0);
  const int tok = row_c / g, hg = row_c - tok * g;
  const int qpos = first_pos + tok;
  const int head = kvh * g + hg;
  const int* table = a.block_table + (size_t)seq * a.table_width;

  f32x4_t o[DB];
#pragma unroll
  for (int i = 0; i < DB; ++i) o[i] = (f32x4_t){0.f, 0.f, 0.f, 0.f};
  float m = -INFINITY, l = 0.f;

  // FUSED (one token per sequence, at position first_pos): the cache holds the keys before it,
  // [lo, first_pos - 1]; the token itself is added from registers below. For the masks of the
  // cache's blocks the token then stands one position earlier with a window one shorter.
  const int own = FUSED ? 1 : 0;
  const int window = FUSED && a.window > 0 ? a.window - 1 : a.window;
  const int qpos_c = qpos - own;
  const int pos_min = first_pos - own, pos_max = first_pos + (max(n_rows, 1) - 1) / g - own;
  const int lo = a.window > 0 ? max(0, first_pos - a.window + 1) : 0;
  int blk_begin, blk_end;
  decode_key_blocks(kv_len, q_len, a.window, FUSED, blk_begin, blk_end);
  // equal parts of the sequence's blocks, or pieces of a fixed length, as many as it has
  const int per = a.items ? a.split_blocks : (blk_end - blk_begin + a.num_splits - 1) / a.num_splits;
  const int last_split = a.items ? max(1, (blk_end - blk_begin + per - 1) / per) - 1 : (int)gridDim.z - 1;
  const int b0 = blk_begin + split * per;
  const int b1 = min(blk_end, b0 + per);
  int b = b0 + wave;

  bf16x8_t qreg[KFULL > 0 ? KFULL : 1];
  bf16x8_t qtail = load_tail((const bf16_t*)nullptr, 2);  // zeros
  // every wave forms the queries it multiplies; the last wave of the last split also takes the
  // token's own key and value, the wave before it stores them into the cache (these have the
  // fewest blocks of cached keys: the blocks go round the waves, and the last split takes what
  // the others left)
  auto own_token = [&]() {
    const bf16_t* raw = a.qkv + (size_t)q_begin * a.qkv_stride;
    const float* rope = a.rope ? a.rope + (size_t)q_begin * D : nullptr;
    head_as_operand(raw + (size_t)head * D, a.q_weight, rope, a.eps, quad, qreg);
    const bool at_end = split == last_split;
    const bool adds_own = at_end && wave == DW - 1, stores_own = at_end && wave == (2 * DW - 2) % DW;
    if (adds_own || stores_own) {  // uniform over the wave
      const bf16_t* kraw = raw + ((size_t)a.nq + kvh) * D;
      const bf16_t* vraw = raw + ((size_t)a.nq + a.nkv + kvh) * D;
      bf16x8_t kreg[KFULL > 0 ? KFULL : 1];
      head_as_operand(kraw, a.k_weight, rope, a.eps, quad, kreg);
      if (stores_own) {
        const int slot = a.slots[q_begin];
        const int page = slot / a.page_size, off = slot - page * a.page_size;
        bf16_t* kdst = (bf16_t*)a.k_cache + (((size_t)page * a.nkv + kvh) * a.page_size + off) * D;
        bf16_t* vdst = (bf16_t*)a.v_cache + ((size_t)page * a.nkv + kvh) * D * a.page_size + off;
        if (r16 == 0) {
#pragma unroll
          for (int i = 0; i < KFULL; ++i) *(bf16x8_t*)(kdst + 32 * i + 8 * quad) = kreg[i];
        }
        for (int d = lane; d < D; d += 64) vdst[(size_t)d * a.page_size] = vraw[d];
      }
      if (adds_own) {
        // a block of keys that holds this one key, in the place of key first_pos: operand row 0
        // of the first half block; the other rows are masked like keys after the token
        f32x4_t sc[2];
        sc[0] = (f32x4_t){0.f, 0.f, 0.f, 0.f};
        sc[1] = sc[0];
#pragma unroll
        for (int i = 0; i < KFULL; ++i) sc[0] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kreg[i], qreg[i], sc[0], 0, 0, 0);
        bf16x8_t vv[DB];
#pragma unroll
        for (int i = 0; i < DB; ++i) {
#pragma unroll
          for (int e = 0; e < 8; ++e) vv[i][e] = (bf16_t)0.0f;
          if (quad == 0) vv[i][0] = vraw[16 * i + r16];
        }
        tile_update(sc, vv, true, first_pos, quad, row_valid, qpos, a.window, a.scale_log2, m, l, o);
      }
    }
  };

  if (n_rows > 0 && b < b1) {
    if (!FUSED) {
      const bf16_t* qp = a.q + ((size_t)(q_begin + tok) * a.nq + head) * D;
#pragma unroll
      for (int i = 0; i < KFULL; ++i) qreg[i] = *(const bf16x8_t*)(qp + 32 * i + 8 * quad);
      if (KTAIL) qtail = load_tail(qp + 32 * KFULL, quad);
    }

    // two blocks of keys and values are on their way while a third is multiplied, and the page
    // numbers of the two after them; past the wave's last block the loads go on (one shape of
    // loop, no load under a branch) but fetch next to nothing
    const int last = b + (b1 - 1 - b) / DW * DW;
    KvBlock A, B;
    int pgA[3], pgB[3];
    block_pages<P2>(table, b << 5, lo, pos_max, a.page_size, r16, quad, pgA);
    block_pages<P2>(table, min(b + DW, last) << 5, lo, pos_max, a.page_size, r16, quad, pgB);
    block_load<P2, DECODE_ONCE>(a, kvh, b << 5, lo, pos_max, r16, quad, pgA, A);
    block_load<P2, DECODE_ONCE>(a, kvh, min(b + DW, last) << 5, lo, pos_max, r16, quad, pgB, B, b + DW <= last);
    block_pages<P2>(table, min(b + 2 * DW, last) << 5, lo, pos_max, a.page_size, r16, quad, pgA);
    block_pages<P2>(table, min(b + 3 * DW, last) << 5, lo, pos_max, a.page_size, r16, quad, pgB);
    if (FUSED) own_token();  // while the first keys and values are on their way
    while (true) {
      block_compute(A, qreg, qtail, b << 5, lo, pos_min, pos_max, quad, row_valid, qpos_c, window, a.scale_log2, m, l, o);
      block_load<P2, DECODE_ONCE>(a, kvh, min(b + 2 * DW, last) << 5, lo, pos_max, r16, quad, pgA, A, b + 2 * DW <= last);
      block_pages<P2>(table, min(b + 4 * DW, last) << 5, lo, pos_max, a.page_size, r16, quad, pgA);
      b += DW;
      if (b >= b1) break;
      block_compute(B, qreg, qtail, b << 5, lo, pos_min, pos_max, quad, row_valid, qpos_c, window, a.scale_log2, m, l, o);
      block_load<P2, DECODE_ONCE>(a, kvh, min(b + 2 * DW, last) << 5, lo, pos_max, r16, quad, pgB, B, b + 2 * DW <= last);
      block_pages<P2>(table, min(b + 4 * DW, last) << 5, lo, pos_max, a.page_size, r16, quad, pgB);
      b += DW;
      if (b >= b1) break;
    }
  } else if (FUSED) {
    own_token();
  }
  l += __shfl_xor(l, 16, 64);
  l += __shfl_xor(l, 32, 64);

  // the waves' parts meet in LDS
  if (quad == 0) {
    lds_m[wave * 16 + r16] = m;
    lds_l[wave * 16 + r16] = l;
  }
#pragma unroll
  for (int i = 0; i < DB; ++i)
#pragma unroll
    for (int r = 0; r < 4; ++r) lds_o[(wave * 16 + r16) * D + 16 * i + 4 * quad + r] = o[i][r];
  __syncthreads();

  const size_t tile_row0 = (size_t)q_begin * a.nq;  // rows of this sequence start here, in units of heads
  for (int idx = threadIdx.x; idx < 16 * D; idx += 64 * DW) {
    const int row = idx / D, d = idx - row * D;
    if (row >= n_rows) continue;
    float mm = -INFINITY;
#pragma unroll
    for (int w = 0; w < DW; ++w) mm = fmaxf(mm, lds_m[w * 16 + row]);
    float num = 0.f, den = 0.f;
    if (mm != -INFINITY) {
#pragma unroll
      for (int w = 0; w < DW; ++w) {
        const float f = exp2f(lds_m[w * 16 + row] - mm);
        num += f * lds_o[(w * 16 + row) * D + d];
        den += f * lds_l[w * 16 + row];
      }
    }
    const int rt = row / g, rh = row - rt * g;
    const size_t row_index = tile_row0 + (size_t)rt * a.nq + kvh * g + rh;
    const float val = den > 0.f ? num / den : 0.f;
    if (a.num_splits == 1) {
      a.out[row_index * D + d] = (bf16_t)val;
    } else {
      a.part_o[(row_index * a.num_splits + split) * D + d] = val;
      if (d == 0) a.part_lse[row_index * a.num_splits + split] = den > 0.f ? mm + log2f(den) : -INFINITY;
    }
  }
  // the pieces this sequence does not have count as empty splits (their parts are never read)
  if (a.items && split == 0) {
    const int missing = a.num_splits - 1 - last_split;
    for (int idx = threadIdx.x; idx < n_rows * missing; idx += 64 * DW) {
      const int row = idx % n_rows, s = last_split + 1 + idx / n_rows;
      const int rt = row / g, rh = row - rt * g;
      a.part_lse[(tile_row0 + (size_t)rt * a.nq + kvh * g + rh) * a.num_splits + s] = -INFINITY;
    }
  }
}

// Fills args->items for a decode launch in pieces of args->split_blocks blocks: needs cu_q,
// kv_lens, tile_seq (or null), num_tiles <= 1024, window, max_items >= the pieces there can be
// (num_tiles * num_splits will do). `fused` as the launch: the tokens' own keys come from the
// product, the cache holds the keys before them.
extern "C" int qrt_attention_work_list(const AttnTileArgs* args, int fused, hipStream_t stream) {
  const AttnTileArgs& a = *args;
  QRT_CHECK(a.items && a.split_blocks > 0 && a.num_tiles >= 0 && a.num_tiles <= LIST_TILES && a.max_items >= a.num_tiles,
            "attention work list: %d sequences (at most %d), %d items, pieces of %d blocks", a.num_tiles, LIST_TILES,
            a.max_items, a.split_blocks);
  if (a.max_items == 0) return 0;
  attention_work_list_kernel<<<1, 256, 0, stream>>>(a, fused);
  QRT_LAUNCH_CHECK("attention_work_list");
  return 0;
}

// every listed sequence at most 16 rows (q_len * g <= 16) and D <= 256; num_tiles = number of
// sequences; tile_seq lists them, or is null for all sequences of the step in order
extern "C" int qrt_attention_bf16_decode(const AttnTileArgs* args, int num_rows_total, hipStream_t stream) {
  AttnTileArgs a = *args;
  QRT_CHECK(a.nq > 0 && a.nkv > 0 && a.nq % a.nkv == 0, "attention: %d query heads do not divide into %d key heads",
            a.nq, a.nkv);
  QRT_CHECK(D <= 256, "attention (decode): head size %d is above 256", D);
  QRT_CHECK(a.page_size > 0 && a.page_size % 8 == 0,
            "attention (bfloat16): page size %d must be a multiple of 8", a.page_size);
  QRT_CHECK(a.num_splits >= 1 && a.num_splits <= 65535 && a.nkv <= 65535, "attention: bad split or head count");
  QRT_CHECK(a.num_splits == 1 || (a.part_o && a.part_lse), "attention: split run without scratch");
  QRT_CHECK(a.table_width > 0 && a.window >= 0, "attention: bad table width or window");
  QRT_CHECK(a.items ? a.split_blocks > 0 && a.max_items >= a.num_tiles && a.max_items <= 65535
                    : a.split_blocks == 0,
            "attention (decode): pieces of %d blocks with a list of %d items for %d sequences", a.split_blocks,
            a.max_items, a.num_tiles);
  if (a.num_tiles == 0) return 0;
  const bool p2 = (a.page_size & (a.page_size - 1)) == 0;  // shifts instead of divisions
  dim3 grid(a.num_tiles, a.nkv, a.num_splits), block(64 * DW);
  if (a.items) grid = dim3(a.nkv, a.max_items, 1);
  constexpr size_t smem = (size_t)(2 * DW * 16 + DW * 16 * D) * sizeof(float);
  if (smem > 64 * 1024) {  // head size 256: a little more LDS than a block gets without asking
    static bool allowed = false;  // once: not again inside every stream capture
    if (!allowed) {
      if (hipFuncSetAttribute((const void*)attention_bf16_decode_kernel<true>,
                              hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem) != hipSuccess ||
          hipFuncSetAttribute((const void*)attention_bf16_decode_kernel<false>,
                              hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem) != hipSuccess)
        return qrt_fail("attention (decode): cannot get %zu bytes of LDS", smem);
      allowed = true;
    }
  }
  if (a.qkv) {
    // one token per sequence, its query, key and value taken from the product that made them
    if constexpr (D % 64 == 0) {
      QRT_CHECK(a.nq / a.nkv <= 16 && a.slots && a.qkv_stride >= (long)(a.nq + 2 * a.nkv) * D && a.qkv_stride % 8 == 0 &&
                    (uintptr_t)a.qkv % 16 == 0,
                "attention (decode, own token from the product): %d query heads per key head, stride %ld",
                a.nq / a.nkv, a.qkv_stride);
      if (smem > 64 * 1024) {
        static bool allowed_fused = false;
        if (!allowed_fused) {
          if (hipFuncSetAttribute((const void*)attention_bf16_decode_kernel<true, true>,
                                  hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem) != hipSuccess ||
              hipFuncSetAttribute((const void*)attention_bf16_decode_kernel<false, true>,
                                  hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem) != hipSuccess)
            return qrt_fail("attention (decode): cannot get %zu bytes of LDS", smem);
          allowed_fused = true;
        }
      }
      if (p2) attention_bf16_decode_kernel<true, true><<<grid, block, smem, stream>>>(a);
      else attention_bf16_decode_kernel<false, true><<<grid, block, smem, stream>>>(a);
    } else {
      return qrt_fail("attention (decode, own token from the product): head size %d is no multiple of 64", D);
    }
  } else if (p2) attention_bf16_decode_kernel<true><<<grid, block, smem, stream>>>(a);
  else attention_bf16_decode_kernel<false><<<grid, block, smem, stream>>>(a);
  QRT_LAUNCH_CHECK("attention_bf16_decode");
  if (a.num_splits > 1) {
    const int merge_rows = a.merge_tokens ? a.num_merge_tokens * a.nq : num_rows_total;
    if (merge_rows > 0)
      attention_merge_kernel<<<dim3(merge_rows), dim3(D >= 64 ? 64 : 32), 0, stream>>>(
          a.part_o, a.part_lse, a.out, a.num_splits, a.merge_tokens, a.nq);
    QRT_LAUNCH_CHECK("attention_merge");
  }
  return 0;
}

extern "C" int qrt_attention_bf16(const AttnTileArgs* args, int num_rows_total, hipStream_t stream) {
  AttnTileArgs a = *args;
  QRT_CHECK(a.nq > 0 && a.nkv > 0 && a.nq % a.nkv == 0, "attention: %d query heads do not divide into %d key heads",
            a.nq, a.nkv);
  QRT_CHECK(a.page_size > 0 && a.page_size % 8 == 0,
            "attention (bfloat16): page size %d must be a multiple of 8", a.page_size);
  QRT_CHECK(a.waves == 1 || a.waves == 2 || a.waves == 4, "attention: waves per block must be 1, 2 or 4");
  QRT_CHECK(a.num_splits >= 1 && a.num_splits <= 65535 && a.nkv <= 65535, "attention: bad split or head count");
  QRT_CHECK(a.num_splits == 1 || (a.part_o && a.part_lse), "attention: split run without scratch");
  QRT_CHECK(a.table_width > 0 && a.window >= 0, "attention: bad table width or window");
  if (a.num_tiles == 0) return 0;
  const bool p2 = (a.page_size & (a.page_size - 1)) == 0;  // shifts instead of divisions
  QRT_CHECK((long long)a.num_tiles * a.nkv < (1ll << 31), "attention: %d tiles x %d key heads is too many blocks", a.num_tiles, a.nkv);
  dim3 grid(a.num_tiles * a.nkv, 1, a.num_splits), block(64 * a.waves);
  // the kernel that shares keys and values through LDS, where its two stages fit what a block
  // may have without asking (64 KB: head sizes up to 208); the general kernel otherwise
  constexpr size_t lds_bytes = 2 * (size_t)STAGE_ELEMS * sizeof(bf16_t);
  if (a.row_tiles == 2 && a.waves == 4 && a.use_lds == 2 && lds_bytes <= 64 * 1024) {
    // two groups of four waves: twice the stages, more LDS than a block gets without asking
    // ... or what the join of the two groups' sums needs afterwards, in the same memory (more than
    // the stages at small head sizes): accumulators [4 waves][2 tiles][DB][64 lanes] of 16 bytes,
    // maxima and sums [4][2][2][64] of 4
    constexpr size_t join_bytes = (size_t)4 * 2 * DB * 64 * 16 + (size_t)4 * 2 * 2 * 64 * 4;
    constexpr size_t smem = 2 * lds_bytes > join_bytes ? 2 * lds_bytes : join_bytes;
    static bool allowed = false;  // once: not again inside every stream capture
    if (!allowed) {
      if (hipFuncSetAttribute((const void*)attention_bf16_prefill_kernel<2, true, 2>,
                              hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem) != hipSuccess ||
          hipFuncSetAttribute((const void*)attention_bf16_prefill_kernel<2, false, 2>,
                              hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem) != hipSuccess)
        return qrt_fail("attention (long portions, two groups): cannot get %zu bytes of LDS", smem);
      allowed = true;
    }
    if (p2) attention_bf16_prefill_kernel<2, true, 2><<<grid, dim3(512), smem, stream>>>(a);
    else attention_bf16_prefill_kernel<2, false, 2><<<grid, dim3(512), smem, stream>>>(a);
  } else if (a.row_tiles == 2 && a.waves == 4 && a.use_lds && lds_bytes <= 64 * 1024) {
    const size_t smem = lds_bytes;
    if (p2) attention_bf16_prefill_kernel<2, true, 1><<<grid, block, smem, stream>>>(a);
    else attention_bf16_prefill_kernel<2, false, 1><<<grid, block, smem, stream>>>(a);
  } else if (a.row_tiles == 1 && p2) attention_bf16_kernel<1, true><<<grid, block, 0, stream>>>(a);
  else if (a.row_tiles == 1) attention_bf16_kernel<1, false><<<grid, block, 0, stream>>>(a);
  else if (a.row_tiles == 2 && p2) attention_bf16_kernel<2, true><<<grid, block, 0, stream>>>(a);
  else if (a.row_tiles == 2) attention_bf16_kernel<2, false><<<grid, block, 0, stream>>>(a);
  else return qrt_fail("attention: %d row tiles per wave at head size %d is not built", a.row_tiles, D);
  QRT_LAUNCH_CHECK("attention_bf16");
  if (a.num_splits > 1) {
    const int merge_rows = a.merge_tokens ? a.num_merge_tokens * a.nq : num_rows_total;
    if (merge_rows > 0)
      attention_merge_kernel<<<dim3(merge_rows), dim3(D >= 64 ? 64 : 32), 0, stream>>>(
          a.part_o, a.part_lse, a.out, a.num_splits, a.merge_tokens, a.nq);
    QRT_LAUNCH_CHECK("attention_merge");
  }
  return 0;
}
