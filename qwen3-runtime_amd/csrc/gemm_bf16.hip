// bfloat16 matrix product on MFMA: C[M, N] = A[M, K] * W[N, K]^T, float32
// accumulation, output bfloat16 or float32.
//
// Both operands are contiguous along K, which is what the 16x16x32 MFMA wants
// in each lane (8 consecutive k), so operands go from global memory straight
// into registers. The product is formed transposed (C^T = W * A^T): the weight
// rows are the MFMA's A operand and the activations its B operand, so that a
// lane ends up with four consecutive n of one output row m and stores them as
// one vector. A wave owns a (16*MT) x (16*NT) tile; a block is four waves side
// by side along N. Skinny M (decode) uses MT = 1.
#include "common.h"

template <bool ALIGNED>
__device__ __forceinline__ bf16x8_t load_k8(const bf16_t* __restrict__ row, int k, int K, bool valid) {
  bf16x8_t v;
#pragma unroll
  for (int e = 0; e < 8; ++e) v[e] = (bf16_t)0.0f;
  if (!valid) return v;
  if (ALIGNED && k + 8 <= K) {
    v = *(const bf16x8_t*)(row + k);
  } else {
#pragma unroll
    for (int e = 0; e < 8; ++e)
      if (k + e < K) v[e] = row[k + e];
  }
  return v;
}

template <int MT, int NT, bool ALIGNED, typename TO>
__global__ __launch_bounds__(256) void gemm_bf16_kernel(const bf16_t* __restrict__ A, const bf16_t* __restrict__ W,
                                                         TO* __restrict__ C, int M, int N, int K) {
  const int lane = threadIdx.x & 63, wave = uniform_wave_number();
  const int r16 = lane & 15, quad = lane >> 4;
  const int m0 = blockIdx.y * (16 * MT);
  const int n0 = (blockIdx.x * 4 + wave) * (16 * NT);
  if (n0 >= N) return;

  f32x4_t acc[MT][NT];
#pragma unroll
  for (int i = 0; i < MT; ++i)
#pragma unroll
    for (int j = 0; j < NT; ++j) acc[i][j] = (f32x4_t){0.f, 0.f, 0.f, 0.f};

  const bf16_t* arow[MT];
  bool avalid[MT];
#pragma unroll
  for (int i = 0; i < MT; ++i) {
    const int m = m0 + 16 * i + r16;
    avalid[i] = m < M;
    arow[i] = A + (size_t)(avalid[i] ? m : 0) * K;
  }
  const bf16_t* wrow[NT];
  bool wvalid[NT];
#pragma unroll
  for (int j = 0; j < NT; ++j) {
    const int n = n0 + 16 * j + r16;
    wvalid[j] = n < N;
    wrow[j] = W + (size_t)(wvalid[j] ? n : 0) * K;
  }

  for (int k0 = 0; k0 < K; k0 += 32) {
    const int k = k0 + 8 * quad;
    bf16x8_t a[MT], w[NT];
#pragma unroll
    for (int i = 0; i < MT; ++i) a[i] = load_k8<ALIGNED>(arow[i], k, K, avalid[i]);
#pragma unroll
    for (int j = 0; j < NT; ++j) w[j] = load_k8<ALIGNED>(wrow[j], k, K, wvalid[j]);
#pragma unroll
    for (int i = 0; i < MT; ++i)
#pragma unroll
      for (int j = 0; j < NT; ++j)
        acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(w[j], a[i], acc[i][j], 0, 0, 0);
  }

  // acc[i][j][r]: output row m0 + 16 i + r16, column n0 + 16 j + 4 quad + r
#pragma unroll
  for (int i = 0; i < MT; ++i) {
    const int m = m0 + 16 * i + r16;
    if (m >= M) continue;
#pragma unroll
    for (int j = 0; j < NT; ++j) {
      const int n = n0 + 16 * j + 4 * quad;
#pragma unroll
      for (int r = 0; r < 4; ++r)
        if (n + r < N) C[(size_t)m * N + n + r] = from_f32<TO>(acc[i][j][r]);
    }
  }
}


// ---------------------------------------------------------------- few rows
// M <= 16 (decoding): the product is a stream of the weight matrix, so the
// layout is chosen for memory parallelism, not for reuse. A block owns NT
// tiles of 16 weight rows and all of K; its NW waves take the 32-wide k-steps
// round-robin, so that in every round the block reads 16 rows x NW x 64
// contiguous bytes per tile. A wave issues the loads of U steps before the
// first MFMA of them. Each wave keeps MB accumulators (16 rows of M each) per
// tile; activations come from L2/L1 (they are tiny). Partial sums meet in LDS
// and are added in wave order, so the result does not depend on timing.
//
// GATED: W holds 2N rows, gate rows then up rows; the block owns matching
// tiles of both and writes silu(gate) * up, so the gated feed-forward's
// intermediate [M, 2N] never reaches memory.
template <int MB, int NW, int NT, int U, bool GATED, bool TILED, typename TO>
__global__ __launch_bounds__(64 * NW) void gemm_bf16_skinny_kernel(const bf16_t* __restrict__ A,
                                                                    const bf16_t* __restrict__ W,
                                                                    TO* __restrict__ C, int M, int N, int K) {
  constexpr int WT = GATED ? 2 * NT : NT;  // weight tiles per block
  extern __shared__ float red[];            // [NW][WT][MB][4][64]
  const int lane = threadIdx.x & 63, wave = uniform_wave_number();
  const int r16 = lane & 15, quad = lane >> 4;
  const int n0 = blockIdx.x * 16 * NT;
  const bf16_t* wrow[WT];
  // TILED: W is stored tile by tile, [row tile of 16][k-step of 32][lane][8 elements], each
  // (tile, step) being exactly the 1 KB a wave loads at once; N is then a multiple of 16
  constexpr int WSTEP = TILED ? 512 : 32;  // elements between consecutive k-steps of a lane
#pragma unroll
  for (int t = 0; t < NT; ++t) {
    if (TILED) {
      const int tile = min(n0 / 16 + t, N / 16 - 1);
      wrow[t] = W + (size_t)tile * 16 * K + 8 * lane;
      if (GATED) wrow[NT + t] = W + (size_t)(N / 16 + tile) * 16 * K + 8 * lane;
    } else {
      const int n = min(n0 + 16 * t + r16, N - 1);
      wrow[t] = W + (size_t)n * K + 8 * quad;
      if (GATED) wrow[NT + t] = W + (size_t)(N + n) * K + 8 * quad;
    }
  }
  const bf16_t* arow[MB];
  bool avalid[MB];
#pragma unroll
  for (int b = 0; b < MB; ++b) {
    const int m = 16 * b + r16;
    avalid[b] = m < M;
    arow[b] = A + (size_t)(avalid[b] ? m : 0) * K + 8 * quad;
  }
  f32x4_t acc[WT][MB];
#pragma unroll
  for (int t = 0; t < WT; ++t)
#pragma unroll
    for (int b = 0; b < MB; ++b) acc[t][b] = (f32x4_t){0.f, 0.f, 0.f, 0.f};

  // gridDim.y blocks share the row tiles; block y takes the y-th part of the k-steps and writes
  // output plane y (the caller adds the planes: used where the result feeds a residual add)
  const int all_steps = K >> 5;  // K is a multiple of 32 here
  const int part = (all_steps + gridDim.y - 1) / gridDim.y;
  const int s_first = blockIdx.y * part, steps = min(all_steps, s_first + part);
  C += (size_t)blockIdx.y * M * N;
  bf16x8_t zero;
#pragma unroll
  for (int e = 0; e < 8; ++e) zero[e] = (bf16_t)0.0f;
  for (int s0 = s_first + wave; s0 < steps; s0 += U * NW) {
    bf16x8_t w[U][WT], a[U][MB];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int s = s0 + u * NW;
      if (s < steps) {  // uniform over the wave
#pragma unroll
        for (int t = 0; t < WT; ++t) w[u][t] = load_once8(wrow[t] + (size_t)s * WSTEP);
#pragma unroll
        for (int b = 0; b < MB; ++b) a[u][b] = avalid[b] ? *(const bf16x8_t*)(arow[b] + (s << 5)) : zero;
      }
    }
#pragma unroll
    for (int u = 0; u < U; ++u) {
      if (s0 + u * NW < steps) {
#pragma unroll
        for (int t = 0; t < WT; ++t)
#pragma unroll
          for (int b = 0; b < MB; ++b)
            acc[t][b] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(w[u][t], a[u][b], acc[t][b], 0, 0, 0);
      }
    }
  }

#pragma unroll
  for (int t = 0; t < WT; ++t)
#pragma unroll
    for (int b = 0; b < MB; ++b)
#pragma unroll
      for (int r = 0; r < 4; ++r) red[(((wave * WT + t) * MB + b) * 4 + r) * 64 + lane] = acc[t][b][r];
  __syncthreads();
  // one thread per (tile, accumulator block, lane) adds the waves' parts in order
  for (int i = threadIdx.x; i < NT * MB * 64; i += 64 * NW) {
    const int l = i & 63, b = (i >> 6) % MB, t = (i >> 6) / MB;
    const int m = 16 * b + (l & 15);
    const int nn = n0 + 16 * t + 4 * (l >> 4);
    float sum[4], sum2[4];
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      float v = 0.f, v2 = 0.f;
      for (int w = 0; w < NW; ++w) {
        v += red[(((w * WT + t) * MB + b) * 4 + r) * 64 + l];
        if (GATED) v2 += red[(((w * WT + NT + t) * MB + b) * 4 + r) * 64 + l];
      }
      sum[r] = v;
      sum2[r] = v2;
    }
    if (m < M) {
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        if (nn + r < N) {
          // the gate and the up value are rounded to bfloat16 first, as the unfused kernels see them
          const float g = (float)(bf16_t)sum[r];
          const float out = GATED ? g / (1.0f + expf(-g)) * (float)(bf16_t)sum2[r] : sum[r];
          C[(size_t)m * N + nn + r] = from_f32<TO>(out);
        }
      }
    }
  }
}

template <int MB, int NW, int NT, int U, bool GATED, bool TILED = false>
static int launch_skinny(const bf16_t* a, const bf16_t* w, void* c, int out_dtype, int M, int N, int K,
                         hipStream_t stream, int k_parts = 1) {
  dim3 grid((N + 16 * NT - 1) / (16 * NT), k_parts), block(64 * NW);
  const size_t smem = (size_t)NW * (GATED ? 2 : 1) * NT * MB * 4 * 64 * sizeof(float);
  if (out_dtype == QRT_BF16)
    gemm_bf16_skinny_kernel<MB, NW, NT, U, GATED, TILED, bf16_t><<<grid, block, smem, stream>>>(a, w, (bf16_t*)c, M, N, K);
  else if (out_dtype == QRT_F32)
    gemm_bf16_skinny_kernel<MB, NW, NT, U, GATED, TILED, float><<<grid, block, smem, stream>>>(a, w, (float*)c, M, N, K);
  else
    return qrt_fail("gemm_bf16: unknown output dtype %d", out_dtype);
  QRT_LAUNCH_CHECK("gemm_bf16_skinny");
  return 0;
}

template <bool GATED>
static int skinny(const bf16_t* a, const bf16_t* w, void* c, int out_dtype, int M, int N, int K, hipStream_t st) {
  const int tiles = (N + 15) / 16;
  if (tiles >= 2048) return launch_skinny<1, 8, 2, 8, GATED>(a, w, c, out_dtype, M, N, K, st);
  if (tiles >= 512 || K < 4096) return launch_skinny<1, 8, 1, 8, GATED>(a, w, c, out_dtype, M, N, K, st);
  return launch_skinny<1, 16, 1, 8, GATED>(a, w, c, out_dtype, M, N, K, st);
}

// Tile-major weights, M <= 16. Configurations from timing 78 of them (2 to 16 waves, 1 to 4 row
// tiles a block, 2 to 12 steps in flight) on the shapes of the 4B, 8B and 32B models at 1 to 16
// rows, on the weight matrices of 36 layers in turn and replayed from a graph: eight waves
// everywhere. Gated: one row tile, eight steps in flight (the best at every size). The whole
// result of a matrix with many row tiles: two tiles a block, so that the activations are read
// half as often; with two steps in flight up to K = 4,096 (the 8B q/k/v product 10.3 us against
// 11.8 with eight), with eight for the vocabulary head (7.0 TB/s). K cut into planes: two tiles
// a block from K = 12,288 on (the 32B down projection at 8 rows 40.4 us against 45.0), four
// steps in flight up to K = 4,096, eight between.
template <bool GATED>
static int skinny_tiled(const bf16_t* a, const bf16_t* w, void* c, int out_dtype, int M, int N, int K,
                        hipStream_t st, int k_parts) {
  const int tiles = N / 16;
  if (GATED) return launch_skinny<1, 8, 1, 8, GATED, true>(a, w, c, out_dtype, M, N, K, st, k_parts);
  if (k_parts == 1) {
    if (tiles >= 2048) return launch_skinny<1, 8, 2, 8, GATED, true>(a, w, c, out_dtype, M, N, K, st);
    if (tiles >= 384 && K <= 4096) return launch_skinny<1, 8, 2, 2, GATED, true>(a, w, c, out_dtype, M, N, K, st);
    return launch_skinny<1, 8, 1, 8, GATED, true>(a, w, c, out_dtype, M, N, K, st);
  }
  if (K >= 12288) return launch_skinny<1, 8, 2, 8, GATED, true>(a, w, c, out_dtype, M, N, K, st, k_parts);
  if (K <= 4096) return launch_skinny<1, 8, 1, 4, GATED, true>(a, w, c, out_dtype, M, N, K, st, k_parts);
  return launch_skinny<1, 8, 1, 8, GATED, true>(a, w, c, out_dtype, M, N, K, st, k_parts);
}

__device__ __forceinline__ void store4(float* p, const float (&o)[4]) {
  *(f32x4_t*)p = (f32x4_t){o[0], o[1], o[2], o[3]};
}
__device__ __forceinline__ void store4(bf16_t* p, const float (&o)[4]) {
  typedef bf16_t bf16x4_t __attribute__((ext_vector_type(4)));
  *(bf16x4_t*)p = (bf16x4_t){(bf16_t)o[0], (bf16_t)o[1], (bf16_t)o[2], (bf16_t)o[3]};
}

// ---------------------------------------------------------------- 17 to 64 rows
// Still a stream of the weight matrix, but the activations now weigh as much as the weights
// if every wave fetches its own: four accumulator blocks of 16 rows want 4 KB of activations
// for each KB of weights. So the waves that walk the same part of K (a K group) share the
// activations through LDS: NWV waves side by side along N, NT tiles each, read one staged
// copy, and the traffic for activations falls to MB / (NWV * NT) of the weights'. KW such
// groups in a block take consecutive parts of the block's k-steps (the block's k-steps being
// part blockIdx.y of all, as in the few-row kernel) and meet in LDS at the end, added in
// group order. Weights, tile-major, go straight to registers, DEPTH chunks of KC k-steps
// ahead; the activations of chunk c + 2 are fetched while chunk c is used and chunk c + 1
// waits in the other LDS buffer, so there is one barrier per chunk. All loads are
// unconditional, at clamped addresses: steps past the end are loaded again and count as zero.
// Blocks start at different chunks of their k-steps and wrap round: every block reads all
// the activations, and in step they would all ask the same L2 channels at the same time.
// What a compute unit can pull through its memory pipeline is the limit (weights and
// activations alike, about 55 GB/s each), so the row tiles are dealt out evenly over
// gridDim.x blocks, chosen by the host as the number of compute units where there are more
// tiles than that: a block gets floor or ceil of tiles / blocks, at most NWV * NT. A wave
// without a tile reads a page of zeros instead, at no cost in memory traffic, and stores nothing.
__device__ bf16x8_t qrt_zero_tile[64];

template <int MB, int KW, int NWV, int NT, int KC, int DEPTH, bool GATED, typename TO>
__global__ __launch_bounds__(64 * KW * NWV) void gemm_bf16_mid_kernel(const bf16_t* __restrict__ A,
                                                                       const bf16_t* __restrict__ W,
                                                                       TO* __restrict__ C, int M, int N, int K) {
  constexpr int WT = GATED ? 2 * NT : NT;  // weight tiles per wave
  constexpr int UPW = KC * MB / NWV;       // 1 KB units of activations a wave stages per chunk
  static_assert(KC * MB % NWV == 0 && KC % 2 == 0, "the waves of a K group stage equal shares of a chunk");
  static_assert(DEPTH == 1 || DEPTH == 2, "the weights run one or two chunks ahead");
  extern __shared__ __align__(16) unsigned char smem_raw[];  // [KW][2] staged chunks
  const int lane = threadIdx.x & 63;
  const int wave = uniform_wave_number();
  const int kg = wave / NWV, nw = wave % NWV;
  const int r16 = lane & 15, quad = lane >> 4;
  const int ntiles = N >> 4;
  const int tile_lo = (int)(blockIdx.x * (unsigned)ntiles / gridDim.x);  // N <= 2^20: no overflow
  const int tile_hi = (int)((blockIdx.x + 1) * (unsigned)ntiles / gridDim.x);
  const int tile0 = tile_lo + nw * NT;

  // the k-steps of this block, then of this K group
  // (K is a multiple of 64 here; parts and groups start at even k-steps: a cache line of
  // activations holds two)
  const int all_steps = K >> 5;
  const int part = 2 * ((all_steps / 2 + gridDim.y - 1) / gridDim.y);
  const int p0 = min(all_steps, (int)blockIdx.y * part), p1 = min(all_steps, p0 + part);
  const int glen = 2 * (((p1 - p0) / 2 + KW - 1) / KW);
  const int g0 = min(p1, p0 + kg * glen), g1 = min(p1, g0 + glen);
  const int chunks = (glen + KC - 1) / KC;  // the same for every group: they share the barriers
  const int last_step = all_steps - 1, last_pair = all_steps - 2;
  const int rot = (int)((blockIdx.x * 5u + blockIdx.y * 3u + kg) % (unsigned)max(chunks, 1));
  // first k-step of the c-th chunk in this block's order; past the last chunk nothing is live
  auto chunk_start = [&](int c) {
    int cc = c + rot;
    if (cc >= chunks) cc -= chunks;
    return c < chunks ? g0 + cc * KC : g1;
  };

  const bf16_t* wbase[WT];  // uniform over the wave: the lane is added at the load
  int wstep[NT];            // elements from one k-step to the next: none in the page of zeros
#pragma unroll
  for (int t = 0; t < NT; ++t) {
    const int tile = tile0 + t;
    const bool mine = tile < tile_hi;
    wstep[t] = mine ? 512 : 0;
    wbase[t] = mine ? W + (size_t)tile * 16 * K : (const bf16_t*)qrt_zero_tile;
    if (GATED) wbase[NT + t] = mine ? W + (size_t)(ntiles + tile) * 16 * K : (const bf16_t*)qrt_zero_tile;
  }
  // Staging of a chunk: unit u = (pair of k-steps u / (2 MB), row block (u / 2) % MB, half u % 2
  // of its 16 rows); this wave stages units nw, nw + NWV, ... A unit is 8 rows x 128 bytes, whole
  // cache lines: lane l reads row 8 half + l / 8, 16-byte piece l % 8 (k-step l % 8 / 4 of the
  // pair, columns 8 (l % 4) .. + 7 of it). In LDS the piece of (k-step s, row block b, column
  // group q, row i) lies at s * SS + b * BS + q * QS + 16 i bytes: the strides are padded so
  // that the 8 pieces of a row, written together, do not all fall into the same banks, while
  // the 16 rows of a column group, read together, stay contiguous. (Counters: a third of the
  // LDS's active cycles are still conflicts; a stride of 288 bytes made it a half. The waves
  // wait for LDS 3 % of their time, so it was left there.)
  constexpr int QS = 256 + 16, BS = 4 * QS, SS = MB * BS + 64;  // bytes
  const bf16_t* abase[UPW];
  int apair[UPW], awrite[UPW];
#pragma unroll
  for (int j = 0; j < UPW; ++j) {
    const int u = nw + NWV * j;
    const int half = u % 2, b = (u / 2) % MB, piece = lane & 7, row = 8 * half + (lane >> 3);
    apair[j] = 2 * (u / (2 * MB));
    abase[j] = A + (size_t)min(16 * b + row, M - 1) * K + 8 * piece;
    awrite[j] = (apair[j] + piece / 4) * SS + b * BS + (piece % 4) * QS + 16 * row;
  }
  unsigned char* group_buf = smem_raw + (size_t)kg * 2 * KC * SS;
  const int aread = quad * QS + 16 * r16;

  f32x4_t acc[WT][MB];
#pragma unroll
  for (int t = 0; t < WT; ++t)
#pragma unroll
    for (int b = 0; b < MB; ++b) acc[t][b] = (f32x4_t){0.f, 0.f, 0.f, 0.f};

  // Every load has the same number of younger loads behind it when it is waited for, in the
  // first chunks as in the later ones (the order of issue before the loop is the loop's), so
  // the waits the compiler counts out leave the rest of the ring in flight.
  bf16x8_t w[DEPTH][KC][WT], ar[UPW], zero;
#pragma unroll
  for (int e = 0; e < 8; ++e) zero[e] = (bf16_t)0.0f;
#pragma unroll
  for (int d = 0; d < DEPTH; ++d) {
    const int s_w = chunk_start(d);
#pragma unroll
    for (int s = 0; s < KC; ++s)
#pragma unroll
      for (int t = 0; t < WT; ++t)
        w[d][s][t] = ((const bf16x8_t*)(wbase[t] + (size_t)min(s_w + s, last_step) * wstep[t % NT]))[lane];
  }
  {
    const int s_a = chunk_start(0);
#pragma unroll
    for (int j = 0; j < UPW; ++j) ar[j] = *(const bf16x8_t*)(abase[j] + (min(s_a + apair[j], last_pair) << 5));
#pragma unroll
    for (int j = 0; j < UPW; ++j) *(bf16x8_t*)(group_buf + awrite[j]) = ar[j];
    const int s_a1 = chunk_start(1);
#pragma unroll
    for (int j = 0; j < UPW; ++j) ar[j] = *(const bf16x8_t*)(abase[j] + (min(s_a1 + apair[j], last_pair) << 5));
  }

  for (int c0 = 0; c0 < chunks; c0 += DEPTH) {
#pragma unroll
    for (int d = 0; d < DEPTH; ++d) {
      const int c = c0 + d;  // with an odd number of chunks and DEPTH 2 the last one is empty
      __syncthreads();       // chunk c is staged, and nobody reads the other buffer any more
      const unsigned char* cur = group_buf + (c & 1) * KC * SS + aread;
      unsigned char* nxt = group_buf + ((c + 1) & 1) * KC * SS;
      const int s_cur = chunk_start(c), s_w = chunk_start(c + DEPTH), s_a = chunk_start(c + 2);
      const int n_live = g1 - s_cur;
      // the activations of step s + 1 leave LDS while the products of step s run
      bf16x8_t a[2][MB];
#pragma unroll
      for (int b = 0; b < MB; ++b) a[0][b] = *(const bf16x8_t*)(cur + b * BS);
#pragma unroll
      for (int s = 0; s < KC; ++s) {
        if (s + 1 < KC) {
#pragma unroll
          for (int b = 0; b < MB; ++b) a[(s + 1) & 1][b] = *(const bf16x8_t*)(cur + (s + 1) * SS + b * BS);
        }
        // a step past the group's end counts as zeros: a select, because a branch round the
        // products would make the accumulators leave their registers at every step
        const bool live = s < n_live;
#pragma unroll
        for (int t = 0; t < WT; ++t) {
          const bf16x8_t wt = live ? w[d][s][t] : zero;
#pragma unroll
          for (int b = 0; b < MB; ++b)
            acc[t][b] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wt, a[s & 1][b], acc[t][b], 0, 0, 0);
        }
#pragma unroll
        for (int t = 0; t < WT; ++t)
          w[d][s][t] = ((const bf16x8_t*)(wbase[t] + (size_t)min(s_w + s, last_step) * wstep[t % NT]))[lane];
      }
      // the activations of chunk c + 1, asked for a chunk ago, go to the other buffer; those
      // of chunk c + 2 are asked for
#pragma unroll
      for (int j = 0; j < UPW; ++j) *(bf16x8_t*)(nxt + awrite[j]) = ar[j];
#pragma unroll
      for (int j = 0; j < UPW; ++j)
        ar[j] = *(const bf16x8_t*)(abase[j] + (min(s_a + apair[j], last_pair) << 5));
    }
  }

  if (KW > 1) {  // the K groups' sums meet in group 0, added in group order
    __syncthreads();
    float* red = (float*)smem_raw;  // [KW - 1][NWV][WT][MB][4][64]
    if (kg > 0) {
#pragma unroll
      for (int t = 0; t < WT; ++t)
#pragma unroll
        for (int b = 0; b < MB; ++b)
#pragma unroll
          for (int r = 0; r < 4; ++r)
            red[(((((kg - 1) * NWV + nw) * WT + t) * MB + b) * 4 + r) * 64 + lane] = acc[t][b][r];
    }
    __syncthreads();
    if (kg > 0) return;
    for (int g = 1; g < KW; ++g)
#pragma unroll
      for (int t = 0; t < WT; ++t)
#pragma unroll
        for (int b = 0; b < MB; ++b)
#pragma unroll
          for (int r = 0; r < 4; ++r)
            acc[t][b][r] += red[(((((g - 1) * NWV + nw) * WT + t) * MB + b) * 4 + r) * 64 + lane];
  }

  // acc[t][b][r]: output row 16 b + r16, column 16 (tile0 + t) + 4 quad + r: one vector store
  C += (size_t)blockIdx.y * M * N;
#pragma unroll
  for (int t = 0; t < NT; ++t) {
    if (tile0 + t >= tile_hi) continue;
    const int n = 16 * (tile0 + t) + 4 * quad;
#pragma unroll
    for (int b = 0; b < MB; ++b) {
      const int m = 16 * b + r16;
      if (m >= M) continue;
      float o[4];
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        if (GATED) {  // gate and up value rounded to bfloat16 first, as the unfused kernels see them
          const float g = (float)(bf16_t)acc[t][b][r];
          o[r] = g / (1.0f + expf(-g)) * (float)(bf16_t)acc[NT + t][b][r];
        } else {
          o[r] = acc[t][b][r];
        }
      }
      store4(C + (size_t)m * N + n, o);
    }
  }
}

template <int MB, int KW, int NWV, int NT, int KC, int DEPTH, bool GATED>
static int launch_mid(const bf16_t* a, const bf16_t* w, void* c, int out_dtype, int M, int N, int K,
                      hipStream_t stream, int k_parts) {
  constexpr int WT = GATED ? 2 * NT : NT;
  const int per_block = NWV * NT, tiles = N / 16;
  // as many blocks as compute units where the tiles allow it, each with its even share
  constexpr int COMPUTE_UNITS = 256;  // of an MI355X
  int blocks = tiles <= COMPUTE_UNITS / k_parts ? tiles
                                                : max(COMPUTE_UNITS / k_parts, (tiles + per_block - 1) / per_block);
  blocks = max(blocks, (tiles + per_block - 1) / per_block);
  dim3 grid(blocks, k_parts), block(64 * KW * NWV);
  const size_t stage = (size_t)KW * 2 * KC * (MB * 4 * (256 + 16) + 64);
  const size_t meet = (size_t)(KW - 1) * NWV * WT * MB * 1024;
  const size_t smem = stage > meet ? stage : meet;
  QRT_CHECK(smem <= 160 * 1024, "gemm_bf16: the staging of this configuration needs %zu bytes of LDS", smem);
#define GO(TO)                                                                                          \
  do {                                                                                                  \
    auto kernel = gemm_bf16_mid_kernel<MB, KW, NWV, NT, KC, DEPTH, GATED, TO>;                          \
    static bool allowed = false; /* once per kernel: not inside a stream capture again and again */    \
    if (smem > 64 * 1024 && !allowed) {                                                                 \
      if (hipFuncSetAttribute((const void*)kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem) != hipSuccess) \
        return qrt_fail("gemm_bf16: cannot get %zu bytes of LDS", smem);                                \
      allowed = true;                                                                                   \
    }                                                                                                   \
    kernel<<<grid, block, smem, stream>>>(a, w, (TO*)c, M, N, K);                                       \
  } while (0)
  if (out_dtype == QRT_BF16) GO(bf16_t);
  else if (out_dtype == QRT_F32) GO(float);
  else return qrt_fail("gemm_bf16: unknown output dtype %d", out_dtype);
#undef GO
  QRT_LAUNCH_CHECK("gemm_bf16_mid");
  return 0;
}

// 17 to 64 rows on tile-major weights. Configurations from timing every combination of 1 to 4
// K groups, 1 to 4 waves a group, 1 or 2 tiles a wave, chunks of 4, 6 or 8 k-steps and weights
// one or two chunks ahead that fits LDS and registers (some 150 per form) on the shapes of the
// 4B and 8B models at 32 and 64 rows, each on the weight matrices of 36 layers in turn (one
// matrix over and over stays in the memory-side cache and flatters every configuration, the
// small products most): K groups of two waves with one tile each where the result is wanted
// whole (three groups from 33 rows on, two below: 12.4 us against 13.6 for the former choice
// at 64 rows of the 4B size, 16.7 against 18.5 at the 8B size); one group of three waves, a
// gate and an up tile each, for the gated form; one group of three waves with two tiles each
// where K is cut over blocks. The weights run one chunk ahead everywhere: two chunks lost 3 to
// 6 % in the gated form.
template <int MB>
static int mid(const bf16_t* a, const bf16_t* w, void* c, int out_dtype, int M, int N, int K, int gated,
               hipStream_t st, int k_parts) {
  if (gated) return launch_mid<MB, 1, 3, 1, 6, 1, true>(a, w, c, out_dtype, M, N, K, st, 1);
  if (k_parts > 1) return launch_mid<MB, 1, 3, 2, 6, 1, false>(a, w, c, out_dtype, M, N, K, st, k_parts);
  // The whole result of an ungated product: up to 64 rows only. Beyond, every block would have to
  // fetch more activations than weights, and the vendor library was measured to be faster.
  if constexpr (MB <= 4) {
    // very many tiles (the vocabulary head): eight tiles share the staged activations
    if (N >= 32768) return launch_mid<MB, 1, 4, 2, 8, 1, false>(a, w, c, out_dtype, M, N, K, st, 1);
    return launch_mid<MB, (MB <= 2 ? 2 : 3), 2, 1, 4, 1, false>(a, w, c, out_dtype, M, N, K, st, 1);
  }
  return qrt_fail("gemm_bf16: above 64 rows only the gated form and products cut along K run on tile-major weights (M=%d)", M);
}

template <int MT, int NT>
static int launch(const bf16_t* a, const bf16_t* w, void* c, int out_dtype, int M, int N, int K, hipStream_t stream) {
  dim3 grid((N + 64 * NT - 1) / (64 * NT), (M + 16 * MT - 1) / (16 * MT)), block(256);
  QRT_CHECK(grid.y <= 65535, "gemm_bf16: M=%d is too large for one launch", M);
  const bool aligned = (K % 8 == 0) && ((uintptr_t)a % 16 == 0) && ((uintptr_t)w % 16 == 0);
#define GO(AL, TO) gemm_bf16_kernel<MT, NT, AL, TO><<<grid, block, 0, stream>>>(a, w, (TO*)c, M, N, K)
  if (out_dtype == QRT_BF16) { if (aligned) GO(true, bf16_t); else GO(false, bf16_t); }
  else if (out_dtype == QRT_F32) { if (aligned) GO(true, float); else GO(false, float); }
  else return qrt_fail("gemm_bf16: unknown output dtype %d", out_dtype);
#undef GO
  QRT_LAUNCH_CHECK("gemm_bf16");
  return 0;
}

// gated = 0: C[M, N] = A W^T with W [N, K].
// gated = 1: W is [2N, K] (gate rows, then up rows) and C[M, N] = silu(A Wg^T) * (A Wu^T).
// tiled = 1 or 2: W is stored tile-major, [rows / 16][K / 32][64 lanes][8]: lane q * 16 + i of tile
// (r, s) holds W[16 r + i][32 s + 8 q .. + 7]; needs N % 16 == 0 and K % 32 == 0. 1: the few-row
// kernel, M <= 16. 2: the kernel that shares the activations through LDS, K % 64 == 0 and M <= 64
// (M <= 128 for the gated form and for K parts).
// k_parts > 1 (tile-major, not gated, float32 out): K is cut into that many parts, each handled
// by blocks of its own, and C is [k_parts, M, N]: planes to be added by the caller.
extern "C" int qrt_gemm_bf16(const void* a, const void* w, void* c, int out_dtype, int M, int N, int K, int gated,
                             int tiled, int k_parts, hipStream_t stream) {
  QRT_CHECK(M >= 0 && N > 0 && K > 0, "gemm_bf16: bad sizes M=%d N=%d K=%d", M, N, K);
  QRT_CHECK(gated == 0 || gated == 1, "gemm_bf16: unknown mode %d", gated);
  QRT_CHECK(k_parts >= 1 && k_parts <= 64, "gemm_bf16: bad number of K parts %d", k_parts);
  QRT_CHECK(k_parts == 1 || (tiled != 0 && !gated && out_dtype == QRT_F32),
            "gemm_bf16: K parts need tile-major weights, no gate and float32 output");
  if (M == 0) return 0;
  const bf16_t* A = (const bf16_t*)a;
  const bf16_t* W = (const bf16_t*)w;
  const bool aligned = (K % 32 == 0) && ((uintptr_t)a % 16 == 0) && ((uintptr_t)w % 16 == 0);
  if (tiled == 1) {  // the few-row kernel
    QRT_CHECK(M <= 16 && N % 16 == 0 && aligned,
              "gemm_bf16: the few-row kernel on tile-major weights needs M <= 16, N %% 16 == 0, K %% 32 == 0 "
              "(M=%d N=%d K=%d)", M, N, K);
    return gated ? skinny_tiled<true>(A, W, c, out_dtype, M, N, K, stream, 1)
                 : skinny_tiled<false>(A, W, c, out_dtype, M, N, K, stream, k_parts);
  }
  if (tiled == 2) {  // the kernel that shares the activations through LDS
    QRT_CHECK(M <= 128 && N % 16 == 0 && N <= (1 << 20) && K % 64 == 0 && aligned,
              "gemm_bf16: the LDS-sharing kernel needs M <= 128, N %% 16 == 0, N <= 2^20, K %% 64 == 0 "
              "(M=%d N=%d K=%d)", M, N, K);
    if (M <= 16) return mid<1>(A, W, c, out_dtype, M, N, K, gated, stream, k_parts);
    if (M <= 32) return mid<2>(A, W, c, out_dtype, M, N, K, gated, stream, k_parts);
    if (M <= 48) return mid<3>(A, W, c, out_dtype, M, N, K, gated, stream, k_parts);
    if (M <= 64) return mid<4>(A, W, c, out_dtype, M, N, K, gated, stream, k_parts);
    if (M <= 96) return mid<6>(A, W, c, out_dtype, M, N, K, gated, stream, k_parts);
    return mid<8>(A, W, c, out_dtype, M, N, K, gated, stream, k_parts);
  }
  QRT_CHECK(tiled == 0, "gemm_bf16: unknown weight layout %d", tiled);
  if (M <= 16 && aligned) return gated ? skinny<true>(A, W, c, out_dtype, M, N, K, stream)
                                       : skinny<false>(A, W, c, out_dtype, M, N, K, stream);
  QRT_CHECK(gated == 0, "gemm_bf16: the gated form needs K a multiple of 32, and M <= 16 or tile-major weights "
            "(M=%d K=%d)", M, K);
  if (M <= 16) return launch<1, 2>(A, W, c, out_dtype, M, N, K, stream);
  if (M <= 32) return launch<2, 2>(A, W, c, out_dtype, M, N, K, stream);
  return launch<4, 4>(A, W, c, out_dtype, M, N, K, stream);
}
