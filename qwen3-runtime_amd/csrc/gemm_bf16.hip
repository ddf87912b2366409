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
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
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
// M <= 64 (decoding): the product is a stream of the weight matrix, so the
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
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
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
        for (int t = 0; t < WT; ++t) w[u][t] = *(const bf16x8_t*)(wrow[t] + (size_t)s * WSTEP);
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
  if (M <= 16) {
    if (tiles >= 2048) return launch_skinny<1, 8, 2, 8, GATED>(a, w, c, out_dtype, M, N, K, st);
    if (tiles >= 512 || K < 4096) return launch_skinny<1, 8, 1, 8, GATED>(a, w, c, out_dtype, M, N, K, st);
    return launch_skinny<1, 16, 1, 8, GATED>(a, w, c, out_dtype, M, N, K, st);
  }
  if (M <= 32) {
    if (tiles >= 512) return launch_skinny<2, 8, 2, 4, GATED>(a, w, c, out_dtype, M, N, K, st);
    return launch_skinny<2, 8, 1, 8, GATED>(a, w, c, out_dtype, M, N, K, st);
  }
  if (tiles >= 512 && !GATED) return launch_skinny<4, 8, 2, 2, GATED>(a, w, c, out_dtype, M, N, K, st);
  return launch_skinny<4, 8, 1, 4, GATED>(a, w, c, out_dtype, M, N, K, st);
}

// Tile-major weights, M <= 16. Configurations from timing all of them on the shapes of the
// 4B model: eight waves and eight steps in flight everywhere; two row tiles per block where
// there are many tiles and no gate (the activations are then read half as often).
template <bool GATED>
static int skinny_tiled(const bf16_t* a, const bf16_t* w, void* c, int out_dtype, int M, int N, int K,
                        hipStream_t st, int k_parts) {
  const int tiles = N / 16;
  if (!GATED && tiles >= 384 && k_parts == 1)
    return launch_skinny<1, 8, 2, 8, GATED, true>(a, w, c, out_dtype, M, N, K, st);
  return launch_skinny<1, 8, 1, 8, GATED, true>(a, w, c, out_dtype, M, N, K, st, k_parts);
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

// Tuning aid: run one named configuration of the few-row kernel (M <= 16), so that
// configurations can be timed against each other on the shapes of a model.
extern "C" int qrt_gemm_bf16_variant(const void* a, const void* w, void* c, int out_dtype, int M, int N, int K,
                                     int gated, int variant, hipStream_t stream) {
  QRT_CHECK(M >= 1 && M <= 16 && K % 32 == 0, "gemm_bf16_variant: M <= 16 and K a multiple of 32 only");
  const bf16_t* A = (const bf16_t*)a;
  const bf16_t* W = (const bf16_t*)w;
#define V(ID, NW, NT, U)                                                                            \
  if (variant == ID)                                                                                \
    return gated ? launch_skinny<1, NW, NT, U, true>(A, W, c, out_dtype, M, N, K, stream)           \
                 : launch_skinny<1, NW, NT, U, false>(A, W, c, out_dtype, M, N, K, stream);
  V(0, 8, 1, 8) V(1, 8, 2, 8) V(2, 16, 1, 8) V(4, 4, 1, 8) V(10, 4, 1, 16)
#undef V
  // 100 + id: the same on tile-major weights
#define V(ID, NW, NT, U)                                                                            \
  if (variant == 100 + ID)                                                                          \
    return gated ? launch_skinny<1, NW, NT, U, true, true>(A, W, c, out_dtype, M, N, K, stream)     \
                 : launch_skinny<1, NW, NT, U, false, true>(A, W, c, out_dtype, M, N, K, stream);
  V(0, 8, 1, 8) V(1, 8, 2, 8) V(2, 16, 1, 8) V(4, 4, 1, 8) V(10, 4, 1, 16)
#undef V
  return qrt_fail("gemm_bf16_variant: no variant %d", variant);
}

// gated = 0: C[M, N] = A W^T with W [N, K].
// gated = 1: W is [2N, K] (gate rows, then up rows) and C[M, N] = silu(A Wg^T) * (A Wu^T).
// tiled = 1: W is stored tile-major, [rows / 16][K / 32][64 lanes][8]: lane q * 16 + i of tile
// (r, s) holds W[16 r + i][32 s + 8 q .. + 7]; needs M <= 16, N % 16 == 0, K % 32 == 0.
// k_parts > 1 (tile-major, not gated, float32 out): K is cut into that many parts, each handled
// by blocks of its own, and C is [k_parts, M, N]: planes to be added by the caller.
extern "C" int qrt_gemm_bf16(const void* a, const void* w, void* c, int out_dtype, int M, int N, int K, int gated,
                             int tiled, int k_parts, hipStream_t stream) {
  QRT_CHECK(M >= 0 && N > 0 && K > 0, "gemm_bf16: bad sizes M=%d N=%d K=%d", M, N, K);
  QRT_CHECK(gated == 0 || gated == 1, "gemm_bf16: unknown mode %d", gated);
  QRT_CHECK(k_parts >= 1 && k_parts <= 64, "gemm_bf16: bad number of K parts %d", k_parts);
  QRT_CHECK(k_parts == 1 || (tiled && !gated && out_dtype == QRT_F32),
            "gemm_bf16: K parts need tile-major weights, no gate and float32 output");
  if (M == 0) return 0;
  const bf16_t* A = (const bf16_t*)a;
  const bf16_t* W = (const bf16_t*)w;
  const bool aligned = (K % 32 == 0) && ((uintptr_t)a % 16 == 0) && ((uintptr_t)w % 16 == 0);
  if (tiled) {
    QRT_CHECK(M <= 16 && N % 16 == 0 && aligned,
              "gemm_bf16: tile-major weights need M <= 16, N %% 16 == 0, K %% 32 == 0 (M=%d N=%d K=%d)", M, N, K);
    return gated ? skinny_tiled<true>(A, W, c, out_dtype, M, N, K, stream, 1)
                 : skinny_tiled<false>(A, W, c, out_dtype, M, N, K, stream, k_parts);
  }
  if (M <= 64 && aligned) return gated ? skinny<true>(A, W, c, out_dtype, M, N, K, stream)
                                       : skinny<false>(A, W, c, out_dtype, M, N, K, stream);
  QRT_CHECK(gated == 0, "gemm_bf16: the gated form needs M <= 64 and K a multiple of 32 (M=%d K=%d)", M, K);
  if (M <= 16) return launch<1, 2>(A, W, c, out_dtype, M, N, K, stream);
  if (M <= 32) return launch<2, 2>(A, W, c, out_dtype, M, N, K, stream);
  return launch<4, 4>(A, W, c, out_dtype, M, N, K, stream);
}
