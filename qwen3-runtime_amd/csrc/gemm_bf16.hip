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
#include <type_traits>

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


// ---------------------------------------------------------------- few rows, K a multiple of 32 only
// M <= 16 (decoding): the product is a stream of the weight matrix, so the
// layout is chosen for memory parallelism, not for reuse. A block owns NT
// tiles of 16 weight rows and all of K; its NW waves take the 32-wide k-steps
// round-robin, so that in every round the block reads 16 rows x NW x 64
// contiguous bytes per tile. A wave issues the loads of U steps before the
// first MFMA of them. Each wave keeps MB accumulators (16 rows of M each) per
// tile; activations come from L2/L1 (they are tiny). Partial sums meet in LDS
// and are added in wave order, so the result does not depend on timing. A
// lane's load is 16 bytes of one of 16 rows, half a cache line: where K is a
// multiple of 64 the kernel after this one, which fetches whole lines, is up
// to twice as fast and takes the product.
//
// GATED: W holds 2N rows, gate rows then up rows; the block owns matching
// tiles of both and writes silu(gate) * up, so the gated feed-forward's
// intermediate [M, 2N] never reaches memory.
template <int MB, int NW, int NT, int U, bool GATED, typename TO>
__global__ __launch_bounds__(64 * NW) void gemm_bf16_skinny_kernel(const bf16_t* __restrict__ A,
                                                                    const bf16_t* __restrict__ W,
                                                                    TO* __restrict__ C, int M, int N, int K) {
  constexpr int WT = GATED ? 2 * NT : NT;  // weight tiles per block
  extern __shared__ float red[];            // [NW][WT][MB][4][64]
  const int lane = threadIdx.x & 63, wave = uniform_wave_number();
  const int r16 = lane & 15, quad = lane >> 4;
  const int n0 = blockIdx.x * 16 * NT;
  const bf16_t* wrow[WT];
#pragma unroll
  for (int t = 0; t < NT; ++t) {
    const int n = min(n0 + 16 * t + r16, N - 1);
    wrow[t] = W + (size_t)n * K + 8 * quad;
    if (GATED) wrow[NT + t] = W + (size_t)(N + n) * K + 8 * quad;
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

  const int steps = K >> 5;  // K is a multiple of 32 here
  bf16x8_t zero;
#pragma unroll
  for (int e = 0; e < 8; ++e) zero[e] = (bf16_t)0.0f;
  for (int s0 = wave; s0 < steps; s0 += U * NW) {
    bf16x8_t w[U][WT], a[U][MB];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int s = s0 + u * NW;
      if (s < steps) {  // uniform over the wave
#pragma unroll
        for (int t = 0; t < WT; ++t) w[u][t] = load_once8(wrow[t] + (size_t)s * 32);
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

template <int MB, int NW, int NT, int U, bool GATED>
static int launch_skinny(const bf16_t* a, const bf16_t* w, void* c, int out_dtype, int M, int N, int K,
                         hipStream_t stream) {
  dim3 grid((N + 16 * NT - 1) / (16 * NT)), block(64 * NW);
  const size_t smem = (size_t)NW * (GATED ? 2 : 1) * NT * MB * 4 * 64 * sizeof(float);
  if (out_dtype == QRT_BF16)
    gemm_bf16_skinny_kernel<MB, NW, NT, U, GATED, bf16_t><<<grid, block, smem, stream>>>(a, w, (bf16_t*)c, M, N, K);
  else if (out_dtype == QRT_F32)
    gemm_bf16_skinny_kernel<MB, NW, NT, U, GATED, float><<<grid, block, smem, stream>>>(a, w, (float*)c, M, N, K);
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

// ---------------------------------------------------------------- few rows, whole cache lines
// M <= 16 on the weights as stored, [N, K] row-major, K a multiple of 64. The MFMA wants, per
// lane, row lane & 15 and 16 bytes at 8 (lane / 16): loaded straight to registers that is
// sixteen half cache lines an instruction, which costs up to half the stream's speed (a
// tile-major second copy of every matrix, each 16 x 32 tile a contiguous KB in the lanes' order,
// was the way round that before; this kernel is as fast on the 4B, 8B and 32B shapes, within
// 3 % either way, and needs no copy). Here the weights go to LDS by direct loads instead, whose
// lanes may take any addresses: lane l fetches 16 bytes of row l / 8, so one instruction brings
// 8 rows x 128 bytes, whole lines, and two of them a tile of 16 rows by a pair of k-steps (64
// columns). The instruction writes lane l's piece to LDS at 16 l, so the pieces of a row are
// permuted on the way in: lane l asks for piece (l & 7) ^ (l / 8) of its row, which puts piece
// c of row r at 128 r + 16 (c ^ (r & 7)), and the operand reads (row lane & 15, piece
// 4 h + lane / 16 for k-step h of the pair) then touch every bank once. The activations' 16
// rows come the same way (rows past M repeat row M - 1; their results are not stored), so the
// loop holds no load to registers and the waits on the loads' counter can be counted by hand
// (the compiler does not count them out for direct loads): every pair is 2 (tiles + 1) loads,
// U pairs are in flight in a ring of the wave's own, and a wave waits until all but the
// youngest U - 1 pairs have landed. The weights are loaded as data used once, so that the
// activations stay in the caches (10 % of the time at the large shapes). A block owns NT tiles
// (and, GATED, the matching up tiles: it writes silu(gate) * up) and part blockIdx.y of K, whose
// result is plane blockIdx.y of the output (the caller adds the planes: used where the result
// feeds a residual add); its NW waves take the pairs round-robin and meet in LDS, added in
// wave order.
#define QRT_WAIT_LOADS(n) asm volatile("s_waitcnt vmcnt(%0)" ::"n"(n) : "memory")
#define QRT_WAIT_LDS() asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory")
// A barrier without the fence of __syncthreads(), which would wait for every direct load to LDS
// in flight: what has to have landed is waited for by hand before it.
#define QRT_BARRIER() asm volatile("s_barrier" ::: "memory")
typedef const void __attribute__((address_space(1)))* global_ptr_t;
typedef void __attribute__((address_space(3)))* lds_ptr_t;

template <int NW, int NT, int U, bool GATED, typename TO>
__global__ __launch_bounds__(64 * NW) void gemm_bf16_rows_kernel(const bf16_t* __restrict__ A,
                                                                  const bf16_t* __restrict__ W,
                                                                  TO* __restrict__ C, int M, int N, int K) {
  constexpr int WT = GATED ? 2 * NT : NT, UNITS = WT + 1, LOADS = 2 * UNITS, SLOT = UNITS * 2048;
  constexpr int ONCE = 2;  // the cache policy of a non-temporal load
  static_assert((U - 1) * LOADS < 64, "the loads' counter holds 63");
  extern __shared__ __align__(16) unsigned char rows_lds[];  // [NW][U][UNITS] x 2 KB, then the partial sums
  const int lane = threadIdx.x & 63, wave = uniform_wave_number();
  const int r16 = lane & 15, quad = lane >> 4;
  const int n0 = blockIdx.x * 16 * NT;
  unsigned char* ring = rows_lds + (size_t)wave * U * SLOT;
  const int sub = lane >> 3, piece = (lane & 7) ^ sub;
  const bf16_t* src[UNITS][2];
#pragma unroll
  for (int j = 0; j < 2; ++j) {
#pragma unroll
    for (int t = 0; t < NT; ++t) {
      const int n = min(n0 + 16 * t + 8 * j + sub, N - 1);  // rows past the end repeat the last; not stored
      src[t][j] = W + (size_t)n * K + 8 * piece;
      if (GATED) src[NT + t][j] = W + (size_t)(N + n) * K + 8 * piece;
    }
    src[WT][j] = A + (size_t)min(8 * j + sub, M - 1) * K + 8 * piece;
  }
  const int all_pairs = K >> 6;
  const int part = (all_pairs + gridDim.y - 1) / gridDim.y;
  const int p_first = blockIdx.y * part, p_end = min(all_pairs, p_first + part);
  const int mine = max(0, (p_end - p_first - wave + NW - 1) / NW);  // pairs of this wave
  C += (size_t)blockIdx.y * M * N;
  auto fetch = [&](int i, int slot) {  // the wave's i-th pair into a slot of its ring
    const size_t at = (size_t)(p_first + wave + i * NW) * 64;
    unsigned char* dst = ring + slot * SLOT;
#pragma unroll
    for (int un = 0; un < UNITS; ++un)
#pragma unroll
      for (int j = 0; j < 2; ++j) {
        if (un < WT)
          __builtin_amdgcn_global_load_lds((global_ptr_t)(src[un][j] + at), (lds_ptr_t)(dst + un * 2048 + j * 1024), 16, 0, ONCE);
        else
          __builtin_amdgcn_global_load_lds((global_ptr_t)(src[un][j] + at), (lds_ptr_t)(dst + un * 2048 + j * 1024), 16, 0, 0);
      }
  };
  f32x4_t acc[WT];
#pragma unroll
  for (int t = 0; t < WT; ++t) acc[t] = (f32x4_t){0.f, 0.f, 0.f, 0.f};
  int fetched = 0;
  for (; fetched < U && fetched < mine; ++fetched) fetch(fetched, fetched);
  const int read_at[2] = {r16 * 128 + 16 * (quad ^ (r16 & 7)), r16 * 128 + 16 * ((4 + quad) ^ (r16 & 7))};
  int slot = 0;
  for (int i = 0; i < mine; ++i) {
    // pair i has landed when at most the U - 1 pairs fetched after it are still on their way;
    // near the end fewer follow it, and the wave waits for all
    if (fetched - i == U) QRT_WAIT_LOADS((U - 1) * LOADS);
    else QRT_WAIT_LOADS(0);
    const unsigned char* at = ring + slot * SLOT;
    bf16x8_t w[WT][2], a[2];
#pragma unroll
    for (int h = 0; h < 2; ++h) {
#pragma unroll
      for (int t = 0; t < WT; ++t) w[t][h] = *(const bf16x8_t*)(at + t * 2048 + read_at[h]);
      a[h] = *(const bf16x8_t*)(at + WT * 2048 + read_at[h]);
    }
    QRT_WAIT_LDS();  // the slot is in registers: the next pair may overwrite it
    if (fetched < mine) {
      fetch(fetched, slot);
      ++fetched;
    }
#pragma unroll
    for (int h = 0; h < 2; ++h)
#pragma unroll
      for (int t = 0; t < WT; ++t) acc[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(w[t][h], a[h], acc[t], 0, 0, 0);
    slot = slot + 1 == U ? 0 : slot + 1;
  }
  __syncthreads();  // every wave has read its last slot: the rings' room now takes the partial sums
  float* red = (float*)rows_lds;  // [NW][WT][4][64]
#pragma unroll
  for (int t = 0; t < WT; ++t)
#pragma unroll
    for (int r = 0; r < 4; ++r) red[((wave * WT + t) * 4 + r) * 64 + lane] = acc[t][r];
  __syncthreads();
  // one thread per (tile, lane) adds the waves' parts in order
  for (int i = threadIdx.x; i < NT * 64; i += 64 * NW) {
    const int l = i & 63, t = i >> 6;
    const int m = l & 15;
    const int nn = n0 + 16 * t + 4 * (l >> 4);
    float sum[4], sum2[4];
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      float v = 0.f, v2 = 0.f;
      for (int w = 0; w < NW; ++w) {
        v += red[((w * WT + t) * 4 + r) * 64 + l];
        if (GATED) v2 += red[((w * WT + NT + t) * 4 + r) * 64 + l];
      }
      sum[r] = v;
      sum2[r] = v2;
    }
    if (m < M) {
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        if (nn + r < N) {
          const float g = (float)(bf16_t)sum[r];  // rounded to bfloat16 first, as the unfused kernels see them
          const float out = GATED ? g / (1.0f + expf(-g)) * (float)(bf16_t)sum2[r] : sum[r];
          C[(size_t)m * N + nn + r] = from_f32<TO>(out);
        }
      }
    }
  }
}

template <int NW, int NT, int U, bool GATED>
static int launch_rows(const bf16_t* a, const bf16_t* w, void* c, int out_dtype, int M, int N, int K,
                       hipStream_t stream, int k_parts) {
  constexpr int WT = GATED ? 2 * NT : NT;
  dim3 grid((N + 16 * NT - 1) / (16 * NT), k_parts), block(64 * NW);
  constexpr size_t smem = (size_t)NW * U * (WT + 1) * 2048;  // the partial sums, NW * WT KB, fit in it
  static_assert(smem <= 160 * 1024, "the rings of this configuration do not fit LDS");
#define GO(TO)                                                                                          \
  do {                                                                                                  \
    auto kernel = gemm_bf16_rows_kernel<NW, NT, U, GATED, TO>;                                          \
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
  QRT_LAUNCH_CHECK("gemm_bf16_rows");
  return 0;
}

// Configurations from timing 16 of them (2 to 8 waves, 1 or 2 row tiles a block, 2 to 6 pairs in
// flight) on the shapes of the 4B, 8B and 32B models at 1, 8 and 16 rows, each on the weight
// matrices of 36 layers in turn: four waves everywhere (several small blocks on a compute unit
// hide each other's ends better than one large one). Gated: one row tile, three pairs in flight
// (19.1 us at the 4B size, 5.2 TB/s; 81.4 at the 32B size, 6.4 TB/s). The whole result: two tiles a block, except where K is a multiple of 2,048 (the rows of
// two tiles then start in the same memory channels: 14.0 us against 11.2 for the 8B q/k/v product)
// and for a few hundred tiles of long rows. K cut into planes: two tiles a block from K = 9,728 on.
template <bool GATED>
static int few_rows(const bf16_t* a, const bf16_t* w, void* c, int out_dtype, int M, int N, int K, hipStream_t st,
                    int k_parts) {
  const int tiles = (N + 15) / 16;
  if (GATED) return launch_rows<4, 1, 3, GATED>(a, w, c, out_dtype, M, N, K, st, 1);
  if (k_parts > 1) {
    if (K >= 9728) return launch_rows<4, 2, 2, GATED>(a, w, c, out_dtype, M, N, K, st, k_parts);
    return launch_rows<4, 1, 2, GATED>(a, w, c, out_dtype, M, N, K, st, k_parts);
  }
  if (K % 2048 == 0) {
    if (tiles >= 2048) return launch_rows<4, 1, 3, GATED>(a, w, c, out_dtype, M, N, K, st, 1);
    return launch_rows<4, 1, 2, GATED>(a, w, c, out_dtype, M, N, K, st, 1);
  }
  if (tiles >= 2048) return launch_rows<4, 2, 3, GATED>(a, w, c, out_dtype, M, N, K, st, 1);
  if (tiles >= 384 && K <= 4096) return launch_rows<4, 2, 2, GATED>(a, w, c, out_dtype, M, N, K, st, 1);
  if (tiles >= 384) return launch_rows<4, 1, 4, GATED>(a, w, c, out_dtype, M, N, K, st, 1);
  return launch_rows<4, 1, 2, GATED>(a, w, c, out_dtype, M, N, K, st, 1);
}

__device__ __forceinline__ void store4(float* p, const float (&o)[4]) {
  *(f32x4_t*)p = (f32x4_t){o[0], o[1], o[2], o[3]};
}
__device__ __forceinline__ void store4(bf16_t* p, const float (&o)[4]) {
  typedef bf16_t bf16x4_t __attribute__((ext_vector_type(4)));
  *(bf16x4_t*)p = (bf16x4_t){(bf16_t)o[0], (bf16_t)o[1], (bf16_t)o[2], (bf16_t)o[3]};
}

// A page of zeros for a wave that has no tile of its own: read at no cost in memory traffic.
__device__ bf16x8_t qrt_zero_tile[64];

// ---------------------------------------------------------------- 17 to 128 rows, weights as stored
// Still a stream of the weight matrix, but the activations now weigh as much as the weights if
// every wave fetches its own: four accumulator blocks of 16 rows want 4 KB of activations for
// each KB of weights. So the waves that walk the same part of K (a K group) share the
// activations through LDS: NWV waves side by side along N, NT tiles each, read one staged copy,
// and the traffic for activations falls to MB / (NWV * NT) of the weights'. KW such groups in a
// block take consecutive parts of the block's k-steps (the block's k-steps being part
// blockIdx.y of all, as in the few-row kernel) and meet in LDS at the end, added in group order.
// Blocks start at different chunks of their k-steps and wrap round: every block reads all the
// activations, and in step they would all ask the same L2 channels at the same time. What a
// compute unit can pull through its memory pipeline is the limit, so the row tiles are dealt out
// evenly over gridDim.x blocks, chosen by the host as the number of compute units where there
// are more tiles than that: a block gets floor or ceil of tiles / blocks, at most NWV * NT. A
// wave without a tile reads a page of zeros instead and stores nothing.
// Both operands come to LDS by direct loads, as in the few-row kernel: a unit is 16 rows by a
// pair of k-steps, two loads of 8 rows x 128 bytes, piece c of row r at 128 r + 16 (c ^ (r & 7)).
// The waves of a K group stage the activations of chunk c + 1 (KC / 2 pairs x MB row blocks,
// shared) while chunk c is used; each wave streams its own tiles' weights into a ring of one
// chunk, a pair being fetched for chunk c + 1 as soon as the same pair of chunk c is in
// registers. No load goes to registers, so the waits are counted by hand. Per chunk a wave issues its ACT loads of activations and then, pair by pair, 2 WT loads
// of weights; the loads land in the order of issue, so
//   - the activations of chunk c + 1 have landed when at most the chunk's KC / 2 pairs of weights
//     issued after them are on their way (before the barrier that opens chunk c + 1);
//   - pair p of chunk c has landed when at most KC / 2 - 1 pairs and one batch of activations are
//     behind it (the first pair of a chunk, read after the barrier), or KC / 2 - 2 pairs and the
//     batch (the others, read one pair ahead of their products).
// Within a chunk, loads past the end of K are issued all the same, at clamped addresses, and count
// as zero; behind the last chunk nothing is fetched, and its waits count accordingly.
template <int MB, int KW, int NWV, int NT, int KC, bool GATED, typename TO>
__global__ __launch_bounds__(64 * KW * NWV) void gemm_bf16_mid_rows_kernel(const bf16_t* __restrict__ A,
                                                                            const bf16_t* __restrict__ W,
                                                                            TO* __restrict__ C, int M, int N, int K) {
  constexpr int WT = GATED ? 2 * NT : NT;  // weight tiles per wave
  constexpr int PAIRS = KC / 2;            // pairs of k-steps per chunk
  constexpr int ACT = KC * MB / NWV;       // loads of activations a wave issues per chunk
  constexpr int WLOADS = 2 * WT;           // loads of weights per pair
  constexpr int ONCE = 2;                  // the cache policy of a non-temporal load
  static_assert(KC % 2 == 0 && KC * MB % NWV == 0 && PAIRS >= 2, "the waves of a K group stage equal shares of a chunk");
  static_assert((PAIRS - 1) * WLOADS + ACT < 64 && PAIRS * WLOADS < 64, "the loads' counter holds 63");
  extern __shared__ __align__(16) unsigned char mid_lds[];  // [KW][2][PAIRS][MB] units, then [waves][PAIRS][WT] units
  const int lane = threadIdx.x & 63;
  const int wave = uniform_wave_number();
  const int kg = wave / NWV, nw = wave % NWV;
  const int r16 = lane & 15, quad = lane >> 4;
  const int sub = lane >> 3, piece = (lane & 7) ^ sub;
  const int ntiles = N >> 4;
  const int tile_lo = (int)(blockIdx.x * (unsigned)ntiles / gridDim.x);  // N <= 2^20: no overflow
  const int tile_hi = (int)((blockIdx.x + 1) * (unsigned)ntiles / gridDim.x);
  const int tile0 = tile_lo + nw * NT;

  // the k-steps of this block, then of this K group (parts and groups start at even k-steps)
  const int all_steps = K >> 5;
  const int part = 2 * ((all_steps / 2 + gridDim.y - 1) / gridDim.y);
  const int p0 = min(all_steps, (int)blockIdx.y * part), p1 = min(all_steps, p0 + part);
  const int glen = 2 * (((p1 - p0) / 2 + KW - 1) / KW);
  const int g0 = min(p1, p0 + kg * glen), g1 = min(p1, g0 + glen);
  const int chunks = (glen + KC - 1) / KC;  // the same for every group: they share the barriers
  const int last_pair = all_steps - 2;
  const int rot = (int)((blockIdx.x * 5u + blockIdx.y * 3u + kg) % (unsigned)max(chunks, 1));
  auto chunk_start = [&](int c) {  // first k-step of the c-th chunk in this block's order
    int cc = c + rot;
    if (cc >= chunks) cc -= chunks;
    return c < chunks ? g0 + cc * KC : g1;
  };

  // weights: unit (tile t, half j) of a pair; a wave without a tile reads the page of zeros
  const bf16_t* wsrc[WT][2];
  int wpair[NT];  // elements from one pair to the next: none in the page of zeros
#pragma unroll
  for (int t = 0; t < NT; ++t) {
    const bool mine = tile0 + t < tile_hi;
    wpair[t] = mine ? 64 : 0;
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      const size_t row = (size_t)16 * (tile0 + t) + 8 * j + sub;
      wsrc[t][j] = mine ? W + row * K + 8 * piece : (const bf16_t*)qrt_zero_tile + 8 * lane;
      if (GATED) wsrc[NT + t][j] = mine ? W + ((size_t)N + row) * K + 8 * piece : (const bf16_t*)qrt_zero_tile + 8 * lane;
    }
  }
  // activations: load u = nw + NWV j of a chunk is (pair u / (2 MB), row block (u / 2) % MB, half u % 2)
  const bf16_t* asrc[ACT];
  int apair[ACT], adst[ACT];
#pragma unroll
  for (int j = 0; j < ACT; ++j) {
    const int u = nw + NWV * j;
    const int half = u % 2, b = (u / 2) % MB;
    apair[j] = u / (2 * MB);
    asrc[j] = A + (size_t)min(16 * b + 8 * half + sub, M - 1) * K + 8 * piece;
    adst[j] = (apair[j] * MB + b) * 2048 + half * 1024;
  }
  constexpr int ABUF = PAIRS * MB * 2048;  // one staged chunk of activations
  unsigned char* group_buf = mid_lds + (size_t)kg * 2 * ABUF;
  unsigned char* ring = mid_lds + (size_t)KW * 2 * ABUF + (size_t)wave * PAIRS * WT * 2048;
  const int read_at[2] = {r16 * 128 + 16 * (quad ^ (r16 & 7)), r16 * 128 + 16 * ((4 + quad) ^ (r16 & 7))};

  auto fetch_activations = [&](int c) {
    const int s_a = chunk_start(c);
    unsigned char* buf = group_buf + (c & 1) * ABUF;
#pragma unroll
    for (int j = 0; j < ACT; ++j)
      __builtin_amdgcn_global_load_lds((global_ptr_t)(asrc[j] + ((size_t)min(s_a + 2 * apair[j], last_pair) << 5)),
                                       (lds_ptr_t)(buf + adst[j]), 16, 0, 0);
  };
  auto fetch_weights = [&](int c, int p) {  // pair p of chunk c into slot p of the ring
    const size_t pair = (size_t)(min(chunk_start(c) + 2 * p, last_pair) >> 1);
#pragma unroll
    for (int t = 0; t < WT; ++t)
#pragma unroll
      for (int j = 0; j < 2; ++j)
        __builtin_amdgcn_global_load_lds((global_ptr_t)(wsrc[t][j] + pair * wpair[t % NT]),
                                         (lds_ptr_t)(ring + (p * WT + t) * 2048 + j * 1024), 16, 0, ONCE);
  };

  f32x4_t acc[WT][MB];
#pragma unroll
  for (int t = 0; t < WT; ++t)
#pragma unroll
    for (int b = 0; b < MB; ++b) acc[t][b] = (f32x4_t){0.f, 0.f, 0.f, 0.f};
  bf16x8_t zero;
#pragma unroll
  for (int e = 0; e < 8; ++e) zero[e] = (bf16_t)0.0f;

  // One chunk. LAST: nothing is fetched behind it, so fewer loads are behind the ones waited for.
  auto run_chunk = [&](int c, auto last) {
    constexpr bool LAST = decltype(last)::value;
    QRT_WAIT_LOADS(PAIRS * WLOADS);  // this wave's share of the activations of chunk c has landed
    QRT_WAIT_LDS();                  // and its reads of the chunk before are in registers
    QRT_BARRIER();                   // everybody's has, and nobody reads the other buffer any more
    if (!LAST) fetch_activations(c + 1);
    const unsigned char* cur = group_buf + (c & 1) * ABUF;
    const int n_live = g1 - chunk_start(c);
    bf16x8_t w[2][WT], a[2][MB];  // operands of this k-step and the next
    QRT_WAIT_LOADS((PAIRS - 1) * WLOADS + (LAST ? 0 : ACT));
#pragma unroll
    for (int t = 0; t < WT; ++t) w[0][t] = *(const bf16x8_t*)(ring + t * 2048 + read_at[0]);
#pragma unroll
    for (int b = 0; b < MB; ++b) a[0][b] = *(const bf16x8_t*)(cur + b * 2048 + read_at[0]);
#pragma unroll
    for (int s = 0; s < KC; ++s) {
      const int p = s >> 1, h = s & 1;
      if (s + 1 < KC) {  // the operands of step s + 1 leave LDS while the products of step s run
        const int pn = (s + 1) >> 1, hn = (s + 1) & 1;
        if (hn == 0) {
          if (LAST) QRT_WAIT_LOADS((PAIRS - 1 - pn) * WLOADS);
          else QRT_WAIT_LOADS((PAIRS - 2) * WLOADS + ACT);
        }
#pragma unroll
        for (int t = 0; t < WT; ++t) w[(s + 1) & 1][t] = *(const bf16x8_t*)(ring + (pn * WT + t) * 2048 + read_at[hn]);
#pragma unroll
        for (int b = 0; b < MB; ++b) a[(s + 1) & 1][b] = *(const bf16x8_t*)(cur + (pn * MB + b) * 2048 + read_at[hn]);
      }
      const bool live = s < n_live;  // a select: a branch round the products would spill the accumulators
#pragma unroll
      for (int t = 0; t < WT; ++t) {
        const bf16x8_t wt = live ? w[s & 1][t] : zero;
#pragma unroll
        for (int b = 0; b < MB; ++b)
          acc[t][b] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wt, a[s & 1][b], acc[t][b], 0, 0, 0);
      }
      if (h == 1 && !LAST) {  // both k-steps of pair p are in registers: its slot takes the same pair of the next chunk
        QRT_WAIT_LDS();
        fetch_weights(c + 1, p);
      }
    }
  };
  if (chunks > 0) {  // the same in every wave of the block
    fetch_activations(0);
#pragma unroll
    for (int p = 0; p < PAIRS; ++p) fetch_weights(0, p);
    for (int c = 0; c + 1 < chunks; ++c) run_chunk(c, std::false_type{});
    run_chunk(chunks - 1, std::true_type{});
  }

  if (KW > 1) {  // the K groups' sums meet in group 0, added in group order
    __syncthreads();
    float* red = (float*)mid_lds;  // [KW - 1][NWV][WT][MB][4][64]
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

template <int MB, int KW, int NWV, int NT, int KC, bool GATED>
static int launch_mid_rows(const bf16_t* a, const bf16_t* w, void* c, int out_dtype, int M, int N, int K,
                           hipStream_t stream, int k_parts) {
  constexpr int WT = GATED ? 2 * NT : NT;
  const int per_block = NWV * NT, tiles = N / 16;
  constexpr int COMPUTE_UNITS = 256;  // of an MI355X
  int blocks = tiles <= COMPUTE_UNITS / k_parts ? tiles
                                                : max(COMPUTE_UNITS / k_parts, (tiles + per_block - 1) / per_block);
  blocks = max(blocks, (tiles + per_block - 1) / per_block);
  dim3 grid(blocks, k_parts), block(64 * KW * NWV);
  constexpr size_t stage = (size_t)KW * 2 * (KC / 2) * MB * 2048 + (size_t)KW * NWV * (KC / 2) * WT * 2048;
  constexpr size_t meet = (size_t)(KW - 1) * NWV * WT * MB * 1024;
  constexpr size_t smem = stage > meet ? stage : meet;
  static_assert(smem <= 160 * 1024, "the staging of this configuration does not fit LDS");
#define GO(TO)                                                                                          \
  do {                                                                                                  \
    auto kernel = gemm_bf16_mid_rows_kernel<MB, KW, NWV, NT, KC, GATED, TO>;                            \
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
  QRT_LAUNCH_CHECK("gemm_bf16_mid_rows");
  return 0;
}

// Configurations from timing 42 of them per form (1 to 4 K groups, 1 to 8 waves a group, 1 or 2
// tiles a wave, chunks of 4 to 12 k-steps) on the shapes of the 4B and 8B models at 32, 64 and
// 128 rows, each on the weight matrices of 36 layers in turn (one matrix over and over stays in
// the memory-side cache and flatters every configuration, the small products most). Gated: one
// group of three waves, a gate and an up tile each (20.7, 23.6 and 33.4 us at the 4B size). K cut
// over blocks: one group whose waves have eight tiles between them, as four waves with two tiles
// each and chunks of eight k-steps, or, where K is a multiple of 2,048 (the rows of a wave's two
// tiles then start in the same memory channels) and from 65 rows on (LDS), as eight waves with
// one tile each and chunks of four (the 8B down projection at 64 rows 19.2 us against 20.5).
// The whole result: K groups of two waves with one tile each, two groups with chunks of eight,
// or three with chunks of four where K is a multiple of 2,048; up to 64 rows only: beyond, every
// block would have to fetch more activations than weights, and the vendor library is faster.
// Very many tiles (the vocabulary head): eight tiles on the staged activations.
template <int MB>
static int mid_rows(const bf16_t* a, const bf16_t* w, void* c, int out_dtype, int M, int N, int K, int gated,
                    hipStream_t st, int k_parts) {
  if (gated) return launch_mid_rows<MB, 1, 3, 1, 6, true>(a, w, c, out_dtype, M, N, K, st, 1);
  if (k_parts > 1) {
    if constexpr (MB % 2 == 0) {
      if (MB > 4 || K % 2048 == 0) return launch_mid_rows<MB, 1, 8, 1, 4, false>(a, w, c, out_dtype, M, N, K, st, k_parts);
    } else {
      if (K % 2048 == 0) return launch_mid_rows<MB, 1, 4, 1, 4, false>(a, w, c, out_dtype, M, N, K, st, k_parts);
    }
    if constexpr (MB <= 4) return launch_mid_rows<MB, 1, 4, 2, 8, false>(a, w, c, out_dtype, M, N, K, st, k_parts);
  }
  if constexpr (MB <= 4) {
    if (N >= 32768) return launch_mid_rows<MB, 1, 4, 2, 8, false>(a, w, c, out_dtype, M, N, K, st, 1);
    if (K % 2048 == 0) return launch_mid_rows<MB, 3, 2, 1, 4, false>(a, w, c, out_dtype, M, N, K, st, 1);
    return launch_mid_rows<MB, 2, 2, 1, 8, false>(a, w, c, out_dtype, M, N, K, st, 1);
  }
  return qrt_fail("gemm_bf16: above 64 rows only the gated form and products cut along K have a kernel of their own (M=%d)", M);
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
// shared = 0: the few-row kernels up to 16 rows (the one through LDS where K % 64 == 0), the plain
// tiled kernel beyond. shared = 1: the kernel that shares the activations through LDS; needs
// N % 16 == 0, K % 64 == 0, K >= 128, and M <= 64 (M <= 128 for the gated form and for K parts).
// k_parts > 1 (not gated, float32 out; K % 64 == 0, and shared or M <= 16): K is cut into that
// many parts, each handled by blocks of its own, and C is [k_parts, M, N]: planes to be added by
// the caller.
extern "C" int qrt_gemm_bf16(const void* a, const void* w, void* c, int out_dtype, int M, int N, int K, int gated,
                             int shared, int k_parts, hipStream_t stream) {
  QRT_CHECK(M >= 0 && N > 0 && K > 0, "gemm_bf16: bad sizes M=%d N=%d K=%d", M, N, K);
  QRT_CHECK(gated == 0 || gated == 1, "gemm_bf16: unknown mode %d", gated);
  QRT_CHECK(shared == 0 || shared == 1, "gemm_bf16: unknown kernel choice %d", shared);
  QRT_CHECK(k_parts >= 1 && k_parts <= 64, "gemm_bf16: bad number of K parts %d", k_parts);
  QRT_CHECK(k_parts == 1 || (!gated && out_dtype == QRT_F32), "gemm_bf16: K parts need no gate and float32 output");
  if (M == 0) return 0;
  const bf16_t* A = (const bf16_t*)a;
  const bf16_t* W = (const bf16_t*)w;
  const bool aligned = (K % 32 == 0) && ((uintptr_t)a % 16 == 0) && ((uintptr_t)w % 16 == 0);
  if (shared) {
    QRT_CHECK(M <= 128 && N % 16 == 0 && N <= (1 << 20) && K % 64 == 0 && K >= 128 && aligned,
              "gemm_bf16: the LDS-sharing kernel needs M <= 128, N %% 16 == 0, N <= 2^20, K %% 64 == 0, K >= 128 "
              "(M=%d N=%d K=%d)", M, N, K);
    if (M <= 16) return mid_rows<1>(A, W, c, out_dtype, M, N, K, gated, stream, k_parts);
    if (M <= 32) return mid_rows<2>(A, W, c, out_dtype, M, N, K, gated, stream, k_parts);
    if (M <= 48) return mid_rows<3>(A, W, c, out_dtype, M, N, K, gated, stream, k_parts);
    if (M <= 64) return mid_rows<4>(A, W, c, out_dtype, M, N, K, gated, stream, k_parts);
    if (M <= 96) return mid_rows<6>(A, W, c, out_dtype, M, N, K, gated, stream, k_parts);
    return mid_rows<8>(A, W, c, out_dtype, M, N, K, gated, stream, k_parts);
  }
  if (M <= 16 && aligned && K % 64 == 0)  // through LDS by direct loads: whole cache lines
    return gated ? few_rows<true>(A, W, c, out_dtype, M, N, K, stream, 1)
                 : few_rows<false>(A, W, c, out_dtype, M, N, K, stream, k_parts);
  QRT_CHECK(k_parts == 1, "gemm_bf16: K parts need M <= 16 or the LDS-sharing kernel, and K %% 64 == 0 (M=%d K=%d)", M, K);
  if (M <= 16 && aligned) return gated ? skinny<true>(A, W, c, out_dtype, M, N, K, stream)
                                       : skinny<false>(A, W, c, out_dtype, M, N, K, stream);
  QRT_CHECK(gated == 0, "gemm_bf16: the gated form needs K a multiple of 32 and M <= 16, or the LDS-sharing kernel "
            "(M=%d K=%d)", M, K);
  if (M <= 16) return launch<1, 2>(A, W, c, out_dtype, M, N, K, stream);
  if (M <= 32) return launch<2, 2>(A, W, c, out_dtype, M, N, K, stream);
  return launch<4, 4>(A, W, c, out_dtype, M, N, K, stream);
}
