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
// layout is chosen for memory parallelism, not for reuse. A block owns 16
// weight rows (one MFMA tile of outputs n) and all of K; its NW waves take the
// 32-wide k-steps round-robin, so that in every round the block reads
// 16 rows x NW x 64 contiguous bytes. Each wave keeps MB accumulators (16 rows
// of M each); activations come from L2/L1 (they are tiny), optionally as
// silu(gate) * up of a [M, 2K] input. Partial sums meet in LDS and are added in
// wave order, so the result does not depend on timing.
template <bool SWIGLU>
__device__ __forceinline__ bf16x8_t load_act(const bf16_t* __restrict__ row, int k, int K, bool valid) {
  bf16x8_t v;
#pragma unroll
  for (int e = 0; e < 8; ++e) v[e] = (bf16_t)0.0f;
  if (!valid) return v;
  if (!SWIGLU) return *(const bf16x8_t*)(row + k);
  const bf16x8_t g = *(const bf16x8_t*)(row + k);
  const bf16x8_t u = *(const bf16x8_t*)(row + K + k);
#pragma unroll
  for (int e = 0; e < 8; ++e) {
    const float gf = (float)g[e];
    v[e] = (bf16_t)(gf / (1.0f + __expf(-gf)) * (float)u[e]);
  }
  return v;
}

template <int MB, int NW, bool SWIGLU, typename TO>
__global__ __launch_bounds__(64 * NW) void gemm_bf16_skinny_kernel(const bf16_t* __restrict__ A,
                                                                    const bf16_t* __restrict__ W,
                                                                    TO* __restrict__ C, int M, int N, int K) {
  extern __shared__ float red[];  // [NW][MB][4][64]
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int r16 = lane & 15, quad = lane >> 4;
  const int n0 = blockIdx.x * 16;
  const int n = n0 + r16;
  const bf16_t* wrow = W + (size_t)(n < N ? n : N - 1) * K;
  const int a_stride = SWIGLU ? 2 * K : K;
  const bf16_t* arow[MB];
  bool avalid[MB];
#pragma unroll
  for (int b = 0; b < MB; ++b) {
    const int m = 16 * b + r16;
    avalid[b] = m < M;
    arow[b] = A + (size_t)(avalid[b] ? m : 0) * a_stride;
  }
  f32x4_t acc[MB];
#pragma unroll
  for (int b = 0; b < MB; ++b) acc[b] = (f32x4_t){0.f, 0.f, 0.f, 0.f};

  const int steps = K >> 5;  // K is a multiple of 32 here
  constexpr int U = 4;
  int s = wave;
  for (; s + (U - 1) * NW < steps; s += U * NW) {
    bf16x8_t w[U];
#pragma unroll
    for (int u = 0; u < U; ++u) w[u] = *(const bf16x8_t*)(wrow + ((s + u * NW) << 5) + 8 * quad);
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int k = ((s + u * NW) << 5) + 8 * quad;
#pragma unroll
      for (int b = 0; b < MB; ++b) {
        const bf16x8_t a = load_act<SWIGLU>(arow[b], k, K, avalid[b]);
        acc[b] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(w[u], a, acc[b], 0, 0, 0);
      }
    }
  }
  for (; s < steps; s += NW) {
    const int k = (s << 5) + 8 * quad;
    const bf16x8_t w = *(const bf16x8_t*)(wrow + k);
#pragma unroll
    for (int b = 0; b < MB; ++b) {
      const bf16x8_t a = load_act<SWIGLU>(arow[b], k, K, avalid[b]);
      acc[b] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(w, a, acc[b], 0, 0, 0);
    }
  }

#pragma unroll
  for (int b = 0; b < MB; ++b)
#pragma unroll
    for (int r = 0; r < 4; ++r) red[((wave * MB + b) * 4 + r) * 64 + lane] = acc[b][r];
  __syncthreads();
  // thread t < MB * 64 finishes accumulator block b = t / 64 of lane t % 64
  for (int t = threadIdx.x; t < MB * 64; t += 64 * NW) {
    const int b = t >> 6, l = t & 63;
    const int m = 16 * b + (l & 15);
    const int nn = n0 + 4 * (l >> 4);
    float sum[4];
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      float v = 0.f;
      for (int w = 0; w < NW; ++w) v += red[((w * MB + b) * 4 + r) * 64 + l];
      sum[r] = v;
    }
    if (m < M) {
#pragma unroll
      for (int r = 0; r < 4; ++r)
        if (nn + r < N) C[(size_t)m * N + nn + r] = from_f32<TO>(sum[r]);
    }
  }
}

template <int MB, int NW, bool SWIGLU>
static int launch_skinny(const bf16_t* a, const bf16_t* w, void* c, int out_dtype, int M, int N, int K,
                         hipStream_t stream) {
  dim3 grid((N + 15) / 16), block(64 * NW);
  const size_t smem = (size_t)NW * MB * 4 * 64 * sizeof(float);
  if (out_dtype == QRT_BF16)
    gemm_bf16_skinny_kernel<MB, NW, SWIGLU, bf16_t><<<grid, block, smem, stream>>>(a, w, (bf16_t*)c, M, N, K);
  else if (out_dtype == QRT_F32)
    gemm_bf16_skinny_kernel<MB, NW, SWIGLU, float><<<grid, block, smem, stream>>>(a, w, (float*)c, M, N, K);
  else
    return qrt_fail("gemm_bf16: unknown output dtype %d", out_dtype);
  QRT_LAUNCH_CHECK("gemm_bf16_skinny");
  return 0;
}

template <bool SWIGLU>
static int skinny(const bf16_t* a, const bf16_t* w, void* c, int out_dtype, int M, int N, int K, hipStream_t st) {
  // more waves per block when there are few blocks or K is long
  const bool many = (N / 16 < 512) || (K >= 8192);
  if (M <= 16) return many ? launch_skinny<1, 16, SWIGLU>(a, w, c, out_dtype, M, N, K, st)
                           : launch_skinny<1, 8, SWIGLU>(a, w, c, out_dtype, M, N, K, st);
  if (M <= 32) return many ? launch_skinny<2, 16, SWIGLU>(a, w, c, out_dtype, M, N, K, st)
                           : launch_skinny<2, 8, SWIGLU>(a, w, c, out_dtype, M, N, K, st);
  return many ? launch_skinny<4, 16, SWIGLU>(a, w, c, out_dtype, M, N, K, st)
              : launch_skinny<4, 8, SWIGLU>(a, w, c, out_dtype, M, N, K, st);
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

// act: 0 = A is [M, K]; 1 = A is [M, 2K] and the operand is silu(A[:, :K]) * A[:, K:]
extern "C" int qrt_gemm_bf16(const void* a, const void* w, void* c, int out_dtype, int M, int N, int K, int act,
                             hipStream_t stream) {
  QRT_CHECK(M >= 0 && N > 0 && K > 0, "gemm_bf16: bad sizes M=%d N=%d K=%d", M, N, K);
  QRT_CHECK(act == 0 || act == 1, "gemm_bf16: unknown activation %d", act);
  if (M == 0) return 0;
  const bf16_t* A = (const bf16_t*)a;
  const bf16_t* W = (const bf16_t*)w;
  const bool aligned = (K % 32 == 0) && ((uintptr_t)a % 16 == 0) && ((uintptr_t)w % 16 == 0);
  if (M <= 64 && aligned) return act ? skinny<true>(A, W, c, out_dtype, M, N, K, stream)
                                     : skinny<false>(A, W, c, out_dtype, M, N, K, stream);
  QRT_CHECK(act == 0, "gemm_bf16: the fused activation needs M <= 64 and K a multiple of 32 (M=%d K=%d)", M, K);
  if (M <= 16) return launch<1, 2>(A, W, c, out_dtype, M, N, K, stream);
  if (M <= 32) return launch<2, 2>(A, W, c, out_dtype, M, N, K, stream);
  return launch<4, 4>(A, W, c, out_dtype, M, N, K, stream);
}
