// True 32-bit matrix product: C[M, N] = A[M, K] * W[N, K]^T, float32 operands,
// float32 fused multiply-adds, no reduced-precision matrix mode.
//
// Each output element is one sequential sum over k = 0 .. K-1, so its value
// depends on neither M nor on which rows share the launch. 64 x 64 tile per
// block of 256 threads, 4 x 4 outputs per thread, operands staged through LDS
// in slices of 16 along K.
#include "common.h"

#define TM 64
#define TN 64
#define TK 16

__global__ __launch_bounds__(256) void gemm_f32_kernel(const float* __restrict__ A, const float* __restrict__ W,
                                                        float* __restrict__ C, int M, int N, int K) {
  __shared__ float As[TK][TM + 4];
  __shared__ float Ws[TK][TN + 4];
  const int tx = threadIdx.x & 15, ty = threadIdx.x >> 4;
  const int m0 = blockIdx.y * TM, n0 = blockIdx.x * TN;
  float acc[4][4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) acc[i][j] = 0.f;

  // loader: 256 threads bring 64 rows x 16 k of each operand; thread -> (row, 4 k)
  const int lrow = threadIdx.x >> 2, lk = (threadIdx.x & 3) * 4;
  for (int k0 = 0; k0 < K; k0 += TK) {
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      const int k = k0 + lk + e;
      const int am = m0 + lrow, wn = n0 + lrow;
      As[lk + e][lrow] = (am < M && k < K) ? A[(size_t)am * K + k] : 0.f;
      Ws[lk + e][lrow] = (wn < N && k < K) ? W[(size_t)wn * K + k] : 0.f;
    }
    __syncthreads();
#pragma unroll
    for (int kk = 0; kk < TK; ++kk) {
      float a[4], w[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) a[i] = As[kk][ty * 4 + i];
#pragma unroll
      for (int j = 0; j < 4; ++j) w[j] = Ws[kk][tx * 4 + j];
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = fmaf(a[i], w[j], acc[i][j]);
    }
    __syncthreads();
  }
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int m = m0 + ty * 4 + i;
    if (m >= M) continue;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int n = n0 + tx * 4 + j;
      if (n < N) C[(size_t)m * N + n] = acc[i][j];
    }
  }
}

extern "C" int qrt_gemm_f32(const float* a, const float* w, float* c, int M, int N, int K, hipStream_t stream) {
  QRT_CHECK(M >= 0 && N > 0 && K > 0, "gemm_f32: bad sizes M=%d N=%d K=%d", M, N, K);
  if (M == 0) return 0;
  dim3 grid((N + TN - 1) / TN, (M + TM - 1) / TM), block(256);
  QRT_CHECK(grid.y <= 65535, "gemm_f32: M=%d is too large for one launch", M);
  gemm_f32_kernel<<<grid, block, 0, stream>>>(a, w, c, M, N, K);
  QRT_LAUNCH_CHECK("gemm_f32");
  return 0;
}
