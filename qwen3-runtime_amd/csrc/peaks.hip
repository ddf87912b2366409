// Two microbenchmarks that say what this device delivers, to stand beside the published
// peaks in a roofline: a read of a large contiguous buffer (HBM bandwidth) and a loop of
// bfloat16 MFMA instructions on registers (dense matrix throughput). Neither has a
// counterpart in the reference; the measurements' host side is bench.py.
#include "common.h"

typedef unsigned u32x4_t __attribute__((ext_vector_type(4)));
typedef float f32x16_t __attribute__((ext_vector_type(16)));

// Every lane reads 16 bytes per load, eight loads in flight, grid-stride over the buffer, with
// loads marked non-temporal (data read once: measured 6.9 TB/s against 6.1 with plain loads).
// The loaded words are folded into a value that is written only if it equals a constant it
// practically never equals, so that no load can be dropped.
__global__ __launch_bounds__(256) void read_kernel(const u32x4_t* __restrict__ p, size_t n16, unsigned* __restrict__ sink) {
  constexpr int U = 8;
  const size_t stride = (size_t)gridDim.x * 256;
  size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
  unsigned acc = 0;
  for (; i + (U - 1) * stride < n16; i += U * stride) {
    u32x4_t v[U];
#pragma unroll
    for (int u = 0; u < U; ++u) v[u] = __builtin_nontemporal_load(p + i + u * stride);
#pragma unroll
    for (int u = 0; u < U; ++u) acc ^= v[u][0] ^ v[u][1] ^ v[u][2] ^ v[u][3];
  }
  for (; i < n16; i += stride) {
    const u32x4_t a = __builtin_nontemporal_load(p + i);
    acc ^= a[0] ^ a[1] ^ a[2] ^ a[3];
  }
  if (acc == 0x9e3779b9u) sink[0] = acc;
}

extern "C" int qrt_peak_read(const void* buffer, size_t bytes, unsigned* sink, int blocks, hipStream_t stream) {
  QRT_CHECK(buffer && sink && bytes >= 16 && blocks > 0 && blocks <= 65535, "peak_read: bad arguments");
  QRT_CHECK(((uintptr_t)buffer & 15) == 0, "peak_read: the buffer must start on a 16-byte boundary");
  read_kernel<<<dim3(blocks), dim3(256), 0, stream>>>((const u32x4_t*)buffer, bytes / 16, sink);
  QRT_LAUNCH_CHECK("peak_read");
  return 0;
}

// Four independent accumulators per wave, so that consecutive MFMAs never wait for each other;
// operands stay in registers. One 32x32x16 bfloat16 MFMA is 2 * 32 * 32 * 16 = 32,768 flop. This
// shape is the faster of the two bfloat16 ones here: measured 1.86 PFLOP/s against 1.37 for
// 16x16x32 with every SIMD busy.
__global__ __launch_bounds__(256) void mfma_kernel(float* __restrict__ sink, int iters) {
  const int lane = threadIdx.x & 63;
  bf16x8_t a, b;
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    a[i] = (bf16_t)(0.37f * (float)((lane * 7 + i * 3) % 11) - 1.5f);
    b[i] = (bf16_t)(0.21f * (float)((lane * 5 + i) % 13) - 1.1f);
  }
  f32x16_t c[4];
#pragma unroll
  for (int j = 0; j < 4; ++j)
#pragma unroll
    for (int e = 0; e < 16; ++e) c[j][e] = 0.f;
  for (int it = 0; it < iters; ++it) {
#pragma unroll
    for (int j = 0; j < 4; ++j) c[j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c[j], 0, 0, 0);
  }
  float s = 0.f;
#pragma unroll
  for (int j = 0; j < 4; ++j)
#pragma unroll
    for (int e = 0; e < 16; ++e) s += c[j][e];
  if (s == 12345.678f) sink[0] = s;
}

// flop of one launch = blocks * 4 waves * iters * 4 * 32,768
extern "C" int qrt_peak_mfma_bf16(float* sink, int blocks, int iters, hipStream_t stream) {
  QRT_CHECK(sink && blocks > 0 && blocks <= 65535 && iters > 0, "peak_mfma: bad arguments");
  mfma_kernel<<<dim3(blocks), dim3(256), 0, stream>>>(sink, iters);
  QRT_LAUNCH_CHECK("peak_mfma");
  return 0;
}
