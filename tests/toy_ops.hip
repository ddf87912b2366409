// A kernel that a part defined in the tests brings with it (tests/test_parts_gpu.py): the toy
// position encoding, q and k scaled by 1 + rate * position. It is registered, built and loaded
// through the same hook as any part's library from outside the package.
#include "common.h"

template <typename T>
__global__ void toy_scale_kernel(const T* __restrict__ in, T* __restrict__ out, const int* __restrict__ positions,
                                 float rate, int per_token, long total) {
  const long i = (long)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= total) return;
  const float f = 1.0f + rate * (float)positions[i / per_token];
  out[i] = from_f32<T>(to_f32<T>(in[i]) * f);
}

extern "C" int toy_scale_by_position(const void* in, void* out, const int* positions, float rate, int num_tokens,
                                     int per_token, int dtype, hipStream_t stream) {
  QRT_CHECK(num_tokens >= 0 && per_token > 0, "toy_scale: bad sizes");
  const long total = (long)num_tokens * per_token;
  if (total == 0) return 0;
  const dim3 grid((unsigned)((total + 255) / 256)), block(256);
  if (dtype == QRT_F32)
    toy_scale_kernel<float><<<grid, block, 0, stream>>>((const float*)in, (float*)out, positions, rate, per_token, total);
  else if (dtype == QRT_BF16)
    toy_scale_kernel<bf16_t><<<grid, block, 0, stream>>>((const bf16_t*)in, (bf16_t*)out, positions, rate, per_token, total);
  else
    return qrt_fail("toy_scale: unknown dtype code %d", dtype);
  QRT_LAUNCH_CHECK("toy_scale");
  return 0;
}
