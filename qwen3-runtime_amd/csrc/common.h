// Shared declarations of the HIP library (gfx950, wave64).
//
// Every entry point is extern "C", takes raw device pointers plus sizes and a
// stream, validates what it can on the host, launches on that stream and
// returns 0, or a negative code after recording a message that
// qrt_last_error() returns. Nothing here allocates device memory.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

typedef __bf16 bf16_t;
typedef __bf16 bf16x4_t __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef float f32x4_t __attribute__((ext_vector_type(4)));
typedef unsigned u32x4_t __attribute__((ext_vector_type(4)));

#define QRT_WAVE 64

// dtype codes shared with the Python side
#define QRT_F32 0
#define QRT_BF16 1

extern "C" const char* qrt_last_error();
int qrt_fail(const char* fmt, ...);

#define QRT_CHECK(cond, ...)                 \
  do {                                       \
    if (!(cond)) return qrt_fail(__VA_ARGS__); \
  } while (0)

#define QRT_LAUNCH_CHECK(name)                                                     \
  do {                                                                             \
    hipError_t e_ = hipGetLastError();                                             \
    if (e_ != hipSuccess) return qrt_fail("%s: launch failed: %s", name, hipGetErrorString(e_)); \
  } while (0)

// The wave's number within its block, in a scalar register: what follows from it (the wave's rows,
// its share of a loop) is then the same for the whole wave to the compiler too, and branches on it
// become scalar branches. For kernels with MFMA instructions this is needed, not only faster:
// MFMA does not look at the EXEC mask, so one inside a branch that the compiler lowered to an
// EXEC mask of zeros, without a jump over it, runs all the same, on registers never loaded.
__device__ __forceinline__ int uniform_wave_number() { return __builtin_amdgcn_readfirstlane(threadIdx.x >> 6); }

// Eight bfloat16 of a matrix that a step reads exactly once (weights streamed past few rows of
// activations): a non-temporal load, which leaves the caches to data that is read again. A plain
// read of 4 GiB runs at 6.1 TB/s on this device, a non-temporal one at 6.9; the few-row products
// of a decode step gain 2 to 5 % by it (the products with 17 to 64 rows lose 2 %, and keep
// plain loads).
__device__ __forceinline__ bf16x8_t load_once8(const bf16_t* p) {
  return __builtin_bit_cast(bf16x8_t, __builtin_nontemporal_load((const u32x4_t*)p));
}

template <typename T> __device__ __forceinline__ float to_f32(T x);
template <> __device__ __forceinline__ float to_f32<float>(float x) { return x; }
template <> __device__ __forceinline__ float to_f32<bf16_t>(bf16_t x) { return (float)x; }

template <typename T> __device__ __forceinline__ T from_f32(float x);
template <> __device__ __forceinline__ float from_f32<float>(float x) { return x; }
template <> __device__ __forceinline__ bf16_t from_f32<bf16_t>(float x) { return (bf16_t)x; }

// Sine and cosine of a rotation angle held in float32 (position times frequency: up to
// millions of radians). The library routine reduces such arguments with a table it loads from
// memory; here the angle is reduced to [-pi, pi] in float64 (exact to 1e-10 rad) first, so the
// routine stays on its short path and the kernel has no loads in its middle. The result is the
// sine and cosine of the float32 angle to within one unit in the last place.
__device__ __forceinline__ void sincos_angle(float angle, float* sn, float* cs) {
  const double turns = (double)angle * 0.15915494309189535;  // 1 / (2 pi)
  const float reduced = (float)((turns - rint(turns)) * 6.283185307179586);
  sincosf(reduced, sn, cs);
}

__device__ __forceinline__ float wave_sum(float x) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) x += __shfl_xor(x, o, 64);
  return x;
}
__device__ __forceinline__ float wave_max(float x) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) x = fmaxf(x, __shfl_xor(x, o, 64));
  return x;
}

// Sum over a block of up to 1024 threads; every thread gets the result.
// `red` is shared memory of at least 17 floats. Order of additions is fixed.
__device__ __forceinline__ float block_sum(float x, float* red) {
  x = wave_sum(x);
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int nw = (blockDim.x + 63) >> 6;
  __syncthreads();
  if (lane == 0) red[wave] = x;
  __syncthreads();
  if (threadIdx.x == 0) {
    float s = 0.f;
    for (int i = 0; i < nw; ++i) s += red[i];
    red[16] = s;
  }
  __syncthreads();
  return red[16];
}
__device__ __forceinline__ float block_max(float x, float* red) {
  x = wave_max(x);
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int nw = (blockDim.x + 63) >> 6;
  __syncthreads();
  if (lane == 0) red[wave] = x;
  __syncthreads();
  if (threadIdx.x == 0) {
    float s = red[0];
    for (int i = 1; i < nw; ++i) s = fmaxf(s, red[i]);
    red[16] = s;
  }
  __syncthreads();
  return red[16];
}
