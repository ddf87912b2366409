// Paged attention in true 32-bit, any head size: the check path.
//
// One wave per (query token, query head). The wave walks the keys its query may
// see in chunks of 64 (one key per lane for the scores), keeps a running
// maximum and sum (online softmax, float32), and accumulates the context with
// each lane owning head elements lane, lane + 64, ... Query head h reads key
// head h / g. The query at position p sees keys j <= p, and j > p - window when
// a window is set. Cache layout: keys [page, head, offset, D], values
// [page, head, D, offset].
#include "common.h"
#include <math.h>

struct AttnArgs {
  const void* q;         // [T, nq * D]
  void* out;             // [T, nq * D]
  const void* k_cache;
  const void* v_cache;
  const int* positions;  // [T] position of each query token
  const int* seq_of_token;  // [T]
  const int* block_table;   // [S, table_width]
  int table_width;
  int num_tokens, nq, nkv, head_dim, page_size, window;  // window 0: none
  float scale;
};

#define MAX_D 512

template <typename T>
__global__ __launch_bounds__(64) void attention_f32_kernel(AttnArgs a) {
  __shared__ float qs[MAX_D];
  const int lane = threadIdx.x;
  const int t = blockIdx.x, h = blockIdx.y;
  const int D = a.head_dim, ps = a.page_size;
  const int kvh = h / (a.nq / a.nkv);
  const int pos = a.positions[t];
  const int* table = a.block_table + (size_t)a.seq_of_token[t] * a.table_width;
  const T* q = (const T*)a.q + ((size_t)t * a.nq + h) * D;
  for (int i = lane; i < D; i += 64) qs[i] = to_f32<T>(q[i]);
  __syncthreads();

  const int lo = a.window > 0 ? max(0, pos - a.window + 1) : 0;
  float m = -INFINITY, l = 0.f;
  float acc[MAX_D / 64];
#pragma unroll
  for (int i = 0; i < MAX_D / 64; ++i) acc[i] = 0.f;

  const T* kc = (const T*)a.k_cache;
  const T* vc = (const T*)a.v_cache;
  for (int j0 = lo; j0 <= pos; j0 += 64) {
    const int j = j0 + lane;
    const bool valid = j <= pos;
    float s = -INFINITY;
    int page = 0, off = 0;
    if (valid) {
      page = table[j / ps];
      off = j % ps;
      const T* kr = kc + (((size_t)page * a.nkv + kvh) * ps + off) * D;
      float dot = 0.f;
      for (int d = 0; d < D; ++d) dot = fmaf(qs[d], to_f32<T>(kr[d]), dot);
      s = dot * a.scale;
    }
    const float m_new = fmaxf(m, wave_max(s));
    const float p = valid ? expf(s - m_new) : 0.f;
    const float corr = expf(m - m_new);  // m = -inf at the first chunk: exp(-inf) = 0
    l = l * corr + wave_sum(p);
    m = m_new;
#pragma unroll
    for (int i = 0; i < MAX_D / 64; ++i) acc[i] *= corr;
    const int n = min(64, pos - j0 + 1);
    for (int jj = 0; jj < n; ++jj) {
      const float pj = __shfl(p, jj, 64);
      const int pg = __shfl(page, jj, 64);
      const int of = __shfl(off, jj, 64);
      const T* vr = vc + ((size_t)pg * a.nkv + kvh) * D * ps + of;
#pragma unroll
      for (int i = 0; i < MAX_D / 64; ++i) {
        const int d = lane + 64 * i;
        if (d < D) acc[i] = fmaf(pj, to_f32<T>(vr[(size_t)d * ps]), acc[i]);
      }
    }
  }
  T* o = (T*)a.out + ((size_t)t * a.nq + h) * D;
  const float inv = l > 0.f ? 1.0f / l : 0.f;
#pragma unroll
  for (int i = 0; i < MAX_D / 64; ++i) {
    const int d = lane + 64 * i;
    if (d < D) o[d] = from_f32<T>(acc[i] * inv);
  }
}

extern "C" int qrt_attention_f32(const AttnArgs* args, int dtype, hipStream_t stream) {
  AttnArgs a = *args;
  QRT_CHECK(a.num_tokens >= 0 && a.nq > 0 && a.nkv > 0 && a.nq % a.nkv == 0,
            "attention: %d query heads do not divide into %d key heads", a.nq, a.nkv);
  QRT_CHECK(a.head_dim > 0 && a.head_dim <= MAX_D, "attention: head size %d is above %d", a.head_dim, MAX_D);
  QRT_CHECK(a.page_size > 0 && a.table_width > 0 && a.window >= 0, "attention: bad page size, table width or window");
  QRT_CHECK(a.nq <= 65535, "attention: too many heads");
  if (a.num_tokens == 0) return 0;
  dim3 grid(a.num_tokens, a.nq), block(64);
  if (dtype == QRT_F32) attention_f32_kernel<float><<<grid, block, 0, stream>>>(a);
  else if (dtype == QRT_BF16) attention_f32_kernel<bf16_t><<<grid, block, 0, stream>>>(a);
  else return qrt_fail("attention: unknown dtype %d", dtype);
  QRT_LAUNCH_CHECK("attention_f32");
  return 0;
}
