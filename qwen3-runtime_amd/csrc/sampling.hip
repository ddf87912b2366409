// Sampling on the device: one block per row of float32 logits (with few rows, the first
// pass over a row is spread over several blocks).
//
// Chain, in the order the reference runs it (qwen3_runtime/sampling.py:120-135):
// penalties from per-slot counts, (greedy: first maximal id), temperature,
// min_p, top_k, top_p, softmax, inverse-CDF draw with a uniform number from a
// counter-based generator keyed by (seed, draw index). All in float32. top_k
// and top_p are found by bisection on the value that bounds the kept set, not
// by sorting; ids that tie with the bound are all kept.
#include "common.h"
#include "sampling.h"
#include <math.h>
#include <mutex>

#define SAMPLE_THREADS 1024

// floats ordered as unsigned integers
__device__ __forceinline__ unsigned f2ord(float f) {
  const unsigned u = __float_as_uint(f);
  return (u & 0x80000000u) ? ~u : (u | 0x80000000u);
}
__device__ __forceinline__ float ord2f(unsigned o) {
  const unsigned u = (o & 0x80000000u) ? (o & 0x7fffffffu) : ~o;
  return __uint_as_float(u);
}

// Philox4x32-10 (Salmon et al. 2011): counter-based, so a draw depends only on
// (seed, index), never on what else was sampled in the batch.
__device__ __forceinline__ unsigned mulhi32(unsigned a, unsigned b) { return __umulhi(a, b); }
__device__ inline float philox_uniform(unsigned long long seed, unsigned long long index) {
  unsigned c0 = (unsigned)index, c1 = (unsigned)(index >> 32), c2 = 0x51ab1e5u, c3 = 0;
  unsigned k0 = (unsigned)seed, k1 = (unsigned)(seed >> 32);
#pragma unroll
  for (int r = 0; r < 10; ++r) {
    const unsigned h0 = mulhi32(0xD2511F53u, c0), l0 = 0xD2511F53u * c0;
    const unsigned h1 = mulhi32(0xCD9E8D57u, c2), l1 = 0xCD9E8D57u * c2;
    const unsigned n0 = h1 ^ c1 ^ k0, n1 = l1, n2 = h0 ^ c3 ^ k1, n3 = l0;
    c0 = n0; c1 = n1; c2 = n2; c3 = n3;
    k0 += 0x9E3779B9u; k1 += 0xBB67AE85u;
  }
  return (float)(c0 >> 8) * (1.0f / 16777216.0f);  // [0, 1)
}

// first maximal index of a row; returns it to every thread
__device__ int block_argmax(const float* __restrict__ x, int n, float* red, int* redi, float* out_max) {
  float best = -INFINITY;
  int besti = 0x7fffffff;
  for (int i = threadIdx.x; i < n; i += blockDim.x) {
    const float v = x[i];
    if (v > best || (v == best && i < besti)) { best = v; besti = i; }
  }
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) {
    const float ov = __shfl_xor(best, o, 64);
    const int oi = __shfl_xor(besti, o, 64);
    if (ov > best || (ov == best && oi < besti)) { best = ov; besti = oi; }
  }
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, nw = (blockDim.x + 63) >> 6;
  __syncthreads();
  if (lane == 0) { red[wave] = best; redi[wave] = besti; }
  __syncthreads();
  if (threadIdx.x == 0) {
    for (int w = 1; w < nw; ++w)
      if (red[w] > red[0] || (red[w] == red[0] && redi[w] < redi[0])) { red[0] = red[w]; redi[0] = redi[w]; }
    if (redi[0] == 0x7fffffff) redi[0] = 0;  // a row of NaNs
  }
  __syncthreads();
  if (out_max) *out_max = red[0];
  return redi[0];
}

__global__ void argmax_kernel(const float* __restrict__ logits, int* __restrict__ out, int vocab) {
  __shared__ float red[32];
  __shared__ int redi[32];
  const int tok = block_argmax(logits + (size_t)blockIdx.x * vocab, vocab, red, redi, nullptr);
  if (threadIdx.x == 0) out[blockIdx.x] = tok;
}

extern "C" int qrt_argmax(const float* logits, int* out, int rows, int vocab, hipStream_t stream) {
  QRT_CHECK(rows >= 0 && vocab > 0, "argmax: bad sizes");
  if (rows == 0) return 0;
  argmax_kernel<<<dim3(rows), dim3(SAMPLE_THREADS), 0, stream>>>(logits, out, vocab);
  QRT_LAUNCH_CHECK("argmax");
  return 0;
}

// The first pass over ids [lo, hi) of a row: penalties (reference:
// qwen3_runtime/sampling.py:63-71) and temperature give the processed value (written to the
// work row if asked); alongside, a running maximum, the first index that reaches it, and the
// sum of exp(value - maximum). lo and hi are multiples of 4 (or hi = V).
struct RowOptions {
  float temp, rep, pres, freq;
  const int* cnt;  // the slot's counts, or null when no penalty is set
  bool greedy, keep;
};

__device__ __forceinline__ RowOptions row_options(const SampleArgs& a, int r) {
  const int sl = a.slot[r];
  const float* fp = a.fparams + (size_t)sl * 8;
  RowOptions o;
  o.temp = fp[0]; o.rep = fp[3]; o.pres = fp[4]; o.freq = fp[5];
  const bool pen = a.counts && (o.rep != 1.0f || o.pres != 0.0f || o.freq != 0.0f);
  o.cnt = pen ? a.counts + (size_t)sl * a.vocab : nullptr;
  o.greedy = o.temp <= 0.f;
  o.keep = !o.greedy || a.write_work;
  return o;
}

__device__ __forceinline__ void first_pass(const RowOptions& o, const float* __restrict__ lg, float* __restrict__ x,
                                           int lo, int hi, int V, float& m, float& ssum, int& bi) {
  const int* cnt = o.cnt;
  const int tid = threadIdx.x;
  auto take = [&](float v, int c, int i) -> float {  // processed value of id i; updates m, ssum, bi
    if (c > 0) {
      v = v > 0.f ? v / o.rep : v * o.rep;
      v -= o.pres;
      v -= o.freq * (float)c;
    }
    if (!o.greedy) v = v / o.temp;
    if (v > m) {
      ssum = ssum * expf(m - v) + 1.0f;  // m = -inf at first: exp(-inf) = 0
      m = v;
      bi = i;
    } else if (v > -INFINITY) {  // neither NaN nor an excluded id (-inf beside m = -inf would give NaN)
      ssum += expf(v - m);
    }
    return v;
  };
  if ((V & 3) == 0) {
    // rows start on 16-byte boundaries: four ids per load, several loads in flight per thread
    typedef float f32x4 __attribute__((ext_vector_type(4)));
    typedef int i32x4 __attribute__((ext_vector_type(4)));
    constexpr int U = 6;
    const int lo4 = lo >> 2, hi4 = hi >> 2;
    for (int i0 = lo4 + tid; i0 < hi4; i0 += U * blockDim.x) {
      f32x4 v[U];
      i32x4 c[U];
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const int i = i0 + u * blockDim.x;
        if (i < hi4) {
          v[u] = ((const f32x4*)lg)[i];
          c[u] = cnt ? ((const i32x4*)cnt)[i] : (i32x4){0, 0, 0, 0};
        }
      }
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const int i = i0 + u * blockDim.x;
        if (i < hi4) {
          f32x4 w;
#pragma unroll
          for (int e = 0; e < 4; ++e) w[e] = take(v[u][e], c[u][e], 4 * i + e);
          if (o.keep) ((f32x4*)x)[i] = w;
        }
      }
    }
  } else {
#pragma unroll 4
    for (int i = lo + tid; i < hi; i += blockDim.x) {
      const float v = take(lg[i], cnt ? cnt[i] : 0, i);
      if (o.keep) x[i] = v;
    }
  }
}

// (maximum, sum, index) of two parts of a row: the larger maximum wins, ties go to the lower index
__device__ __forceinline__ void merge_parts(float& m, float& ssum, int& bi, float om, float os, int oi) {
  const float mm = fmaxf(m, om);
  const float f1 = m == -INFINITY ? 0.f : expf(m - mm), f2 = om == -INFINITY ? 0.f : expf(om - mm);
  ssum = ssum * f1 + os * f2;
  if (om > m || (om == m && oi < bi)) bi = oi;
  m = mm;
}

// wave, then block: every thread leaves with the block's values in red[24], red[25], redi[24]
__device__ __forceinline__ void block_merge(float m, float ssum, int bi, float* red, float* part, int* redi) {
  const int tid = threadIdx.x;
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) {
    const float om = __shfl_xor(m, o, 64), os = __shfl_xor(ssum, o, 64);
    const int oi = __shfl_xor(bi, o, 64);
    merge_parts(m, ssum, bi, om, os, oi);
  }
  const int lane = tid & 63, wave = tid >> 6, nw = (blockDim.x + 63) >> 6;
  if (lane == 0) { red[wave] = m; part[wave] = ssum; redi[wave] = bi; }
  __syncthreads();
  if (tid == 0) {
    float mm = red[0], ss = part[0];
    int ii = redi[0];
    for (int w = 1; w < nw; ++w) merge_parts(mm, ss, ii, red[w], part[w], redi[w]);
    red[24] = mm; red[25] = ss; redi[24] = ii;
  }
  __syncthreads();
}

// With few rows one block per row would leave the chip idle while it reads the whole
// vocabulary: the first pass is then spread over `parts` blocks per row, and sample_kernel
// starts from their results.
__global__ __launch_bounds__(256) void sample_first_pass_kernel(SampleArgs a) {
  __shared__ float red[32];
  __shared__ int redi[32];
  __shared__ float part[32];
  const int r = blockIdx.x, p = blockIdx.y, V = a.vocab;
  const RowOptions o = row_options(a, r);
  const int chunk = (((V + a.parts - 1) / a.parts) + 3) & ~3;
  const int lo = min(p * chunk, V), hi = min(lo + chunk, V);
  float m = -INFINITY, ssum = 0.f;
  int bi = 0x7fffffff;
  first_pass(o, a.logits + (size_t)r * V, a.work + (size_t)r * V, lo, hi, V, m, ssum, bi);
  block_merge(m, ssum, bi, red, part, redi);
  if (threadIdx.x == 0) {
    float* dst = a.partials + ((size_t)r * a.parts + p) * 4;
    dst[0] = red[24];
    dst[1] = red[25];
    dst[2] = __int_as_float(redi[24]);
  }
}

__global__ __launch_bounds__(SAMPLE_THREADS) void sample_kernel(SampleArgs a) {
  __shared__ float red[32];
  __shared__ int redi[32];
  __shared__ float part[SAMPLE_THREADS];
  const int r = blockIdx.x, V = a.vocab, tid = threadIdx.x;
  const float* lg = a.logits + (size_t)r * V;
  float* x = a.work + (size_t)r * V;
  const int sl = a.slot[r];
  const float* fp = a.fparams + (size_t)sl * 8;
  const float temp = fp[0], topp = fp[1], minp = fp[2];
  const RowOptions o = row_options(a, r);
  const bool greedy = o.greedy;
  float m = -INFINITY, ssum = 0.f;
  int bi = 0x7fffffff;
  if (a.parts > 0) {  // the first pass has run; its parts are merged in order
    if (tid < a.parts) {
      const float* src = a.partials + ((size_t)r * a.parts + tid) * 4;
      m = src[0]; ssum = src[1]; bi = __float_as_int(src[2]);
    }
  } else {
    first_pass(o, lg, x, 0, V, V, m, ssum, bi);
  }
  block_merge(m, ssum, bi, red, part, redi);
  if (tid == 0 && redi[24] == 0x7fffffff) redi[24] = 0;  // a row of NaNs
  __syncthreads();
  const float mx = red[24];
  const int best = redi[24];

  if (greedy) {  // logprob = log_softmax(processed)[tok] = -log(sum of exp(x - max))
    if (tid == 0) {
      a.out_token[r] = best;
      a.out_logprob[r] = -logf(red[25]);
    }
    return;
  }
  __syncthreads();

  // min_p: drop ids with p < min_p * p_max  <=>  x < max + log(min_p)
  if (minp > 0.f) {
    const float bound = mx + logf(minp);
    for (int i = tid; i < V; i += blockDim.x)
      if (x[i] < bound) x[i] = -INFINITY;
    __syncthreads();
  }

  // top_k: keep values >= the k-th largest (reference: qwen3_runtime/sampling.py:98-101)
  const int k = a.iparams[(size_t)sl * 2];
  if (k > 0 && k < V) {
    unsigned lo = f2ord(-INFINITY), hi = f2ord(mx);  // largest t with count(x >= t) >= k
    while (lo < hi) {
      const unsigned mid = lo + (hi - lo + 1u) / 2u;
      const float t = ord2f(mid);
      float c = 0.f;
      for (int i = tid; i < V; i += blockDim.x) c += (x[i] >= t) ? 1.f : 0.f;
      c = block_sum(c, red);
      if (c >= (float)k) lo = mid; else hi = mid - 1u;
    }
    const float t = ord2f(lo);
    for (int i = tid; i < V; i += blockDim.x)
      if (x[i] < t) x[i] = -INFINITY;
    __syncthreads();
  }

  // top_p: keep an id iff the mass of ids strictly above it is <= top_p
  // (reference: qwen3_runtime/sampling.py:102-109: the first id past the mass stays)
  if (topp < 1.0f) {
    float z = 0.f;
    for (int i = tid; i < V; i += blockDim.x) z += expf(x[i] - mx);
    z = block_sum(z, red);
    unsigned lo = f2ord(-INFINITY), hi = f2ord(mx);  // smallest t with mass(x > t) <= top_p * z
    while (lo < hi) {
      const unsigned mid = lo + (hi - lo) / 2u;
      const float t = ord2f(mid);
      float c = 0.f;
      for (int i = tid; i < V; i += blockDim.x) c += (x[i] > t) ? expf(x[i] - mx) : 0.f;
      c = block_sum(c, red);
      if (c <= topp * z) hi = mid; else lo = mid + 1u;
    }
    const float t = ord2f(lo);
    for (int i = tid; i < V; i += blockDim.x)
      if (x[i] < t) x[i] = -INFINITY;
    __syncthreads();
  }

  // softmax + inverse CDF (reference: qwen3_runtime/sampling.py:208-227)
  const int chunk = (V + blockDim.x - 1) / blockDim.x;
  const int c0 = min(V, tid * chunk), c1 = min(V, c0 + chunk);
  float local = 0.f;
  for (int i = c0; i < c1; ++i) local += expf(x[i] - mx);
  part[tid] = local;
  __syncthreads();
  if (tid == 0) {
    float run = 0.f;
    for (int i = 0; i < (int)blockDim.x; ++i) { const float v = part[i]; part[i] = run; run += v; }
    red[20] = run;
  }
  __syncthreads();
  const float z = red[20];
  const unsigned long long seed = a.seeds[(size_t)sl * 2], draw = a.seeds[(size_t)sl * 2 + 1];
  const float u = philox_uniform(seed, draw) * z;
  if (tid == 0) redi[20] = -1;
  __syncthreads();
  // the chunk whose span of the cumulative sum holds u; the last non-empty one if rounding overshoots
  const float before = part[tid];
  const float after = (tid + 1 < (int)blockDim.x) ? part[tid + 1] : z;
  if (local > 0.f && (u < after || after >= z) && u >= before) atomicMax(&redi[20], tid);
  __syncthreads();
  int owner = redi[20];
  if (owner < 0) {  // u fell in no chunk because of rounding: take the last chunk with mass
    if (local > 0.f) atomicMax(&redi[20], tid);
    __syncthreads();
    owner = redi[20];
  }
  if (tid == owner) {
    float run = before;
    int pick = -1, last = -1;
    for (int i = c0; i < c1; ++i) {
      const float pe = expf(x[i] - mx);
      if (pe > 0.f) {
        last = i;
        run += pe;
        if (run > u) { pick = i; break; }
      }
    }
    if (pick < 0) pick = last;
    a.out_token[r] = pick;
    a.out_logprob[r] = logf(fmaxf(expf(x[pick] - mx) / z, 1e-30f));
    a.seeds[(size_t)sl * 2 + 1] = draw + 1;
  }
}

// both entry points: `a.partials` is already where the first pass may write
static int launch_sample(const SampleArgs& a, hipStream_t stream) {
  if (a.parts > 0) {
    QRT_CHECK(a.rows <= 65535, "sample: %d rows in parts", a.rows);
    sample_first_pass_kernel<<<dim3(a.rows, a.parts), dim3(256), 0, stream>>>(a);
    QRT_LAUNCH_CHECK("sample (first pass)");
  }
  sample_kernel<<<dim3(a.rows), dim3(SAMPLE_THREADS), 0, stream>>>(a);
  QRT_LAUNCH_CHECK("sample");
  return 0;
}

extern "C" int qrt_sample(const SampleArgs* args, hipStream_t stream) {
  SampleArgs a = *args;
  QRT_CHECK(a.rows >= 0 && a.vocab > 0, "sample: bad sizes");
  if (a.rows == 0) return 0;
  QRT_CHECK(a.parts >= 0 && a.parts <= 64 && (a.parts == 0 || a.partials), "sample: bad number of parts %d", a.parts);
  return launch_sample(a, stream);
}

// ---- the entry point that allocates nothing (declared and described in sampling.h) ----------
//
// The partial results of the first pass live in this array, one copy per GPU, each at its own
// address. In host code the array's name is only a handle for hipGetSymbolAddress, never an
// address: kernels get the pointer that call returned for the current device.
// No device code names the array (kernels get its address as an argument); it stays in the device
// image, as a global symbol the runtime can look up, because host code below names it. (Marked
// `used` it would stay a local symbol instead, which hipGetSymbolAddress cannot find.)
static __device__ __align__(256) unsigned char scratch[QRT_SAMPLE_SCRATCH_BYTES];

#define QRT_MAX_DEVICES 64
static void* g_scratch_of_device[QRT_MAX_DEVICES] = {};
static std::mutex g_scratch_mutex;

// The current device's copy of `scratch`; looked up once per device, with that device current.
static int scratch_for_current_device(void** out) {
  int dev = -1;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return qrt_fail("sample_noalloc: hipGetDevice: %s", hipGetErrorString(e));
  QRT_CHECK(dev >= 0 && dev < QRT_MAX_DEVICES, "sample_noalloc: device %d is beyond the %d this library counts",
            dev, QRT_MAX_DEVICES);
  std::lock_guard<std::mutex> lock(g_scratch_mutex);
  if (!g_scratch_of_device[dev]) {
    void* ptr = nullptr;
    e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
    if (e != hipSuccess || !ptr)
      return qrt_fail("sample_noalloc: hipGetSymbolAddress on device %d: %s", dev, hipGetErrorString(e));
    g_scratch_of_device[dev] = ptr;
  }
  *out = g_scratch_of_device[dev];
  return 0;
}

// Optional: look the buffer up now (for the current device), so that the first sampling call,
// which may sit inside a stream capture, finds it ready.
extern "C" int qrt_sample_noalloc_setup() {
  void* ptr = nullptr;
  return scratch_for_current_device(&ptr);
}

extern "C" int qrt_sample_noalloc(const SampleArgs* args, hipStream_t stream) {
  SampleArgs a = *args;
  QRT_CHECK(a.rows >= 0 && a.vocab > 0, "sample_noalloc: bad sizes");
  if (a.rows == 0) return 0;
  QRT_CHECK(a.parts >= 0 && a.parts <= 64, "sample_noalloc: bad number of parts %d", a.parts);
  const size_t need = (size_t)a.rows * (size_t)a.parts * 4 * sizeof(float);
  QRT_CHECK(need <= QRT_SAMPLE_SCRATCH_BYTES,
            "sample_noalloc: %d rows in %d parts need %zu bytes for the first pass's results; the buffer built "
            "into the library holds %d (fewer parts, or qrt_sample with a buffer of the caller's)",
            a.rows, a.parts, need, QRT_SAMPLE_SCRATCH_BYTES);
  a.partials = nullptr;
  if (a.parts > 0) {
    void* ptr = nullptr;
    if (scratch_for_current_device(&ptr) != 0) return -1;
    a.partials = (float*)ptr;  // every entry [row, part] is written by the first pass before it is read
  }
  return launch_sample(a, stream);
}

// counts[slot[i], token[i]] += 1   (ids a request has seen: prompt and output)
__global__ void count_tokens_kernel(int* counts, const int* slot, const int* token, int n, int vocab) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n && token[i] >= 0 && token[i] < vocab) atomicAdd(&counts[(size_t)slot[i] * vocab + token[i]], 1);
}

extern "C" int qrt_count_tokens(int* counts, const int* slot, const int* token, int n, int vocab, hipStream_t stream) {
  if (n <= 0) return 0;
  count_tokens_kernel<<<dim3((n + 255) / 256), dim3(256), 0, stream>>>(counts, slot, token, n, vocab);
  QRT_LAUNCH_CHECK("count_tokens");
  return 0;
}

// logits[row[i], token[i]] += value[i]   (logit bias; reference: qwen3_runtime/sampling.py:35-41)
__global__ void add_bias_kernel(float* logits, const int* row, const int* token, const float* value, int n, int vocab) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n && token[i] >= 0 && token[i] < vocab) atomicAdd(&logits[(size_t)row[i] * vocab + token[i]], value[i]);
}

extern "C" int qrt_add_bias(float* logits, const int* row, const int* token, const float* value, int n, int vocab,
                            hipStream_t stream) {
  if (n <= 0) return 0;
  add_bias_kernel<<<dim3((n + 255) / 256), dim3(256), 0, stream>>>(logits, row, token, value, n, vocab);
  QRT_LAUNCH_CHECK("add_bias");
  return 0;
}
