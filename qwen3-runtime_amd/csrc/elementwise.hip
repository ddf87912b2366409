// Memory-bound ops between the matrix products: embedding gather, residual add
// + RMSNorm, per-head q/k RMSNorm + rotary encoding + cache write, SwiGLU.
// All reductions, the norms, the rotation angles and the residual sum are
// float32; each row's reduction order is fixed, whatever else is in the batch.
#include "common.h"
#include <math.h>

// ---------------------------------------------------------------- embedding
// residual[t, :] = float(table[ids[t], :])            (no scaling of embeddings)
template <typename TW>
__global__ void embed_kernel(const int* __restrict__ ids, const TW* __restrict__ table,
                             float* __restrict__ out, int hidden) {
  const int t = blockIdx.x;
  const TW* row = table + (size_t)ids[t] * hidden;
  float* o = out + (size_t)t * hidden;
  for (int i = threadIdx.x; i < hidden; i += blockDim.x) o[i] = to_f32<TW>(row[i]);
}

extern "C" int qrt_embed(const int* ids, const void* table, int table_dtype, float* out,
                         int num_tokens, int vocab, int hidden, hipStream_t stream) {
  QRT_CHECK(num_tokens >= 0 && vocab > 0 && hidden > 0, "embed: bad sizes T=%d V=%d H=%d", num_tokens, vocab, hidden);
  if (num_tokens == 0) return 0;
  dim3 grid(num_tokens), block(256);
  if (table_dtype == QRT_F32)
    embed_kernel<float><<<grid, block, 0, stream>>>(ids, (const float*)table, out, hidden);
  else if (table_dtype == QRT_BF16)
    embed_kernel<bf16_t><<<grid, block, 0, stream>>>(ids, (const bf16_t*)table, out, hidden);
  else
    return qrt_fail("embed: unknown table dtype %d", table_dtype);
  QRT_LAUNCH_CHECK("embed");
  return 0;
}

// ------------------------------------------------ rotation table of a step
// out[t, j] = cos(pos[t] * inv_freq[j]), out[t, half + j] = sin(...), j < half: the angles of a
// step's tokens, float32. Every layer of a step rotates by the same angles, so a step that
// rotates inside its attention kernel computes them once, here, and the layers look them up.
__global__ void rope_table_kernel(const int* __restrict__ positions, const float* __restrict__ inv_freq,
                                  float* __restrict__ out, int half) {
  const float pos = (float)positions[blockIdx.x];
  float* row = out + (size_t)blockIdx.x * 2 * half;
  for (int j = threadIdx.x; j < half; j += blockDim.x) {
    float sn, cs;
    sincos_angle(pos * inv_freq[j], &sn, &cs);
    row[j] = cs;
    row[half + j] = sn;
  }
}

extern "C" int qrt_rope_table(const int* positions, const float* inv_freq, float* out, int num_tokens, int half,
                              hipStream_t stream) {
  QRT_CHECK(num_tokens >= 0 && half > 0, "rope_table: bad sizes T=%d half=%d", num_tokens, half);
  if (num_tokens == 0) return 0;
  rope_table_kernel<<<dim3(num_tokens), dim3(half <= 64 ? 64 : 128), 0, stream>>>(positions, inv_freq, out, half);
  QRT_LAUNCH_CHECK("rope_table");
  return 0;
}

// ------------------------------------------------------- add + RMSNorm
// r = rows ? rows[b] : b
// x = residual[r] (+ delta[r]);  without `rows` the sum is written back.
// out[b] = x * rsqrt(mean(x^2) + eps) * weight
// One block of 256 threads per row. Each thread keeps its elements of the row in registers
// (rows up to 256 * VEC * KEEP wide; wider rows are read a second time), all loads of a row are
// issued before the first use, squares are summed over the block in a fixed order.
// delta may come as `planes` planes [planes, T, H] that are added in order (the parts of a product
// whose K was cut). PL is the number of planes where it is known when compiling (0: no delta):
// residual, planes and weights are then all loaded at once, unconditionally (clamped index), so
// that a row costs one round of memory latency instead of one per plane and one for the weights;
// PL = -1 loops over any number of planes.
template <typename TD, typename TO, int VEC, int KEEP, int PL>
__global__ __launch_bounds__(256) void add_rmsnorm_kernel(float* __restrict__ residual, const TD* __restrict__ delta,
                                                          const float* __restrict__ weight,
                                                          const int* __restrict__ rows, TO* __restrict__ out,
                                                          int hidden, float eps, int planes, size_t plane_stride) {
  typedef float fvec_t __attribute__((ext_vector_type(VEC)));
  typedef TD dvec_t __attribute__((ext_vector_type(VEC)));
  typedef TO ovec_t __attribute__((ext_vector_type(VEC)));
  __shared__ float red[32];
  const int b = blockIdx.x;
  const int r = rows ? rows[b] : b;
  float* res = residual + (size_t)r * hidden;
  const TD* del = delta ? delta + (size_t)r * hidden : nullptr;
  const bool write_back = del && !rows;
  constexpr int STRIDE = 256 * VEC;
  const int i0 = threadIdx.x * VEC;

  fvec_t x[KEEP], w[KEEP];
  float ss = 0.f;
  if (PL >= 0) {
    dvec_t d[PL > 0 ? PL : 1][KEEP];
#pragma unroll
    for (int j = 0; j < KEEP; ++j) {
      const int ic = min(i0 + j * STRIDE, hidden - VEC);  // beyond the row: some element of it, dropped below
      x[j] = *(const fvec_t*)(res + ic);
      w[j] = *(const fvec_t*)(weight + ic);
#pragma unroll
      for (int p = 0; p < PL; ++p) d[p][j] = *(const dvec_t*)(del + p * plane_stride + ic);
    }
#pragma unroll
    for (int p = 0; p < PL; ++p)
#pragma unroll
      for (int j = 0; j < KEEP; ++j)
#pragma unroll
        for (int e = 0; e < VEC; ++e) x[j][e] += to_f32<TD>(d[p][j][e]);
  } else {
#pragma unroll
    for (int j = 0; j < KEEP; ++j) {
      const int ic = min(i0 + j * STRIDE, hidden - VEC);
      x[j] = *(const fvec_t*)(res + ic);
      w[j] = *(const fvec_t*)(weight + ic);
    }
    if (del) {
      for (int p = 0; p < planes; ++p) {
#pragma unroll
        for (int j = 0; j < KEEP; ++j) {
          const int ic = min(i0 + j * STRIDE, hidden - VEC);
          const dvec_t d = *(const dvec_t*)(del + p * plane_stride + ic);
#pragma unroll
          for (int e = 0; e < VEC; ++e) x[j][e] += to_f32<TD>(d[e]);
        }
      }
    }
  }
#pragma unroll
  for (int j = 0; j < KEEP; ++j) {
    const int i = i0 + j * STRIDE;
    if (i < hidden) {
      if (write_back) *(fvec_t*)(res + i) = x[j];
#pragma unroll
      for (int e = 0; e < VEC; ++e) ss += x[j][e] * x[j][e];
    }
  }
  // the part of a row beyond what the registers hold
  for (int i = i0 + KEEP * STRIDE; i < hidden; i += STRIDE) {
    fvec_t v = *(const fvec_t*)(res + i);
    if (del) {
      for (int p = 0; p < planes; ++p) {
        const dvec_t d = *(const dvec_t*)(del + p * plane_stride + i);
#pragma unroll
        for (int e = 0; e < VEC; ++e) v[e] += to_f32<TD>(d[e]);
      }
      if (write_back) *(fvec_t*)(res + i) = v;
    }
#pragma unroll
    for (int e = 0; e < VEC; ++e) ss += v[e] * v[e];
  }
  const float inv = rsqrtf(block_sum(ss, red) / (float)hidden + eps);
  TO* o = out + (size_t)b * hidden;
#pragma unroll
  for (int j = 0; j < KEEP; ++j) {
    const int i = i0 + j * STRIDE;
    if (i < hidden) {
      ovec_t y;
#pragma unroll
      for (int e = 0; e < VEC; ++e) y[e] = from_f32<TO>(x[j][e] * inv * w[j][e]);
      *(ovec_t*)(o + i) = y;
    }
  }
  for (int i = i0 + KEEP * STRIDE; i < hidden; i += STRIDE) {
    fvec_t v = *(const fvec_t*)(res + i);  // already summed if written back
    if (del && !write_back) {
      for (int p = 0; p < planes; ++p) {
        const dvec_t d = *(const dvec_t*)(del + p * plane_stride + i);
#pragma unroll
        for (int e = 0; e < VEC; ++e) v[e] += to_f32<TD>(d[e]);
      }
    }
    const fvec_t wv = *(const fvec_t*)(weight + i);
    ovec_t y;
#pragma unroll
    for (int e = 0; e < VEC; ++e) y[e] = from_f32<TO>(v[e] * inv * wv[e]);
    *(ovec_t*)(o + i) = y;
  }
}

extern "C" int qrt_add_rmsnorm(float* residual, const void* delta, int delta_dtype, const float* weight,
                               const int* rows, void* out, int out_dtype, int num_out_rows, int hidden,
                               float eps, int planes, long plane_stride, hipStream_t stream) {
  QRT_CHECK(hidden > 0 && num_out_rows >= 0, "add_rmsnorm: bad sizes rows=%d H=%d", num_out_rows, hidden);
  QRT_CHECK(planes >= 1 && planes <= 64 && plane_stride >= 0, "add_rmsnorm: bad delta planes %d", planes);
  if (num_out_rows == 0) return 0;
  dim3 grid(num_out_rows), block(256);
  const bool vec4 = hidden % 4 == 0 && (uintptr_t)residual % 16 == 0 && (uintptr_t)weight % 16 == 0 &&
                    (uintptr_t)out % 16 == 0 && (!delta || (uintptr_t)delta % 16 == 0) && plane_stride % 4 == 0;
  // planes known to the compiler (0: no delta) up to eight of them
  const int pl = !delta ? 0 : planes >= 1 && planes <= 8 ? planes : -1;
#define GO(TD, TO, VEC, KEEP, PL)                                                                               \
  add_rmsnorm_kernel<TD, TO, VEC, KEEP, PL><<<grid, block, 0, stream>>>(residual, (const TD*)delta, weight,     \
                                                                        rows, (TO*)out, hidden, eps, planes,    \
                                                                        (size_t)plane_stride)
#define LAUNCH(TD, TO)                                                                                          \
  do {                                                                                                          \
    if (!vec4) GO(TD, TO, 1, 8, -1);                                                                            \
    else if (pl == 0) GO(TD, TO, 4, 4, 0);                                                                      \
    else if (pl == 1) GO(TD, TO, 4, 4, 1);                                                                      \
    else if (pl == 2) GO(TD, TO, 4, 4, 2);                                                                      \
    else if (pl == 3) GO(TD, TO, 4, 4, 3);                                                                      \
    else if (pl == 4) GO(TD, TO, 4, 4, 4);                                                                      \
    else if (pl == 5) GO(TD, TO, 4, 4, 5);                                                                      \
    else if (pl == 6) GO(TD, TO, 4, 4, 6);                                                                      \
    else if (pl == 7) GO(TD, TO, 4, 4, 7);                                                                      \
    else if (pl == 8) GO(TD, TO, 4, 4, 8);                                                                      \
    else GO(TD, TO, 4, 4, -1);                                                                                  \
  } while (0)
  if (delta_dtype == QRT_F32 && out_dtype == QRT_F32) LAUNCH(float, float);
  else if (delta_dtype == QRT_BF16 && out_dtype == QRT_BF16) LAUNCH(bf16_t, bf16_t);
  else if (delta_dtype == QRT_F32 && out_dtype == QRT_BF16) LAUNCH(float, bf16_t);
  else if (delta_dtype == QRT_BF16 && out_dtype == QRT_F32) LAUNCH(bf16_t, float);
  else return qrt_fail("add_rmsnorm: unknown dtypes %d %d", delta_dtype, out_dtype);
#undef LAUNCH
#undef GO
  QRT_LAUNCH_CHECK("add_rmsnorm");
  return 0;
}

// ------------------------------------------------------------------ SwiGLU
// out[t, i] = silu(gu[t, i]) * gu[t, I + i],  silu(x) = x / (1 + exp(-x)), in float32.
// VEC elements per thread and access: 8 for bfloat16 rows whose halves start on 16 bytes.
template <typename T, int VEC>
__global__ __launch_bounds__(256) void swiglu_kernel(const T* __restrict__ gu, T* __restrict__ out, int inter) {
  typedef T vec_t __attribute__((ext_vector_type(VEC)));
  // a block per token: no division to find the row, and two loads of each half in flight per thread
  // (120 MB read and written for 2,048 tokens of the 4B shape in 23.6 us, 5.1 TB/s, as the
  // grid-stride form before it: the mix of reads and writes is what bounds it)
  const T* g_row = gu + (size_t)blockIdx.x * 2 * inter;
  const T* u_row = g_row + inter;
  T* o_row = out + (size_t)blockIdx.x * inter;
  constexpr int U = 2;
  for (int i0 = threadIdx.x * VEC; i0 < inter; i0 += U * 256 * VEC) {
    vec_t g[U], u[U];
#pragma unroll
    for (int k = 0; k < U; ++k) {
      const int i = i0 + k * 256 * VEC;
      if (i < inter) {
        g[k] = *(const vec_t*)(g_row + i);
        u[k] = *(const vec_t*)(u_row + i);
      }
    }
#pragma unroll
    for (int k = 0; k < U; ++k) {
      const int i = i0 + k * 256 * VEC;
      if (i < inter) {
        vec_t o;
#pragma unroll
        for (int e = 0; e < VEC; ++e) {
          const float gf = to_f32<T>(g[k][e]);
          o[e] = from_f32<T>(gf / (1.0f + expf(-gf)) * to_f32<T>(u[k][e]));
        }
        *(vec_t*)(o_row + i) = o;
      }
    }
  }
}

template <typename T, int VEC>
static void swiglu_launch(const void* gate_up, void* out, int num_tokens, int inter, hipStream_t stream) {
  swiglu_kernel<T, VEC><<<dim3((unsigned)num_tokens), 256, 0, stream>>>((const T*)gate_up, (T*)out, inter);
}

extern "C" int qrt_swiglu(const void* gate_up, void* out, int dtype, int num_tokens, int inter,
                          hipStream_t stream) {
  QRT_CHECK(num_tokens >= 0 && inter > 0, "swiglu: bad sizes T=%d I=%d", num_tokens, inter);
  if ((size_t)num_tokens * inter == 0) return 0;
  const bool aligned = ((uintptr_t)gate_up % 16 == 0) && ((uintptr_t)out % 16 == 0);
  if (dtype == QRT_F32) {
    if (aligned && inter % 4 == 0) swiglu_launch<float, 4>(gate_up, out, num_tokens, inter, stream);
    else swiglu_launch<float, 1>(gate_up, out, num_tokens, inter, stream);
  } else if (dtype == QRT_BF16) {
    if (aligned && inter % 8 == 0) swiglu_launch<bf16_t, 8>(gate_up, out, num_tokens, inter, stream);
    else swiglu_launch<bf16_t, 1>(gate_up, out, num_tokens, inter, stream);
  } else {
    return qrt_fail("swiglu: unknown dtype %d", dtype);
  }
  QRT_LAUNCH_CHECK("swiglu");
  return 0;
}

// ------------------------------- per-head norm + rotary + cache write
// One wave per (token, head) over the nq query heads, nkv key heads and nkv
// value heads of a token. Query and key heads: optional RMSNorm over the head
// (weight [D]), optional NeoX rotation with angle = float(pos) * inv_freq[j]
// pairing element j with j + D/2. Value heads are copied. Keys and values go to
// the paged cache (keys [page, head, offset, D], values [page, head, D, offset])
// and/or to dense outputs; queries go to q_out.
struct QkArgs {
  const void* q_in;  long q_stride;   // elements between tokens
  const void* k_in;  long k_stride;
  const void* v_in;  long v_stride;
  const float* q_weight;  // null: no norm
  const float* k_weight;
  const float* inv_freq;  // null: no rotation
  const int* positions;
  const int* slots;       // null: no cache write
  void* q_out;            // [T, nq, D] or null
  void* k_out;            // [T, nkv, D] or null
  void* v_out;            // [T, nkv, D] or null
  void* k_cache;
  void* v_cache;
  int num_tokens, nq, nkv, nv, head_dim, page_size;
  float eps;
  // [T, head_dim] or null: the cosines of the tokens' head_dim / 2 angles, then their sines, as
  // rope_table makes them. The kernel for many tokens looks them up instead of computing them in
  // every layer (inv_freq and positions are still given: the kernel for few tokens computes).
  const float* rope;
};

template <typename T>
__global__ void qk_norm_rope_store_kernel(QkArgs a) {
  const int lane = threadIdx.x & 63;
  const int heads = a.nq + a.nkv + a.nv;
  const long item = (long)blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
  if (item >= (long)a.num_tokens * heads) return;
  const int t = (int)(item / heads);
  const int h = (int)(item - (long)t * heads);
  const int D = a.head_dim, half = D >> 1;

  if (h >= a.nq + a.nkv) {  // value head: copy
    const int hv = h - a.nq - a.nkv;
    const T* src = (const T*)a.v_in + (size_t)t * a.v_stride + (size_t)hv * D;
    if (a.v_out) {
      T* dst = (T*)a.v_out + ((size_t)t * a.nv + hv) * D;
      for (int i = lane; i < D; i += 64) dst[i] = src[i];
    }
    if (a.slots) {
      const int slot = a.slots[t];
      const int page = slot / a.page_size, off = slot - page * a.page_size;
      T* dst = (T*)a.v_cache + ((size_t)page * a.nv + hv) * D * a.page_size + off;
      for (int i = lane; i < D; i += 64) dst[(size_t)i * a.page_size] = src[i];
    }
    return;
  }

  const bool is_q = h < a.nq;
  const int hh = is_q ? h : h - a.nq;
  const T* src = is_q ? (const T*)a.q_in + (size_t)t * a.q_stride + (size_t)hh * D
                      : (const T*)a.k_in + (size_t)t * a.k_stride + (size_t)hh * D;
  const float* w = is_q ? a.q_weight : a.k_weight;

  // each lane owns the pairs (p, p + D/2) for p = lane, lane + 64, ... (D <= 512).
  // Everything the lane will need is loaded before the first use (norm weights, position,
  // frequencies, slot), so that the kernel costs one round of memory latency, not four.
  float x1[4], x2[4], w1[4], w2[4], fr[4];
  float ss = 0.f;
  const float pos = a.inv_freq ? (float)a.positions[t] : 0.f;
  const int slot = (!is_q && a.slots) ? a.slots[t] : 0;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int p = lane + 64 * i;
    x1[i] = x2[i] = 0.f;
    w1[i] = w2[i] = 1.f;
    fr[i] = 0.f;
    if (p < half) {
      x1[i] = to_f32<T>(src[p]);
      x2[i] = to_f32<T>(src[p + half]);
      if (w) {
        w1[i] = w[p];
        w2[i] = w[p + half];
      }
      if (a.inv_freq) fr[i] = a.inv_freq[p];
    }
  }
#pragma unroll
  for (int i = 0; i < 4; ++i) ss += x1[i] * x1[i] + x2[i] * x2[i];
  if (w) {
    ss = wave_sum(ss);
    const float inv = rsqrtf(ss / (float)D + a.eps);
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      x1[i] = x1[i] * inv * w1[i];
      x2[i] = x2[i] * inv * w2[i];
    }
  }
  if (a.inv_freq) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int p = lane + 64 * i;
      if (p < half) {
        const float ang = pos * fr[i];
        float sn, c;
        sincos_angle(ang, &sn, &c);
        const float y1 = x1[i] * c - x2[i] * sn;
        const float y2 = x2[i] * c + x1[i] * sn;
        x1[i] = y1;
        x2[i] = y2;
      }
    }
  }
  T* dense = nullptr;
  if (is_q && a.q_out) dense = (T*)a.q_out + ((size_t)t * a.nq + hh) * D;
  if (!is_q && a.k_out) dense = (T*)a.k_out + ((size_t)t * a.nkv + hh) * D;
  T* paged = nullptr;
  if (!is_q && a.slots) {
    const int page = slot / a.page_size, off = slot - page * a.page_size;
    paged = (T*)a.k_cache + (((size_t)page * a.nkv + hh) * a.page_size + off) * D;
  }
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int p = lane + 64 * i;
    if (p < half) {
      const T y1 = from_f32<T>(x1[i]), y2 = from_f32<T>(x2[i]);
      if (dense) { dense[p] = y1; dense[p + half] = y2; }
      if (paged) { paged[p] = y1; paged[p + half] = y2; }
    }
  }
}

// The same work for head sizes 16, 32, ..., 512 (powers of two) with every access 8 elements
// wide. Norm and rotation: a lane owns 8 neighbouring elements of the first half of a head and
// their partners in the second half, head_dim / 16 lanes share a head, a wave covers
// 64 / (head_dim / 16) heads per pass and computes the sines and cosines of its token once for
// all passes it makes. Values: a wave takes 8 tokens of one head, turns them round in LDS and
// writes, for each head element, the 8 tokens as one piece of the transposed page; that needs
// the 8 slots to be neighbours that start on a multiple of 8, as the tokens of a prompt
// portion usually are, otherwise it writes element by element.
template <typename T> struct alignas(sizeof(T) * 8) Vec8 { T v[8]; };

template <typename T>
__global__ __launch_bounds__(256) void qk_norm_rope_store_wide_kernel(QkArgs a, int lph, int rope_blocks,
                                                                      int passes_per_wave) {
  extern __shared__ __align__(32) unsigned char smem_raw[];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int D = a.head_dim, half = D >> 1;

  if ((int)blockIdx.x < rope_blocks) {
    const int hp = 64 / lph, nh = a.nq + a.nkv;
    const int passes = (nh + hp - 1) / hp;
    const int groups = (passes + passes_per_wave - 1) / passes_per_wave;
    const long item = (long)blockIdx.x * 4 + wave;
    if (item >= (long)a.num_tokens * groups) return;
    const int t = (int)(item / groups), grp = (int)(item - (long)t * groups);
    const int c = lane & (lph - 1), hl = lane / lph;
    float sn[8], cs[8];
    if (a.rope) {
      const float* angles = a.rope + (size_t)t * D + 8 * c;
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        cs[e] = angles[e];
        sn[e] = angles[half + e];
      }
    } else if (a.inv_freq) {
      const float pos = (float)a.positions[t];
#pragma unroll
      for (int e = 0; e < 8; ++e) sincos_angle(pos * a.inv_freq[8 * c + e], &sn[e], &cs[e]);
    }
    const int slot = a.slots ? a.slots[t] : 0;
    const int page = slot / a.page_size, off = slot - page * a.page_size;
    const int pass_end = min(passes, (grp + 1) * passes_per_wave);
    for (int ps = grp * passes_per_wave; ps < pass_end; ++ps) {
      const int h = ps * hp + hl;
      if (h >= nh) continue;  // whole groups of lph lanes leave together
      const bool is_q = h < a.nq;
      const int hh = is_q ? h : h - a.nq;
      const T* src = is_q ? (const T*)a.q_in + (size_t)t * a.q_stride + (size_t)hh * D
                          : (const T*)a.k_in + (size_t)t * a.k_stride + (size_t)hh * D;
      const float* w = is_q ? a.q_weight : a.k_weight;
      const Vec8<T> r1 = *(const Vec8<T>*)(src + 8 * c), r2 = *(const Vec8<T>*)(src + half + 8 * c);
      float x1[8], x2[8];
      float ss = 0.f;
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        x1[e] = to_f32<T>(r1.v[e]);
        x2[e] = to_f32<T>(r2.v[e]);
        ss += x1[e] * x1[e] + x2[e] * x2[e];
      }
      if (w) {
        for (int o = lph >> 1; o > 0; o >>= 1) ss += __shfl_xor(ss, o, 64);
        const float inv = rsqrtf(ss / (float)D + a.eps);
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          x1[e] = x1[e] * inv * w[8 * c + e];
          x2[e] = x2[e] * inv * w[half + 8 * c + e];
        }
      }
      Vec8<T> y1, y2;
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        float u1 = x1[e], u2 = x2[e];
        if (a.inv_freq) {
          u1 = x1[e] * cs[e] - x2[e] * sn[e];
          u2 = x2[e] * cs[e] + x1[e] * sn[e];
        }
        y1.v[e] = from_f32<T>(u1);
        y2.v[e] = from_f32<T>(u2);
      }
      T* dense = nullptr;
      if (is_q && a.q_out) dense = (T*)a.q_out + ((size_t)t * a.nq + hh) * D;
      if (!is_q && a.k_out) dense = (T*)a.k_out + ((size_t)t * a.nkv + hh) * D;
      if (dense) {
        *(Vec8<T>*)(dense + 8 * c) = y1;
        *(Vec8<T>*)(dense + half + 8 * c) = y2;
      }
      if (!is_q && a.slots) {
        T* paged = (T*)a.k_cache + (((size_t)page * a.nkv + hh) * a.page_size + off) * D;
        *(Vec8<T>*)(paged + 8 * c) = y1;
        *(Vec8<T>*)(paged + half + 8 * c) = y2;
      }
    }
    return;
  }

  // values: 8 tokens of one head
  const long item = (long)(blockIdx.x - rope_blocks) * 4 + wave;
  const int token_groups = (a.num_tokens + 7) >> 3;
  if (item >= (long)token_groups * a.nv) return;
  const int tg = (int)(item / a.nv), hv = (int)(item - (long)tg * a.nv);
  const int t0 = 8 * tg, nvalid = min(8, a.num_tokens - t0);
  const int row = D + 8;  // padded: the 8 tokens of an element lie in different banks
  T* tile = (T*)smem_raw + (size_t)wave * 8 * row;
  const int chunks = D >> 3;
  for (int idx = lane; idx < 8 * chunks; idx += 64) {
    const int j = idx / chunks, c = idx - j * chunks;
    if (j < nvalid) {
      const Vec8<T> r = *(const Vec8<T>*)((const T*)a.v_in + (size_t)(t0 + j) * a.v_stride + (size_t)hv * D + 8 * c);
      *(Vec8<T>*)(tile + j * row + 8 * c) = r;
      if (a.v_out) *(Vec8<T>*)((T*)a.v_out + ((size_t)(t0 + j) * a.nv + hv) * D + 8 * c) = r;
    }
  }
  if (!a.slots) return;
  __builtin_amdgcn_wave_barrier();  // the wave reads below what it wrote above; LDS keeps a wave's order
  const int my_slot = a.slots[t0 + min(lane, nvalid - 1)];
  const int s0 = __shfl(my_slot, 0, 64);
  const bool in_line = lane >= 8 || my_slot == s0 + lane;
  const bool wide = nvalid == 8 && (s0 & 7) == 0 && (a.page_size & 7) == 0 && __all(in_line);
  if (wide) {
    const int page = s0 / a.page_size, off = s0 - page * a.page_size;
    T* base = (T*)a.v_cache + ((size_t)page * a.nv + hv) * D * a.page_size + off;
    for (int d = lane; d < D; d += 64) {
      Vec8<T> o;
#pragma unroll
      for (int j = 0; j < 8; ++j) o.v[j] = tile[j * row + d];
      *(Vec8<T>*)(base + (size_t)d * a.page_size) = o;
    }
  } else {
    for (int j = 0; j < nvalid; ++j) {
      const int sj = __shfl(my_slot, j, 64);
      const int page = sj / a.page_size, off = sj - page * a.page_size;
      T* base = (T*)a.v_cache + ((size_t)page * a.nv + hv) * D * a.page_size + off;
      for (int d = lane; d < D; d += 64) base[(size_t)d * a.page_size] = tile[j * row + d];
    }
  }
}

extern "C" int qrt_qk_norm_rope_store(const QkArgs* args, int dtype, long num_cache_pages, hipStream_t stream) {
  QkArgs a = *args;
  QRT_CHECK(a.num_tokens >= 0 && a.nq >= 0 && a.nkv >= 0 && a.nv >= 0, "qk_norm_rope_store: negative size");
  QRT_CHECK(a.head_dim >= 2 && a.head_dim % 2 == 0 && a.head_dim <= 512,
            "qk_norm_rope_store: head size %d must be even and at most 512", a.head_dim);
  QRT_CHECK(a.nq == 0 || a.q_in, "qk_norm_rope_store: query heads without input");
  QRT_CHECK(a.nkv == 0 || a.k_in, "qk_norm_rope_store: key heads without input");
  QRT_CHECK(a.nv == 0 || a.v_in, "qk_norm_rope_store: value heads without input");
  QRT_CHECK(!a.inv_freq || a.positions, "qk_norm_rope_store: rotation without positions");
  if (a.slots) {
    QRT_CHECK(a.k_cache && a.v_cache && a.page_size > 0 && num_cache_pages > 0,
              "qk_norm_rope_store: cache write without cache");
    QRT_CHECK(a.nkv == a.nv, "qk_norm_rope_store: cache write needs as many key as value heads");
  }
  const long items = (long)a.num_tokens * (a.nq + a.nkv + a.nv);
  if (items == 0) return 0;
  const int waves = 4;
  const size_t esize = dtype == QRT_F32 ? 4 : 2;
  auto lined_up = [&](const void* ptr) { return ((uintptr_t)ptr % (8 * esize)) == 0; };
  const int D = a.head_dim;
  // few tokens (decoding): the time is the launch and one round of memory latency, and the
  // one-head-per-wave kernel has the shorter chain
  const bool wide = a.num_tokens >= 32 && D >= 16 && (D & (D - 1)) == 0 && a.q_stride % 8 == 0 && a.k_stride % 8 == 0 &&
                    a.v_stride % 8 == 0 && lined_up(a.q_in) && lined_up(a.k_in) && lined_up(a.v_in) &&
                    lined_up(a.q_out) && lined_up(a.k_out) && lined_up(a.v_out) && lined_up(a.k_cache) &&
                    lined_up(a.v_cache);
  if (wide) {
    const int lph = D / 16, hp = 64 / lph, nh = a.nq + a.nkv;
    const int passes = (nh + hp - 1) / hp;
    // many tokens: a wave makes all passes of its token and computes its sines and cosines once
    const int ppw = (long)a.num_tokens * passes >= 4096 ? (passes > 0 ? passes : 1) : 1;
    const int groups = passes > 0 ? (passes + ppw - 1) / ppw : 0;
    const long rope_items = (long)a.num_tokens * groups;
    const long v_items = (long)((a.num_tokens + 7) / 8) * a.nv;
    const long rope_blocks = (rope_items + waves - 1) / waves, v_blocks = (v_items + waves - 1) / waves;
    QRT_CHECK(rope_blocks + v_blocks < (1l << 31), "qk_norm_rope_store: too many tokens");
    dim3 grid((unsigned)(rope_blocks + v_blocks)), block(64 * waves);
    const size_t smem = (size_t)waves * 8 * (D + 8) * esize;
    if (dtype == QRT_F32)
      qk_norm_rope_store_wide_kernel<float><<<grid, block, smem, stream>>>(a, lph, (int)rope_blocks, ppw);
    else if (dtype == QRT_BF16)
      qk_norm_rope_store_wide_kernel<bf16_t><<<grid, block, smem, stream>>>(a, lph, (int)rope_blocks, ppw);
    else return qrt_fail("qk_norm_rope_store: unknown dtype %d", dtype);
    QRT_LAUNCH_CHECK("qk_norm_rope_store (wide)");
    return 0;
  }
  dim3 grid((unsigned)((items + waves - 1) / waves)), block(64 * waves);
  if (dtype == QRT_F32) qk_norm_rope_store_kernel<float><<<grid, block, 0, stream>>>(a);
  else if (dtype == QRT_BF16) qk_norm_rope_store_kernel<bf16_t><<<grid, block, 0, stream>>>(a);
  else return qrt_fail("qk_norm_rope_store: unknown dtype %d", dtype);
  QRT_LAUNCH_CHECK("qk_norm_rope_store");
  return 0;
}
