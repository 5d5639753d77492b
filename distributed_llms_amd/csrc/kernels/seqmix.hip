// Kernels of layer-list models with per-sequence state (ops/seqmix.py): a float32 residual stream
// with RMS norms before and after every sublayer, short causal convolutions whose tail lives in a
// state slot, the real-gated linear recurrent unit (gates, then a chunked linear scan), the
// attention input stages (convolution + per-head norm + interleaved rotation + paged append; whole-
// projection norm + half-split rotation + paged append), embedding (+ learned positions) + norm, the close of
// pre-norm sublayers (one or two outputs, each normed apart), a token shift whose previous row lives in a state
// slot, the entry of a looped span, the averaged keys / values of blocks of positions, a clipped GLU and the
// logit soft cap.
//
// Every kernel is a template over the activation type T (bf16 or float): the float32 build is the
// exact path (true 32-bit everywhere), the bf16 build keeps in float32 what feeds a norm, a
// rotation, a gate of the recurrence or the state.  Sizes are runtime values with bounds checks,
// no divisibility assumed: widths, head sizes, taps and block counts come from the model's config.
#include <math.h>

#include "common.h"
#include "launchers.h"
#include "stream_common.h"

namespace dllm {

// --------------------------------------------------------------------------- embedding -> f32
template <typename T>
__global__ void __launch_bounds__(256) sm_embed_kernel(float* __restrict__ out, const int32_t* __restrict__ ids,
                                                       const void* __restrict__ table_, int width, int vocab) {
  const T* table = (const T*)table_;
  int id = ids[blockIdx.x];
  id = id < 0 ? 0 : (id >= vocab ? vocab - 1 : id);
  const T* src = table + (size_t)id * width;
  float* dst = out + (size_t)blockIdx.x * width;
  for (int i = threadIdx.x; i < width; i += 256) dst[i] = ldf(src + i);
}

void sm_embed_f32(uintptr_t out, uintptr_t ids, uintptr_t table, int tokens, int width, int vocab, int f32,
                  uintptr_t stream) {
  if (tokens <= 0) return;
  DLLM_HOST_CHECK(width > 0 && vocab > 0, "embed sizes");
  SM_DISPATCH(f32, sm_embed_kernel, dim3(tokens), dim3(256), 0, stream, (float*)out, (const int32_t*)ids,
              (const void*)table, width, vocab);
}

// --------------------------------------------------------------------------- embedding + RMS norm -> f32 stream
// x = e / sqrt(mean(e^2) + eps) * (offset + w) for e = table[id] * scale (+ pos_table[position], a learned
// vector per position, when given), as the float32 stream and -- when h is given -- also in the activation
// type (the input of a first sublayer that reads the stream unnormed).
template <typename T>
__global__ void __launch_bounds__(256) sm_embed_norm_kernel(float* __restrict__ x, void* __restrict__ h_,
                                                            const int32_t* __restrict__ ids,
                                                            const void* __restrict__ table_, const void* __restrict__ w_,
                                                            int width, int vocab, float eps, float offset, float scale,
                                                            const void* __restrict__ pos_table_,
                                                            const int32_t* __restrict__ positions, int max_pos) {
  __shared__ float red[16];
  const T* table = (const T*)table_;
  const T* w = (const T*)w_;
  int id = ids[blockIdx.x];
  id = id < 0 ? 0 : (id >= vocab ? vocab - 1 : id);
  const T* src = table + (size_t)id * width;
  const T* prow = nullptr;
  if (pos_table_) {
    int p = positions[blockIdx.x];
    p = p < 0 ? 0 : (p >= max_pos ? max_pos - 1 : p);
    prow = (const T*)pos_table_ + (size_t)p * width;
  }
  float ss = 0.f;
  for (int i = threadIdx.x; i < width; i += 256) {
    const float v = ldf(src + i) * scale + (prow ? ldf(prow + i) : 0.f);
    ss += v * v;
  }
  ss = block_sum(ss, red);
  const float inv = 1.0f / sqrtf(ss / (float)width + eps);
  float* dst = x + (size_t)blockIdx.x * width;
  T* h = h_ ? (T*)h_ + (size_t)blockIdx.x * width : nullptr;
  for (int i = threadIdx.x; i < width; i += 256) {
    const float e = ldf(src + i) * scale + (prow ? ldf(prow + i) : 0.f);
    const float v = e * inv * (offset + ldf(w + i));
    dst[i] = v;
    if (h) stf(h + i, v);
  }
}

void sm_embed_norm(uintptr_t x, uintptr_t h, uintptr_t ids, uintptr_t table, uintptr_t w, int tokens, int width,
                   int vocab, float eps, float offset, float scale, uintptr_t pos_table, uintptr_t positions,
                   int max_pos, int f32, uintptr_t stream) {
  if (tokens <= 0) return;
  DLLM_HOST_CHECK(width > 0 && vocab > 0 && x && w && (!pos_table || (positions && max_pos > 0)),
                  "embed_norm arguments");
  SM_DISPATCH(f32, sm_embed_norm_kernel, dim3(tokens), dim3(256), 0, stream, (float*)x, (void*)h, (const int32_t*)ids,
              (const void*)table, (const void*)w, width, vocab, eps, offset, scale, (const void*)pos_table,
              (const int32_t*)positions, max_pos);
}

// --------------------------------------------------------------------------- RMS norm of an f32 row
// y = x * rsqrt(mean(x^2) + eps) * (offset + w); one workgroup per row, V elements per lane and step.
template <typename T, int V>
__global__ void __launch_bounds__(256) sm_rms_norm_kernel(void* __restrict__ y_, const float* __restrict__ x,
                                                          const void* __restrict__ w_, int width, float eps,
                                                          float offset) {
  __shared__ float red[16];
  T* y = (T*)y_ + (size_t)blockIdx.x * width;
  const T* w = (const T*)w_;
  const float* xr = x + (size_t)blockIdx.x * width;
  float ss = 0.f;
  for (int i = threadIdx.x * V; i < width; i += 256 * V) {
    float v[V];
    ldv<V>(xr + i, v);
#pragma unroll
    for (int j = 0; j < V; ++j) ss += v[j] * v[j];
  }
  ss = block_sum(ss, red);
  const float inv = 1.0f / sqrtf(ss / (float)width + eps);
  for (int i = threadIdx.x * V; i < width; i += 256 * V) {
    float v[V], g[V];
    ldv<V>(xr + i, v);
    ldv<V>(w + i, g);
#pragma unroll
    for (int j = 0; j < V; ++j) v[j] = v[j] * inv * (offset + g[j]);
    stv<V>(y + i, v);
  }
}

void sm_rms_norm(uintptr_t y, uintptr_t x, uintptr_t w, int rows, int width, float eps, float offset, int f32,
                 uintptr_t stream) {
  if (rows <= 0) return;
  DLLM_HOST_CHECK(width > 0, "norm width");
  SM_DISPATCH_V(f32, width % 8 == 0, sm_rms_norm_kernel, dim3(rows), dim3(256), 0, stream, (void*)y, (const float*)x,
                (const void*)w, width, eps, offset);
}

// --------------------------------------------------------------------------- close of a sublayer
// x += mult * rms_norm(v) * (offset + w_post) with v = o + bias, or v = s1 o + s2 o2 when a second input is
// given (two mixers side by side);  h = rms_norm(x) * (offset + w_next) when w_next, else, when h is
// given, the new stream itself in the activation type (a following sublayer that reads x unnormed)
// (offset 1: weights stored around zero; 0: plain weights).
template <typename T, int V>
__global__ void __launch_bounds__(256) sm_post_norm_add_kernel(float* __restrict__ x, const void* __restrict__ o_,
                                                               const void* __restrict__ bias_,
                                                               const void* __restrict__ wp_,
                                                               const void* __restrict__ wn_, void* __restrict__ h_,
                                                               int width, float eps, float mult, float offset,
                                                               const void* __restrict__ o2_, float s1, float s2) {
  __shared__ float red[16];
  const T* o = (const T*)o_ + (size_t)blockIdx.x * width;
  const T* o2 = o2_ ? (const T*)o2_ + (size_t)blockIdx.x * width : nullptr;
  const T* bias = (const T*)bias_;
  const T* wp = (const T*)wp_;
  const T* wn = (const T*)wn_;
  float* xr = x + (size_t)blockIdx.x * width;
  float ss = 0.f;
  for (int i = threadIdx.x * V; i < width; i += 256 * V) {
    float v[V], bb[V];
    ldv<V>(o + i, v);
    if (o2) {
      ldv<V>(o2 + i, bb);
#pragma unroll
      for (int j = 0; j < V; ++j) v[j] = s1 * v[j] + s2 * bb[j];
    }
    if (bias) {
      ldv<V>(bias + i, bb);
#pragma unroll
      for (int j = 0; j < V; ++j) v[j] += bb[j];
    }
#pragma unroll
    for (int j = 0; j < V; ++j) ss += v[j] * v[j];
  }
  ss = block_sum(ss, red);
  const float inv = 1.0f / sqrtf(ss / (float)width + eps);
  float sq = 0.f;
  for (int i = threadIdx.x * V; i < width; i += 256 * V) {
    float v[V], bb[V], g[V], xv[V];
    ldv<V>(o + i, v);
    if (o2) {
      ldv<V>(o2 + i, bb);
#pragma unroll
      for (int j = 0; j < V; ++j) v[j] = s1 * v[j] + s2 * bb[j];
    }
    if (bias) {
      ldv<V>(bias + i, bb);
#pragma unroll
      for (int j = 0; j < V; ++j) v[j] += bb[j];
    }
    ldv<V>(wp + i, g);
    ldv<V>(xr + i, xv);
#pragma unroll
    for (int j = 0; j < V; ++j) {
      xv[j] = xv[j] + mult * (v[j] * inv * (offset + g[j]));
      sq += xv[j] * xv[j];
    }
    stv<V>(xr + i, xv);
    if (!wn && h_) stv<V>((T*)h_ + (size_t)blockIdx.x * width + i, xv);
  }
  if (!wn) return;
  sq = block_sum(sq, red);
  const float inv2 = 1.0f / sqrtf(sq / (float)width + eps);
  T* h = (T*)h_ + (size_t)blockIdx.x * width;
  for (int i = threadIdx.x * V; i < width; i += 256 * V) {      // each lane re-reads what it wrote itself
    float xv[V], g[V];
    ldv<V>(xr + i, xv);
    ldv<V>(wn + i, g);
#pragma unroll
    for (int j = 0; j < V; ++j) xv[j] = xv[j] * inv2 * (offset + g[j]);
    stv<V>(h + i, xv);
  }
}

void sm_post_norm_add(uintptr_t x, uintptr_t o, uintptr_t bias, uintptr_t w_post, uintptr_t w_next, uintptr_t h,
                      int rows, int width, float eps, float mult, float offset, uintptr_t o2, float s1, float s2,
                      int f32, uintptr_t stream) {
  if (rows <= 0) return;
  DLLM_HOST_CHECK(width > 0 && (!w_next || h), "post_norm_add arguments");
  SM_DISPATCH_V(f32, width % 8 == 0, sm_post_norm_add_kernel, dim3(rows), dim3(256), 0, stream, (float*)x,
                (const void*)o, (const void*)bias, (const void*)w_post, (const void*)w_next, (void*)h, width, eps, mult,
                offset, (const void*)o2, s1, s2);
}

// --------------------------------------------------------------------------- entry of a looped span
// x += x0 (a second float32 stream, when given) + vec (one row [width] of the activation type for every
// token, when given), in place.
template <typename T>
__global__ void __launch_bounds__(256) sm_stream_enter_kernel(float* __restrict__ x, const float* __restrict__ x0,
                                                              const void* __restrict__ vec_, long n, int width) {
  const T* vec = (const T*)vec_;
  for (long i = (long)blockIdx.x * 256 + threadIdx.x; i < n; i += (long)gridDim.x * 256) {
    float v = x[i];
    if (x0) v += x0[i];
    if (vec) v += ldf(vec + (int)(i % width));
    x[i] = v;
  }
}

void sm_stream_enter(uintptr_t x, uintptr_t x0, uintptr_t vec, int rows, int width, int f32, uintptr_t stream) {
  if (rows <= 0) return;
  DLLM_HOST_CHECK(width > 0 && x, "stream_enter arguments");
  const long n = (long)rows * width;
  const unsigned grid = (unsigned)std::min<long>((n + 255) / 256, 65535);
  SM_DISPATCH(f32, sm_stream_enter_kernel, dim3(grid), dim3(256), 0, stream, (float*)x, (const float*)x0,
              (const void*)vec, n, width);
}

// --------------------------------------------------------------------------- close of a pre-norm sublayer
// x += coef * (f(o, w1) + f(o2, w2)) with f(o, w) = o / sqrt(mean(o^2) + eps) * w when w is given and o itself
// otherwise (o2 null: one term): two mixer outputs are normed apart, each with its own plain weight, before
// they are summed.  With wn: h = x / sqrt(mean(x^2) + eps) * wn, the next sublayer's input.
template <typename T, int V>
__global__ void __launch_bounds__(256) sm_mix_add_kernel(float* __restrict__ x, const void* __restrict__ o_,
                                                         const void* __restrict__ w1_, const void* __restrict__ o2_,
                                                         const void* __restrict__ w2_, const void* __restrict__ wn_,
                                                         void* __restrict__ h_, int width, float eps, float coef) {
  __shared__ float red[16];
  const T* o = (const T*)o_ + (size_t)blockIdx.x * width;
  const T* o2 = o2_ ? (const T*)o2_ + (size_t)blockIdx.x * width : nullptr;
  const T* w1 = (const T*)w1_;
  const T* w2 = (const T*)w2_;
  const T* wn = (const T*)wn_;
  float* xr = x + (size_t)blockIdx.x * width;
  float inv1 = 1.f, inv2 = 1.f;
  if (w1 || (o2 && w2)) {
    float s1 = 0.f, s2 = 0.f;
    for (int i = threadIdx.x * V; i < width; i += 256 * V) {
      float v[V];
      if (w1) {
        ldv<V>(o + i, v);
#pragma unroll
        for (int j = 0; j < V; ++j) s1 += v[j] * v[j];
      }
      if (o2 && w2) {
        ldv<V>(o2 + i, v);
#pragma unroll
        for (int j = 0; j < V; ++j) s2 += v[j] * v[j];
      }
    }
    if (w1) inv1 = 1.0f / sqrtf(block_sum(s1, red) / (float)width + eps);
    if (o2 && w2) inv2 = 1.0f / sqrtf(block_sum(s2, red) / (float)width + eps);
  }
  float sq = 0.f;
  for (int i = threadIdx.x * V; i < width; i += 256 * V) {
    float v[V], g[V], xv[V], y[V];
    ldv<V>(o + i, v);
    if (w1) {
      ldv<V>(w1 + i, g);
#pragma unroll
      for (int j = 0; j < V; ++j) v[j] = v[j] * inv1 * g[j];
    }
#pragma unroll
    for (int j = 0; j < V; ++j) y[j] = v[j];
    if (o2) {
      ldv<V>(o2 + i, v);
      if (w2) {
        ldv<V>(w2 + i, g);
#pragma unroll
        for (int j = 0; j < V; ++j) v[j] = v[j] * inv2 * g[j];
      }
#pragma unroll
      for (int j = 0; j < V; ++j) y[j] += v[j];
    }
    ldv<V>(xr + i, xv);
#pragma unroll
    for (int j = 0; j < V; ++j) {
      xv[j] = xv[j] + coef * y[j];
      sq += xv[j] * xv[j];
    }
    stv<V>(xr + i, xv);
  }
  if (!wn) return;
  sq = block_sum(sq, red);
  const float invn = 1.0f / sqrtf(sq / (float)width + eps);
  T* h = (T*)h_ + (size_t)blockIdx.x * width;
  for (int i = threadIdx.x * V; i < width; i += 256 * V) {      // each lane re-reads what it wrote itself
    float xv[V], g[V];
    ldv<V>(xr + i, xv);
    ldv<V>(wn + i, g);
#pragma unroll
    for (int j = 0; j < V; ++j) xv[j] = xv[j] * invn * g[j];
    stv<V>(h + i, xv);
  }
}

void sm_mix_add(uintptr_t x, uintptr_t o, uintptr_t w1, uintptr_t o2, uintptr_t w2, uintptr_t w_next, uintptr_t h,
                int rows, int width, float eps, float coef, int f32, uintptr_t stream) {
  if (rows <= 0) return;
  DLLM_HOST_CHECK(width > 0 && x && o && (!w_next || h) && (!w2 || o2), "mix_add arguments");
  SM_DISPATCH_V(f32, width % 8 == 0, sm_mix_add_kernel, dim3(rows), dim3(256), 0, stream, (float*)x, (const void*)o,
                (const void*)w1, (const void*)o2, (const void*)w2, (const void*)w_next, (void*)h, width, eps, coef);
}

// --------------------------------------------------------------------------- token shift
// y_t = h_t + (h_(t-1) - h_t) * w per channel, h_(t-1) the UNBLENDED previous row of the same sequence: the
// batch row before it, for a chunk's first token the row the state slot keeps (zeros at position 0).  One
// workgroup per token; the workgroup of a chunk's FIRST token also brings the slot up to date -- it writes
// the chunk's last row there after it has read the old one, and nobody else touches that slot in the launch.
template <typename T, int V>
__global__ void __launch_bounds__(256) sm_token_shift_kernel(void* __restrict__ y_, const void* __restrict__ h_,
                                                             const void* __restrict__ w_, void* __restrict__ state_,
                                                             const int32_t* __restrict__ cu,
                                                             const int32_t* __restrict__ positions,
                                                             const int32_t* __restrict__ tok_seq,
                                                             const int32_t* __restrict__ slots, int width) {
  const int t = blockIdx.x, b = tok_seq[t];
  const int lo = cu[b], hi = cu[b + 1];
  const T* h = (const T*)h_ + (size_t)t * width;
  const T* w = (const T*)w_;
  T* y = (T*)y_ + (size_t)t * width;
  const bool first = t == lo;
  T* st = (T*)state_ + (size_t)slots[b] * width;
  const T* prev = first ? st : h - width;
  const bool zero = first && positions[t] == 0;
  const T* last = (const T*)h_ + (size_t)(hi - 1) * width;
  for (int i = threadIdx.x * V; i < width; i += 256 * V) {
    float c[V], p[V], g[V];
    ldv<V>(h + i, c);
    ldv<V>(w + i, g);
    if (zero) {
#pragma unroll
      for (int j = 0; j < V; ++j) p[j] = 0.f;
    } else {
      ldv<V>(prev + i, p);
    }
#pragma unroll
    for (int j = 0; j < V; ++j) c[j] = c[j] + (p[j] - c[j]) * g[j];
    stv<V>(y + i, c);
    if (first) {                                // same thread read st[i ..] just above
      ldv<V>(last + i, p);
      stv<V>(st + i, p);
    }
  }
}

void sm_token_shift(uintptr_t y, uintptr_t h, uintptr_t w, uintptr_t state, uintptr_t cu, uintptr_t positions,
                    uintptr_t tok_seq, uintptr_t slots, int tokens, int width, int f32, uintptr_t stream) {
  if (tokens <= 0) return;
  DLLM_HOST_CHECK(width > 0 && y && h && w && state && cu && positions && tok_seq && slots && y != h,
                  "token_shift arguments");
  const int esz = f32 ? 4 : 2;
  const bool vec = width % 8 == 0 && y % (8 * esz) == 0 && h % (8 * esz) == 0 && w % (8 * esz) == 0 && state % (8 * esz) == 0;
  SM_DISPATCH_V(f32, vec, sm_token_shift_kernel, dim3(tokens), dim3(256), 0, stream, (void*)y, (const void*)h,
                (const void*)w, (void*)state, (const int32_t*)cu, (const int32_t*)positions, (const int32_t*)tok_seq,
                (const int32_t*)slots, width);
}

// --------------------------------------------------------------------------- causal convolution with state
// (conv_input / conv_input_v, the reads of a token's earlier inputs, are in stream_common.h)
template <typename T, typename OT, int V>
__global__ void __launch_bounds__(256) sm_causal_conv_kernel(void* __restrict__ y_, const void* __restrict__ u_,
                                                             long stride, const void* __restrict__ w_,
                                                             const void* __restrict__ bias_,
                                                             const void* __restrict__ in_bias_,
                                                             const void* __restrict__ state_,
                                                             const int32_t* __restrict__ cu,
                                                             const int32_t* __restrict__ positions,
                                                             const int32_t* __restrict__ tok_seq,
                                                             const int32_t* __restrict__ slots, int C, int taps,
                                                             int act) {
  const int t = blockIdx.x;
  const int b = tok_seq[t];
  const int tl = t - cu[b], pos = positions[t];
  const T* u = (const T*)u_;
  const T* w = (const T*)w_;
  const T* st = (const T*)state_ + (size_t)slots[b] * (taps - 1) * C;
  const T* bias = (const T*)bias_;
  const T* in_bias = (const T*)in_bias_;
  OT* y = (OT*)y_ + (size_t)t * C;
  for (int c = (blockIdx.y * 256 + threadIdx.x) * V; c < C; c += gridDim.y * 256 * V) {
    float acc[V], ib[V], xv[V], wv[V];
#pragma unroll
    for (int j = 0; j < V; ++j) acc[j] = 0.f, ib[j] = 0.f;
    if (bias) ldv<V>(bias + c, acc);
    if (in_bias) ldv<V>(in_bias + c, ib);
    for (int j = 0; j < taps; ++j) {
      if (!conv_input_v<T, V>(u, stride, st, t, tl, pos, taps - 1 - j, taps, c, C, xv)) continue;
      ldv<V>(w + (size_t)j * C + c, wv);
#pragma unroll
      for (int e = 0; e < V; ++e) acc[e] += wv[e] * (xv[e] + ib[e]);
    }
    if (act == 1) {                                  // silu, in float32 with the exact exponential
#pragma unroll
      for (int e = 0; e < V; ++e) acc[e] = acc[e] / (1.0f + expf(-acc[e]));
    }
    stv<V>(y + c, acc);
  }
}

// New tail of every sequence: row j of the state becomes the input at position end - (taps - 1) + j
// (end = the chunk's last position + 1).  One thread per (sequence, V channels) walks j upwards: row j
// of the old tail is read (as row j + n, n the chunk's length) only before it is overwritten.
template <typename T, int V>
__global__ void __launch_bounds__(256) sm_conv_state_kernel(void* __restrict__ state_, const void* __restrict__ u_,
                                                            long stride, const int32_t* __restrict__ cu,
                                                            const int32_t* __restrict__ positions,
                                                            const int32_t* __restrict__ slots, int C, int taps) {
  const int b = blockIdx.x;
  const int lo = cu[b], n = cu[b + 1] - lo;
  if (n <= 0) return;
  const int start = positions[lo];
  T* st = (T*)state_ + (size_t)slots[b] * (taps - 1) * C;
  const T* u = (const T*)u_;
  for (int c = (blockIdx.y * 256 + threadIdx.x) * V; c < C; c += gridDim.y * 256 * V) {
    for (int j = 0; j < taps - 1; ++j) {
      const int tl = n - (taps - 1) + j;              // local index of the row that lands in tail row j
      float v[V];
#pragma unroll
      for (int e = 0; e < V; ++e) v[e] = 0.f;
      if (tl >= 0) ldv<V>(u + (size_t)(lo + tl) * stride + c, v);
      else if (start + tl >= 0) ldv<V>(st + (size_t)(j + n) * C + c, v);
      stv<V>(st + (size_t)j * C + c, v);
    }
  }
}

static void launch_conv_state(uintptr_t state, uintptr_t u, long stride, uintptr_t cu, uintptr_t positions,
                              uintptr_t slots, int seqs, int C, int taps, int f32, int vec, uintptr_t stream) {
  const int per = 256 * (vec ? 8 : 1);
  SM_DISPATCH_V(f32, vec, sm_conv_state_kernel, dim3(seqs, std::min(8, (C + per - 1) / per)), dim3(256), 0, stream,
                (void*)state, (const void*)u, stride, (const int32_t*)cu, (const int32_t*)positions,
                (const int32_t*)slots, C, taps);
}

// The tail update alone (a caller that ran the convolution in a kernel of its own).
void sm_conv_tail(uintptr_t state, uintptr_t u, long stride, uintptr_t cu, uintptr_t positions, uintptr_t slots, int seqs,
                  int C, int taps, int f32, uintptr_t stream) {
  if (seqs <= 0 || taps <= 1) return;
  DLLM_HOST_CHECK(C > 0 && stride >= C, "conv sizes");
  const int esz = f32 ? 4 : 2;
  launch_conv_state(state, u, stride, cu, positions, slots, seqs, C, taps, f32,
                    C % 8 == 0 && stride % 8 == 0 && (u % (8 * esz)) == 0, stream);
}

void sm_causal_conv(uintptr_t y, uintptr_t u, long stride, uintptr_t w, uintptr_t bias, uintptr_t in_bias,
                    uintptr_t state, uintptr_t cu, uintptr_t positions, uintptr_t tok_seq, uintptr_t slots,
                    int tokens, int seqs, int C, int taps, int f32, int out_f32, int act, uintptr_t stream) {
  if (tokens <= 0 || seqs <= 0) return;
  DLLM_HOST_CHECK(C > 0 && taps >= 1 && stride >= C && (act == 0 || act == 1), "conv sizes");
  const int esz = f32 ? 4 : 2;
  const int vec = C % 8 == 0 && stride % 8 == 0 && (u % (8 * esz)) == 0;
  const int per = 256 * (vec ? 8 : 1);
  const dim3 grid(tokens, std::min(8, (C + per - 1) / per));
  hipStream_t s = (hipStream_t)stream;
#define SM_CONV(T, OT, V)                                                                                    \
  hipLaunchKernelGGL(HIP_KERNEL_NAME(sm_causal_conv_kernel<T, OT, V>), grid, dim3(256), 0, s, (void*)y, (const void*)u, \
                     stride, (const void*)w, (const void*)bias, (const void*)in_bias, (const void*)state,     \
                     (const int32_t*)cu, (const int32_t*)positions, (const int32_t*)tok_seq, (const int32_t*)slots, C, taps, act)
  if (f32) { if (vec) SM_CONV(float, float, 8); else SM_CONV(float, float, 1); }
  else if (out_f32) { if (vec) SM_CONV(bf16, float, 8); else SM_CONV(bf16, float, 1); }
  else { if (vec) SM_CONV(bf16, bf16, 8); else SM_CONV(bf16, bf16, 1); }
#undef SM_CONV
  DLLM_HIP_CHECK(hipGetLastError());
  if (taps > 1) launch_conv_state(state, u, stride, cu, positions, slots, seqs, C, taps, f32, vec, stream);
}

// --------------------------------------------------------------------------- RG-LRU gates
// a = exp(-scale * sigmoid(Ra_b u_b + ra_b) * softplus(lam)),  g = sqrt(1 - a^2) * sigmoid(Ri_b u_b + ri_b) * u,
// with the transposed gate matrices [nb, in, out] (consecutive lanes on consecutive outputs).
__device__ __forceinline__ float sigmoid_f(float x) { return 1.0f / (1.0f + expf(-x)); }
__device__ __forceinline__ float softplus_f(float x) { return fmaxf(x, 0.f) + log1pf(expf(-fabsf(x))); }

// Few tokens (decode): GT tokens x one block of bw channels per workgroup on the vector ALUs; the
// token tile's u_b sits in LDS, every weight is read once per workgroup.
constexpr int GT = 4;

template <typename T>
__global__ void __launch_bounds__(256) sm_rglru_gates_small_kernel(float* __restrict__ a_out, float* __restrict__ g_out,
                                                                   const float* __restrict__ u,
                                                                   const void* __restrict__ ra_t_,
                                                                   const void* __restrict__ ra_b_,
                                                                   const void* __restrict__ ri_t_,
                                                                   const void* __restrict__ ri_b_,
                                                                   const void* __restrict__ lam_, int tokens, int nb,
                                                                   int bw, float scale) {
  extern __shared__ float ubs[];                      // [GT][bw]
  const int t0 = blockIdx.x * GT, b = blockIdx.y, C = nb * bw;
  const int nt = min(GT, tokens - t0);
  for (int i = threadIdx.x; i < GT * bw; i += 256) {
    const int k = i / bw, c = i - k * bw;
    ubs[i] = k < nt ? u[(size_t)(t0 + k) * C + b * bw + c] : 0.f;
  }
  __syncthreads();
  const T* ra = (const T*)ra_t_ + (size_t)b * bw * bw;
  const T* ri = (const T*)ri_t_ + (size_t)b * bw * bw;
  for (int o = threadIdx.x; o < bw; o += 256) {
    float ar[GT], ai[GT];
    const float br = ldf((const T*)ra_b_ + b * bw + o), bi = ldf((const T*)ri_b_ + b * bw + o);
#pragma unroll
    for (int k = 0; k < GT; ++k) ar[k] = br, ai[k] = bi;
    int i = 0;
    for (; i + 8 <= bw; i += 8) {                      // 16 weight loads in flight, then their FMAs
      float wr[8], wi[8];
#pragma unroll
      for (int j = 0; j < 8; ++j) wr[j] = ldf(ra + (size_t)(i + j) * bw + o), wi[j] = ldf(ri + (size_t)(i + j) * bw + o);
#pragma unroll
      for (int j = 0; j < 8; ++j) {
#pragma unroll
        for (int k = 0; k < GT; ++k) {
          const float x = ubs[k * bw + i + j];
          ar[k] = fmaf(wr[j], x, ar[k]);
          ai[k] = fmaf(wi[j], x, ai[k]);
        }
      }
    }
    for (; i < bw; ++i) {
      const float wr = ldf(ra + (size_t)i * bw + o), wi = ldf(ri + (size_t)i * bw + o);
#pragma unroll
      for (int k = 0; k < GT; ++k) {
        const float x = ubs[k * bw + i];
        ar[k] = fmaf(wr, x, ar[k]);
        ai[k] = fmaf(wi, x, ai[k]);
      }
    }
    const float sp = softplus_f(ldf((const T*)lam_ + b * bw + o));
#pragma unroll
    for (int k = 0; k < GT; ++k) {
      if (k < nt) {
        const float av = expf(-scale * sigmoid_f(ar[k]) * sp);
        const size_t idx = (size_t)(t0 + k) * C + b * bw + o;
        a_out[idx] = av;
        g_out[idx] = sqrtf(1.0f - av * av) * sigmoid_f(ai[k]) * ubs[k * bw + o];
      }
    }
  }
}

// The same for blocks whose width is a multiple of 8: a lane loads 8 consecutive outputs of one input
// row (16 bytes of bf16) and the workgroup's 8 lane groups take every 8th input row; their partial
// sums meet in LDS.  256 outputs of block b per workgroup.
template <typename T>
__global__ void __launch_bounds__(256) sm_rglru_gates_small_vec_kernel(
    float* __restrict__ a_out, float* __restrict__ g_out, const float* __restrict__ u, const void* __restrict__ ra_t_,
    const void* __restrict__ ra_b_, const void* __restrict__ ri_t_, const void* __restrict__ ri_b_,
    const void* __restrict__ lam_, int tokens, int nb, int bw, float scale) {
  extern __shared__ float smem[];
  float* ubs = smem;                                  // [GT][bw]
  float* red = smem + GT * bw;                        // [8 groups][GT][256]
  const int t0 = blockIdx.x * GT, b = blockIdx.y, C = nb * bw, o0 = blockIdx.z * 256;
  const int nt = min(GT, tokens - t0);
  const int tid = threadIdx.x, og = tid & 31, kg = tid >> 5;
  for (int i = tid; i < GT * bw; i += 256) {
    const int k = i / bw, c = i - k * bw;
    ubs[i] = k < nt ? u[(size_t)(t0 + k) * C + b * bw + c] : 0.f;
  }
  __syncthreads();
  const T* ra = (const T*)ra_t_ + (size_t)b * bw * bw;
  const T* ri = (const T*)ri_t_ + (size_t)b * bw * bw;
  const int ob = o0 + 8 * og;                         // this lane's 8 outputs
  float ar[GT][8], ai[GT][8];
#pragma unroll
  for (int k = 0; k < GT; ++k)
#pragma unroll
    for (int j = 0; j < 8; ++j) ar[k][j] = 0.f, ai[k][j] = 0.f;
  if (ob < bw) {
    for (int i = kg; i < bw; i += 8) {
      float wr[8], wi[8];
      ldv<8>(ra + (size_t)i * bw + ob, wr);
      ldv<8>(ri + (size_t)i * bw + ob, wi);
#pragma unroll
      for (int k = 0; k < GT; ++k) {
        const float x = ubs[k * bw + i];
#pragma unroll
        for (int j = 0; j < 8; ++j) ar[k][j] = fmaf(wr[j], x, ar[k][j]), ai[k][j] = fmaf(wi[j], x, ai[k][j]);
      }
    }
  }
  // the 8 lane groups' partial sums meet in LDS, one gate after the other (the same 32 KiB)
  float sr[GT], si[GT];
#pragma unroll
  for (int pass = 0; pass < 2; ++pass) {
    __syncthreads();
#pragma unroll
    for (int k = 0; k < GT; ++k)
#pragma unroll
      for (int j = 0; j < 8; ++j) red[(kg * GT + k) * 256 + 8 * og + j] = pass ? ai[k][j] : ar[k][j];
    __syncthreads();
#pragma unroll
    for (int k = 0; k < GT; ++k) {                    // this thread finishes (token k, output o0 + tid)
      float sum = 0.f;
#pragma unroll
      for (int g8 = 0; g8 < 8; ++g8) sum += red[(g8 * GT + k) * 256 + tid];
      if (pass) si[k] = sum; else sr[k] = sum;
    }
  }
  const int o = o0 + tid;
  if (o >= bw) return;
  const int ch = b * bw + o;
  const float sp = softplus_f(ldf((const T*)lam_ + ch));
  const float rb = ldf((const T*)ra_b_ + ch), ib = ldf((const T*)ri_b_ + ch);
#pragma unroll
  for (int k = 0; k < GT; ++k) {
    if (k < nt) {
      const float av = expf(-scale * sigmoid_f(sr[k] + rb) * sp);
      const size_t at = (size_t)(t0 + k) * C + ch;
      a_out[at] = av;
      g_out[at] = sqrtf(1.0f - av * av) * sigmoid_f(si[k] + ib) * ubs[k * bw + o];
    }
  }
}

// Many tokens (prompts): the two block-diagonal products on the float32 matrix cores
// (v_mfma_f32_32x32x2_f32: true 32-bit operands and sums, which the gates of the recurrence require).
// One workgroup per (64 tokens, block b, 128 outputs of the block): each wave owns 32 outputs and, for
// both gates, two 32 x 32 accumulators (token rows 0-31 and 32-63).  The token tile's u_b passes through
// LDS in K chunks of kGK (A operand: lane l = row l % 32, k l / 32); the gate matrices are the B operand
// from global memory, kGU k-steps of loads issued ahead of the MFMAs that use them.
constexpr int kGT = 64;       // tokens per workgroup
constexpr int kGK = 128;      // K chunk in LDS
constexpr int kGU = 8;        // k-steps (of 2) per group of loads

template <typename T>
__global__ void __launch_bounds__(256) sm_rglru_gates_kernel(float* __restrict__ a_out, float* __restrict__ g_out,
                                                             const float* __restrict__ u,
                                                             const void* __restrict__ ra_t_,
                                                             const void* __restrict__ ra_b_,
                                                             const void* __restrict__ ri_t_,
                                                             const void* __restrict__ ri_b_,
                                                             const void* __restrict__ lam_, int tokens, int nb, int bw,
                                                             float scale) {
  __shared__ float ub[kGT][kGK + 1];
  const int t0 = blockIdx.x * kGT, b = blockIdx.y, C = nb * bw;
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63, n = lane & 31, half = lane >> 5;
  const int o = blockIdx.z * 128 + wave * 32 + n;            // this lane's output channel inside block b
  const int oc = min(o, bw - 1);
  const T* ra = (const T*)ra_t_ + (size_t)b * bw * bw;
  const T* ri = (const T*)ri_t_ + (size_t)b * bw * bw;
  f32x16 cr0, ci0, cr1, ci1;
#pragma unroll
  for (int i = 0; i < 16; ++i) cr0[i] = ci0[i] = cr1[i] = ci1[i] = 0.f;
  for (int kc = 0; kc < bw; kc += kGK) {
    const int kn = min(kGK, bw - kc);
    __syncthreads();
    for (int i = tid; i < kGT * kGK; i += 256) {
      const int r = i / kGK, k = i - r * kGK;
      ub[r][k] = (t0 + r < tokens && k < kn) ? u[(size_t)(t0 + r) * C + b * bw + kc + k] : 0.f;
    }
    __syncthreads();
    // groups of kGU k-steps: the next group's weights and u values are loaded before the current
    // group's 4 kGU MFMAs issue, so their latency hides behind 64-cycle matrix instructions
    float br[2][kGU], bi[2][kGU], a0[2][kGU], a1[2][kGU];
    auto load_group = [&](int ks0, int buf) {
#pragma unroll
      for (int j = 0; j < kGU; ++j) {
        const int k = 2 * (ks0 + j) + half;                  // inside the chunk
        const bool ok = k < kn && o < bw;
        const size_t at = (size_t)(kc + min(k, kn - 1)) * bw + oc;
        const float wr = ldf(ra + at), wi = ldf(ri + at);
        br[buf][j] = ok ? wr : 0.f;
        bi[buf][j] = ok ? wi : 0.f;
        const int kk = min(k, kGK - 1);
        a0[buf][j] = k < kn ? ub[n][kk] : 0.f;
        a1[buf][j] = k < kn ? ub[32 + n][kk] : 0.f;
      }
    };
    auto mma_group = [&](int buf) {
#pragma unroll
      for (int j = 0; j < kGU; ++j) {
        cr0 = __builtin_amdgcn_mfma_f32_32x32x2f32(a0[buf][j], br[buf][j], cr0, 0, 0, 0);
        ci0 = __builtin_amdgcn_mfma_f32_32x32x2f32(a0[buf][j], bi[buf][j], ci0, 0, 0, 0);
        cr1 = __builtin_amdgcn_mfma_f32_32x32x2f32(a1[buf][j], br[buf][j], cr1, 0, 0, 0);
        ci1 = __builtin_amdgcn_mfma_f32_32x32x2f32(a1[buf][j], bi[buf][j], ci1, 0, 0, 0);
      }
    };
    load_group(0, 0);
    for (int ks0 = 0; 2 * ks0 < kn; ks0 += 2 * kGU) {
      const bool more1 = 2 * (ks0 + kGU) < kn, more2 = 2 * (ks0 + 2 * kGU) < kn;
      if (more1) load_group(ks0 + kGU, 1);
      mma_group(0);
      if (more1) {
        if (more2) load_group(ks0 + 2 * kGU, 0);
        mma_group(1);
      }
    }
  }
  if (o >= bw) return;
  const int ch = b * bw + o;
  const float rb = ldf((const T*)ra_b_ + ch), ib = ldf((const T*)ri_b_ + ch);
  const float sp = softplus_f(ldf((const T*)lam_ + ch));
#pragma unroll
  for (int hh = 0; hh < 2; ++hh) {
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      const int row = 32 * hh + 8 * (i >> 2) + 4 * half + (i & 3);    // accumulator register i of this lane
      const int t = t0 + row;
      if (t < tokens) {
        const float av = expf(-scale * sigmoid_f((hh ? cr1[i] : cr0[i]) + rb) * sp);
        const size_t idx = (size_t)t * C + ch;
        a_out[idx] = av;
        g_out[idx] = sqrtf(1.0f - av * av) * sigmoid_f((hh ? ci1[i] : ci0[i]) + ib) * u[idx];
      }
    }
  }
}

void sm_rglru_gates(uintptr_t a, uintptr_t g, uintptr_t u, uintptr_t ra_t, uintptr_t ra_b, uintptr_t ri_t,
                    uintptr_t ri_b, uintptr_t lam, int tokens, int nb, int bw, float scale, int f32,
                    uintptr_t stream) {
  if (tokens <= 0) return;
  DLLM_HOST_CHECK(nb > 0 && bw > 0 && nb <= 65535 && (bw + 127) / 128 <= 65535, "rglru gate sizes");
  const size_t lds = (size_t)GT * bw * sizeof(float);
  const size_t lds_vec = lds + (size_t)8 * GT * 256 * sizeof(float);
  if (tokens <= 64 && bw % 8 == 0 && lds_vec <= 64 * 1024) {
    SM_DISPATCH(f32, sm_rglru_gates_small_vec_kernel, dim3((tokens + GT - 1) / GT, nb, (bw + 255) / 256), dim3(256),
                lds_vec, stream, (float*)a, (float*)g, (const float*)u, (const void*)ra_t, (const void*)ra_b,
                (const void*)ri_t, (const void*)ri_b, (const void*)lam, tokens, nb, bw, scale);
    return;
  }
  if (tokens <= 64 && lds <= 48 * 1024) {
    SM_DISPATCH(f32, sm_rglru_gates_small_kernel, dim3((tokens + GT - 1) / GT, nb), dim3(256), lds, stream, (float*)a,
                (float*)g, (const float*)u, (const void*)ra_t, (const void*)ra_b, (const void*)ri_t,
                (const void*)ri_b, (const void*)lam, tokens, nb, bw, scale);
    return;
  }
  SM_DISPATCH(f32, sm_rglru_gates_kernel, dim3((tokens + kGT - 1) / kGT, nb, (bw + 127) / 128), dim3(256), 0, stream,
              (float*)a, (float*)g, (const float*)u, (const void*)ra_t, (const void*)ra_b, (const void*)ri_t,
              (const void*)ri_b, (const void*)lam, tokens, nb, bw, scale);
}

// --------------------------------------------------------------------------- RG-LRU scan
// S_t = a_t S_(t-1) + g_t per (sequence, channel), from the slot's state (zero at position 0);
// out_t = S_t * gelu_tanh(y_raw_t + y_bias).  One thread per channel walks its sequence's chunk.
__device__ __forceinline__ float gelu_tanh_f(float z) {
  return 0.5f * z * (1.0f + tanhf(0.7978845608028654f * (z + 0.044715f * z * z * z)));
}

template <typename T>
__global__ void __launch_bounds__(64) sm_rglru_scan_kernel(void* __restrict__ out_, const float* __restrict__ a,
                                                           const float* __restrict__ g,
                                                           const void* __restrict__ y_raw_, long y_stride,
                                                           const void* __restrict__ y_bias_,
                                                           float* __restrict__ state, const int32_t* __restrict__ cu,
                                                           const int32_t* __restrict__ positions,
                                                           const int32_t* __restrict__ slots, int C) {
  const int b = blockIdx.y;
  const int c = blockIdx.x * 64 + threadIdx.x;
  const int lo = cu[b], hi = cu[b + 1];
  if (c >= C || hi <= lo) return;
  const T* y_raw = (const T*)y_raw_;
  T* out = (T*)out_;
  float* sp = state + (size_t)slots[b] * C + c;
  float s = positions[lo] > 0 ? *sp : 0.f;
  const float yb = ldf((const T*)y_bias_ + c);
  // the recurrence is a dependent chain, its operands are not: 8 steps' loads go out together
  int t = lo;
  for (; t + 8 <= hi; t += 8) {
    float av[8], gv[8], yv[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const size_t i = (size_t)(t + j) * C + c;
      av[j] = a[i];
      gv[j] = g[i];
      yv[j] = ldf(y_raw + (size_t)(t + j) * y_stride + c);
    }
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      s = fmaf(av[j], s, gv[j]);
      stf(out + (size_t)(t + j) * C + c, s * gelu_tanh_f(yv[j] + yb));
    }
  }
  for (; t < hi; ++t) {
    const size_t i = (size_t)t * C + c;
    s = fmaf(a[i], s, g[i]);
    stf(out + i, s * gelu_tanh_f(ldf(y_raw + (size_t)t * y_stride + c) + yb));
  }
  *sp = s;
}

// Long chunks of few sequences: the recurrence S_t = a_t S_(t-1) + g_t is affine in S, so a chunk cut
// into segments of kSeg tokens is scanned in two launches.  The first reduces every segment to its
// composition (A = prod a_t, B = the segment scanned from zero); the second gives every (sequence,
// segment) its start state -- the slot's state folded through the earlier segments' (A, B) -- and scans
// the segment with outputs.  sequences x segments x channels / 64 waves instead of sequences x channels / 64.
constexpr int kSeg = 128;

__global__ void __launch_bounds__(64) sm_rglru_seg_reduce_kernel(float* __restrict__ ab, float* __restrict__ s0,
                                                                 const float* __restrict__ a,
                                                                 const float* __restrict__ g,
                                                                 const float* __restrict__ state,
                                                                 const int32_t* __restrict__ cu,
                                                                 const int32_t* __restrict__ positions,
                                                                 const int32_t* __restrict__ slots, int C, int nseg) {
  const int b = blockIdx.y, sg = blockIdx.z;
  const int c = blockIdx.x * 64 + threadIdx.x;
  const int lo = cu[b] + sg * kSeg, hi = min(cu[b + 1], lo + kSeg);
  if (c >= C || lo >= hi) return;
  // the sequence's state before this step, copied where the second launch reads it: that launch's last
  // segment overwrites the slot while other segments may not have started yet
  if (sg == 0) s0[(size_t)b * C + c] = positions[lo] > 0 ? state[(size_t)slots[b] * C + c] : 0.f;
  float A = 1.f, B = 0.f;
  int t = lo;
  for (; t + 8 <= hi; t += 8) {
    float av[8], gv[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) av[j] = a[(size_t)(t + j) * C + c], gv[j] = g[(size_t)(t + j) * C + c];
#pragma unroll
    for (int j = 0; j < 8; ++j) A *= av[j], B = fmaf(av[j], B, gv[j]);
  }
  for (; t < hi; ++t) {
    const float av = a[(size_t)t * C + c];
    A *= av, B = fmaf(av, B, g[(size_t)t * C + c]);
  }
  float* o = ab + (((size_t)b * nseg + sg) * 2) * C + c;
  o[0] = A;
  o[C] = B;
}

template <typename T>
__global__ void __launch_bounds__(64) sm_rglru_seg_scan_kernel(void* __restrict__ out_, const float* __restrict__ a,
                                                               const float* __restrict__ g,
                                                               const void* __restrict__ y_raw_, long y_stride,
                                                               const void* __restrict__ y_bias_,
                                                               float* __restrict__ state, const float* __restrict__ ab,
                                                               const float* __restrict__ s0,
                                                               const int32_t* __restrict__ cu,
                                                               const int32_t* __restrict__ slots, int C, int nseg) {
  const int b = blockIdx.y, sg = blockIdx.z;
  const int c = blockIdx.x * 64 + threadIdx.x;
  const int first = cu[b], end = cu[b + 1];
  const int lo = first + sg * kSeg, hi = min(end, lo + kSeg);
  if (c >= C || lo >= hi) return;
  const T* y_raw = (const T*)y_raw_;
  T* out = (T*)out_;
  float s = s0[(size_t)b * C + c];
  for (int j = 0; j < sg; ++j) {                          // the earlier segments, composed
    const float* p = ab + (((size_t)b * nseg + j) * 2) * C + c;
    s = fmaf(p[0], s, p[C]);
  }
  const float yb = ldf((const T*)y_bias_ + c);
  int t = lo;
  for (; t + 8 <= hi; t += 8) {
    float av[8], gv[8], yv[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const size_t i = (size_t)(t + j) * C + c;
      av[j] = a[i];
      gv[j] = g[i];
      yv[j] = ldf(y_raw + (size_t)(t + j) * y_stride + c);
    }
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      s = fmaf(av[j], s, gv[j]);
      stf(out + (size_t)(t + j) * C + c, s * gelu_tanh_f(yv[j] + yb));
    }
  }
  for (; t < hi; ++t) {
    const size_t i = (size_t)t * C + c;
    s = fmaf(a[i], s, g[i]);
    stf(out + i, s * gelu_tanh_f(ldf(y_raw + (size_t)t * y_stride + c) + yb));
  }
  if (hi == end) state[(size_t)slots[b] * C + c] = s;     // the sequence's last segment leaves the new state
}

// ab: workspace of seqs x (ceil(max_q_len / kSeg) x 2 + 1) x C floats (0: always the one-launch scan)
void sm_rglru_scan(uintptr_t out, uintptr_t a, uintptr_t g, uintptr_t y_raw, long y_stride, uintptr_t y_bias,
                   uintptr_t state, uintptr_t cu, uintptr_t positions, uintptr_t slots, int seqs, int C, int max_q_len,
                   uintptr_t ab, int f32, uintptr_t stream) {
  if (seqs <= 0) return;
  DLLM_HOST_CHECK(C > 0 && y_stride >= C && seqs <= 65535, "rglru scan sizes");
  const int nseg = (max_q_len + kSeg - 1) / kSeg;
  if (ab && nseg > 1 && nseg <= 65535) {
    const dim3 grid((C + 63) / 64, seqs, nseg);
    float* s0 = (float*)ab + (size_t)seqs * nseg * 2 * C;
    hipLaunchKernelGGL(sm_rglru_seg_reduce_kernel, grid, dim3(64), 0, (hipStream_t)stream, (float*)ab, s0,
                       (const float*)a, (const float*)g, (const float*)state, (const int32_t*)cu,
                       (const int32_t*)positions, (const int32_t*)slots, C, nseg);
    DLLM_HIP_CHECK(hipGetLastError());
    SM_DISPATCH(f32, sm_rglru_seg_scan_kernel, grid, dim3(64), 0, stream, (void*)out, (const float*)a, (const float*)g,
                (const void*)y_raw, y_stride, (const void*)y_bias, (float*)state, (const float*)ab, (const float*)s0,
                (const int32_t*)cu, (const int32_t*)slots, C, nseg);
    return;
  }
  SM_DISPATCH(f32, sm_rglru_scan_kernel, dim3((C + 63) / 64, seqs), dim3(64), 0, stream, (void*)out, (const float*)a,
              (const float*)g, (const void*)y_raw, y_stride, (const void*)y_bias, (float*)state, (const int32_t*)cu,
              (const int32_t*)positions, (const int32_t*)slots, C);
}

// --------------------------------------------------------------------------- clipped GLU
template <typename T, int V>
__global__ void __launch_bounds__(256) sm_clipped_glu_kernel(void* __restrict__ out_, const void* __restrict__ gu_,
                                                             const void* __restrict__ bias_, int F, float limit,
                                                             float alpha) {
  const T* gu = (const T*)gu_ + (size_t)blockIdx.x * 2 * F;
  const T* bias = (const T*)bias_;
  T* out = (T*)out_ + (size_t)blockIdx.x * F;
  for (int c = (blockIdx.y * 256 + threadIdx.x) * V; c < F; c += gridDim.y * 256 * V) {
    float gv[V], uv[V], b1[V], b2[V];
    ldv<V>(gu + c, gv);
    ldv<V>(gu + F + c, uv);
    if (bias) {
      ldv<V>(bias + c, b1);
      ldv<V>(bias + F + c, b2);
#pragma unroll
      for (int j = 0; j < V; ++j) gv[j] += b1[j], uv[j] += b2[j];
    }
#pragma unroll
    for (int j = 0; j < V; ++j) {
      const float g = fminf(gv[j], limit), u = fminf(fmaxf(uv[j], -limit), limit);
      gv[j] = g * (1.0f / (1.0f + expf(-alpha * g))) * (u + 1.0f);
    }
    stv<V>(out + c, gv);
  }
}

void sm_clipped_glu(uintptr_t out, uintptr_t gu, uintptr_t bias, int tokens, int F, float limit, float alpha, int f32,
                    uintptr_t stream) {
  if (tokens <= 0 || F <= 0) return;
  const int vec = F % 8 == 0;
  const int per = 256 * (vec ? 8 : 1);
  SM_DISPATCH_V(f32, vec, sm_clipped_glu_kernel, dim3(tokens, std::min(16, (F + per - 1) / per)), dim3(256), 0, stream,
                (void*)out, (const void*)gu, (const void*)bias, F, limit, alpha);
}

// --------------------------------------------------------------------------- logit soft cap
template <typename T>
__global__ void __launch_bounds__(256) sm_softcap_kernel(float* __restrict__ out, const void* __restrict__ x_, long n,
                                                         float cap) {
  const T* x = (const T*)x_;
  for (long i = (long)blockIdx.x * 256 + threadIdx.x; i < n; i += (long)gridDim.x * 256) {
    const float v = ldf(x + i);
    out[i] = cap > 0.f ? cap * tanhf(v / cap) : v;
  }
}

void sm_softcap(uintptr_t out, uintptr_t x, long n, float cap, int f32, uintptr_t stream) {
  if (n <= 0) return;
  const int grid = (int)std::min<long>((n + 255) / 256, 65535);
  SM_DISPATCH(f32, sm_softcap_kernel, dim3(grid), dim3(256), 0, stream, (float*)out, (const void*)x, n, cap);
}

// --------------------------------------------------------------------------- attention input stage
// One wave per (token, head) of the fused projection [q heads | k heads | v heads]: the causal
// convolution of the head's channels, then for q / k the RMS norm over the head (plain weight) and
// the rotation of pairs (2i, 2i + 1), i < nrot, by pos * freqs[i] (cos and sin scaled by mag);
// q goes to q_out [T, H, D], k / v to the paged caches [NB, G, BS, D] / [NB, G, Dv, BS] (V transposed
// inside a block).
template <typename T>
__global__ void __launch_bounds__(64) sm_attn_prep_kernel(
    void* __restrict__ q_out_, const void* __restrict__ qkv_, const void* __restrict__ conv_w_,
    const void* __restrict__ state_, const void* __restrict__ q_norm_, const void* __restrict__ k_norm_,
    const float* __restrict__ freqs, int nrot, float mag, float eps, void* __restrict__ k_cache_,
    void* __restrict__ v_cache_, const int32_t* __restrict__ slot_mapping, const int32_t* __restrict__ cu,
    const int32_t* __restrict__ positions, const int32_t* __restrict__ tok_seq, const int32_t* __restrict__ slots,
    int H, int G, int D, int Dv, int taps, int bs) {
  extern __shared__ float hv[];                      // the head's values [max(D, Dv)]
  const int t = blockIdx.x, head = blockIdx.y, lane = threadIdx.x;
  const int C = H * D + G * (D + Dv);
  const int b = tok_seq[t];
  const int tl = t - cu[b], pos = positions[t];
  const T* qkv = (const T*)qkv_;
  const T* w = (const T*)conv_w_;
  const T* st = (const T*)state_ + (size_t)slots[b] * (taps - 1) * C;
  // channel range and kind of this head
  int c0, n, kind;                                   // kind 0 q, 1 k, 2 v
  if (head < H) c0 = head * D, n = D, kind = 0;
  else if (head < H + G) c0 = H * D + (head - H) * D, n = D, kind = 1;
  else c0 = H * D + G * D + (head - H - G) * Dv, n = Dv, kind = 2;
  float ss = 0.f;
  for (int e = lane; e < n; e += 64) {
    const int c = c0 + e;
    float acc = 0.f;
    for (int j = 0; j < taps; ++j)
      acc += ldf(w + (size_t)j * C + c) * conv_input(qkv, (long)C, st, t, tl, pos, taps - 1 - j, taps, c, C);
    hv[e] = acc;
    ss += acc * acc;
  }
  T* dst;
  if (kind == 0) dst = (T*)q_out_ + ((size_t)t * H + head) * D;
  else {
    const int slot = slot_mapping[t];
    const int blk = slot / bs, off = slot - blk * bs;
    if (kind == 1) dst = (T*)k_cache_ + (((size_t)blk * G + (head - H)) * bs + off) * D;
    else dst = (T*)v_cache_ + ((size_t)blk * G + (head - H - G)) * Dv * bs + off;
  }
  if (kind == 2) {
    for (int e = lane; e < n; e += 64) stf(dst + (size_t)e * bs, hv[e]);
    return;
  }
  ss = wave_sum(ss);
  const float inv = 1.0f / sqrtf(ss / (float)n + eps);
  const T* nw = (const T*)(kind == 0 ? q_norm_ : k_norm_);
  __syncthreads();
  for (int e = lane; e < n; e += 64) hv[e] = hv[e] * inv * ldf(nw + e);
  __syncthreads();
  const float fpos = (float)pos;
  for (int i = lane; 2 * i < n; i += 64) {
    float x0 = hv[2 * i], x1 = 2 * i + 1 < n ? hv[2 * i + 1] : 0.f;
    if (i < nrot) {
      const float ang = fpos * freqs[i];
      const float cs = cosf(ang) * mag, sn = sinf(ang) * mag;
      const float r0 = x0 * cs - x1 * sn, r1 = x1 * cs + x0 * sn;
      x0 = r0, x1 = r1;
    }
    stf(dst + 2 * i, x0);
    if (2 * i + 1 < n) stf(dst + 2 * i + 1, x1);
  }
}

// The same with even head sizes: a lane owns rotation pairs (channels 2e, 2e + 1), so the convolution
// reads 2-element vectors, the rotation needs no exchange through LDS, and q / k leave as 2-element
// stores.  Heads up to 512 wide (4 pairs per lane).
constexpr int kPrepPairs = 4;

template <typename T>
__global__ void __launch_bounds__(256) sm_attn_prep_pair_kernel(
    void* __restrict__ q_out_, const void* __restrict__ qkv_, const void* __restrict__ conv_w_,
    const void* __restrict__ state_, const void* __restrict__ q_norm_, const void* __restrict__ k_norm_,
    const float* __restrict__ freqs, int nrot, float mag, float eps, void* __restrict__ k_cache_,
    void* __restrict__ v_cache_, const int32_t* __restrict__ slot_mapping, const int32_t* __restrict__ cu,
    const int32_t* __restrict__ positions, const int32_t* __restrict__ tok_seq, const int32_t* __restrict__ slots,
    int H, int G, int D, int Dv, int taps, int bs) {
  const int t = blockIdx.x, head = blockIdx.y * 4 + (threadIdx.x >> 6), lane = threadIdx.x & 63;   // a wave per head
  if (head >= H + 2 * G) return;
  const int C = H * D + G * (D + Dv);
  const int b = tok_seq[t];
  const int tl = t - cu[b], pos = positions[t];
  const T* qkv = (const T*)qkv_;
  const T* w = (const T*)conv_w_;
  const T* st = (const T*)state_ + (size_t)slots[b] * (taps - 1) * C;
  int c0, n, kind;                                   // kind 0 q, 1 k, 2 v
  if (head < H) c0 = head * D, n = D, kind = 0;
  else if (head < H + G) c0 = H * D + (head - H) * D, n = D, kind = 1;
  else c0 = H * D + G * D + (head - H - G) * Dv, n = Dv, kind = 2;
  float x[kPrepPairs][2];
  float ss = 0.f;
#pragma unroll
  for (int r = 0; r < kPrepPairs; ++r) {
    const int e = 2 * (lane + 64 * r);
    x[r][0] = x[r][1] = 0.f;
    if (e < n) {
      const int c = c0 + e;
      for (int j = 0; j < taps; ++j) {
        const int d = taps - 1 - j;
        if (d > pos) continue;
        float xv[2], wv[2];
        if (d <= tl) ldv<2>(qkv + (size_t)(t - d) * C + c, xv);
        else ldv<2>(st + (size_t)(tl - d + taps - 1) * C + c, xv);
        ldv<2>(w + (size_t)j * C + c, wv);
        x[r][0] += wv[0] * xv[0];
        x[r][1] += wv[1] * xv[1];
      }
      ss += x[r][0] * x[r][0] + x[r][1] * x[r][1];
    }
  }
  if (kind == 2) {
    const int slot = slot_mapping[t];
    const int blk = slot / bs, off = slot - blk * bs;
    T* dst = (T*)v_cache_ + ((size_t)blk * G + (head - H - G)) * Dv * bs + off;
#pragma unroll
    for (int r = 0; r < kPrepPairs; ++r) {
      const int e = 2 * (lane + 64 * r);
      if (e < n) stf(dst + (size_t)e * bs, x[r][0]), stf(dst + (size_t)(e + 1) * bs, x[r][1]);
    }
    return;
  }
  T* dst;
  if (kind == 0) dst = (T*)q_out_ + ((size_t)t * H + head) * D;
  else {
    const int slot = slot_mapping[t];
    const int blk = slot / bs, off = slot - blk * bs;
    dst = (T*)k_cache_ + (((size_t)blk * G + (head - H)) * bs + off) * D;
  }
  ss = wave_sum(ss);
  const float inv = 1.0f / sqrtf(ss / (float)n + eps);
  const T* nw = (const T*)(kind == 0 ? q_norm_ : k_norm_);
  const float fpos = (float)pos;
#pragma unroll
  for (int r = 0; r < kPrepPairs; ++r) {
    const int i = lane + 64 * r, e = 2 * i;
    if (e < n) {
      float g2[2], o[2];
      ldv<2>(nw + e, g2);
      float x0 = x[r][0] * inv * g2[0], x1 = x[r][1] * inv * g2[1];
      if (i < nrot) {
        const float ang = fpos * freqs[i];
        const float cs = cosf(ang) * mag, sn = sinf(ang) * mag;
        const float r0 = x0 * cs - x1 * sn, r1 = x1 * cs + x0 * sn;
        x0 = r0, x1 = r1;
      }
      o[0] = x0, o[1] = x1;
      stv<2>(dst + e, o);
    }
  }
}

void sm_attn_prep(uintptr_t q_out, uintptr_t qkv, uintptr_t conv_w, uintptr_t state, uintptr_t q_norm,
                  uintptr_t k_norm, uintptr_t freqs, int nrot, float mag, float eps, uintptr_t k_cache,
                  uintptr_t v_cache, uintptr_t slot_mapping, uintptr_t cu, uintptr_t positions, uintptr_t tok_seq,
                  uintptr_t slots, int tokens, int seqs, int H, int G, int D, int Dv, int taps, int bs, int f32,
                  uintptr_t stream) {
  if (tokens <= 0 || seqs <= 0) return;
  DLLM_HOST_CHECK(H > 0 && G >= 0 && D > 0 && Dv > 0 && taps >= 1 && bs > 0 && 2 * nrot <= D, "attn_prep sizes");
  DLLM_HOST_CHECK(G == 0 || (k_cache && v_cache && k_norm), "attn_prep caches");
  DLLM_HOST_CHECK(H + 2 * G <= 65535, "attn_prep heads");
  const int C = H * D + G * (D + Dv);
  const size_t lds = (size_t)std::max(D, Dv) * sizeof(float);
  if (D % 2 == 0 && Dv % 2 == 0 && std::max(D, Dv) <= 128 * kPrepPairs)
    SM_DISPATCH(f32, sm_attn_prep_pair_kernel, dim3(tokens, (H + 2 * G + 3) / 4), dim3(256), 0, stream, (void*)q_out,
                (const void*)qkv, (const void*)conv_w, (const void*)state, (const void*)q_norm, (const void*)k_norm,
                (const float*)freqs, nrot, mag, eps, (void*)k_cache, (void*)v_cache, (const int32_t*)slot_mapping,
                (const int32_t*)cu, (const int32_t*)positions, (const int32_t*)tok_seq, (const int32_t*)slots, H, G, D,
                Dv, taps, bs);
  else
  SM_DISPATCH(f32, sm_attn_prep_kernel, dim3(tokens, H + 2 * G), dim3(64), lds, stream, (void*)q_out, (const void*)qkv,
              (const void*)conv_w, (const void*)state, (const void*)q_norm, (const void*)k_norm, (const float*)freqs,
              nrot, mag, eps, (void*)k_cache, (void*)v_cache, (const int32_t*)slot_mapping, (const int32_t*)cu,
              (const int32_t*)positions, (const int32_t*)tok_seq, (const int32_t*)slots, H, G, D, Dv, taps, bs);
  // the projection's last taps - 1 rows of every sequence become its new tail
  if (taps > 1)
    launch_conv_state(state, qkv, (long)C, cu, positions, slots, seqs, C, taps, f32, C % 8 == 0, stream);
}

// --------------------------------------------------------------------------- attention input: row norm + half-split rotation + append
// From a fused projection row [.. | q (H D) | k (G D) | v (G Dv) | ..] (row stride ld, q at column `col0`):
// an RMS norm over the WHOLE q projection and over the whole k projection (all heads at once, plain
// weights qw [H D] / kw [G D]; both null: no norm), then the half-split rotation of the first 2 nrot
// dimensions of every head: dimension i < nrot is paired with dimension i + nrot, the pair turns by
// float(pos) * freqs[i] (cos and sin times `mag`).  q goes to q_out [T, H, D]; k and v (unchanged) are appended
// at slot_mapping to caches k [NB, G, BS, D] / v [NB, G, Dv, BS].  `v_from_k`: the row has no v columns and
// the values are the k columns as projected, before norm and rotation (Dv = D).
// One workgroup per token; norms, angles and the rotation are float32.
template <typename T>
__global__ void __launch_bounds__(256) sm_rownorm_rope_kernel(
    void* __restrict__ q_out_, const void* __restrict__ qkv_, long ld, int col0, const void* __restrict__ qw_,
    const void* __restrict__ kw_, const float* __restrict__ freqs, int nrot, float eps, void* __restrict__ k_cache_,
    void* __restrict__ v_cache_, const int32_t* __restrict__ slot_mapping, const int32_t* __restrict__ positions, int H,
    int G, int D, int Dv, int bs, float mag, int v_from_k) {
  __shared__ float red[16];
  extern __shared__ float csn[];                   // cos | sin of the token's nrot angles
  const int t = blockIdx.x, tid = threadIdx.x;
  const float fpos = (float)positions[t];
  for (int i = tid; i < nrot; i += 256) {
    const float ang = fpos * freqs[i];
    csn[i] = cosf(ang) * mag;
    csn[nrot + i] = sinf(ang) * mag;
  }
  const T* q = (const T*)qkv_ + (size_t)t * ld + col0;
  const T* k = q + (size_t)H * D;
  const T* v = v_from_k ? k : k + (size_t)G * D;
  const T* qw = (const T*)qw_;
  const T* kw = (const T*)kw_;
  const int nq = H * D, nk = G * D, nv = G * Dv;
  float iq = 1.f, ik = 1.f;
  if (qw) {
    float sq = 0.f, sk = 0.f;
    for (int e = tid; e < nq; e += 256) { const float x = ldf(q + e); sq += x * x; }
    for (int e = tid; e < nk; e += 256) { const float x = ldf(k + e); sk += x * x; }
    sq = block_sum(sq, red);
    sk = block_sum(sk, red);
    iq = 1.0f / sqrtf(sq / (float)nq + eps), ik = 1.0f / sqrtf(sk / (float)nk + eps);
  } else {
    __syncthreads();                               // csn is complete
  }
  const int slot = slot_mapping[t], blk = slot / bs, off = slot - blk * bs;
  T* q_out = (T*)q_out_ + (size_t)t * nq;
  T* kc = (T*)k_cache_;
  T* vc = (T*)v_cache_;
  for (int e = tid; e < nq + nk; e += 256) {
    const bool isq = e < nq;
    const int ee = isq ? e : e - nq;
    const T* src = isq ? q : k;
    const T* w = isq ? qw : kw;
    const float inv = isq ? iq : ik;
    const int hd = ee / D, d = ee - hd * D;
    float x = ldf(src + ee);
    if (w) x = x * inv * ldf(w + ee);
    if (d < 2 * nrot) {
      const int i = d < nrot ? d : d - nrot;
      const int pe = d < nrot ? ee + nrot : ee - nrot;          // the pair's other dimension
      float y = ldf(src + pe);
      if (w) y = y * inv * ldf(w + pe);
      const float cs = csn[i], sn = csn[nrot + i];
      x = d < nrot ? x * cs - y * sn : x * cs + y * sn;
    }
    if (isq) stf(q_out + ee, x);
    else stf(kc + (((size_t)blk * G + hd) * bs + off) * D + d, x);
  }
  for (int e = tid; e < nv; e += 256) {
    const int g = e / Dv, c = e - g * Dv;
    vc[(((size_t)blk * G + g) * Dv + c) * bs + off] = v[e];
  }
}

// The same with 8 consecutive dimensions per lane (16-byte loads and stores for bf16): head size, rotated
// half, row stride and first column are multiples of 8, so a lane's 8 dimensions and their 8 partners are
// one aligned piece each.
template <typename T>
__global__ void __launch_bounds__(256) sm_rownorm_rope_vec_kernel(
    void* __restrict__ q_out_, const void* __restrict__ qkv_, long ld, int col0, const void* __restrict__ qw_,
    const void* __restrict__ kw_, const float* __restrict__ freqs, int nrot, float eps, void* __restrict__ k_cache_,
    void* __restrict__ v_cache_, const int32_t* __restrict__ slot_mapping, const int32_t* __restrict__ positions, int H,
    int G, int D, int Dv, int bs, float mag, int v_from_k) {
  __shared__ float red[32];
  extern __shared__ float csn[];                   // cos | sin of the token's nrot angles
  const int t = blockIdx.x, tid = threadIdx.x, lane = tid & 63, wid = tid >> 6;
  const float fpos = (float)positions[t];
  for (int i = tid; i < nrot; i += 256) {
    const float ang = fpos * freqs[i];
    csn[i] = cosf(ang) * mag;
    csn[nrot + i] = sinf(ang) * mag;
  }
  const T* q = (const T*)qkv_ + (size_t)t * ld + col0;
  const int nq = H * D, nk = G * D, nv = G * Dv;
  const T* v = v_from_k ? q + nq : q + nq + nk;
  const bool normed = qw_ != nullptr;
  float sq = 0.f, sk = 0.f;
  if (normed) {
    for (int e = tid * 8; e < nq + nk; e += 2048) {
      float x[8];
      ldv<8>(q + e, x);
      float a = 0.f;
#pragma unroll
      for (int i = 0; i < 8; ++i) a += x[i] * x[i];
      if (e < nq) sq += a; else sk += a;
    }
    sq = wave_sum(sq);
    sk = wave_sum(sk);
    if (lane == 0) red[wid] = sq, red[4 + wid] = sk;
  }
  __syncthreads();                                 // also: csn is complete
  float iq = 1.f, ik = 1.f;
  if (normed) {
    sq = red[0] + red[1] + red[2] + red[3];
    sk = red[4] + red[5] + red[6] + red[7];
    iq = 1.0f / sqrtf(sq / (float)nq + eps), ik = 1.0f / sqrtf(sk / (float)nk + eps);
  }
  const int slot = slot_mapping[t], blk = slot / bs, off = slot - blk * bs;
  T* q_out = (T*)q_out_ + (size_t)t * nq;
  T* kc = (T*)k_cache_;
  T* vc = (T*)v_cache_;
  for (int e = tid * 8; e < nq + nk; e += 2048) {
    const bool isq = e < nq;
    const int ee = isq ? e : e - nq;
    const T* w = (isq ? (const T*)qw_ : (const T*)kw_) + ee;
    const float inv = isq ? iq : ik;
    const int hd = ee / D, d = ee - hd * D;
    float x[8], g[8];
    ldv<8>(q + e, x);
    if (normed) {
      ldv<8>(w, g);
#pragma unroll
      for (int i = 0; i < 8; ++i) x[i] *= inv * g[i];
    }
    if (d < 2 * nrot) {
      const bool first = d < nrot;
      const int po = first ? nrot : -nrot, i0 = first ? d : d - nrot;
      float y[8], gy[8];
      ldv<8>(q + e + po, y);
      if (normed) {
        ldv<8>(w + po, gy);
#pragma unroll
        for (int i = 0; i < 8; ++i) y[i] *= inv * gy[i];
      }
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        const float cs = csn[i0 + i], sn = csn[nrot + i0 + i];
        x[i] = first ? x[i] * cs - y[i] * sn : x[i] * cs + y[i] * sn;
      }
    }
    if (isq) stv<8>(q_out + ee, x);
    else stv<8>(kc + (((size_t)blk * G + hd) * bs + off) * D + d, x);
  }
  for (int e = tid; e < nv; e += 256) {
    const int g = e / Dv, c = e - g * Dv;
    vc[(((size_t)blk * G + g) * Dv + c) * bs + off] = v[e];
  }
}

void sm_rownorm_rope(uintptr_t q_out, uintptr_t qkv, long ld, int col0, uintptr_t q_norm, uintptr_t k_norm,
                     uintptr_t freqs, int nrot, float eps, uintptr_t k_cache, uintptr_t v_cache, uintptr_t slot_mapping,
                     uintptr_t positions, int tokens, int H, int G, int D, int Dv, int bs, float mag, int v_from_k,
                     int f32, uintptr_t stream) {
  if (tokens <= 0) return;
  DLLM_HOST_CHECK(H > 0 && G > 0 && D > 0 && Dv > 0 && bs > 0 && nrot >= 0 && 2 * nrot <= D && col0 >= 0 &&
                      ld >= col0 + (long)H * D + (long)G * D + (v_from_k ? 0 : (long)G * Dv) && (!v_from_k || Dv == D),
                  "rownorm_rope sizes");
  DLLM_HOST_CHECK(q_out && k_cache && v_cache && (!q_norm == !k_norm) && (nrot == 0 || freqs), "rownorm_rope arguments");
  const int esz = f32 ? 4 : 2;
  if (D % 8 == 0 && nrot % 8 == 0 && ld % 8 == 0 && col0 % 8 == 0 && qkv % (8 * esz) == 0 && q_norm % (8 * esz) == 0 &&
      k_norm % (8 * esz) == 0 && q_out % (8 * esz) == 0 && k_cache % (8 * esz) == 0) {
    SM_DISPATCH(f32, sm_rownorm_rope_vec_kernel, dim3(tokens), dim3(256), 2 * (size_t)nrot * sizeof(float), stream,
                (void*)q_out, (const void*)qkv, ld, col0, (const void*)q_norm, (const void*)k_norm, (const float*)freqs, nrot,
                eps, (void*)k_cache, (void*)v_cache, (const int32_t*)slot_mapping, (const int32_t*)positions, H, G, D, Dv, bs,
                mag, v_from_k);
    return;
  }
  SM_DISPATCH(f32, sm_rownorm_rope_kernel, dim3(tokens), dim3(256), 2 * (size_t)nrot * sizeof(float), stream, (void*)q_out, (const void*)qkv, ld, col0,
              (const void*)q_norm, (const void*)k_norm, (const float*)freqs, nrot, eps, (void*)k_cache, (void*)v_cache,
              (const int32_t*)slot_mapping, (const int32_t*)positions, H, G, D, Dv, bs, mag, v_from_k);
}

// --------------------------------------------------------------------------- averaged blocks of old keys
// For every block of `pool` positions whose LAST position p (p + 1 a multiple of pool) is a token of this
// step: the float32 mean of the block's keys and of its values AS THE CACHES HOLD THEM (k [NB, G, BS, D],
// v [NB, G, Dv, BS], read through the sequence's block table; earlier steps may have written some of them)
// goes to entry b = (p + 1) / pool - 1 of the averaged caches kp [NB, G, PB, D] / vp [NB, G, Dv, PB] (entry b
// at block b / PB of the same table, place b % PB).  One workgroup per (block that a chunk may complete, K/V
// head, sequence); V consecutive key dimensions per lane.  Runs after the step's append.
template <typename T, int V>
__global__ void __launch_bounds__(128) sm_pool_blocks_kernel(const void* __restrict__ k_cache_,
                                                             const void* __restrict__ v_cache_, void* __restrict__ kp_,
                                                             void* __restrict__ vp_,
                                                             const int32_t* __restrict__ block_tables, int max_blocks,
                                                             const int32_t* __restrict__ cu,
                                                             const int32_t* __restrict__ positions, int G, int D, int Dv,
                                                             int bs, int pb, int pool) {
  const int s = blockIdx.z, g = blockIdx.y;
  const int lo = cu[s], n = cu[s + 1] - lo;
  if (n <= 0) return;
  const int start = positions[lo], end = start + n - 1;          // positions of the chunk's tokens
  const int b = (start + pool) / pool - 1 + (int)blockIdx.x;     // first block whose last position is >= start
  if ((long)b * pool + pool - 1 > end) return;
  const int32_t* bt = block_tables + (size_t)s * max_blocks;
  const T* kc = (const T*)k_cache_;
  const T* vc = (const T*)v_cache_;
  const int pblk = bt[b / pb], poff = b % pb;
  T* kp = (T*)kp_ + (((size_t)pblk * G + g) * pb + poff) * D;
  T* vp = (T*)vp_ + ((size_t)pblk * G + g) * Dv * pb + poff;
  const float fpool = (float)pool;
  const int j0 = b * pool;
  for (int c = threadIdx.x * V; c < D; c += 128 * V) {
    float a[V];
#pragma unroll
    for (int i = 0; i < V; ++i) a[i] = 0.f;
    for (int j = j0; j < j0 + pool; ++j) {
      float x[V];
      ldv<V>(kc + (((size_t)bt[j / bs] * G + g) * bs + j % bs) * D + c, x);
#pragma unroll
      for (int i = 0; i < V; ++i) a[i] += x[i];
    }
#pragma unroll
    for (int i = 0; i < V; ++i) a[i] /= fpool;
    stv<V>(kp + c, a);
  }
  for (int c = threadIdx.x; c < Dv; c += 128) {
    float a = 0.f;
    for (int j = j0; j < j0 + pool; ++j) a += ldf(vc + (((size_t)bt[j / bs] * G + g) * Dv + c) * bs + j % bs);
    stf(vp + (size_t)c * pb, a / fpool);
  }
}

void sm_pool_blocks(uintptr_t k_cache, uintptr_t v_cache, uintptr_t kp_cache, uintptr_t vp_cache, uintptr_t block_tables,
                    int max_blocks, uintptr_t cu, uintptr_t positions, int seqs, int max_q_len, int G, int D, int Dv,
                    int bs, int pb, int pool, int f32, uintptr_t stream) {
  if (seqs <= 0 || max_q_len <= 0) return;
  DLLM_HOST_CHECK(G > 0 && G <= 65535 && seqs <= 65535 && D > 0 && Dv > 0 && bs > 0 && pb > 0 && pool > 0 &&
                      (long)pb * pool >= bs && max_blocks > 0 && k_cache && v_cache && kp_cache && vp_cache && cu && positions,
                  "pool_blocks arguments");
  const int esz = f32 ? 4 : 2;
  const bool vec = D % 8 == 0 && k_cache % (8 * esz) == 0 && kp_cache % (8 * esz) == 0;
  // a chunk of n tokens completes at most (n + pool - 1) / pool blocks
  SM_DISPATCH_V(f32, vec, sm_pool_blocks_kernel, dim3((max_q_len + pool - 1) / pool, G, seqs), dim3(128), 0, stream,
                (const void*)k_cache, (const void*)v_cache, (void*)kp_cache, (void*)vp_cache,
                (const int32_t*)block_tables, max_blocks, (const int32_t*)cu, (const int32_t*)positions, G, D, Dv, bs, pb,
                pool);
}

}  // namespace dllm
