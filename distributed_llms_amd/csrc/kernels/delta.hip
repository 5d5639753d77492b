// Gated delta rule (ops/delta.py): a linear-attention mixer whose per-head state S [dim, vdim] is a
// float32 matrix carried from token to token,
//     S <- g S;   u = beta (v - S^T k);   S <- S + k u^T;   o = S^T q
// with unit-length q and k, a write strength beta in (0, 1) and a decay g in (0, 1) per head and token.
// Everything here is float32 whatever the activation type: the inputs of the recurrence, the state and
// the read-out; only the gate, the norm weight and the result of the output norm are activations.
//
//   dr_prep_kernel      per token: q and k of every K/V head to unit length (q also times `qscale`), beta =
//                       sigmoid(b), g = exp(-exp(A_log) softplus(a + dt_bias))
//   dr_conv_prep_kernel the same behind the short convolutions + silu of q | k | v, one launch from the fused
//                       projection (what the mixer runs)
//   dr_scan_kernel      the recurrence over a varlen batch: a workgroup per (sequence, head, 64 value
//                       columns); a column's state is thread-local (split over 4 lanes along dim), so a
//                       step costs no exchange besides two 4-lane sums
//   dr_out_norm_kernel  per (token, head): o / rms(o) * w * silu(gate) (or sigmoid(gate))
#include <math.h>

#include "common.h"
#include "launchers.h"
#include "stream_common.h"

namespace dllm {

__device__ __forceinline__ float dr_sigmoid(float x) { return 1.0f / (1.0f + expf(-x)); }
__device__ __forceinline__ float dr_softplus(float x) { return fmaxf(x, 0.f) + log1pf(expf(-fabsf(x))); }

// u [T, ld] float32 holds q [G, dim] at column 0 and k [G, dim] at column G dim (normalised in place).
// ab_ [T, ldab] (activation type) holds the H write logits at column `bcol` and the H decay logits
// at `bcol + H`; bd [T, 2 H] float32 receives beta | g.
template <typename T>
__global__ void __launch_bounds__(256) dr_prep_kernel(float* __restrict__ u, long ld, const void* __restrict__ ab_,
                                                      long ldab, int bcol, const float* __restrict__ a_log,
                                                      const float* __restrict__ dt_bias, float* __restrict__ bd,
                                                      int H, int G, int dim, float qscale, float unit_eps) {
  const int t = blockIdx.x, lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  float* row = u + (size_t)t * ld;
  for (int unit = wave; unit < 2 * G; unit += 4) {          // units 0 .. G - 1: q heads, G .. 2 G - 1: k heads
    float* x = row + (size_t)unit * dim;
    float ss = 0.f;
    for (int i = lane; i < dim; i += 64) ss += x[i] * x[i];
    ss = wave_sum(ss);
    const float m = (unit < G ? qscale : 1.0f) / sqrtf(ss + unit_eps);
    for (int i = lane; i < dim; i += 64) x[i] *= m;
  }
  const T* ab = (const T*)ab_ + (size_t)t * ldab + bcol;
  for (int h = threadIdx.x; h < H; h += 256) {
    bd[(size_t)t * 2 * H + h] = dr_sigmoid(ldf(ab + h));
    bd[(size_t)t * 2 * H + H + h] = expf(-expf(a_log[h]) * dr_softplus(ldf(ab + H + h) + dt_bias[h]));
  }
}

void dr_prep(uintptr_t u, long ld, uintptr_t ab, long ldab, int bcol, uintptr_t a_log, uintptr_t dt_bias, uintptr_t bd,
             int tokens, int H, int G, int dim, float qscale, float unit_eps, int f32, uintptr_t stream) {
  if (tokens <= 0) return;
  DLLM_HOST_CHECK(H > 0 && G > 0 && H % G == 0 && dim > 0 && ld >= 2L * G * dim && ldab >= bcol + 2L * H && bcol >= 0,
                  "delta rule prep sizes");
  SM_DISPATCH(f32, dr_prep_kernel, dim3(tokens), dim3(256), 0, stream, (float*)u, ld, (const void*)ab, ldab, bcol,
              (const float*)a_log, (const float*)dt_bias, (float*)bd, H, G, dim, qscale, unit_eps);
}

// The mixer's input stage in one launch, a workgroup per token: the causal convolutions of q | k | v (columns
// col0 .. of the projection `x`, weights [taps, C] tap-major, tail in `state`, see sm_causal_conv_kernel) with
// silu, then dr_prep_kernel's work on the result -- unit q and k (held in LDS between the two phases: 2 G dim
// floats), beta and g -- into u [T, C] float32 and bd [T, 2 H].  The tail update stays a launch of its own
// (sm_conv_tail): it must see every token's rows unchanged.
template <typename T, int V>
__global__ void __launch_bounds__(256) dr_conv_prep_kernel(
    float* __restrict__ u, float* __restrict__ bd, const void* __restrict__ x_, long ld, int col0, int bcol,
    const void* __restrict__ w_, const void* __restrict__ state_, const float* __restrict__ a_log,
    const float* __restrict__ dt_bias, const int32_t* __restrict__ cu, const int32_t* __restrict__ positions,
    const int32_t* __restrict__ tok_seq, const int32_t* __restrict__ slots, int H, int G, int dim, int vdim, int taps,
    float qscale, float unit_eps) {
  extern __shared__ float qk[];                    // [2 G dim]
  const int t = blockIdx.x, tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int b = tok_seq[t];
  const int tl = t - cu[b], pos = positions[t];
  const int nqk = 2 * G * dim, C = nqk + H * vdim;
  const T* x = (const T*)x_ + col0;
  const T* w = (const T*)w_;
  const T* st = (const T*)state_ + (size_t)slots[b] * (taps - 1) * C;
  float* row = u + (size_t)t * C;
  for (int c = tid * V; c < C; c += 256 * V) {
    float acc[V], xv[V], wv[V];
#pragma unroll
    for (int e = 0; e < V; ++e) acc[e] = 0.f;
    for (int j = 0; j < taps; ++j) {
      if (!conv_input_v<T, V>(x, ld, st, t, tl, pos, taps - 1 - j, taps, c, C, xv)) continue;
      ldv<V>(w + (size_t)j * C + c, wv);
#pragma unroll
      for (int e = 0; e < V; ++e) acc[e] += wv[e] * xv[e];
    }
#pragma unroll
    for (int e = 0; e < V; ++e) acc[e] = acc[e] / (1.0f + expf(-acc[e]));
    if (c < nqk) stv<V>(qk + c, acc);              // V divides dim: a piece lies in one part
    else stv<V>(row + c, acc);
  }
  __syncthreads();
  const int lpu = dim >> 3;                                 // lanes per unit when a lane takes 8 dimensions
  if (V == 8 && lpu <= 64 && (lpu & (lpu - 1)) == 0) {
    // units 0 .. G - 1: q heads, G .. 2 G - 1: k heads; 256 / lpu units per pass, each on an aligned lane group
    for (int p0 = 0; p0 < nqk; p0 += 2048) {
      const int c = p0 + tid * 8;
      const bool ok = c < nqk;
      float xv[8];
#pragma unroll
      for (int e = 0; e < 8; ++e) xv[e] = 0.f;
      if (ok) ldv<8>(qk + c, xv);
      float ss = 0.f;
#pragma unroll
      for (int e = 0; e < 8; ++e) ss += xv[e] * xv[e];
      for (int m = lpu >> 1; m > 0; m >>= 1) ss += __shfl_xor(ss, m, 64);
      const float m = (c < G * dim ? qscale : 1.0f) / sqrtf(ss + unit_eps);
#pragma unroll
      for (int e = 0; e < 8; ++e) xv[e] *= m;
      if (ok) stv<8>(row + c, xv);
    }
  } else {
    for (int unit = wave; unit < 2 * G; unit += 4) {
      const float* xq = qk + (size_t)unit * dim;
      float ss = 0.f;
      for (int i = lane; i < dim; i += 64) ss += xq[i] * xq[i];
      ss = wave_sum(ss);
      const float m = (unit < G ? qscale : 1.0f) / sqrtf(ss + unit_eps);
      for (int i = lane; i < dim; i += 64) row[(size_t)unit * dim + i] = xq[i] * m;
    }
  }
  const T* ab = (const T*)x_ + (size_t)t * ld + bcol;
  for (int h = tid; h < H; h += 256) {
    bd[(size_t)t * 2 * H + h] = dr_sigmoid(ldf(ab + h));
    bd[(size_t)t * 2 * H + H + h] = expf(-expf(a_log[h]) * dr_softplus(ldf(ab + H + h) + dt_bias[h]));
  }
}

void dr_conv_prep(uintptr_t u, uintptr_t bd, uintptr_t x, long ld, int col0, int bcol, uintptr_t w, uintptr_t state,
                  uintptr_t a_log, uintptr_t dt_bias, uintptr_t cu, uintptr_t positions, uintptr_t tok_seq, uintptr_t slots,
                  int tokens, int H, int G, int dim, int vdim, int taps, float qscale, float unit_eps, int f32,
                  uintptr_t stream) {
  if (tokens <= 0) return;
  const long C = 2L * G * dim + (long)H * vdim;
  DLLM_HOST_CHECK(H > 0 && G > 0 && H % G == 0 && dim > 0 && vdim > 0 && taps >= 1 && col0 >= 0 && bcol >= 0 &&
                      ld >= col0 + C && ld >= bcol + 2L * H,
                  "delta rule input stage sizes");
  const size_t lds = sizeof(float) * 2 * (size_t)G * dim;
  DLLM_HOST_CHECK(lds <= 48 * 1024, "delta rule input stage: q | k too wide for LDS");
  const int esz = f32 ? 4 : 2;
  const int vec = dim % 8 == 0 && vdim % 8 == 0 && ld % 8 == 0 && col0 % 8 == 0 && (x % (8 * esz)) == 0 &&
                  (w % (8 * esz)) == 0 && (state % (8 * esz)) == 0;
  SM_DISPATCH_V(f32, vec, dr_conv_prep_kernel, dim3(tokens), dim3(256), lds, stream, (float*)u, (float*)bd,
                (const void*)x, ld, col0, bcol, (const void*)w, (const void*)state, (const float*)a_log,
                (const float*)dt_bias, (const int32_t*)cu, (const int32_t*)positions, (const int32_t*)tok_seq,
                (const int32_t*)slots, H, G, dim, vdim, taps, qscale, unit_eps);
}

// The recurrence.  Lane (part = lane / 16, jj = lane % 16) of wave w owns rows [part DK/4, (part + 1) DK/4) of
// value column j = 64 z + 16 w + jj of the state of head h: S^T k and S^T q are DK/4 FMAs and a sum over the
// four parts.  k and q (zero-padded to DK) and the gates of kDrTB tokens are staged in LDS for the
// workgroup's NT / 64 waves (fewer waves and value columns per workgroup when few sequences and heads would
// leave CUs idle: the chain of a token's steps, not the arithmetic, bounds a lone wave); the next block's global loads are issued before the current block's steps and
// land in LDS after them.  A chunk that starts at position 0 starts from a zero state; the state goes back
// to its slot after the chunk's last token.
constexpr int kDrTB = 8;

template <int DK, int CPL, int NT>
__global__ void __launch_bounds__(NT) dr_scan_kernel(float* __restrict__ o, const float* __restrict__ u, long ld,
                                                      const float* __restrict__ bd, float* __restrict__ state, const int32_t* __restrict__ cu,
                                                      const int32_t* __restrict__ positions,
                                                      const int32_t* __restrict__ slots, int H, int G, int dim,
                                                      int vdim) {
  constexpr int R = DK / 4;
  constexpr int NST = kDrTB * 2 * DK / NT;                    // staged k / q elements per thread and block
  constexpr int NW = NT / 64;                                 // waves: 16 NW CPL value columns per workgroup
  __shared__ __attribute__((aligned(16))) float kq[kDrTB][2][DK];
  __shared__ float gates[kDrTB][2];
  const int b = blockIdx.x, h = blockIdx.y;
  const int lo = cu[b], n = cu[b + 1] - lo;
  if (n <= 0) return;
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63, part = lane >> 4, jj = lane & 15;
  // CPL value columns per lane, 64 apart: every k / q element a lane reads from LDS feeds CPL columns (the
  // LDS reads, not the FMAs, bound the CPL = 1 form on long chunks)
  int j[CPL];
  bool jok[CPL];
#pragma unroll
  for (int c = 0; c < CPL; ++c) {
    j[c] = (blockIdx.z * CPL + c) * (16 * NW) + wave * 16 + jj;
    jok[c] = j[c] < vdim;
  }
  const int g = h / (H / G);
  const size_t kcol = (size_t)G * dim + (size_t)g * dim, qcol = (size_t)g * dim, vcol = 2 * (size_t)G * dim + (size_t)h * vdim;
  float* S = state + ((size_t)slots[b] * H + h) * dim * vdim;
  const bool fresh = positions[lo] == 0;
  float s[CPL][R];
#pragma unroll
  for (int c = 0; c < CPL; ++c)
#pragma unroll
    for (int r = 0; r < R; ++r) {
      const int i = part * R + r;
      s[c][r] = (!fresh && jok[c] && i < dim) ? S[(size_t)i * vdim + j[c]] : 0.f;
    }
  float st[NST], vn[CPL][kDrTB], gn = 0.f;
  auto fetch = [&](int t0) {                                  // global loads of the block that starts at t0
    const int nt = min(kDrTB, n - t0);
#pragma unroll
    for (int r = 0; r < NST; ++r) {
      const int idx = tid + NT * r;
      const int tt = idx / (2 * DK), rem = idx - tt * 2 * DK, which = rem / DK, i = rem - which * DK;
      st[r] = (tt < nt && i < dim) ? u[(size_t)(lo + t0 + tt) * ld + (which ? qcol : kcol) + i] : 0.f;
    }
#pragma unroll
    for (int c = 0; c < CPL; ++c)
#pragma unroll
      for (int tt = 0; tt < kDrTB; ++tt)
        vn[c][tt] = (tt < nt && jok[c]) ? u[(size_t)(lo + t0 + tt) * ld + vcol + j[c]] : 0.f;
    if (tid < nt * 2) {
      const int tt = tid >> 1, w = tid & 1;
      gn = bd[(size_t)(lo + t0 + tt) * 2 * H + w * H + h];
    }
  };
  fetch(0);
  for (int t0 = 0; t0 < n; t0 += kDrTB) {
    const int nt = min(kDrTB, n - t0);
    __syncthreads();                                          // the previous block's reads are done
#pragma unroll
    for (int r = 0; r < NST; ++r) {
      const int idx = tid + NT * r;
      (&kq[0][0][0])[idx] = st[r];
    }
    if (tid < nt * 2) gates[tid >> 1][tid & 1] = gn;
    float vv[CPL][kDrTB];
#pragma unroll
    for (int c = 0; c < CPL; ++c)
#pragma unroll
      for (int tt = 0; tt < kDrTB; ++tt) vv[c][tt] = vn[c][tt];
    __syncthreads();
    if (t0 + kDrTB < n) fetch(t0 + kDrTB);
#pragma unroll
    for (int tt = 0; tt < kDrTB; ++tt) {
      if (tt < nt) {
        const float* kk = &kq[tt][0][part * R];
        const float* qq = &kq[tt][1][part * R];
        const float beta = gates[tt][0], dec = gates[tt][1];
        float a4[CPL][4], o4[CPL][4], uj[CPL];
#pragma unroll
        for (int c = 0; c < CPL; ++c)
#pragma unroll
          for (int e = 0; e < 4; ++e) a4[c][e] = o4[c][e] = 0.f;
#pragma unroll
        for (int r = 0; r < R; ++r) {
          const float kr = kk[r];
#pragma unroll
          for (int c = 0; c < CPL; ++c) {
            s[c][r] *= dec;
            a4[c][r & 3] = fmaf(s[c][r], kr, a4[c][r & 3]);
          }
        }
#pragma unroll
        for (int c = 0; c < CPL; ++c)
          uj[c] = beta * (vv[c][tt] - rows_sum((a4[c][0] + a4[c][1]) + (a4[c][2] + a4[c][3])));
#pragma unroll
        for (int r = 0; r < R; ++r) {
          const float kr = kk[r], qr = qq[r];
#pragma unroll
          for (int c = 0; c < CPL; ++c) {
            s[c][r] = fmaf(kr, uj[c], s[c][r]);
            o4[c][r & 3] = fmaf(s[c][r], qr, o4[c][r & 3]);
          }
        }
#pragma unroll
        for (int c = 0; c < CPL; ++c) {
          const float oo = rows_sum((o4[c][0] + o4[c][1]) + (o4[c][2] + o4[c][3]));
          if (part == 0 && jok[c]) o[((size_t)(lo + t0 + tt) * H + h) * vdim + j[c]] = oo;
        }
      }
    }
  }
#pragma unroll
  for (int c = 0; c < CPL; ++c)
#pragma unroll
    for (int r = 0; r < R; ++r) {
      const int i = part * R + r;
      if (jok[c] && i < dim) S[(size_t)i * vdim + j[c]] = s[c][r];
    }
}

// u [T, ld] float32: unit q | unit k | v; bd [T, 2 H]: beta | g.
void dr_scan(uintptr_t o, uintptr_t u, long ld, uintptr_t bd, uintptr_t state, uintptr_t cu, uintptr_t positions,
             uintptr_t slots, int seqs, int max_q_len, int H, int G, int dim, int vdim, uintptr_t stream) {
  if (seqs <= 0) return;
  DLLM_HOST_CHECK(H > 0 && G > 0 && H % G == 0 && dim > 0 && dim <= 256 && vdim > 0 && H <= 65535 &&
                      ld >= 2L * G * dim + (long)H * vdim,
                  "delta rule sizes (key size up to 256)");
  // long chunks with keys up to 128 wide: two value columns per lane (half the LDS reads per FMA, 2 DK / 4 state
  // registers); one-token rows and short portions: one column, twice the workgroups; and while the grid
  // leaves CUs idle, fewer waves (value columns) per workgroup
  int cpl = (max_q_len > 16 && vdim > 64 && dim <= 128) ? 2 : 1;
  if ((long)seqs * H * ((vdim + 127) / 128) < 256) cpl = 1;
  int nt = 256;
  while (nt > 64 && vdim > nt / 8 && (long)seqs * H * ((vdim + nt / 4 - 1) / (nt / 4)) < 512) nt /= 2;
  const int cols = cpl * nt / 4;
  const dim3 grid(seqs, H, (vdim + cols - 1) / cols);
  hipStream_t s = (hipStream_t)stream;
#define DR_ARGS                                                                                                   \
  (float*)o, (const float*)u, ld, (const float*)bd, (float*)state, (const int32_t*)cu, (const int32_t*)positions, \
      (const int32_t*)slots, H, G, dim, vdim
#define DR_SCAN(DK)                                                                                               \
  do {                                                                                                            \
    if (cpl == 2)                                                                                                 \
      hipLaunchKernelGGL(HIP_KERNEL_NAME(dr_scan_kernel<(DK <= 128 ? DK : 128), 2, 256>), grid, dim3(256), 0, s, DR_ARGS); \
    else if (nt == 256)                                                                                           \
      hipLaunchKernelGGL(HIP_KERNEL_NAME(dr_scan_kernel<DK, 1, 256>), grid, dim3(256), 0, s, DR_ARGS);           \
    else if (nt == 128)                                                                                           \
      hipLaunchKernelGGL(HIP_KERNEL_NAME(dr_scan_kernel<DK, 1, 128>), grid, dim3(128), 0, s, DR_ARGS);           \
    else                                                                                                          \
      hipLaunchKernelGGL(HIP_KERNEL_NAME(dr_scan_kernel<DK, 1, 64>), grid, dim3(64), 0, s, DR_ARGS);             \
  } while (0)
  if (dim <= 32) DR_SCAN(32);
  else if (dim <= 64) DR_SCAN(64);
  else if (dim <= 128) DR_SCAN(128);
  else DR_SCAN(256);
#undef DR_SCAN
#undef DR_ARGS
  DLLM_HIP_CHECK(hipGetLastError());
}

// y[t, h, :] = o / sqrt(mean(o^2) + eps) * w * silu(gate[t, gcol + h vdim + :]) * out_scale in the
// activation type; o [T, H, vdim] float32, w [vdim] shared by the heads, y rows `ldy` apart.
template <typename T>
__global__ void __launch_bounds__(64) dr_out_norm_kernel(void* __restrict__ y_, long ldy, const float* __restrict__ o,
                                                         const void* __restrict__ gate_, long ldg, int gcol,
                                                         const void* __restrict__ w_, int H, int vdim, float eps,
                                                         float out_scale, int gate_sig) {
  const int t = blockIdx.x, h = blockIdx.y, lane = threadIdx.x;
  const float* row = o + ((size_t)t * H + h) * vdim;
  const T* gate = (const T*)gate_ + (size_t)t * ldg + gcol + (size_t)h * vdim;
  const T* w = (const T*)w_;
  T* y = (T*)y_ + (size_t)t * ldy + (size_t)h * vdim;
  float ss = 0.f;
  for (int e = lane; e < vdim; e += 64) ss += row[e] * row[e];
  ss = wave_sum(ss);
  const float inv = out_scale / sqrtf(ss / (float)vdim + eps);
  for (int e = lane; e < vdim; e += 64) {
    const float z = ldf(gate + e);
    stf(y + e, row[e] * inv * ldf(w + e) * (gate_sig ? dr_sigmoid(z) : z * dr_sigmoid(z)));
  }
}

// The same with 8 channels per lane, vdim / 8 (a power of two) lanes per (token, head) on an aligned lane group.
template <typename T>
__global__ void __launch_bounds__(256) dr_out_norm_vec_kernel(void* __restrict__ y_, long ldy, const float* __restrict__ o,
                                                             const void* __restrict__ gate_, long ldg, int gcol,
                                                             const void* __restrict__ w_, long heads_total, int H,
                                                             int vdim, float eps, float out_scale, int gate_sig) {
  const int lph = vdim >> 3;
  const long idx = (long)blockIdx.x * 256 + threadIdx.x;
  const long th = idx / lph;
  const int c = (int)(idx - th * lph) * 8;
  const bool ok = th < heads_total;
  const long thc = ok ? th : heads_total - 1;
  const long t = thc / H;
  const int h = (int)(thc - t * H);
  float xv[8], gv[8], wv[8];
  ldv<8>(o + (size_t)thc * vdim + c, xv);
  float ss = 0.f;
#pragma unroll
  for (int e = 0; e < 8; ++e) ss += xv[e] * xv[e];
  for (int m = lph >> 1; m > 0; m >>= 1) ss += __shfl_xor(ss, m, 64);
  const float inv = out_scale / sqrtf(ss / (float)vdim + eps);
  ldv<8>((const T*)gate_ + (size_t)t * ldg + gcol + (size_t)h * vdim + c, gv);
  ldv<8>((const T*)w_ + c, wv);
#pragma unroll
  for (int e = 0; e < 8; ++e) xv[e] = xv[e] * inv * wv[e] * (gate_sig ? dr_sigmoid(gv[e]) : gv[e] * dr_sigmoid(gv[e]));
  if (ok) stv<8>((T*)y_ + (size_t)t * ldy + (size_t)h * vdim + c, xv);
}

// The same for groups wider than 512 channels (one norm over many heads at once): a workgroup per (token, group),
// 8 channels per lane and step.
template <typename T>
__global__ void __launch_bounds__(256) dr_out_norm_wide_kernel(void* __restrict__ y_, long ldy, const float* __restrict__ o,
                                                              const void* __restrict__ gate_, long ldg, int gcol,
                                                              const void* __restrict__ w_, int H, int vdim, float eps,
                                                              float out_scale, int gate_sig) {
  __shared__ float red[16];
  const int t = blockIdx.x, h = blockIdx.y;
  const float* row = o + ((size_t)t * H + h) * vdim;
  const T* gate = (const T*)gate_ + (size_t)t * ldg + gcol + (size_t)h * vdim;
  const T* w = (const T*)w_;
  T* y = (T*)y_ + (size_t)t * ldy + (size_t)h * vdim;
  float ss = 0.f;
  for (int e = threadIdx.x * 8; e < vdim; e += 2048) {
    float xv[8];
    ldv<8>(row + e, xv);
#pragma unroll
    for (int i = 0; i < 8; ++i) ss += xv[i] * xv[i];
  }
  ss = block_sum(ss, red);
  const float inv = out_scale / sqrtf(ss / (float)vdim + eps);
  for (int e = threadIdx.x * 8; e < vdim; e += 2048) {
    float xv[8], gv[8], wv[8];
    ldv<8>(row + e, xv);
    ldv<8>(gate + e, gv);
    ldv<8>(w + e, wv);
#pragma unroll
    for (int i = 0; i < 8; ++i) xv[i] = xv[i] * inv * wv[i] * (gate_sig ? dr_sigmoid(gv[i]) : gv[i] * dr_sigmoid(gv[i]));
    stv<8>(y + e, xv);
  }
}

void dr_out_norm(uintptr_t y, long ldy, uintptr_t o, uintptr_t gate, long ldg, int gcol, uintptr_t w, int tokens, int H,
                 int vdim, float eps, float out_scale, int gate_sig, int f32, uintptr_t stream) {
  if (tokens <= 0) return;
  DLLM_HOST_CHECK(H > 0 && H <= 65535 && vdim > 0 && ldy >= (long)H * vdim && ldg >= gcol + (long)H * vdim && gcol >= 0,
                  "delta rule output norm sizes");
  const int esz = f32 ? 4 : 2, lph = vdim >> 3;
  if (vdim % 8 == 0 && vdim > 512 && ldy % 8 == 0 && ldg % 8 == 0 && gcol % 8 == 0 && y % (8 * esz) == 0 &&
      gate % (8 * esz) == 0 && w % (8 * esz) == 0 && o % 32 == 0) {
    SM_DISPATCH(f32, dr_out_norm_wide_kernel, dim3(tokens, H), dim3(256), 0, stream, (void*)y, ldy, (const float*)o,
                (const void*)gate, ldg, gcol, (const void*)w, H, vdim, eps, out_scale, gate_sig);
    return;
  }
  if (vdim % 8 == 0 && lph <= 64 && (lph & (lph - 1)) == 0 && ldy % 8 == 0 && ldg % 8 == 0 && gcol % 8 == 0 &&
      y % (8 * esz) == 0 && gate % (8 * esz) == 0 && w % (8 * esz) == 0 && o % 32 == 0) {
    const long heads_total = (long)tokens * H, lanes = heads_total * lph;
    DLLM_HOST_CHECK((lanes + 255) / 256 < (1L << 31), "delta rule output norm grid");
    SM_DISPATCH(f32, dr_out_norm_vec_kernel, dim3((unsigned)((lanes + 255) / 256)), dim3(256), 0, stream, (void*)y, ldy,
                (const float*)o, (const void*)gate, ldg, gcol, (const void*)w, heads_total, H, vdim, eps, out_scale, gate_sig);
    return;
  }
  SM_DISPATCH(f32, dr_out_norm_kernel, dim3(tokens, H), dim3(64), 0, stream, (void*)y, ldy, (const float*)o,
              (const void*)gate, ldg, gcol, (const void*)w, H, vdim, eps, out_scale, gate_sig);
}

}  // namespace dllm
