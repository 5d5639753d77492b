// Gated delta rule (ops/delta.py): a linear-attention mixer whose per-head state S [dim, vdim] is a
// float32 matrix carried from token to token,
//     S <- g S;   u = beta (v - S^T k);   S <- S + k u^T;   o = S^T q
// with unit-length q and k, a write strength beta in (0, 1) and a decay g in (0, 1) per head and token.
// Everything here is float32 whatever the activation type: the inputs of the recurrence, the state and
// the read-out; only the gate, the norm weight and the result of the output norm are activations.
//
//   dr_prep_kernel      per token: q and k of every K/V head to unit length (q also times `qscale`), beta =
//                       sigmoid(b), g = exp(-exp(A_log) softplus(a + dt_bias))
//   dr_scan_kernel      the recurrence over a varlen batch: a workgroup per (sequence, head, 64 value
//                       columns); a column's state is thread-local (split over 4 lanes along dim), so a
//                       step costs no exchange besides two 4-lane sums
//   dr_out_norm_kernel  per (token, head): o / rms(o) * w * silu(gate)
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

// The recurrence.  Lane (part = lane / 16, jj = lane % 16) of wave w owns rows [part DK/4, (part + 1) DK/4) of
// value column j = 64 z + 16 w + jj of the state of head h: S^T k and S^T q are DK/4 FMAs and a sum over the
// four parts.  k and q (zero-padded to DK) and the gates of kDrTB tokens are staged in LDS for the
// workgroup's four waves.  A chunk that starts at position 0 starts from a zero state; the state goes
// back to its slot after the chunk's last token.
constexpr int kDrTB = 8;

template <int DK>
__global__ void __launch_bounds__(256) dr_scan_kernel(float* __restrict__ o, const float* __restrict__ u, long ld,
                                                      const float* __restrict__ bd, float* __restrict__ state,
                                                      const int32_t* __restrict__ cu,
                                                      const int32_t* __restrict__ positions,
                                                      const int32_t* __restrict__ slots, int H, int G, int dim,
                                                      int vdim) {
  constexpr int R = DK / 4;
  __shared__ __attribute__((aligned(16))) float kq[kDrTB][2][DK];
  __shared__ float gates[kDrTB][2];
  const int b = blockIdx.x, h = blockIdx.y;
  const int lo = cu[b], n = cu[b + 1] - lo;
  if (n <= 0) return;
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63, part = lane >> 4, jj = lane & 15;
  const int j = blockIdx.z * 64 + wave * 16 + jj;
  const bool jok = j < vdim;
  const int g = h / (H / G);
  const size_t kcol = (size_t)G * dim + (size_t)g * dim, qcol = (size_t)g * dim, vcol = 2 * (size_t)G * dim + (size_t)h * vdim;
  float* S = state + ((size_t)slots[b] * H + h) * dim * vdim;
  const bool fresh = positions[lo] == 0;
  float s[R];
#pragma unroll
  for (int r = 0; r < R; ++r) {
    const int i = part * R + r;
    s[r] = (!fresh && jok && i < dim) ? S[(size_t)i * vdim + j] : 0.f;
  }
  for (int t0 = 0; t0 < n; t0 += kDrTB) {
    const int nt = min(kDrTB, n - t0);
    __syncthreads();                                          // the previous block's reads are done
    for (int idx = tid; idx < nt * 2 * DK; idx += 256) {
      const int tt = idx / (2 * DK), rem = idx - tt * 2 * DK, which = rem / DK, i = rem - which * DK;
      const float* row = u + (size_t)(lo + t0 + tt) * ld;
      kq[tt][which][i] = i < dim ? row[(which ? qcol : kcol) + i] : 0.f;
    }
    if (tid < nt * 2) gates[tid >> 1][tid & 1] = bd[(size_t)(lo + t0 + (tid >> 1)) * 2 * H + (tid & 1) * H + h];
    float vv[kDrTB];
#pragma unroll
    for (int tt = 0; tt < kDrTB; ++tt) vv[tt] = (tt < nt && jok) ? u[(size_t)(lo + t0 + tt) * ld + vcol + j] : 0.f;
    __syncthreads();
#pragma unroll
    for (int tt = 0; tt < kDrTB; ++tt) {
      if (tt < nt) {
        const float* kk = &kq[tt][0][part * R];
        const float* qq = &kq[tt][1][part * R];
        const float beta = gates[tt][0], dec = gates[tt][1];
        float acc = 0.f;
#pragma unroll
        for (int r = 0; r < R; ++r) {
          s[r] *= dec;
          acc = fmaf(s[r], kk[r], acc);
        }
        acc = rows_sum(acc);
        const float uj = beta * (vv[tt] - acc);
        float oo = 0.f;
#pragma unroll
        for (int r = 0; r < R; ++r) {
          s[r] = fmaf(kk[r], uj, s[r]);
          oo = fmaf(s[r], qq[r], oo);
        }
        oo = rows_sum(oo);
        if (part == 0 && jok) o[((size_t)(lo + t0 + tt) * H + h) * vdim + j] = oo;
      }
    }
  }
#pragma unroll
  for (int r = 0; r < R; ++r) {
    const int i = part * R + r;
    if (jok && i < dim) S[(size_t)i * vdim + j] = s[r];
  }
}

void dr_scan(uintptr_t o, uintptr_t u, long ld, uintptr_t bd, uintptr_t state, uintptr_t cu, uintptr_t positions,
             uintptr_t slots, int seqs, int H, int G, int dim, int vdim, uintptr_t stream) {
  if (seqs <= 0) return;
  DLLM_HOST_CHECK(H > 0 && G > 0 && H % G == 0 && dim > 0 && dim <= 256 && vdim > 0 && H <= 65535 &&
                      ld >= 2L * G * dim + (long)H * vdim,
                  "delta rule sizes (key size up to 256)");
  const dim3 grid(seqs, H, (vdim + 63) / 64);
  hipStream_t s = (hipStream_t)stream;
#define DR_SCAN(DK)                                                                                              \
  hipLaunchKernelGGL(HIP_KERNEL_NAME(dr_scan_kernel<DK>), grid, dim3(256), 0, s, (float*)o, (const float*)u, ld, \
                     (const float*)bd, (float*)state, (const int32_t*)cu, (const int32_t*)positions,             \
                     (const int32_t*)slots, H, G, dim, vdim)
  if (dim <= 32) DR_SCAN(32);
  else if (dim <= 64) DR_SCAN(64);
  else if (dim <= 128) DR_SCAN(128);
  else DR_SCAN(256);
#undef DR_SCAN
  DLLM_HIP_CHECK(hipGetLastError());
}

// y[t, h, :] = o / sqrt(mean(o^2) + eps) * w * silu(gate[t, gcol + h vdim + :]) * out_scale in the
// activation type; o [T, H, vdim] float32, w [vdim] shared by the heads, y rows `ldy` apart.
template <typename T>
__global__ void __launch_bounds__(64) dr_out_norm_kernel(void* __restrict__ y_, long ldy, const float* __restrict__ o,
                                                         const void* __restrict__ gate_, long ldg, int gcol,
                                                         const void* __restrict__ w_, int H, int vdim, float eps,
                                                         float out_scale) {
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
    stf(y + e, row[e] * inv * ldf(w + e) * (z * dr_sigmoid(z)));
  }
}

void dr_out_norm(uintptr_t y, long ldy, uintptr_t o, uintptr_t gate, long ldg, int gcol, uintptr_t w, int tokens, int H,
                 int vdim, float eps, float out_scale, int f32, uintptr_t stream) {
  if (tokens <= 0) return;
  DLLM_HOST_CHECK(H > 0 && H <= 65535 && vdim > 0 && ldy >= (long)H * vdim && ldg >= gcol + (long)H * vdim && gcol >= 0,
                  "delta rule output norm sizes");
  SM_DISPATCH(f32, dr_out_norm_kernel, dim3(tokens, H), dim3(64), 0, stream, (void*)y, ldy, (const float*)o,
              (const void*)gate, ldg, gcol, (const void*)w, H, vdim, eps, out_scale);
}

}  // namespace dllm
