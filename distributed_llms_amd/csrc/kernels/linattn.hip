// Linear attention with a decayed float32 matrix state per head (ops/linattn.py):
//
//     S <- diag(a) S + k v^T;   o = S^T q          S [dim, vdim] per (sequence, head)
//
// with the decay a either one fixed number per head or, per key channel and token, sigmoid(z + bias)^(1 / tau)
// evaluated as exp(log_sigmoid(z + bias) / tau).  q, k and v are columns of a fused projection of the
// activation type T (bf16 or float); silu and the query scale are applied as they are read.  Everything
// after the read is float32.
//
//   la_scan_kernel   one workgroup per (sequence, head, 64 value columns); a value column of S lives in the
//                    registers of 4 neighbouring lanes (DK / 4 key channels each, DK >= dim zero padded), so a
//                    token costs DK / 4 x (fma, fma) per lane and one 4-lane sum, no exchange of state.  q, k
//                    and the decays of 8 tokens are staged in LDS for the workgroup; the next 8 tokens' global
//                    loads are in flight during the steps.  The state pool is [slots, H, vdim, dim]: a column's
//                    key channels are contiguous, a lane reads and writes its share as 16-byte pieces.
#include <math.h>

#include "common.h"
#include "launchers.h"
#include "stream_common.h"

namespace dllm {

constexpr int kLaTB = 8;        // tokens per staged block
constexpr int kLaCols = 64;     // value columns per workgroup (4 lanes each)

__device__ __forceinline__ float la_silu(float x) { return x / (1.0f + expf(-x)); }
// sigmoid(x)^(inv_tau) = exp(log_sigmoid(x) * inv_tau), log_sigmoid(x) = min(x, 0) - log1p(exp(-|x|))
__device__ __forceinline__ float la_decay(float x, float inv_tau) {
  return expf((fminf(x, 0.f) - log1pf(expf(-fabsf(x)))) * inv_tau);
}

template <typename T, int DK>
__global__ void __launch_bounds__(256) la_scan_kernel(
    float* __restrict__ o, const void* __restrict__ proj_, long ld, int qcol, int kcol, int vcol,
    const float* __restrict__ decay, const void* __restrict__ z_, const float* __restrict__ z_bias, float inv_tau,
    float q_scale, int silu, float* __restrict__ state, const int32_t* __restrict__ cu,
    const int32_t* __restrict__ positions, const int32_t* __restrict__ slots, int H, int D, int Dv) {
  constexpr int R = DK / 4;                        // key channels per lane
  constexpr int NS = (kLaTB * DK) / 256;           // staged (token, channel) pairs per thread
  constexpr int NV = (kLaTB * kLaCols) / 256;      // staged values per thread
  __shared__ __attribute__((aligned(16))) float sq[kLaTB][DK];
  __shared__ __attribute__((aligned(16))) float sk[kLaTB][DK];
  __shared__ __attribute__((aligned(16))) float sa[kLaTB][DK];
  __shared__ float sv[kLaTB][kLaCols];
  const int b = blockIdx.x, h = blockIdx.y, tid = threadIdx.x;
  const int lo = cu[b], hi = cu[b + 1];
  if (hi <= lo) return;
  const int c = tid >> 2, j = tid & 3;
  const int vc = blockIdx.z * kLaCols + c;
  const bool col_ok = vc < Dv;
  const T* proj = (const T*)proj_;
  const T* z = (const T*)z_;
  const float hdecay = decay ? decay[h] : 1.f;
  float* srow = state + (((size_t)slots[b] * H + h) * Dv + (col_ok ? vc : 0)) * D;
  float S[R];
#pragma unroll
  for (int r = 0; r < R; ++r) S[r] = 0.f;
  if (col_ok && positions[lo] > 0) {
    if ((D & 3) == 0) {
#pragma unroll
      for (int r = 0; r < R; r += 4) {
        const int d = j * R + r;
        if (d < D) {
          const f32x4 v = *reinterpret_cast<const f32x4*>(srow + d);
          S[r] = v[0], S[r + 1] = v[1], S[r + 2] = v[2], S[r + 3] = v[3];
        }
      }
    } else {
#pragma unroll
      for (int r = 0; r < R; ++r) {
        const int d = j * R + r;
        if (d < D) S[r] = srow[d];
      }
    }
  }
  // staging registers: this thread's pairs (token tt, channel d) of a block, the same for every block
  float rq[NS], rk[NS], ra[NS], rv[NV];
  auto fetch = [&](int t0) {
#pragma unroll
    for (int i = 0; i < NS; ++i) {
      const int idx = tid + 256 * i, tt = idx / DK, d = idx - tt * DK;
      const int t = t0 + tt;
      float q = 0.f, k = 0.f, a = 1.f;
      if (t < hi && d < D) {
        const T* row = proj + (size_t)t * ld;
        q = ldf(row + qcol + h * D + d);
        k = ldf(row + kcol + h * D + d);
        if (silu) q = la_silu(q), k = la_silu(k);
        q *= q_scale;
        a = z ? la_decay(ldf(z + (size_t)t * H * D + h * D + d) + z_bias[h * D + d], inv_tau) : hdecay;
      }
      rq[i] = q, rk[i] = k, ra[i] = a;
    }
#pragma unroll
    for (int i = 0; i < NV; ++i) {
      const int idx = tid + 256 * i, tt = idx / kLaCols, cc = idx - tt * kLaCols;
      const int t = t0 + tt, col = blockIdx.z * kLaCols + cc;
      float v = 0.f;
      if (t < hi && col < Dv) {
        v = ldf(proj + (size_t)t * ld + vcol + h * Dv + col);
        if (silu) v = la_silu(v);
      }
      rv[i] = v;
    }
  };
  auto stage = [&]() {
#pragma unroll
    for (int i = 0; i < NS; ++i) {
      const int idx = tid + 256 * i, tt = idx / DK, d = idx - tt * DK;
      sq[tt][d] = rq[i], sk[tt][d] = rk[i], sa[tt][d] = ra[i];
    }
#pragma unroll
    for (int i = 0; i < NV; ++i) {
      const int idx = tid + 256 * i;
      sv[idx / kLaCols][idx % kLaCols] = rv[i];
    }
  };
  fetch(lo);
  for (int t0 = lo; t0 < hi; t0 += kLaTB) {
    __syncthreads();                               // every lane is done with the previous block
    stage();
    __syncthreads();
    if (t0 + kLaTB < hi) fetch(t0 + kLaTB);
    const int nt = min(kLaTB, hi - t0);
    for (int tt = 0; tt < nt; ++tt) {
      const float v = sv[tt][c];
      float acc = 0.f;
#pragma unroll
      for (int r = 0; r < R; r += 4) {
        const f32x4 a4 = *reinterpret_cast<const f32x4*>(&sa[tt][j * R + r]);
        const f32x4 k4 = *reinterpret_cast<const f32x4*>(&sk[tt][j * R + r]);
        const f32x4 q4 = *reinterpret_cast<const f32x4*>(&sq[tt][j * R + r]);
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          S[r + e] = fmaf(a4[e], S[r + e], k4[e] * v);
          acc = fmaf(S[r + e], q4[e], acc);
        }
      }
      acc += __shfl_xor(acc, 1, 64);
      acc += __shfl_xor(acc, 2, 64);
      if (j == 0 && col_ok) o[((size_t)(t0 + tt) * H + h) * Dv + vc] = acc;
    }
  }
  if (col_ok) {
    if ((D & 3) == 0) {
#pragma unroll
      for (int r = 0; r < R; r += 4) {
        const int d = j * R + r;
        if (d < D) *reinterpret_cast<f32x4*>(srow + d) = f32x4{S[r], S[r + 1], S[r + 2], S[r + 3]};
      }
    } else {
#pragma unroll
      for (int r = 0; r < R; ++r) {
        const int d = j * R + r;
        if (d < D) srow[d] = S[r];
      }
    }
  }
}

template <typename T, int DK>
static void la_launch(uintptr_t o, uintptr_t proj, long ld, int qcol, int kcol, int vcol, uintptr_t decay, uintptr_t z,
                      uintptr_t z_bias, float inv_tau, float q_scale, int silu, uintptr_t state, uintptr_t cu,
                      uintptr_t positions, uintptr_t slots, int seqs, int H, int D, int Dv, uintptr_t stream) {
  hipLaunchKernelGGL(HIP_KERNEL_NAME(la_scan_kernel<T, DK>), dim3(seqs, H, (Dv + kLaCols - 1) / kLaCols), dim3(256), 0,
                     (hipStream_t)stream, (float*)o, (const void*)proj, ld, qcol, kcol, vcol, (const float*)decay,
                     (const void*)z, (const float*)z_bias, inv_tau, q_scale, silu, (float*)state, (const int32_t*)cu,
                     (const int32_t*)positions, (const int32_t*)slots, H, D, Dv);
  DLLM_HIP_CHECK(hipGetLastError());
}

// o [T, H, Dv] float32; proj [T, ld] of the activation type with q [H, D] at column qcol, k at kcol, v [H, Dv]
// at vcol; decay [H] float32 or z [T, H D] (activation type) + z_bias [H D] float32; state [slots, H, Dv, D].
void la_scan(uintptr_t o, uintptr_t proj, long ld, int qcol, int kcol, int vcol, uintptr_t decay, uintptr_t z,
             uintptr_t z_bias, float inv_tau, float q_scale, int silu, uintptr_t state, uintptr_t cu, uintptr_t positions,
             uintptr_t slots, int seqs, int max_q_len, int H, int D, int Dv, int f32, uintptr_t stream) {
  if (seqs <= 0 || max_q_len <= 0) return;
  DLLM_HOST_CHECK(H > 0 && H <= 65535 && D > 0 && D <= 256 && Dv > 0 && (Dv + kLaCols - 1) / kLaCols <= 65535 &&
                      qcol >= 0 && kcol >= 0 && vcol >= 0 && ld >= (long)qcol + (long)H * D && ld >= (long)kcol + (long)H * D &&
                      ld >= (long)vcol + (long)H * Dv,
                  "linear attention scan sizes");
  DLLM_HOST_CHECK(o && proj && state && cu && positions && slots && (!decay != !z) && (!z || z_bias) &&
                      state % 16 == 0,
                  "linear attention scan arguments");
#define LA_GO(T, DK)                                                                                              \
  la_launch<T, DK>(o, proj, ld, qcol, kcol, vcol, decay, z, z_bias, inv_tau, q_scale, silu, state, cu, positions, \
                   slots, seqs, H, D, Dv, stream)
  if (f32) {
    if (D <= 32) LA_GO(float, 32);
    else if (D <= 64) LA_GO(float, 64);
    else if (D <= 128) LA_GO(float, 128);
    else LA_GO(float, 256);
  } else {
    if (D <= 32) LA_GO(bf16, 32);
    else if (D <= 64) LA_GO(bf16, 64);
    else if (D <= 128) LA_GO(bf16, 128);
    else LA_GO(bf16, 256);
  }
#undef LA_GO
}

}  // namespace dllm
