// Linear attention with a decayed float32 matrix state per head (ops/linattn.py):
//
//     S <- diag(a) S + k v^T;   o = S^T q          S [dim, vdim] per (sequence, head)
//
// with the decay a either one fixed number per head or, per key channel and token, sigmoid(z + bias)^(1 / tau)
// evaluated as exp(log_sigmoid(z + bias) / tau).  q, k and v are columns of a fused projection of the
// activation type T (bf16 or float); silu and the query scale are applied as they are read.  Everything
// after the read is float32.
//
//   la_scan_kernel   one workgroup per (sequence, head, a slice of value columns).  The key channels of a value
//                    column are split over PARTS lanes (4: the lanes 16 apart, 8: also the lanes 8 apart inside a
//                    16-lane row), DK / PARTS channels each (DK >= dim, zero padded), and a lane holds CPL such
//                    columns: a token costs DK / PARTS x (mul, fma, fma) per column and lane and one sum over the
//                    parts (VALU row swaps and a row rotation, no LDS), no exchange of state.  q, k and the decays
//                    of 8 tokens are staged in LDS for the workgroup; every element a lane reads there feeds CPL
//                    columns -- on long chunks the LDS reads, not the FMAs, bound the forms with few columns per
//                    lane (PARTS = 4, CPL = 1: 24 16-byte reads per 96 FMAs; PARTS = 8, CPL = 4: 12 per 192) --
//                    and a fixed decay per head is not read from LDS at all.  The next 8 tokens' global loads are
//                    in flight during the steps.  The state pool is [slots, H, vdim, dim]: a column's key channels
//                    are contiguous, a lane reads and writes its share as 16-byte pieces.
#include <math.h>

#include "common.h"
#include "launchers.h"
#include "stream_common.h"

namespace dllm {

constexpr int kLaTB = 8;        // tokens per staged block

// Sum over the PARTS lanes that share a value column: lanes 16 and 32 apart, and for PARTS = 8 also the lane
// 8 apart inside the 16-lane row (a DPP row rotation: VALU, no LDS round trip).
template <int PARTS>
__device__ __forceinline__ float la_parts_sum(float v) {
  if constexpr (PARTS == 8)
    v += __int_as_float(__builtin_amdgcn_mov_dpp(__float_as_int(v), 0x128 /* row_ror:8 */, 0xf, 0xf, false));
  return rows_sum(v);
}

__device__ __forceinline__ float la_silu(float x) { return x * __builtin_amdgcn_rcpf(1.0f + expf(-x)); }
// sigmoid(x)^(inv_tau) = exp(log_sigmoid(x) * inv_tau), log_sigmoid(x) = min(x, 0) - log1p(exp(-|x|))
__device__ __forceinline__ float la_decay(float x, float inv_tau) {
  return expf((fminf(x, 0.f) - log1pf(expf(-fabsf(x)))) * inv_tau);
}

template <typename T, int DK, int PARTS, int CPL>
__global__ void __launch_bounds__(256) la_scan_kernel(
    float* __restrict__ o, const void* __restrict__ proj_, long ld, int qcol, int kcol, int vcol,
    const float* __restrict__ decay, const void* __restrict__ z_, const float* __restrict__ z_bias, float inv_tau,
    float q_scale, int silu, float* __restrict__ state, const int32_t* __restrict__ cu,
    const int32_t* __restrict__ positions, const int32_t* __restrict__ slots, int H, int D, int Dv) {
  constexpr int R = DK / PARTS;                    // key channels per lane
  constexpr int LPW = 64 / PARTS;                  // value columns per wave and column set
  constexpr int CSET = 4 * LPW;                    // columns of one set in the workgroup (4 waves)
  constexpr int COLS = CSET * CPL;                 // value columns per workgroup
  constexpr int NS = (kLaTB * DK) / 256;           // staged (token, channel) pairs per thread
  constexpr int NV = (kLaTB * COLS + 255) / 256;   // staged values per thread
  static_assert(R % 4 == 0 && (kLaTB * DK) % 256 == 0, "key channels per lane in 16-byte pieces");
  // a part's channels are followed by 4 floats of padding: the parts' 16-byte reads of one step then fall on
  // different banks (unpadded, parts R = 16 or 32 floats apart share a bank: every read a 4-way conflict)
  constexpr int RP = R + 4, DKP = PARTS * RP;
  __shared__ __attribute__((aligned(16))) float sq[kLaTB][DKP];
  __shared__ __attribute__((aligned(16))) float sk[kLaTB][DKP];
  __shared__ __attribute__((aligned(16))) float sa[kLaTB][DKP];
  __shared__ float sv[kLaTB][COLS];
  const int b = blockIdx.x, h = blockIdx.y, tid = threadIdx.x;
  const int lo = cu[b], hi = cu[b + 1];
  if (hi <= lo) return;
  const int wave = tid >> 6, lane = tid & 63, part = lane / LPW, jj = lane % LPW;
  const int col0 = blockIdx.z * COLS;
  const T* proj = (const T*)proj_;
  const T* z = (const T*)z_;
  const bool perch = z != nullptr;                 // a decay per key channel and token (else one per head)
  const float hdecay = decay ? decay[h] : 1.f;
  float* sbase = state + ((size_t)slots[b] * H + h) * Dv * D;
  const bool resume = positions[lo] > 0;
  int cl[CPL];                                     // this lane's columns inside the workgroup's COLS
  bool cok[CPL];
  float S[CPL][R];
#pragma unroll
  for (int c = 0; c < CPL; ++c) {
    cl[c] = c * CSET + wave * LPW + jj;
    cok[c] = col0 + cl[c] < Dv;
    const float* srow = sbase + (size_t)(cok[c] ? col0 + cl[c] : 0) * D;
#pragma unroll
    for (int r = 0; r < R; ++r) S[c][r] = 0.f;
    if (cok[c] && resume) {
      if ((D & 3) == 0) {
#pragma unroll
        for (int r = 0; r < R; r += 4) {
          const int d = part * R + r;
          if (d < D) {
            const f32x4 v = *reinterpret_cast<const f32x4*>(srow + d);
            S[c][r] = v[0], S[c][r + 1] = v[1], S[c][r + 2] = v[2], S[c][r + 3] = v[3];
          }
        }
      } else {
#pragma unroll
        for (int r = 0; r < R; ++r) {
          const int d = part * R + r;
          if (d < D) S[c][r] = srow[d];
        }
      }
    }
  }
  // staging registers: this thread's pairs (token tt, channel d) of a block, the same for every block.  fetch()
  // only issues the loads (raw values of the activation type): their math (silu, the decay's exp / log) waits
  // until stage(), after the steps of the block before, so the loads' latency hides behind those steps.
  T rq[NS], rk[NS], rz[NS], rv[NV];
  float rb[NS];
  auto fetch = [&](int t0) {
#pragma unroll
    for (int i = 0; i < NS; ++i) {
      const int idx = tid + 256 * i, tt = idx / DK, d = idx - tt * DK;
      const int t = t0 + tt;
      if (t < hi && d < D) {
        const T* row = proj + (size_t)t * ld;
        rq[i] = row[qcol + h * D + d];
        rk[i] = row[kcol + h * D + d];
        if (perch) rz[i] = z[(size_t)t * H * D + h * D + d], rb[i] = z_bias[h * D + d];
      }
    }
#pragma unroll
    for (int i = 0; i < NV; ++i) {
      const int idx = tid + 256 * i, tt = idx / COLS, cc = idx - tt * COLS;
      const int t = t0 + tt, col = col0 + cc;
      if (tt < kLaTB && t < hi && col < Dv) rv[i] = proj[(size_t)t * ld + vcol + h * Dv + col];
    }
  };
  auto stage = [&](int t0) {
#pragma unroll
    for (int i = 0; i < NS; ++i) {
      const int idx = tid + 256 * i, tt = idx / DK, d = idx - tt * DK;
      const int dp = d + 4 * (d / R);
      float q = 0.f, k = 0.f, a = 1.f;
      if (t0 + tt < hi && d < D) {
        q = (float)rq[i], k = (float)rk[i];
        if (silu) q = la_silu(q), k = la_silu(k);
        q *= q_scale;
        if (perch) a = la_decay((float)rz[i] + rb[i], inv_tau);
      }
      sq[tt][dp] = q, sk[tt][dp] = k;
      if (perch) sa[tt][dp] = a;
    }
#pragma unroll
    for (int i = 0; i < NV; ++i) {
      const int idx = tid + 256 * i, tt = idx / COLS, cc = idx - tt * COLS;
      float v = 0.f;
      if (tt < kLaTB && t0 + tt < hi && col0 + cc < Dv) {
        v = (float)rv[i];
        if (silu) v = la_silu(v);
      }
      if (idx < kLaTB * COLS) sv[tt][cc] = v;
    }
  };
  fetch(lo);
  for (int t0 = lo; t0 < hi; t0 += kLaTB) {
    __syncthreads();                               // every lane is done with the previous block
    stage(t0);
    __syncthreads();
    if (t0 + kLaTB < hi) fetch(t0 + kLaTB);
    const int nt = min(kLaTB, hi - t0);
    for (int tt = 0; tt < nt; ++tt) {
      float v[CPL], acc[CPL][4];
#pragma unroll
      for (int c = 0; c < CPL; ++c) {
        v[c] = sv[tt][cl[c]];
#pragma unroll
        for (int e = 0; e < 4; ++e) acc[c][e] = 0.f;
      }
#pragma unroll
      for (int r = 0; r < R; r += 4) {
        f32x4 a4 = {hdecay, hdecay, hdecay, hdecay};
        if (perch) a4 = *reinterpret_cast<const f32x4*>(&sa[tt][part * RP + r]);     // wave-uniform branch
        const f32x4 k4 = *reinterpret_cast<const f32x4*>(&sk[tt][part * RP + r]);
        const f32x4 q4 = *reinterpret_cast<const f32x4*>(&sq[tt][part * RP + r]);
#pragma unroll
        for (int e = 0; e < 4; ++e) {
#pragma unroll
          for (int c = 0; c < CPL; ++c) {
            S[c][r + e] = fmaf(a4[e], S[c][r + e], k4[e] * v[c]);
            acc[c][e] = fmaf(S[c][r + e], q4[e], acc[c][e]);
          }
        }
      }
#pragma unroll
      for (int c = 0; c < CPL; ++c) {
        const float oo = la_parts_sum<PARTS>((acc[c][0] + acc[c][1]) + (acc[c][2] + acc[c][3]));
        if (part == 0 && cok[c]) o[((size_t)(t0 + tt) * H + h) * Dv + col0 + cl[c]] = oo;
      }
    }
  }
#pragma unroll
  for (int c = 0; c < CPL; ++c) {
    if (!cok[c]) continue;
    float* srow = sbase + (size_t)(col0 + cl[c]) * D;
    if ((D & 3) == 0) {
#pragma unroll
      for (int r = 0; r < R; r += 4) {
        const int d = part * R + r;
        if (d < D) *reinterpret_cast<f32x4*>(srow + d) = f32x4{S[c][r], S[c][r + 1], S[c][r + 2], S[c][r + 3]};
      }
    } else {
#pragma unroll
      for (int r = 0; r < R; ++r) {
        const int d = part * R + r;
        if (d < D) srow[d] = S[c][r];
      }
    }
  }
}

template <typename T, int DK, int PARTS, int CPL>
static void la_launch(uintptr_t o, uintptr_t proj, long ld, int qcol, int kcol, int vcol, uintptr_t decay, uintptr_t z,
                      uintptr_t z_bias, float inv_tau, float q_scale, int silu, uintptr_t state, uintptr_t cu,
                      uintptr_t positions, uintptr_t slots, int seqs, int H, int D, int Dv, uintptr_t stream) {
  constexpr int COLS = 4 * (64 / PARTS) * CPL;
  hipLaunchKernelGGL(HIP_KERNEL_NAME(la_scan_kernel<T, DK, PARTS, CPL>), dim3(seqs, H, (Dv + COLS - 1) / COLS),
                     dim3(256), 0, (hipStream_t)stream, (float*)o, (const void*)proj, ld, qcol, kcol, vcol,
                     (const float*)decay, (const void*)z, (const float*)z_bias, inv_tau, q_scale, silu, (float*)state,
                     (const int32_t*)cu, (const int32_t*)positions, (const int32_t*)slots, H, D, Dv);
  DLLM_HIP_CHECK(hipGetLastError());
}

// o [T, H, Dv] float32; proj [T, ld] of the activation type with q [H, D] at column qcol, k at kcol, v [H, Dv]
// at vcol; decay [H] float32 or z [T, H D] (activation type) + z_bias [H D] float32; state [slots, H, Dv, D].
void la_scan(uintptr_t o, uintptr_t proj, long ld, int qcol, int kcol, int vcol, uintptr_t decay, uintptr_t z,
             uintptr_t z_bias, float inv_tau, float q_scale, int silu, uintptr_t state, uintptr_t cu, uintptr_t positions,
             uintptr_t slots, int seqs, int max_q_len, int H, int D, int Dv, int f32, uintptr_t stream) {
  if (seqs <= 0 || max_q_len <= 0) return;
  DLLM_HOST_CHECK(H > 0 && H <= 65535 && D > 0 && D <= 256 && Dv > 0 && (Dv + 31) / 32 <= 65535 &&
                      qcol >= 0 && kcol >= 0 && vcol >= 0 && ld >= (long)qcol + (long)H * D && ld >= (long)kcol + (long)H * D &&
                      ld >= (long)vcol + (long)H * Dv,
                  "linear attention scan sizes");
  DLLM_HOST_CHECK(o && proj && state && cu && positions && slots && (!decay != !z) && (!z || z_bias) &&
                      state % 16 == 0,
                  "linear attention scan arguments");
  // long chunks: four value columns per lane with the key channels over 8 lanes (a quarter of the LDS reads per
  // FMA; two columns for keys wider than 128, whose state would not fit the registers); short chunks (decode)
  // and narrow value heads: one column over 4 lanes, so that more workgroups share the state traffic
  // (also for long chunks of few sequences and heads: with four columns per lane they would leave most CUs idle,
  // and the chain of one token's steps on a lone wave, not the arithmetic, bounds them)
  const long wide_wgs = (long)seqs * H * ((Dv + 127) / 128);
  const bool wide = max_q_len >= 16 && Dv > 64 && wide_wgs >= 256;
#define LA_GO(T, DK, PARTS, CPL)                                                                                   \
  la_launch<T, DK, PARTS, CPL>(o, proj, ld, qcol, kcol, vcol, decay, z, z_bias, inv_tau, q_scale, silu, state, cu, \
                               positions, slots, seqs, H, D, Dv, stream)
#define LA_BY_DIM(T)                                                                  \
  do {                                                                                \
    if (D <= 32) { if (wide) LA_GO(T, 32, 8, 4); else LA_GO(T, 32, 4, 1); }           \
    else if (D <= 64) { if (wide) LA_GO(T, 64, 8, 4); else LA_GO(T, 64, 4, 1); }      \
    else if (D <= 128) { if (wide) LA_GO(T, 128, 8, 4); else LA_GO(T, 128, 4, 1); }   \
    else { if (wide) LA_GO(T, 256, 8, 2); else LA_GO(T, 256, 4, 1); }                 \
  } while (0)
  if (f32) LA_BY_DIM(float);
  else LA_BY_DIM(bf16);
#undef LA_BY_DIM
#undef LA_GO
}

}  // namespace dllm
