// Sliding-window attention over a paged K/V cache whose key and value head sizes differ
// (ops/seqmix.py window_attention): caches k [NB, G, BS, D] (one row per key), v [NB, G, Dv, BS]
// (transposed inside a block: 8 keys of one value channel are one 16-byte load),
// query head h reads K/V head h / (H / G), a query at position p sees the keys j of its sequence with
// 0 <= p - j < window and, with `chunk` > 0, floor(j / chunk) = floor(p / chunk) (attention inside fixed
// chunks of positions); `sinks` (float32 [H], or null) adds exp(sink_h) to head h's softmax denominator
// (a learned per-head logit that takes part in the normalisation only).  `softcap` > 0 turns every scaled
// score s into softcap tanh(s / softcap).  Averaged caches kp [NB, G, PB, D] / vp [NB, G, Dv, PB] with `pool` > 0
// (the K/V layouts with PB entries per block, a power of two >= 8, behind the same block table): beside its
// window a query at position p also sees entries b < npool(p) = floor(max(p - window + 1, 0) / pool) -- one
// mean key and value per block of `pool` positions that lies wholly before the window -- in the same softmax;
// every kernel visits those entries first (32-entry tiles from entry 0), then the window's tokens.
// Scores, softmax weights and the weighted sum are float32; T is the storage
// type (bf16 or float).  Head sizes, window and block size are runtime values.
//
//   window_attn_row_kernel   one workgroup per (query token, head): keys in tiles of 256, one key per
//                            thread for q.k, an online softmax across tiles, then P.V with the
//                            threads laid out (value channel, key subgroup).  Decode rows, and prompt
//                            chunks in float32.
//   window_attn_tile_kernel  bf16 prompt chunks on MFMA (v_mfma_f32_16x16x32_bf16): one workgroup per
//                            (64-query tile of a chunk, head), 4 waves x 16 queries, keys in tiles of 32 (the next tile's
//                            global loads are in flight during the current tile's MFMAs)
//                            staged through LDS (K rows permuted so that the S^T = K Q^T accumulator
//                            hands each lane 8 consecutive keys, V transposed so that P.V reads 8 keys
//                            of one value channel in one 16-byte load).  The softmax weights stay
//                            float32: P is fed to the matrix cores as a bf16 pair (upper half + the
//                            remainder), two MFMAs per tile, so P.V carries 16 significand bits.
#include <math.h>

#include "common.h"
#include "launchers.h"

namespace dllm {

template <typename T> __device__ __forceinline__ float wld(const T* p) { return (float)*p; }

// Oldest key position a query at `pos` sees: inside its window and -- with chunk > 0 -- inside its own
// chunk of `chunk` positions, chunks counted from position 0 of the sequence (a query never looks across
// a chunk border, wherever the prompt was cut for processing).  Not decreasing in pos.
__device__ __forceinline__ int win_lo(int pos, int window, int chunk) {
  int lo = max(0, pos - window + 1);
  if (chunk > 0) lo = max(lo, pos - pos % chunk);
  return lo;
}

// Averaged entries a query at `pos` sees: the blocks of `pool` positions that end at or before pos - window.
__device__ __forceinline__ int win_npool(int pos, int window, int pool) {
  return pool > 0 ? max(pos - window + 1, 0) / pool : 0;
}

// softcap tanh(s / softcap) from exp2 and a reciprocal (the matrix-core kernels; the row kernel, which is
// the float32 path, calls tanhf): tanh(x) = 1 - 2 / (e^(2x) + 1), exact at both ends (e -> inf, e -> 0)
__device__ __forceinline__ float fast_tanh(float x) {
  const float e = __builtin_amdgcn_exp2f(x * 2.8853900817779268f);
  return 1.0f - 2.0f * __builtin_amdgcn_rcpf(e + 1.0f);
}

constexpr int kWinTile = 256;     // keys per tile = threads per workgroup
constexpr int kWinMaxAcc = 2;     // value channels per thread: Dv <= 256 * kWinMaxAcc

template <typename T>
__device__ __forceinline__ float dot_row(const float* __restrict__ qs, const T* __restrict__ k, int D) {
  float s = 0.f;
  for (int d = 0; d < D; ++d) s = fmaf(qs[d], wld(k + d), s);
  return s;
}

// 16-byte loads when rows are 16-byte aligned (D % 8 == 0)
template <>
__device__ __forceinline__ float dot_row<bf16>(const float* __restrict__ qs, const bf16* __restrict__ k, int D) {
  float s = 0.f;
  if ((D & 7) == 0) {
    const bf16x8* kv = reinterpret_cast<const bf16x8*>(k);
    for (int d = 0; d < D; d += 8) {
      const bf16x8 v = kv[d >> 3];
#pragma unroll
      for (int j = 0; j < 8; ++j) s = fmaf(qs[d + j], bf2f(v[j]), s);
    }
    return s;
  }
  for (int d = 0; d < D; ++d) s = fmaf(qs[d], bf2f(k[d]), s);
  return s;
}

template <>
__device__ __forceinline__ float dot_row<float>(const float* __restrict__ qs, const float* __restrict__ k, int D) {
  float s = 0.f;
  if ((D & 3) == 0) {
    const f32x4* kv = reinterpret_cast<const f32x4*>(k);
    for (int d = 0; d < D; d += 4) {
      const f32x4 v = kv[d >> 2];
      s = fmaf(qs[d], v[0], s);
      s = fmaf(qs[d + 1], v[1], s);
      s = fmaf(qs[d + 2], v[2], s);
      s = fmaf(qs[d + 3], v[3], s);
    }
    return s;
  }
  for (int d = 0; d < D; ++d) s = fmaf(qs[d], k[d], s);
  return s;
}

template <typename T>
__global__ void __launch_bounds__(kWinTile) window_attn_row_kernel(
    void* __restrict__ out_, const void* __restrict__ q_, const void* __restrict__ k_cache_,
    const void* __restrict__ v_cache_, const int32_t* __restrict__ block_tables, int max_blocks,
    const int32_t* __restrict__ positions, const int32_t* __restrict__ tok_seq, int t0, int H, int G, int D, int Dv,
    int bs, int window, int chunk, float scale, const float* __restrict__ sinks, float softcap,
    const void* __restrict__ kp_, const void* __restrict__ vp_, int pool, int pbs) {
  extern __shared__ float lds[];
  float* qs = lds;                       // [D]
  float* p = qs + D;                     // [kWinTile]
  int* rows = reinterpret_cast<int*>(p + kWinTile);   // [kWinTile] cache row of each key of the tile
  float* red = reinterpret_cast<float*>(rows + kWinTile);   // [16]
  float* part = red + 16;                // [nsub][Dv] at the end
  const int t = t0 + blockIdx.x, h = blockIdx.y, tid = threadIdx.x;
  const int g = h / (H / G);
  const int pos = positions[t], b = tok_seq[t];
  const int lo = win_lo(pos, window, chunk);
  const T* q = (const T*)q_ + ((size_t)t * H + h) * D;
  const int32_t* bt = block_tables + (size_t)b * max_blocks;
  for (int d = tid; d < D; d += kWinTile) qs[d] = wld(q + d);
  // P.V layout: thread = (channel e of ew, key subgroup sub of nsub); channels beyond ew loop
  const int ew = min(kWinTile, ((Dv + 63) / 64) * 64);
  const int nsub = kWinTile / ew;
  const int e0 = tid % ew, sub = tid / ew;
  float acc[kWinMaxAcc];
#pragma unroll
  for (int i = 0; i < kWinMaxAcc; ++i) acc[i] = 0.f;
  float m = -INFINITY, l = 0.f;
  __syncthreads();
  // keys first .. last (all visible) of a cache pair with `cbs` keys per block
  auto run = [&](const T* kc, const T* vc, int cbs, int first, int last) {
    for (int k0 = first; k0 <= last; k0 += kWinTile) {
      const int j = k0 + tid;
      float s = -INFINITY;
      if (j <= last) {
        const int blk = bt[j / cbs];
        const int row = (blk * G + g) * cbs + (j % cbs);
        rows[tid] = row;                                    // K row; V element (e) at ((row / cbs) * Dv + e) * cbs + row % cbs
        s = dot_row<T>(qs, kc + (size_t)row * D, D) * scale;
        if (softcap > 0.f) s = softcap * tanhf(s / softcap);
      }
      const float m_new = fmaxf(m, block_max(s, red));
      const float pj = j <= last ? expf(s - m_new) : 0.f;
      p[tid] = pj;
      const float psum = block_sum(pj, red);      // ends with a barrier: p and rows are visible
      const float corr = expf(m - m_new);         // 0 at the first tile (m = -inf)
      l = l * corr + psum;
      m = m_new;
      const int nk = min(kWinTile, last + 1 - k0);
#pragma unroll
      for (int i = 0; i < kWinMaxAcc; ++i) {
        const int e = e0 + i * ew;
        if (sub < nsub && e < Dv) {
          float a = acc[i] * corr;
          for (int k = sub; k < nk; k += nsub) {
            const int row = rows[k], hb = row / cbs;
            a = fmaf(p[k], wld(vc + ((size_t)hb * Dv + e) * cbs + (row - hb * cbs)), a);
          }
          acc[i] = a;
        }
      }
      __syncthreads();                            // before the next tile overwrites p and rows
    }
  };
  const int np = win_npool(pos, window, pool);
  if (np > 0) run((const T*)kp_, (const T*)vp_, pbs, 0, np - 1);
  run((const T*)k_cache_, (const T*)v_cache_, bs, lo, pos);
  // a sink adds exp(sink) to the denominator; nothing is attended to through it
  float fin = 1.0f / l;
  if (sinks) {
    const float sk = sinks[h], mf = fmaxf(m, sk), cf = expf(m - mf);
    fin = cf / (l * cf + expf(sk - mf));
  }
  // sum the key subgroups
  T* out = (T*)out_ + ((size_t)t * H + h) * Dv;
#pragma unroll
  for (int i = 0; i < kWinMaxAcc; ++i) {
    const int e = e0 + i * ew;
    if (sub < nsub && e < Dv) part[sub * Dv + e] = acc[i];
    __syncthreads();
    if (sub == 0 && e < Dv) {
      float a = 0.f;
      for (int s2 = 0; s2 < nsub; ++s2) a += part[s2 * Dv + e];
      out[e] = (T)(a * fin);
    }
    __syncthreads();
  }
}

static size_t win_row_lds(int D, int Dv) {
  const int ew = std::min(kWinTile, ((Dv + 63) / 64) * 64);
  return sizeof(float) * ((size_t)D + kWinTile + kWinTile + 16 + (size_t)(kWinTile / ew) * Dv);
}

static void launch_rows(uintptr_t out, uintptr_t q, uintptr_t k_cache, uintptr_t v_cache, uintptr_t block_tables,
                        int max_blocks, uintptr_t positions, uintptr_t tok_seq, int t0, int rows, int H, int G, int D,
                        int Dv, int bs, int window, int chunk, float scale, uintptr_t sinks, float softcap, uintptr_t kp,
                        uintptr_t vp, int pool, int pbs, int f32, uintptr_t stream) {
  DLLM_HOST_CHECK(H > 0 && G > 0 && H % G == 0 && D > 0 && Dv > 0 && Dv <= kWinTile * kWinMaxAcc, "window attention heads");
  DLLM_HOST_CHECK(pool == 0 || (pool > 0 && kp && vp && pbs > 0 && chunk == 0), "window attention averaged caches");
  DLLM_HOST_CHECK(bs > 0 && window >= 1 && chunk >= 0 && max_blocks > 0 && H <= 65535, "window attention sizes");
  const size_t lds = win_row_lds(D, Dv);
  DLLM_HOST_CHECK(lds <= 64 * 1024, "window attention head size");
  if (f32)
    hipLaunchKernelGGL(HIP_KERNEL_NAME(window_attn_row_kernel<float>), dim3(rows, H), dim3(kWinTile), lds,
                       (hipStream_t)stream, (void*)out, (const void*)q, (const void*)k_cache, (const void*)v_cache,
                       (const int32_t*)block_tables, max_blocks, (const int32_t*)positions, (const int32_t*)tok_seq, t0,
                       H, G, D, Dv, bs, window, chunk, scale, (const float*)sinks, softcap, (const void*)kp, (const void*)vp,
                       pool, pbs);
  else
    hipLaunchKernelGGL(HIP_KERNEL_NAME(window_attn_row_kernel<bf16>), dim3(rows, H), dim3(kWinTile), lds,
                       (hipStream_t)stream, (void*)out, (const void*)q, (const void*)k_cache, (const void*)v_cache,
                       (const int32_t*)block_tables, max_blocks, (const int32_t*)positions, (const int32_t*)tok_seq, t0,
                       H, G, D, Dv, bs, window, chunk, scale, (const float*)sinks, softcap, (const void*)kp, (const void*)vp,
                       pool, pbs);
  DLLM_HIP_CHECK(hipGetLastError());
}

// Softmax weights for the matrix cores without giving up their float32 value: e = hi + lo with hi the
// upper 16 bits of e (a bf16 by truncation), lo = e - hi (exact in float32) cut to bf16 the same way;
// hi + lo carries 16 significand bits of e.  Two values are packed into a dword with one byte permute.
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
__device__ __forceinline__ void split_pack(const float (&e)[8], bf16x8& ph, bf16x8& pl) {
  u32x4 h, l;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const uint32_t a = __float_as_uint(e[2 * i]), b = __float_as_uint(e[2 * i + 1]);
    const float la = e[2 * i] - __uint_as_float(a & 0xffff0000u), lb = e[2 * i + 1] - __uint_as_float(b & 0xffff0000u);
    h[i] = __builtin_amdgcn_perm(b, a, 0x07060302u);
    l[i] = __builtin_amdgcn_perm(__float_as_uint(lb), __float_as_uint(la), 0x07060302u);
  }
  ph = __builtin_bit_cast(bf16x8, h);
  pl = __builtin_bit_cast(bf16x8, l);
}

// --------------------------------------------------------------------------- MFMA prompt kernel (bf16)
// QT (template): MFMA column tiles (16 queries) per wave.  1 keeps heads up to 128 wide at <= 128 VGPRs
// (4 waves per SIMD, so one wave's softmax overlaps another's MFMAs; 2 measured slower there at 1 wave
// per SIMD).  2 halves the LDS reads per MFMA: every K / V^T fragment a wave reads feeds both of its
// column tiles.  A workgroup has 4 waves x QT column tiles = 64 QT queries.
constexpr int kTK = 32;          // keys per tile
constexpr int kPad = 8;          // bf16 elements of row padding in LDS (16 bytes: rows start on different banks)
constexpr float kLog2e = 1.4426950408889634f;

// NQK: 32-wide K-dim steps of q.k (D <= 32 NQK); NDV: 16-wide tiles of value channels (Dv <= 16 NDV).
// Every K / V^T fragment a wave reads from LDS feeds both of its query column tiles; the next key tile's
// global loads are issued before the current tile's MFMAs and land in LDS after them.
template <int NQK, int NDV, int QT>
__global__ void __launch_bounds__(256) window_attn_tile_kernel(
    bf16* __restrict__ out, const bf16* __restrict__ q, const bf16* __restrict__ k_cache,
    const bf16* __restrict__ v_cache, const int32_t* __restrict__ block_tables, int max_blocks,
    const int32_t* __restrict__ cu, const int32_t* __restrict__ positions, int seq0, int nseq, int nqt, int H, int G,
    int D, int Dv, int bs, int window, int chunk, float scale, const float* __restrict__ sinks, int sub, float softcap,
    const bf16* __restrict__ kp_cache, const bf16* __restrict__ vp_cache, int pool, int pbs) {
  constexpr int kQT = QT, kTQ = 64 * QT;
  constexpr int DP = 32 * NQK, KROW = DP + kPad, VROW = kTK + kPad;
  constexpr int KPT = (kTK * (DP / 8) + 255) / 256, VPT = (16 * NDV * (kTK / 8) + 255) / 256;   // 16-byte pieces per thread
  __shared__ __attribute__((aligned(16))) bf16 ks[kTK * KROW];          // K tile, key j at row krow32(j)
  __shared__ __attribute__((aligned(16))) bf16 vs[16 * NDV * VROW];     // V^T tile [channel][key]
  // Workgroups are dealt to the 8 XCDs round-robin by their linear id.  The id is decoded so that
  // every tile that reads one (sequence, K/V head) pair -- all its query tiles and the heads of the
  // group -- runs on the same XCD, whose L2 then serves the re-reads of that pair's keys and values;
  // within a pair the longest query tiles (most keys, causal) start first.  With fewer pairs than XCDs
  // (few sequences that share one K/V head) a pair's tiles are dealt to `sub` XCDs in turn, so that no
  // XCD stays idle.
  const int R = H / G, per_pair = nqt * R, pairs = nseq * G;
  const int per_part = (per_pair + sub - 1) / sub;
  const int xcd = blockIdx.x & 7, slot = blockIdx.x >> 3;
  const int vpair = (slot / per_part) * 8 + xcd;
  const int pair = vpair / sub, rem = (slot % per_part) * sub + vpair % sub;
  if (pair >= pairs || rem >= per_pair) return;
  const int b = seq0 + pair / G, g = pair % G;
  const int h = g * R + rem % R;
  const int lo_t = cu[b], n = cu[b + 1] - lo_t;
  const int q0 = (nqt - 1 - rem / R) * kTQ;                            // first local query of the tile
  if (q0 >= n) return;
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63, col = lane & 15, grp = lane >> 4;
  const int start = positions[lo_t];                                   // position of the chunk's first token
  const int bsh = __ffs(bs) - 1;                                       // bs is a power of two here
  const int32_t* bt = block_tables + (size_t)b * max_blocks;
  // this lane's two queries (MFMA columns of the wave's two column tiles)
  int ql[kQT], qpos[kQT], qlo[kQT];
  bool qok[kQT];
  bf16x8 qf[kQT][NQK];
#pragma unroll
  for (int c2 = 0; c2 < kQT; ++c2) {
    ql[c2] = q0 + wave * 16 * kQT + c2 * 16 + col;
    qok[c2] = ql[c2] < n;
    qpos[c2] = start + min(ql[c2], n - 1);
    qlo[c2] = win_lo(qpos[c2], window, chunk);
    const bf16* qrow = q + ((size_t)(lo_t + min(ql[c2], n - 1)) * H + h) * D;
#pragma unroll
    for (int s2 = 0; s2 < NQK; ++s2) {
      const int d0 = 32 * s2 + 8 * grp;
      bf16x8 v;
#pragma unroll
      for (int j = 0; j < 8; ++j) v[j] = (bf16)0.f;
      if (d0 + 8 <= D) v = *reinterpret_cast<const bf16x8*>(qrow + d0);
      qf[c2][s2] = v;
    }
  }
  // zero both tiles once: the K padding columns (d in [D, DP)) and the V^T rows of channels >= Dv are
  // never written again
  for (int i = tid; i < kTK * KROW; i += 256) ks[i] = (bf16)0.f;
  for (int i = tid; i < 16 * NDV * VROW; i += 256) vs[i] = (bf16)0.f;
  f32x4 acc[kQT][NDV];
#pragma unroll
  for (int c2 = 0; c2 < kQT; ++c2)
#pragma unroll
    for (int i = 0; i < NDV; ++i) acc[c2][i] = f32x4{0.f, 0.f, 0.f, 0.f};
  float m[kQT], l[kQT];
#pragma unroll
  for (int c2 = 0; c2 < kQT; ++c2) m[c2] = -INFINITY, l[c2] = 0.f;
  const int d8 = D >> 3;
  const float sc2 = scale * kLog2e;
  const float cap_in = softcap > 0.f ? scale / softcap : 0.f, cap_out = softcap * kLog2e;   // capped scores in log2 units
  // the cache pair, block size and key range of the phase that runs: averaged entries first, then tokens
  const bf16* ck = k_cache;
  const bf16* cv = v_cache;
  int cbs = bs, cbsh = bsh, last_pos = 0;
  int lo_q[kQT], hi_q[kQT];                                            // keys this lane's queries see in the phase
  bf16x8 kreg[KPT], vreg[VPT];
  // this thread's 16-byte pieces of a tile: K piece r = (key kj[r], columns 8 kc[r] ..), V piece r =
  // (channel vch[r], keys 8 vc[r] ..); the same for every tile
  int kj[KPT], kc[KPT], vch[VPT], vc[VPT];
#pragma unroll
  for (int r = 0; r < KPT; ++r) {
    const int i = tid + 256 * r;
    kj[r] = i < kTK * d8 ? i / d8 : -1;
    kc[r] = i - max(kj[r], 0) * d8;
  }
#pragma unroll
  for (int r = 0; r < VPT; ++r) {
    const int i = tid + 256 * r;
    vch[r] = i < Dv * (kTK / 8) ? i / (kTK / 8) : -1;
    vc[r] = i & (kTK / 8 - 1);
  }
  auto fetch = [&](int k0) {
#pragma unroll
    for (int r = 0; r < KPT; ++r) {
      if (kj[r] >= 0) {
        const int j = kj[r], c = kc[r];
        const int kp = min(k0 + j, last_pos);
        const size_t row = ((size_t)bt[kp >> cbsh] * G + g) * cbs + (kp & (cbs - 1));
        kreg[r] = *reinterpret_cast<const bf16x8*>(ck + row * D + 8 * c);
      }
    }
#pragma unroll
    for (int r = 0; r < VPT; ++r) {
      if (vch[r] >= 0) {
        const int ch = vch[r], c = vc[r];
        const int kp = min(k0 + 8 * c, last_pos & ~7);     // 8 keys of one block (bs % 8 == 0)
        const size_t at = (((size_t)bt[kp >> cbsh] * G + g) * Dv + ch) * cbs + (kp & (cbs - 1));
        vreg[r] = *reinterpret_cast<const bf16x8*>(cv + at);
      }
    }
  };
  auto stage = [&]() {
#pragma unroll
    for (int r = 0; r < KPT; ++r)
      if (kj[r] >= 0) *reinterpret_cast<bf16x8*>(ks + krow32(kj[r]) * KROW + 8 * kc[r]) = kreg[r];
#pragma unroll
    for (int r = 0; r < VPT; ++r)
      if (vch[r] >= 0) *reinterpret_cast<bf16x8*>(vs + vch[r] * VROW + 8 * vc[r]) = vreg[r];
  };
  // One phase: key tiles from `kfirst` (32-aligned) to last_pos; the wave's queries see keys [wlo, whi], and a
  // tile inside [full_lo, full_hi] is seen whole by every query of the wave (no mask).
  const int wq0 = q0 + wave * 16 * kQT;
  const bool wave_full = wq0 + 16 * kQT <= n;
  auto run = [&](int kfirst, int wlo, int whi, int full_lo, int full_hi) {
  fetch(kfirst);
  for (int k0 = kfirst; k0 <= last_pos; k0 += kTK) {
    __syncthreads();                       // every wave is done with the previous tile
    stage();
    __syncthreads();
    if (k0 + kTK <= last_pos) fetch(k0 + kTK);
    if (k0 <= whi && k0 + kTK - 1 >= wlo) {
      // ---- S^T = K Q^T: lane (col, grp) gets keys k0 + 8 grp + (0..7) of its query in each column tile
      f32x4 s0[kQT], s1[kQT];
#pragma unroll
      for (int c2 = 0; c2 < kQT; ++c2) s0[c2] = f32x4{0.f, 0.f, 0.f, 0.f}, s1[c2] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int s2 = 0; s2 < NQK; ++s2) {
        const bf16x8 ka = *reinterpret_cast<const bf16x8*>(ks + col * KROW + 32 * s2 + 8 * grp);
        const bf16x8 kb = *reinterpret_cast<const bf16x8*>(ks + (16 + col) * KROW + 32 * s2 + 8 * grp);
#pragma unroll
        for (int c2 = 0; c2 < kQT; ++c2) {
          s0[c2] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ka, qf[c2][s2], s0[c2], 0, 0, 0);
          s1[c2] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kb, qf[c2][s2], s1[c2], 0, 0, 0);
        }
      }
      const bool nomask = wave_full && k0 + kTK - 1 <= full_hi && k0 >= full_lo;    // wave-uniform
      bf16x8 ph[kQT], pl[kQT];
      float alpha[kQT];
#pragma unroll
      for (int c2 = 0; c2 < kQT; ++c2) {
        float p[8];
        float cm = -INFINITY;
#pragma unroll
        for (int i = 0; i < 8; ++i) {
          const float raw = i < 4 ? s0[c2][i] : s1[c2][i - 4];
          p[i] = softcap > 0.f ? fast_tanh(raw * cap_in) * cap_out : raw * sc2;      // wave-uniform choice
        }
        if (nomask) {                                      // wave-uniform: no per-element mask work
#pragma unroll
          for (int i = 0; i < 8; ++i) cm = fmaxf(cm, p[i]);
        } else {
#pragma unroll
          for (int i = 0; i < 8; ++i) {
            const int kp = k0 + 8 * grp + i;
            const bool ok = qok[c2] && kp <= hi_q[c2] && kp >= lo_q[c2];
            p[i] = ok ? p[i] : -INFINITY;
            cm = fmaxf(cm, p[i]);
          }
        }
        cm = rows_max(cm);
        const float m_new = fmaxf(m[c2], cm);
        const float m_use = m_new == -INFINITY ? 0.f : m_new;
        alpha[c2] = m[c2] == -INFINITY ? 0.f : __builtin_amdgcn_exp2f(m[c2] - m_new);
        float ps = 0.f;
#pragma unroll
        for (int i = 0; i < 8; ++i) {
          p[i] = __builtin_amdgcn_exp2f(p[i] - m_use);
          ps += p[i];
        }
        split_pack(p, ph[c2], pl[c2]);
        l[c2] = l[c2] * alpha[c2] + rows_sum(ps);
        m[c2] = m_new;
      }
      bool diff = false;
#pragma unroll
      for (int c2 = 0; c2 < kQT; ++c2) diff = diff || alpha[c2] != 1.0f;
      const bool rescale = __any(diff);
#pragma unroll
      for (int dt = 0; dt < NDV; ++dt) {
        if (16 * dt < Dv) {
          // A operand: V^T[channel 16 dt + col][keys 8 grp .. + 7]
          const bf16x8 va = *reinterpret_cast<const bf16x8*>(vs + (16 * dt + col) * VROW + 8 * grp);
#pragma unroll
          for (int c2 = 0; c2 < kQT; ++c2) {
            f32x4 a = acc[c2][dt];
            if (rescale) a *= alpha[c2];                   // wave-uniform: skipped once every row's maximum has settled
            a = __builtin_amdgcn_mfma_f32_16x16x32_bf16(va, ph[c2], a, 0, 0, 0);
            acc[c2][dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(va, pl[c2], a, 0, 0, 0);
          }
        }
      }
    }
  }
  };
  const int tile_last = start + min(q0 + kTQ, n) - 1;                  // position of the tile's last query
  const int wave_last = start + min(wq0 + 16 * kQT - 1, n - 1);        // of the wave's last query
  // ---- phase 1: the averaged entries (entry indices are the keys): query at p sees [0, npool(p) - 1]
  const int np_tile = win_npool(tile_last, window, pool);
  if (np_tile > 0) {                                                   // uniform over the workgroup
    ck = kp_cache, cv = vp_cache, cbs = pbs, cbsh = __ffs(pbs) - 1, last_pos = np_tile - 1;
#pragma unroll
    for (int c2 = 0; c2 < kQT; ++c2) lo_q[c2] = 0, hi_q[c2] = win_npool(qpos[c2], window, pool) - 1;
    run(0, 0, win_npool(wave_last, window, pool) - 1, 0, win_npool(start + wq0, window, pool) - 1);
    __syncthreads();                                                   // before the next phase's first fetch lands in LDS
  }
  // ---- phase 2: the tokens of the window
  {
    ck = k_cache, cv = v_cache, cbs = bs, cbsh = bsh, last_pos = tile_last;
#pragma unroll
    for (int c2 = 0; c2 < kQT; ++c2) lo_q[c2] = qlo[c2], hi_q[c2] = qpos[c2];
    const int first_pos = win_lo(start + q0, window, chunk);           // oldest key any query of the tile sees
    // keys the wave's queries see: [wlo, whi]; a tile whose keys every query of the wave sees needs no mask:
    // all keys <= the wave's first query's position and inside the window of its last one
    run(first_pos & ~(kTK - 1), win_lo(start + wq0, window, chunk), wave_last, win_lo(wave_last, window, chunk),
        start + wq0);
  }
  // O^T accumulator: lane (col, grp) holds channels 16 dt + 4 grp + (0..3) of its query
#pragma unroll
  for (int c2 = 0; c2 < kQT; ++c2) {
    if (!qok[c2]) continue;
    float inv = 1.0f / l[c2];
    if (sinks) {                                   // exp(sink) joins the denominator (scores here are in log2 units)
      const float sk = sinks[h] * kLog2e, mf = fmaxf(m[c2], sk), cf = __builtin_amdgcn_exp2f(m[c2] - mf);
      inv = cf / (l[c2] * cf + __builtin_amdgcn_exp2f(sk - mf));
    }
    bf16* orow = out + ((size_t)(lo_t + ql[c2]) * H + h) * Dv;
#pragma unroll
    for (int dt = 0; dt < NDV; ++dt) {
      const int e0 = 16 * dt + 4 * grp;
      if (e0 + 4 <= Dv) {
        bf16x4 o4;
#pragma unroll
        for (int i = 0; i < 4; ++i) o4[i] = (bf16)(acc[c2][dt][i] * inv);
        *reinterpret_cast<bf16x4*>(orow + e0) = o4;
      }
    }
  }
}

template <int NQK, int NDV, int QT>
static void launch_tile(uintptr_t out, uintptr_t q, uintptr_t k_cache, uintptr_t v_cache, uintptr_t block_tables,
                        int max_blocks, uintptr_t cu, uintptr_t positions, int seq0, int nseq, int max_q_len, int H,
                        int G, int D, int Dv, int bs, int window, int chunk, float scale, uintptr_t sinks, float softcap,
                        uintptr_t kp, uintptr_t vp, int pool, int pbs, uintptr_t stream) {
  constexpr int kTQ = 64 * QT;
  const int nqt = (max_q_len + kTQ - 1) / kTQ;
  const int pairs = nseq * G, per_pair = nqt * (H / G);
  const int sub = pairs < 8 ? 8 : 1;                                    // XCDs that share a pair's tiles
  const long per_xcd = (long)(((long)pairs * sub + 7) / 8) * ((per_pair + sub - 1) / sub);   // workgroups of one XCD
  DLLM_HOST_CHECK(per_xcd * 8 < (1L << 31), "window attention grid");
  hipLaunchKernelGGL(HIP_KERNEL_NAME(window_attn_tile_kernel<NQK, NDV, QT>), dim3((unsigned)(per_xcd * 8)),
                     dim3(256), 0, (hipStream_t)stream, (bf16*)out, (const bf16*)q, (const bf16*)k_cache,
                     (const bf16*)v_cache, (const int32_t*)block_tables, max_blocks, (const int32_t*)cu,
                     (const int32_t*)positions, seq0, nseq, nqt, H, G, D, Dv, bs, window, chunk, scale, (const float*)sinks, sub,
                     softcap, (const bf16*)kp, (const bf16*)vp, pool, pbs);
  DLLM_HIP_CHECK(hipGetLastError());
}

// --------------------------------------------------------------------------- MFMA decode kernel (bf16)
// One workgroup per (one-token sequence, K/V head, 16 query heads of its group): the 16 MFMA columns are
// query heads of the group, so the keys and values of a K/V head are read once for 16 of them.  The wave's key tiles
// (32 keys, tile index mod kDW = wave) go from global memory straight into MFMA fragments: K rows as
// the A operand of S^T = K Q^T (row r of a 16-key half holds the key that makes the accumulator hand
// each lane 8 consecutive keys), V^T pieces (8 keys of one channel, 16 bytes) as the A operand of
// O^T = V^T P^T.  Each wave keeps an online softmax; the waves' partial results meet in LDS.
constexpr int kDW = 4;

template <int NQK, int NDV>
__global__ void __launch_bounds__(64 * kDW) window_attn_decode_kernel(
    bf16* __restrict__ out, const bf16* __restrict__ q, const bf16* __restrict__ k_cache,
    const bf16* __restrict__ v_cache, const int32_t* __restrict__ block_tables, int max_blocks,
    const int32_t* __restrict__ positions, const int32_t* __restrict__ tok_seq, int H, int G, int D, int Dv, int bs,
    int window, int chunk, float scale, const float* __restrict__ sinks, int hpw, int splits, float* __restrict__ ws,
    float softcap, const bf16* __restrict__ kp_cache, const bf16* __restrict__ vp_cache, int pool, int pbs) {
  constexpr int DVP = 16 * NDV;
  __shared__ float so[kDW][16][DVP + 1];
  __shared__ float sml[kDW][2][16];
  // the query heads of a K/V head are dealt to workgroups hpw (<= 16) at a time: part p runs heads
  // hpw p .. of the group (fewer heads per workgroup when few rows would leave most CUs idle)
  const int t = blockIdx.x;
  const int R = H / G, parts = (R + hpw - 1) / hpw;
  const int g = blockIdx.y / parts, part = blockIdx.y - g * parts;
  const int hb = g * R + hpw * part, nh = min(hpw, R - hpw * part);    // first head and heads of this workgroup
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63, col = lane & 15, grp = lane >> 4;
  const int pos = positions[t], b = tok_seq[t];
  const int lo = win_lo(pos, window, chunk);
  const int bsh = __ffs(bs) - 1;                     // bs is a power of two here
  const int32_t* bt = block_tables + (size_t)b * max_blocks;
  bf16x8 qf[NQK];
  {
    const bf16* qrow = q + ((size_t)t * H + hb + min(col, nh - 1)) * D;
#pragma unroll
    for (int s2 = 0; s2 < NQK; ++s2) {
      const int d0 = 32 * s2 + 8 * grp;
      bf16x8 v;
#pragma unroll
      for (int j = 0; j < 8; ++j) v[j] = (bf16)0.f;
      if (d0 + 8 <= D && col < nh) v = *reinterpret_cast<const bf16x8*>(qrow + d0);
      qf[s2] = v;
    }
  }
  f32x4 acc[NDV];
#pragma unroll
  for (int i = 0; i < NDV; ++i) acc[i] = f32x4{0.f, 0.f, 0.f, 0.f};
  float m = -INFINITY, l = 0.f;
  // keys of this lane's A rows inside a tile: first half row col -> key 8 (col / 4) + col % 4, second half + 4
  const int jr = 8 * (col >> 2) + (col & 3);
  // The row's tiles of 32 keys: first the averaged entries (tiles 0 .. ptile - 1 over entries [0, np - 1] of
  // the averaged caches), then the window's tokens (tiles from the 32-aligned k00 over positions [lo, pos]).
  const int np = win_npool(pos, window, pool), ptile = (np + 31) >> 5;
  const int pbsh = pool > 0 ? __ffs(pbs) - 1 : 0;
  const int k00 = lo & ~31, ntile = ptile + ((pos - k00) >> 5) + 1;
  bf16x8 ka[NQK], kb[NQK];
  auto load_k = [&](int ti) {
    const bool pooled = ti < ptile;
    const int k0 = pooled ? 32 * ti : k00 + 32 * (ti - ptile), hi = pooled ? np - 1 : pos;
    const bf16* kc = pooled ? kp_cache : k_cache;
    const int cb = pooled ? pbs : bs, sh = pooled ? pbsh : bsh;
    const int j1 = min(k0 + jr, hi), j2 = min(k0 + jr + 4, hi);
    const bf16* r1 = kc + (((size_t)bt[j1 >> sh] * G + g) * cb + (j1 & (cb - 1))) * D;
    const bf16* r2 = kc + (((size_t)bt[j2 >> sh] * G + g) * cb + (j2 & (cb - 1))) * D;
#pragma unroll
    for (int s2 = 0; s2 < NQK; ++s2) {
      const int d0 = 32 * s2 + 8 * grp;
#pragma unroll
      for (int j = 0; j < 8; ++j) ka[s2][j] = kb[s2][j] = (bf16)0.f;
      if (d0 + 8 <= D) {
        ka[s2] = *reinterpret_cast<const bf16x8*>(r1 + d0);
        kb[s2] = *reinterpret_cast<const bf16x8*>(r2 + d0);
      }
    }
  };
  // the tiles are cut into `splits` runs, one per workgroup along z (long contexts of few
  // rows: the partial results meet in window_attn_merge_kernel); inside a run, tile index mod kDW = wave
  const int tps = (ntile + splits - 1) / splits;
  const int tstop = min(ntile, ((int)blockIdx.z + 1) * tps);
  const int tbeg = (int)blockIdx.z * tps + wave;
  const float cap_in = softcap > 0.f ? scale / softcap : 0.f;
  if (tbeg < tstop) load_k(tbeg);
  for (int ti = tbeg; ti < tstop; ti += kDW) {
    const bool pooled = ti < ptile;
    const int k0 = pooled ? 32 * ti : k00 + 32 * (ti - ptile);
    const int rlo = pooled ? 0 : lo, rhi = pooled ? np - 1 : pos;
    const bf16* vcache = pooled ? vp_cache : v_cache;
    const int cb = pooled ? pbs : bs, sh = pooled ? pbsh : bsh;
    // this tile's V^T pieces (8 keys from k0 + 8 grp, clamped to the last piece that exists) go out first
    const int kp8 = min(k0 + 8 * grp, rhi & ~7);
    const bf16* vbase = vcache + ((size_t)bt[kp8 >> sh] * G + g) * Dv * cb + (kp8 & (cb - 1));
    bf16x8 va[NDV];
#pragma unroll
    for (int dt = 0; dt < NDV; ++dt) {
      const int ch = 16 * dt + col;
#pragma unroll
      for (int j = 0; j < 8; ++j) va[dt][j] = (bf16)0.f;
      if (ch < Dv) va[dt] = *reinterpret_cast<const bf16x8*>(vbase + (size_t)ch * cb);
    }
    f32x4 s0 = {0.f, 0.f, 0.f, 0.f}, s1 = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int s2 = 0; s2 < NQK; ++s2) {
      if (32 * s2 < D) {
        s0 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ka[s2], qf[s2], s0, 0, 0, 0);
        s1 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kb[s2], qf[s2], s1, 0, 0, 0);
      }
    }
    // the wave's next tile's K rows are in flight during this tile's softmax and P.V
    if (ti + kDW < tstop) load_k(ti + kDW);
    float p[8];
    float cm = -INFINITY;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const int kp = k0 + 8 * grp + i;
      const float raw = i < 4 ? s0[i] : s1[i - 4];
      const float sv = softcap > 0.f ? softcap * fast_tanh(raw * cap_in) : raw * scale;
      p[i] = (kp >= rlo && kp <= rhi) ? sv : -INFINITY;
      cm = fmaxf(cm, p[i]);
    }
    cm = rows_max(cm);
    const float m_new = fmaxf(m, cm);
    const float m_use = m_new == -INFINITY ? 0.f : m_new;
    const float alpha = m == -INFINITY ? 0.f : expf(m - m_new);
    float ps = 0.f;
    bf16x8 ph, pl;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      p[i] = expf(p[i] - m_use);
      ps += p[i];
    }
    split_pack(p, ph, pl);
    l = l * alpha + rows_sum(ps);
    m = m_new;
#pragma unroll
    for (int dt = 0; dt < NDV; ++dt) {
      if (16 * dt < Dv) {
        f32x4 a = acc[dt] * alpha;
        a = __builtin_amdgcn_mfma_f32_16x16x32_bf16(va[dt], ph, a, 0, 0, 0);
        acc[dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(va[dt], pl, a, 0, 0, 0);
      }
    }
  }
  // partial results: lane (col, grp) holds channels 16 dt + 4 grp + i of head col
  if (grp == 0) sml[wave][0][col] = m, sml[wave][1][col] = l;
#pragma unroll
  for (int dt = 0; dt < NDV; ++dt)
#pragma unroll
    for (int i = 0; i < 4; ++i) so[wave][col][16 * dt + 4 * grp + i] = acc[dt][i];
  __syncthreads();
  for (int idx = tid; idx < nh * Dv; idx += 64 * kDW) {
    const int hh = idx / Dv, e = idx - hh * Dv;
    float mm = -INFINITY;
#pragma unroll
    for (int w = 0; w < kDW; ++w) mm = fmaxf(mm, sml[w][0][hh]);
    float ll = 0.f, o = 0.f;
    if (splits > 1) {                              // unnormalised partial: Dv sums, then their maximum and weight
#pragma unroll
      for (int w = 0; w < kDW; ++w) {
        const float f = sml[w][0][hh] == -INFINITY ? 0.f : expf(sml[w][0][hh] - mm);
        ll += sml[w][1][hh] * f;
        o += so[w][hh][e] * f;
      }
      float* part = ws + (((size_t)t * H + hb + hh) * splits + blockIdx.z) * (Dv + 2);
      part[e] = o;
      if (e == 0) part[Dv] = mm, part[Dv + 1] = ll;
      continue;
    }
    if (sinks) {                                   // exp(sink) joins the denominator
      const float sk = sinks[hb + hh];
      mm = fmaxf(mm, sk);
      ll = expf(sk - mm);
    }
#pragma unroll
    for (int w = 0; w < kDW; ++w) {
      const float f = sml[w][0][hh] == -INFINITY ? 0.f : expf(sml[w][0][hh] - mm);
      ll += sml[w][1][hh] * f;
      o += so[w][hh][e] * f;
    }
    out[((size_t)t * H + hb + hh) * Dv + e] = (bf16)(o / ll);
  }
}

// Sum of a row's partial results over the context splits: ws [rows, H, splits, Dv + 2] (Dv unnormalised
// sums relative to the split's maximum, the maximum, the weight sum) -> out [rows, H, Dv]
__global__ void __launch_bounds__(64) window_attn_merge_kernel(bf16* __restrict__ out, const float* __restrict__ ws,
                                                               int H, int Dv, int splits,
                                                               const float* __restrict__ sinks) {
  const int t = blockIdx.x, h = blockIdx.y;
  const float* part = ws + ((size_t)t * H + h) * splits * (Dv + 2);
  float mm = sinks ? sinks[h] : -INFINITY;
  for (int s2 = 0; s2 < splits; ++s2) mm = fmaxf(mm, part[s2 * (Dv + 2) + Dv]);
  float ll = sinks ? expf(sinks[h] - mm) : 0.f;
  for (int s2 = 0; s2 < splits; ++s2) {
    const float m = part[s2 * (Dv + 2) + Dv];
    if (m != -INFINITY) ll += part[s2 * (Dv + 2) + Dv + 1] * expf(m - mm);
  }
  for (int e = threadIdx.x; e < Dv; e += 64) {
    float o = 0.f;
    for (int s2 = 0; s2 < splits; ++s2) {
      const float m = part[s2 * (Dv + 2) + Dv];
      if (m != -INFINITY) o += part[s2 * (Dv + 2) + e] * expf(m - mm);
    }
    out[((size_t)t * H + h) * Dv + e] = (bf16)(o / ll);
  }
}

template <int NQK, int NDV>
static void launch_decode(uintptr_t out, uintptr_t q, uintptr_t k_cache, uintptr_t v_cache, uintptr_t block_tables,
                          int max_blocks, uintptr_t positions, uintptr_t tok_seq, int rows, int H, int G, int D,
                          int Dv, int bs, int window, int chunk, float scale, uintptr_t sinks, int splits, uintptr_t ws,
                          float softcap, uintptr_t kp, uintptr_t vp, int pool, int pbs, uintptr_t stream) {
  // heads per workgroup: 16 (all MFMA columns) when rows x K/V heads x key runs fill the chip, else halved
  // until about half the CUs have a workgroup -- the keys are re-read from L2, the columns left idle cost
  // nothing.  Key runs come first: a workgroup holds a CU's registers alone, so the call takes
  // (workgroups / CUs) rounds of one run's load chain, and head groups multiply the rounds, runs shorten them.
  const int R = H / G;
  splits = ws ? std::max(1, std::min(splits, 64)) : 1;
  int hpw = std::min(16, R);
  while (hpw > 2 && (long)rows * G * ((R + hpw - 1) / hpw) * splits < 128) hpw = (hpw + 1) / 2;
  hipLaunchKernelGGL(HIP_KERNEL_NAME(window_attn_decode_kernel<NQK, NDV>),
                     dim3(rows, G * ((R + hpw - 1) / hpw), splits), dim3(64 * kDW), 0,
                     (hipStream_t)stream, (bf16*)out, (const bf16*)q, (const bf16*)k_cache, (const bf16*)v_cache,
                     (const int32_t*)block_tables, max_blocks, (const int32_t*)positions, (const int32_t*)tok_seq, H, G,
                     D, Dv, bs, window, chunk, scale, (const float*)sinks, hpw, splits, (float*)ws, softcap, (const bf16*)kp,
                     (const bf16*)vp, pool, pbs);
  DLLM_HIP_CHECK(hipGetLastError());
  if (splits > 1) {
    hipLaunchKernelGGL(window_attn_merge_kernel, dim3(rows, H), dim3(64), 0, (hipStream_t)stream, (bf16*)out,
                       (const float*)ws, H, Dv, splits, (const float*)sinks);
    DLLM_HIP_CHECK(hipGetLastError());
  }
}

// bf16 with 16-byte rows and pieces goes to the matrix cores; float32 (the exact path), odd head sizes
// and heads wider than 256 take the row kernel
static bool win_mfma_ok(int f32, int H, int G, int D, int Dv, int bs, int pool, int pbs) {
  return !f32 && D % 8 == 0 && Dv % 8 == 0 && bs % 8 == 0 && (bs & (bs - 1)) == 0 && D <= 256 && Dv <= 256 && G > 0 &&
         H % G == 0 && (pool == 0 || (pbs % 8 == 0 && (pbs & (pbs - 1)) == 0));
}

// Decode rows: tokens [0, rows) are one-token sequences.  `splits` > 1 with `ws` (float32
// [rows, H, splits, Dv + 2]) cuts every row's keys into that many runs on separate workgroups (the MFMA
// kernel only; the row kernel ignores it).
void sm_window_attn_decode(uintptr_t out, uintptr_t q, uintptr_t k_cache, uintptr_t v_cache, uintptr_t block_tables,
                           int max_blocks, uintptr_t positions, uintptr_t tok_seq, int rows, int H, int G, int D,
                           int Dv, int bs, int window, int chunk, float scale, uintptr_t sinks, int splits, uintptr_t ws,
                           float softcap, uintptr_t kp, uintptr_t vp, int pool, int pbs, int f32, uintptr_t stream) {
  if (rows <= 0) return;
  if (win_mfma_ok(f32, H, G, D, Dv, bs, pool, pbs) && (long)G * ((H / G + 1) / 2) <= 65535) {
    DLLM_HOST_CHECK(window >= 1 && chunk >= 0 && max_blocks > 0, "window attention sizes");
    DLLM_HOST_CHECK(pool == 0 || (pool > 0 && kp && vp && chunk == 0), "window attention averaged caches");
#define WIN_DEC(NQK, NDV)                                                                                       \
  launch_decode<NQK, NDV>(out, q, k_cache, v_cache, block_tables, max_blocks, positions, tok_seq, rows, H, G, D, Dv, \
                          bs, window, chunk, scale, sinks, splits, ws, softcap, kp, vp, pool, pbs, stream)
    if (D <= 64 && Dv <= 64) WIN_DEC(2, 4);
    else if (D <= 128 && Dv <= 128) WIN_DEC(4, 8);
    else WIN_DEC(8, 16);
#undef WIN_DEC
    return;
  }
  launch_rows(out, q, k_cache, v_cache, block_tables, max_blocks, positions, tok_seq, 0, rows, H, G, D, Dv, bs, window,
              chunk, scale, sinks, softcap, kp, vp, pool, pbs, f32, stream);
}

// Prompt chunks: tokens [t0 .. tokens) of sequences [seq0, seqs).
void sm_window_attn_prefill(uintptr_t out, uintptr_t q, uintptr_t k_cache, uintptr_t v_cache, uintptr_t block_tables,
                            int max_blocks, uintptr_t cu, uintptr_t positions, uintptr_t tok_seq, int seq0, int seqs,
                            int tokens, int max_q_len, int H, int G, int D, int Dv, int bs, int window, int chunk,
                            float scale, uintptr_t sinks, float softcap, uintptr_t kp, uintptr_t vp, int pool, int pbs,
                            int f32, uintptr_t stream) {
  // tokens of the decode rows come first: one per sequence before seq0
  const int t0 = seq0;
  if (tokens <= t0) return;
  if (win_mfma_ok(f32, H, G, D, Dv, bs, pool, pbs) && seqs > seq0 && max_q_len > 1) {
    DLLM_HOST_CHECK(H > 0 && G > 0 && H % G == 0 && H <= 65535 && seqs - seq0 <= 65535, "window attention heads");
    DLLM_HOST_CHECK(bs > 0 && window >= 1 && chunk >= 0 && max_blocks > 0, "window attention sizes");
    DLLM_HOST_CHECK(pool == 0 || (pool > 0 && kp && vp && chunk == 0), "window attention averaged caches");
#define WIN_TILE(NQK, NDV, QT)                                                                                  \
  launch_tile<NQK, NDV, QT>(out, q, k_cache, v_cache, block_tables, max_blocks, cu, positions, seq0, seqs - seq0, \
                            max_q_len, H, G, D, Dv, bs, window, chunk, scale, sinks, softcap, kp, vp, pool, pbs, stream)
    if (D <= 64 && Dv <= 64) WIN_TILE(2, 4, 1);
    else if (D <= 128 && Dv <= 128) WIN_TILE(4, 8, 1);
    else WIN_TILE(8, 16, 2);     // wide heads: 2b-size latent attention prompts 32 x 1024 +7 %, 4 x 4096 +29 % over QT = 1
#undef WIN_TILE
    return;
  }
  launch_rows(out, q, k_cache, v_cache, block_tables, max_blocks, positions, tok_seq, t0, tokens - t0, H, G, D, Dv, bs,
              window, chunk, scale, sinks, softcap, kp, vp, pool, pbs, f32, stream);
}

}  // namespace dllm
