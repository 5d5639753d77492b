// K11 + K12: Mixtral mixture-of-experts on gfx950, graph-capturable (no host round trip).
//
//  moe_route    : router logits [T,E] -> softmax -> top-k -> renormalise (Mixtral); per-expert
//                 counts, offsets and the expert-sorted assignment list (slot -> token) plus the
//                 inverse map ((t,j) -> slot), in ONE 1024-thread workgroup (LDS counters + scan).
//  moe_grouped  : per-expert weight-streaming GEMM (grid = column tiles x experts), A rows
//                 gathered through the sorted list, rows processed in 64-row chunks; epilogue
//                 SwiGLU (gate|up experts weight [E, 2I, H]) or plain store (down [E, H, I]).
//                 Every expert's weights stream once per chunk; the decode regime has <= 64 rows
//                 per expert, i.e. one pass.
//  moe_combine  : out[t] = sum_j w[t,j] * y[inv[t,j]]   (fixed j order: deterministic)
#include "skinny_common.h"
#include "launchers.h"
#include "stream_common.h"

namespace dllm {

constexpr int kMaxExperts = 64;

__global__ void __launch_bounds__(1024) moe_route_kernel(const bf16* __restrict__ logits, int T, int E, int k,
                                                         float* __restrict__ topk_w, int* __restrict__ topk_ids,
                                                         int* __restrict__ counts, int* __restrict__ offsets,
                                                         int* __restrict__ sorted_tok, int* __restrict__ inv) {
  __shared__ int cnt[kMaxExperts], cur[kMaxExperts];
  for (int e = threadIdx.x; e < E; e += blockDim.x) cnt[e] = 0;
  __syncthreads();
  for (int t = threadIdx.x; t < T; t += blockDim.x) {
    float p[kMaxExperts];
    float mx = -INFINITY;
    for (int e = 0; e < E; ++e) {
      p[e] = bf2f(logits[(size_t)t * E + e]);
      mx = fmaxf(mx, p[e]);
    }
    float s = 0.f;
    for (int e = 0; e < E; ++e) {
      p[e] = __expf(p[e] - mx);
      s += p[e];
    }
    float tot = 0.f;
    int ids[8];
    float ws[8];
    for (int j = 0; j < k; ++j) {
      int best = 0;
      float bv = -1.f;
      for (int e = 0; e < E; ++e)
        if (p[e] > bv) { bv = p[e]; best = e; }
      ids[j] = best;
      ws[j] = bv / s;
      tot += ws[j];
      p[best] = -2.f;
    }
    for (int j = 0; j < k; ++j) {
      topk_ids[t * k + j] = ids[j];
      topk_w[t * k + j] = ws[j] / tot;
      atomicAdd(&cnt[ids[j]], 1);
    }
  }
  __syncthreads();
  if (threadIdx.x == 0) {
    int acc = 0;
    for (int e = 0; e < E; ++e) {
      offsets[e] = acc;
      cur[e] = acc;
      counts[e] = cnt[e];
      acc += cnt[e];
    }
    offsets[E] = acc;
  }
  __syncthreads();
  for (int t = threadIdx.x; t < T; t += blockDim.x) {
    for (int j = 0; j < k; ++j) {
      const int e = topk_ids[t * k + j];
      const int slot = atomicAdd(&cur[e], 1);
      sorted_tok[slot] = t;
      inv[t * k + j] = slot;
    }
  }
}

// Router GEMV + top-k fused (decode): one wave per token computes its E router logits
// (H split over the 64 lanes, 16-B loads, wave reductions), rounds them to bf16 like the
// library-GEMM path it replaces, then lane 0 applies softmax -> top-k -> renormalise.
// moe_scatter_kernel (one workgroup) then counts per expert in LDS, scans, and writes the
// offsets and the expert-sorted slot lists (no global counters: nothing to zero first, so the
// pair stays a plain two-node piece of a captured graph).  Replaces linear(x, W_router) + the single-workgroup moe_route_kernel
// (14 + 11 us per layer at T = 256).
template <int E>
__global__ void __launch_bounds__(256) moe_router_kernel(const bf16* __restrict__ x, const bf16* __restrict__ w, int T,
                                                         int H, int k, float* __restrict__ topk_w,
                                                         int* __restrict__ topk_ids) {
  // one workgroup per token, the 4 waves split H (a wave per token left 3/4 of the CUs idle at
  // T = 256 and walked 8 dependent load rounds: 10.5 us per Mixtral layer)
  __shared__ float part[4][E];
  const int lane = threadIdx.x & 63, wv = threadIdx.x >> 6;
  const int t = blockIdx.x;
  float acc[E];
#pragma unroll
  for (int e = 0; e < E; ++e) acc[e] = 0.f;
  const bf16* xr = x + (size_t)t * H;
  const int hq = H / 4;
  for (int c = wv * hq + lane * 8; c < (wv + 1) * hq; c += 64 * 8) {
    const bf16x8 xv = *reinterpret_cast<const bf16x8*>(xr + c);
#pragma unroll
    for (int e = 0; e < E; ++e) {
      const bf16x8 wt = *reinterpret_cast<const bf16x8*>(w + (size_t)e * H + c);
#pragma unroll
      for (int i = 0; i < 8; ++i) acc[e] += bf2f(xv[i]) * bf2f(wt[i]);
    }
  }
#pragma unroll
  for (int e = 0; e < E; ++e) acc[e] = wave_sum(acc[e]);
  if (lane == 0) {
#pragma unroll
    for (int e = 0; e < E; ++e) part[wv][e] = acc[e];
  }
  __syncthreads();
  if (threadIdx.x != 0) return;
  float p[E];
  float mx = -INFINITY;
#pragma unroll
  for (int e = 0; e < E; ++e) {
    p[e] = bf2f(f2bf(((part[0][e] + part[1][e]) + part[2][e]) + part[3][e]));
    mx = fmaxf(mx, p[e]);
  }
  float sum = 0.f;
#pragma unroll
  for (int e = 0; e < E; ++e) {
    p[e] = __expf(p[e] - mx);
    sum += p[e];
  }
  int ids[8];
  float ws[8];
  float tot = 0.f;
  for (int j = 0; j < k; ++j) {
    int best = 0;
    float bv = -1.f;
#pragma unroll
    for (int e = 0; e < E; ++e)
      if (p[e] > bv) { bv = p[e]; best = e; }
    ids[j] = best;
    ws[j] = bv / sum;
    tot += ws[j];
    p[best] = -2.f;
  }
  for (int j = 0; j < k; ++j) {
    topk_ids[t * k + j] = ids[j];
    topk_w[t * k + j] = ws[j] / tot;
  }
}

__global__ void __launch_bounds__(1024) moe_scatter_kernel(const int* __restrict__ topk_ids, int T, int E, int k,
                                                           int* __restrict__ counts, int* __restrict__ offsets,
                                                           int* __restrict__ sorted_tok, int* __restrict__ inv) {
  __shared__ int cnt[kMaxExperts], cur[kMaxExperts];
  for (int e = threadIdx.x; e < E; e += blockDim.x) cnt[e] = 0;
  __syncthreads();
  for (int i = threadIdx.x; i < T * k; i += blockDim.x) atomicAdd(&cnt[topk_ids[i]], 1);
  __syncthreads();
  if (threadIdx.x == 0) {
    int acc = 0;
    for (int e = 0; e < E; ++e) {
      offsets[e] = acc;
      cur[e] = acc;
      counts[e] = cnt[e];
      acc += cnt[e];
    }
    offsets[E] = acc;
  }
  __syncthreads();
  for (int i = threadIdx.x; i < T * k; i += blockDim.x) {
    const int slot = atomicAdd(&cur[topk_ids[i]], 1);
    sorted_tok[slot] = i / k;
    inv[i] = slot;
  }
}

constexpr int MOE_EPI_STORE = 0;
constexpr int MOE_EPI_SWIGLU = 1;
constexpr int MOE_EPI_RELU2 = 2;          // store max(v, 0)^2: the activation of two-matrix experts

// Rows [0, cnt) of one expert in chunks of MT*16 rows; every chunk streams the WG's W column
// tile once (K split over the WAVES waves, partial tiles summed through LDS).
template <int MT, int NT, int WAVES, int EPI>
__device__ __forceinline__ void moe_rows(float* red, bf16* __restrict__ y, const bf16* __restrict__ x,
                                         const int* __restrict__ gather, const bf16* const (&wrow)[NT], int cnt,
                                         int off, int K, int ldy, int g0, int g1, int lane) {
  constexpr int BM = MT * 16, BN = NT * 16, NTHR = WAVES * 64;
  const int r = lane & 15, g = lane >> 4;
  for (int r0 = 0; r0 < cnt; r0 += BM) {
    const int rows = min(BM, cnt - r0);
    for (int i = threadIdx.x; i < BM * BN; i += NTHR) red[i] = 0.f;
    const bf16* xrow[MT];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
      const int slot = off + r0 + min(mt * 16 + r, rows - 1);
      const int src = gather ? gather[slot] : slot;
      xrow[mt] = x + (size_t)src * K + 8 * g;
    }
    f32x4 acc[MT][NT];
    sk_mainloop<MT, NT>(acc, xrow, wrow, g0, g1);
    __syncthreads();
    sk_reduce_lds<MT, NT, WAVES>(red, acc, lane, threadIdx.x >> 6);
    if (EPI == MOE_EPI_SWIGLU) {
      constexpr int HB = BN / 2;
      for (int q = threadIdx.x; q < rows * HB; q += NTHR) {
        const int m = q / HB, c = q % HB;
        y[(size_t)(off + r0 + m) * ldy + blockIdx.x * HB + c] = f2bf(silu_f(red[m * BN + c]) * red[m * BN + HB + c]);
      }
    } else {
      for (int q = threadIdx.x; q < rows * BN; q += NTHR) {
        const int m = q / BN, c = q % BN;
        float v = red[m * BN + c];
        if (EPI == MOE_EPI_RELU2) v = fmaxf(v, 0.f) * fmaxf(v, 0.f);
        y[(size_t)(off + r0 + m) * ldy + blockIdx.x * BN + c] = f2bf(v);
      }
    }
    __syncthreads();
  }
}

// Grouped expert GEMM: grid (N / (NT*16), E).  The row tile is chosen PER EXPERT from its
// actual count (a workgroup-uniform branch): 16-row tiles for <= 16 rows, 32 for <= 32, else
// MTMAX*16-row chunks -- so routing imbalance never makes an expert re-stream its weights
// while it fits one chunk, and a decode expert with 10 rows does not gather 64.
template <int MTMAX, int NT, int WAVES, int EPI>
__global__ void __launch_bounds__(WAVES * 64, 1) moe_grouped_kernel(bf16* __restrict__ y, const bf16* __restrict__ x,
                                                                    const int* __restrict__ gather,
                                                                    const bf16* __restrict__ w,
                                                                    const int* __restrict__ counts,
                                                                    const int* __restrict__ offsets, int N, int K,
                                                                    int ldy) {
  constexpr int BN = NT * 16;
  __shared__ __attribute__((aligned(16))) float red[MTMAX * 16 * BN];
  const int e = blockIdx.y;
  const int cnt = counts[e];
  if (cnt == 0) return;                       // uniform across the workgroup
  const int off = offsets[e];
  const int lane = threadIdx.x & 63, wv = threadIdx.x >> 6;
  const int r = lane & 15, g = lane >> 4;
  const bf16* we = w + (size_t)e * N * K;
  const bf16* wrow[NT];
#pragma unroll
  for (int nt = 0; nt < NT; ++nt) {
    int n0;
    if (EPI == MOE_EPI_SWIGLU) n0 = (nt < NT / 2 ? 0 : N / 2) + blockIdx.x * (BN / 2) + (nt % (NT / 2)) * 16;
    else n0 = blockIdx.x * BN + nt * 16;
    wrow[nt] = we + (size_t)(n0 + r) * K + 8 * g;
  }
  const int ngroups = K >> 7;
  const int per = (ngroups + WAVES - 1) / WAVES;
  const int g0 = wv * per, g1 = min(ngroups, g0 + per);
  if (MTMAX == 1 || cnt <= 16) {
    moe_rows<1, NT, WAVES, EPI>(red, y, x, gather, wrow, cnt, off, K, ldy, g0, g1, lane);
  } else if constexpr (MTMAX >= 2) {
    if (MTMAX == 2 || cnt <= 32) moe_rows<2, NT, WAVES, EPI>(red, y, x, gather, wrow, cnt, off, K, ldy, g0, g1, lane);
    else if constexpr (MTMAX >= 4) moe_rows<4, NT, WAVES, EPI>(red, y, x, gather, wrow, cnt, off, K, ldy, g0, g1, lane);
  }
}

__global__ void __launch_bounds__(256) moe_combine_kernel(bf16* __restrict__ out, const bf16* __restrict__ ysorted,
                                                          const float* __restrict__ topk_w,
                                                          const int* __restrict__ inv, int H, int k) {
  const int t = blockIdx.x;
  for (int v = threadIdx.x; v < (H >> 3); v += 256) {
    float acc[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
    for (int j = 0; j < k; ++j) {
      const float wj = topk_w[t * k + j];
      const bf16x8 yv = *reinterpret_cast<const bf16x8*>(ysorted + (size_t)inv[t * k + j] * H + v * 8);
#pragma unroll
      for (int i = 0; i < 8; ++i) acc[i] += wj * bf2f(yv[i]);
    }
    bf16x8 o;
#pragma unroll
    for (int i = 0; i < 8; ++i) o[i] = f2bf(acc[i]);
    *reinterpret_cast<bf16x8*>(out + (size_t)t * H + v * 8) = o;
  }
}

// ------------------------------------------------------------------ launchers
void moe_route(uintptr_t logits, int T, int E, int k, uintptr_t topk_w, uintptr_t topk_ids, uintptr_t counts,
               uintptr_t offsets, uintptr_t sorted_tok, uintptr_t inv, uintptr_t stream) {
  DLLM_HOST_CHECK(E >= 1 && E <= kMaxExperts, "1 <= experts <= 64");
  DLLM_HOST_CHECK(k >= 1 && k <= 8 && k <= E, "1 <= top_k <= min(8, experts)");
  hipLaunchKernelGGL(moe_route_kernel, dim3(1), dim3(1024), 0, reinterpret_cast<hipStream_t>(stream),
                     (const bf16*)logits, T, E, k, (float*)topk_w, (int*)topk_ids, (int*)counts, (int*)offsets,
                     (int*)sorted_tok, (int*)inv);
  DLLM_HIP_CHECK(hipGetLastError());
}

// router GEMV + top-k + scatter (decode): x [T, H], w_router [E, H]
void moe_router_route(uintptr_t x, uintptr_t w, int T, int H, int E, int k, uintptr_t topk_w, uintptr_t topk_ids,
                      uintptr_t counts, uintptr_t offsets, uintptr_t sorted_tok, uintptr_t inv, uintptr_t stream) {
  DLLM_HOST_CHECK(E == 8 || E == 16, "fused router: 8 or 16 experts");
  DLLM_HOST_CHECK(k >= 1 && k <= 8 && k <= E, "1 <= top_k <= min(8, experts)");
  DLLM_HOST_CHECK(H % 8 == 0, "H % 8");
  if (T == 0) return;
  hipStream_t s = reinterpret_cast<hipStream_t>(stream);
  DLLM_HOST_CHECK(H % 32 == 0, "router: H % 32 (4 waves x 8-element vectors)");
  const dim3 grid(T);
  if (E == 8)
    hipLaunchKernelGGL(moe_router_kernel<8>, grid, dim3(256), 0, s, (const bf16*)x, (const bf16*)w, T, H, k,
                       (float*)topk_w, (int*)topk_ids);
  else
    hipLaunchKernelGGL(moe_router_kernel<16>, grid, dim3(256), 0, s, (const bf16*)x, (const bf16*)w, T, H, k,
                       (float*)topk_w, (int*)topk_ids);
  DLLM_HIP_CHECK(hipGetLastError());
  hipLaunchKernelGGL(moe_scatter_kernel, dim3(1), dim3(1024), 0, s, (const int*)topk_ids, T, E, k, (int*)counts,
                     (int*)offsets, (int*)sorted_tok, (int*)inv);
  DLLM_HIP_CHECK(hipGetLastError());
}

template <int MTMAX, int NT, int WAVES>
static void launch_grouped(hipStream_t s, bf16* y, const bf16* x, const int* gather, const bf16* w, const int* counts,
                           const int* offsets, int E, int N, int K, int mode) {
  constexpr int BN = NT * 16;
  if (mode == 1) {
    DLLM_HOST_CHECK(N % BN == 0, "moe grouped: 2I must be a multiple of the column tile");
    hipLaunchKernelGGL((moe_grouped_kernel<MTMAX, NT, WAVES, MOE_EPI_SWIGLU>), dim3(N / BN, E), dim3(WAVES * 64), 0,
                       s, y, x, gather, w, counts, offsets, N, K, N / 2);
  } else if (mode == 2) {
    DLLM_HOST_CHECK(N % BN == 0, "moe grouped: N must be a multiple of the column tile");
    hipLaunchKernelGGL((moe_grouped_kernel<MTMAX, NT, WAVES, MOE_EPI_RELU2>), dim3(N / BN, E), dim3(WAVES * 64), 0, s,
                       y, x, gather, w, counts, offsets, N, K, N);
  } else {
    DLLM_HOST_CHECK(N % BN == 0, "moe grouped: N must be a multiple of the column tile");
    hipLaunchKernelGGL((moe_grouped_kernel<MTMAX, NT, WAVES, MOE_EPI_STORE>), dim3(N / BN, E), dim3(WAVES * 64), 0, s,
                       y, x, gather, w, counts, offsets, N, K, N);
  }
}

// mode 1 (SwiGLU): w [E, 2I, K] -> y [T*k, I]; mode 0: w [E, N, K] -> y [T*k, N]; mode 2: as 0, storing max(v, 0)^2.
// rows_hint = expected rows per expert (T*k/E) picks the kernel family; variant > 0 forces one
// (benchmarking: 1 = <1,4,8>, 2 = <2,4,8>, 3 = <4,2,8>, 4 = <2,4,4>, 5 = <4,4,4>, 6 = <2,2,8>).
void moe_grouped_gemm(uintptr_t y, uintptr_t x, uintptr_t gather, uintptr_t w, uintptr_t counts, uintptr_t offsets,
                      int E, int N, int K, int mode, int rows_hint, int variant, uintptr_t stream) {
  DLLM_HOST_CHECK(K % 128 == 0, "K % 128");
  DLLM_HOST_CHECK(N % 64 == 0, "N % 64");   // every column tile (32 or 64) divides N
  hipStream_t s = reinterpret_cast<hipStream_t>(stream);
  auto args = [&](auto f) {
    f(s, (bf16*)y, (const bf16*)x, (const int*)gather, (const bf16*)w, (const int*)counts, (const int*)offsets, E, N,
      K, mode);
  };
  // measured (bench/moe_bench.py, Mixtral shapes): 4-wave <4,4,4> is best or tied at every
  // decode token count -- 4.4 TB/s at T=16, 3.8 at T=64, 3.0 at T=128 -- the 8-wave forms
  // spill and split K too finely (profiles/moe_grouped_variants.txt)
  (void)rows_hint;
  if (variant <= 0) variant = 5;
  switch (variant) {
    case 1: args(launch_grouped<1, 4, 8>); break;
    case 2: args(launch_grouped<2, 4, 8>); break;
    case 3: args(launch_grouped<4, 2, 8>); break;
    case 4: args(launch_grouped<2, 4, 4>); break;
    case 5: args(launch_grouped<4, 4, 4>); break;
    case 6: args(launch_grouped<2, 2, 8>); break;
    default: DLLM_HOST_CHECK(false, "moe grouped: unknown variant");
  }
  DLLM_HIP_CHECK(hipGetLastError());
}

void moe_combine(uintptr_t out, uintptr_t ysorted, uintptr_t topk_w, uintptr_t inv, int T, int H, int k,
                 uintptr_t stream) {
  DLLM_HOST_CHECK(H % 8 == 0, "H % 8");
  if (T == 0) return;
  hipLaunchKernelGGL(moe_combine_kernel, dim3(T), dim3(256), 0, reinterpret_cast<hipStream_t>(stream), (bf16*)out,
                     (const bf16*)ysorted, (const float*)topk_w, (const int*)inv, H, k);
  DLLM_HIP_CHECK(hipGetLastError());
}

// ------------------------------------------------------------------ grouped-choice router
// s = sigmoid(logit) (float32 logits [T, ld], the first E columns).  SELECTION ranks s + correction[e]:
// the experts are split into `groups` contiguous blocks of equal size, blocks are ranked by the sum of
// their top two selection values, experts outside the `keep` highest-ranked blocks are masked with -inf,
// and the k highest remaining values are selected.  The mixing WEIGHTS are the selected experts' plain
// s, normalised to sum one (+ 1e-20 in the divisor) and multiplied by `scale`.  One thread per token, 128 tokens per
// workgroup; moe_scatter_wide_kernel (one workgroup, LDS counters) then makes the counts / offsets /
// expert-sorted slot lists that the grouped GEMMs and the combine read.
// `softmax_top` != 0 is the other router form: selection ranks the logits plus `correction` (here a bias
// that is part of the logit), and the mixing weights are the softmax over the selected logits only,
// times `scale`; groups do not apply.
constexpr int kMaxGroups = 64;
constexpr int kMaxChoiceExperts = 256;

// one token's selection from its E logits `lg`
template <int EMAX>
__device__ __forceinline__ void choose_groups(const float* __restrict__ lg, const float* __restrict__ correction, int E,
                                              int k, int groups, int keep, float scale, int softmax_top,
                                              float* __restrict__ tw, int* __restrict__ ti) {
  const int gsz = E / groups;
  float sc[EMAX], ch[EMAX];
  for (int e = 0; e < E; ++e) {
    if (softmax_top) {
      sc[e] = ch[e] = lg[e] + (correction ? correction[e] : 0.f);
    } else {
      sc[e] = 1.0f / (1.0f + expf(-lg[e]));
      ch[e] = sc[e] + (correction ? correction[e] : 0.f);
    }
  }
  if (keep < groups && !softmax_top) {
    float gs[kMaxGroups];
    for (int g = 0; g < groups; ++g) {
      float a = -INFINITY, b = -INFINITY;          // top two of the block
      for (int e = g * gsz; e < (g + 1) * gsz; ++e) {
        if (ch[e] > a) { b = a; a = ch[e]; }
        else if (ch[e] > b) b = ch[e];
      }
      gs[g] = gsz > 1 ? a + b : a;
    }
    unsigned long long kept = 0ull;
    for (int j = 0; j < keep; ++j) {
      int best = -1;
      float bv = -INFINITY;
      for (int g = 0; g < groups; ++g)
        if (!((kept >> g) & 1ull) && (best < 0 || gs[g] > bv)) { bv = gs[g]; best = g; }
      kept |= 1ull << best;
    }
    for (int g = 0; g < groups; ++g)
      if (!((kept >> g) & 1ull))
        for (int e = g * gsz; e < (g + 1) * gsz; ++e) ch[e] = -INFINITY;
  }
  int ids[16];
  float tot = 0.f;
  for (int j = 0; j < k; ++j) {
    int best = -1;
    float bv = -INFINITY;
    for (int e = 0; e < E; ++e) {
      bool taken = false;
      for (int i = 0; i < j; ++i) taken = taken || ids[i] == e;
      if (!taken && (best < 0 || ch[e] > bv)) { bv = ch[e]; best = e; }
    }
    ids[j] = best;
    tot += softmax_top ? expf(sc[best] - sc[ids[0]]) : sc[best];      // ids[0] holds the largest logit
  }
  for (int j = 0; j < k; ++j) {
    ti[j] = ids[j];
    tw[j] = softmax_top ? expf(sc[ids[j]] - sc[ids[0]]) / tot * scale : sc[ids[j]] / (tot + 1e-20f) * scale;
  }
}

template <int EMAX>
__global__ void __launch_bounds__(128) moe_choice_groups_kernel(
    const float* __restrict__ logits, long ld, const float* __restrict__ correction, int T, int E, int k, int groups,
    int keep, float scale, int softmax_top, float* __restrict__ topk_w, int* __restrict__ topk_ids) {
  const int t = blockIdx.x * 128 + threadIdx.x;
  if (t >= T) return;
  choose_groups<EMAX>(logits + (size_t)t * ld, correction, E, k, groups, keep, scale, softmax_top,
                      topk_w + (size_t)t * k, topk_ids + (size_t)t * k);
}

// Few tokens (decode steps): the router product and the selection in one launch, a workgroup per token.
// x [T, K] (bf16 or float) times the float32 rows w [rows, K] (the E router rows, then any further rows
// such as a shared expert's gate), float32 sums, written to logits [T, rows]; then one thread selects.
template <typename TX, int EMAX>
__global__ void __launch_bounds__(256) moe_router_groups_kernel(
    const TX* __restrict__ x, const float* __restrict__ w, int K, int rows, float* __restrict__ logits,
    const float* __restrict__ correction, int E, int k, int groups, int keep, float scale, int softmax_top,
    float* __restrict__ topk_w, int* __restrict__ topk_ids) {
  __shared__ float lg[kMaxChoiceExperts + 8];
  const int t = blockIdx.x, lane = threadIdx.x & 63, wv = threadIdx.x >> 6;
  const TX* xr = x + (size_t)t * K;
  for (int r = wv; r < rows; r += 4) {
    const float* wr = w + (size_t)r * K;
    float acc = 0.f;
    if ((K & 7) == 0) {                            // 8 elements per lane and step: 16- and 32-byte loads
      for (int c = lane * 8; c < K; c += 512) {
        float xv[8], wv8[8];
        ldv<8>(xr + c, xv);
        ldv<8>(wr + c, wv8);
#pragma unroll
        for (int i = 0; i < 8; ++i) acc = fmaf(xv[i], wv8[i], acc);
      }
    } else {
      for (int c = lane; c < K; c += 64) acc = fmaf((float)xr[c], wr[c], acc);
    }
    acc = wave_sum(acc);
    if (lane == 0) {
      lg[r] = acc;
      logits[(size_t)t * rows + r] = acc;
    }
  }
  __syncthreads();
  if (threadIdx.x == 0)
    choose_groups<EMAX>(lg, correction, E, k, groups, keep, scale, softmax_top, topk_w + (size_t)t * k,
                        topk_ids + (size_t)t * k);
}

__global__ void __launch_bounds__(1024) moe_scatter_wide_kernel(const int* __restrict__ topk_ids, int T, int E, int k,
                                                                int* __restrict__ counts, int* __restrict__ offsets,
                                                                int* __restrict__ sorted_tok, int* __restrict__ inv) {
  __shared__ int cnt[kMaxChoiceExperts], cur[kMaxChoiceExperts];
  for (int e = threadIdx.x; e < E; e += blockDim.x) cnt[e] = 0;
  __syncthreads();
  for (int i = threadIdx.x; i < T * k; i += blockDim.x) atomicAdd(&cnt[topk_ids[i]], 1);
  __syncthreads();
  if (threadIdx.x == 0) {
    int acc = 0;
    for (int e = 0; e < E; ++e) {
      offsets[e] = acc;
      cur[e] = acc;
      counts[e] = cnt[e];
      acc += cnt[e];
    }
    offsets[E] = acc;
  }
  __syncthreads();
  for (int i = threadIdx.x; i < T * k; i += blockDim.x) {
    const int slot = atomicAdd(&cur[topk_ids[i]], 1);
    sorted_tok[slot] = i / k;
    inv[i] = slot;
  }
}

void moe_route_groups(uintptr_t logits, long ld, uintptr_t correction, int T, int E, int k, int groups, int keep,
                      float scale, int softmax_top, uintptr_t topk_w, uintptr_t topk_ids, uintptr_t counts,
                      uintptr_t offsets, uintptr_t sorted_tok, uintptr_t inv, uintptr_t stream) {
  DLLM_HOST_CHECK(E >= 1 && E <= kMaxChoiceExperts && ld >= E, "1 <= experts <= 256");
  DLLM_HOST_CHECK(k >= 1 && k <= 16 && k <= E, "1 <= top <= min(16, experts)");
  DLLM_HOST_CHECK(groups >= 1 && groups <= kMaxGroups && E % groups == 0 && keep >= 1 && keep <= groups &&
                      keep * (E / groups) >= k,
                  "expert groups");
  if (T <= 0) return;
  hipStream_t s = reinterpret_cast<hipStream_t>(stream);
#define ROUTE_G(EMAX)                                                                                              \
  hipLaunchKernelGGL(moe_choice_groups_kernel<EMAX>, dim3((T + 127) / 128), dim3(128), 0, s, (const float*)logits, \
                     ld, (const float*)correction, T, E, k, groups, keep, scale, softmax_top, (float*)topk_w,    \
                     (int*)topk_ids)
  if (E <= 16) ROUTE_G(16);
  else if (E <= 64) ROUTE_G(64);
  else ROUTE_G(256);
#undef ROUTE_G
  DLLM_HIP_CHECK(hipGetLastError());
  hipLaunchKernelGGL(moe_scatter_wide_kernel, dim3(1), dim3(1024), 0, s, (const int*)topk_ids, T, E, k, (int*)counts,
                     (int*)offsets, (int*)sorted_tok, (int*)inv);
  DLLM_HIP_CHECK(hipGetLastError());
}

void moe_router_groups(uintptr_t x, uintptr_t w, int K, int rows, uintptr_t logits, uintptr_t correction, int T, int E,
                       int k, int groups, int keep, float scale, int softmax_top, uintptr_t topk_w, uintptr_t topk_ids,
                       uintptr_t counts, uintptr_t offsets, uintptr_t sorted_tok, uintptr_t inv, int f32,
                       uintptr_t stream) {
  DLLM_HOST_CHECK(E >= 1 && E <= kMaxChoiceExperts && rows >= E && rows <= kMaxChoiceExperts + 8 && K > 0,
                  "1 <= experts <= 256, up to 8 further rows");
  DLLM_HOST_CHECK(k >= 1 && k <= 16 && k <= E, "1 <= top <= min(16, experts)");
  DLLM_HOST_CHECK(groups >= 1 && groups <= kMaxGroups && E % groups == 0 && keep >= 1 && keep <= groups &&
                      keep * (E / groups) >= k,
                  "expert groups");
  if (T <= 0) return;
  hipStream_t s = reinterpret_cast<hipStream_t>(stream);
#define ROUTER_G(TX, EMAX)                                                                                       \
  hipLaunchKernelGGL((moe_router_groups_kernel<TX, EMAX>), dim3(T), dim3(256), 0, s, (const TX*)x, (const float*)w, \
                     K, rows, (float*)logits, (const float*)correction, E, k, groups, keep, scale, softmax_top,     \
                     (float*)topk_w, (int*)topk_ids)
  if (f32) { if (E <= 16) ROUTER_G(float, 16); else if (E <= 64) ROUTER_G(float, 64); else ROUTER_G(float, 256); }
  else { if (E <= 16) ROUTER_G(bf16, 16); else if (E <= 64) ROUTER_G(bf16, 64); else ROUTER_G(bf16, 256); }
#undef ROUTER_G
  DLLM_HIP_CHECK(hipGetLastError());
  hipLaunchKernelGGL(moe_scatter_wide_kernel, dim3(1), dim3(1024), 0, s, (const int*)topk_ids, T, E, k, (int*)counts,
                     (int*)offsets, (int*)sorted_tok, (int*)inv);
  DLLM_HIP_CHECK(hipGetLastError());
}

// y <- max(y, 0)^2 in place (activation of experts of the form down(act(up x)))
template <typename T>
__global__ void __launch_bounds__(256) relu_sq_kernel(T* __restrict__ y, long n) {
  for (long i = (long)blockIdx.x * 256 + threadIdx.x; i < n; i += (long)gridDim.x * 256) {
    const float v = fmaxf((float)y[i], 0.f);
    y[i] = (T)(v * v);
  }
}

void relu_sq(uintptr_t y, long n, int f32, uintptr_t stream) {
  if (n <= 0) return;
  const int grid = (int)std::min<long>((n + 255) / 256, 256L * 32);
  hipStream_t s = reinterpret_cast<hipStream_t>(stream);
  if (f32) hipLaunchKernelGGL(relu_sq_kernel<float>, dim3(grid), dim3(256), 0, s, (float*)y, n);
  else hipLaunchKernelGGL(relu_sq_kernel<bf16>, dim3(grid), dim3(256), 0, s, (bf16*)y, n);
  DLLM_HIP_CHECK(hipGetLastError());
}

// out[t] = sum_j w[t, j] y[inv[t, j]]  (+ sigmoid(gate_logits[t * gate_ld]) * shared[t]: an expert that
// every token uses, scaled by one gate per token); T = bf16 or float, V elements per lane and step
template <typename T, int V>
__global__ void __launch_bounds__(256) moe_combine_gated_kernel(T* __restrict__ out, const T* __restrict__ ysorted,
                                                                const float* __restrict__ topk_w,
                                                                const int* __restrict__ inv,
                                                                const T* __restrict__ shared,
                                                                const float* __restrict__ gate_logits, long gate_ld,
                                                                int H, int k) {
  const int t = blockIdx.x;
  float gate = 1.f;
  if (shared && gate_logits) gate = 1.0f / (1.0f + expf(-gate_logits[(size_t)t * gate_ld]));
  for (int i = threadIdx.x * V; i < H; i += 256 * V) {
    float acc[V];
#pragma unroll
    for (int e = 0; e < V; ++e) acc[e] = 0.f;
    for (int j = 0; j < k; ++j) {
      const float wj = topk_w[t * k + j];
      float y[V];
      ldv<V>(ysorted + (size_t)inv[t * k + j] * H + i, y);
#pragma unroll
      for (int e = 0; e < V; ++e) acc[e] += wj * y[e];
    }
    if (shared) {
      float y[V];
      ldv<V>(shared + (size_t)t * H + i, y);
#pragma unroll
      for (int e = 0; e < V; ++e) acc[e] += gate * y[e];
    }
    stv<V>(out + (size_t)t * H + i, acc);
  }
}

void moe_combine_gated(uintptr_t out, uintptr_t ysorted, uintptr_t topk_w, uintptr_t inv, uintptr_t shared,
                       uintptr_t gate_logits, long gate_ld, int T, int H, int k, int f32, uintptr_t stream) {
  if (T == 0) return;
  DLLM_HOST_CHECK(H > 0 && k >= 1 && out && ysorted && topk_w && inv, "moe combine arguments");
  hipStream_t s = reinterpret_cast<hipStream_t>(stream);
#define COMBINE_G(TY, V)                                                                                          \
  hipLaunchKernelGGL((moe_combine_gated_kernel<TY, V>), dim3(T), dim3(256), 0, s, (TY*)out, (const TY*)ysorted,   \
                     (const float*)topk_w, (const int*)inv, (const TY*)shared, (const float*)gate_logits, gate_ld, \
                     H, k)
  if (f32) { if (H % 8 == 0) COMBINE_G(float, 8); else COMBINE_G(float, 1); }
  else { if (H % 8 == 0) COMBINE_G(bf16, 8); else COMBINE_G(bf16, 1); }
#undef COMBINE_G
  DLLM_HIP_CHECK(hipGetLastError());
}

}  // namespace dllm
