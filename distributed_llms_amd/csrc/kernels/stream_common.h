// Helpers shared by the kernels of layer-list models (seqmix.hip, latent.hip, delta.hip): loads and stores
// of V consecutive elements of the activation type T (bf16 or float) as float registers, the reads of a
// causal convolution's earlier inputs (batch rows, then the state tail, then zeros), and the launch macros
// that pick the float32 or bf16 build of a kernel template.
#pragma once
#include <math.h>

#include "common.h"

namespace dllm {

template <typename T> __device__ __forceinline__ float ldf(const T* p) { return (float)*p; }
template <typename T> __device__ __forceinline__ void stf(T* p, float v) { *p = (T)v; }

// V consecutive elements <-> float registers: V = 8 moves 16 bytes of bf16 (32 of float) per lane and
// needs the address aligned to 8 elements; V = 1 is the any-size form.
template <int V> __device__ __forceinline__ void ldv(const bf16* p, float (&o)[V]) {
  if constexpr (V == 2) {
    const bf16x2 v = *reinterpret_cast<const bf16x2*>(p);
    o[0] = bf2f(v[0]), o[1] = bf2f(v[1]);
  } else if constexpr (V == 8) {
    const bf16x8 v = *reinterpret_cast<const bf16x8*>(p);
#pragma unroll
    for (int j = 0; j < 8; ++j) o[j] = bf2f(v[j]);
  } else {
#pragma unroll
    for (int j = 0; j < V; ++j) o[j] = bf2f(p[j]);
  }
}
template <int V> __device__ __forceinline__ void ldv(const float* p, float (&o)[V]) {
  if constexpr (V == 2) {
    const f32x2 v = *reinterpret_cast<const f32x2*>(p);
    o[0] = v[0], o[1] = v[1];
  } else if constexpr (V == 8) {
    const f32x4 a = *reinterpret_cast<const f32x4*>(p), b = *reinterpret_cast<const f32x4*>(p + 4);
#pragma unroll
    for (int j = 0; j < 4; ++j) o[j] = a[j], o[4 + j] = b[j];
  } else {
#pragma unroll
    for (int j = 0; j < V; ++j) o[j] = p[j];
  }
}
template <int V> __device__ __forceinline__ void stv(bf16* p, const float (&o)[V]) {
  if constexpr (V == 2) {
    bf16x2 v;
    v[0] = f2bf(o[0]), v[1] = f2bf(o[1]);
    *reinterpret_cast<bf16x2*>(p) = v;
  } else if constexpr (V == 8) {
    bf16x8 v;
#pragma unroll
    for (int j = 0; j < 8; ++j) v[j] = f2bf(o[j]);
    *reinterpret_cast<bf16x8*>(p) = v;
  } else {
#pragma unroll
    for (int j = 0; j < V; ++j) p[j] = f2bf(o[j]);
  }
}
template <int V> __device__ __forceinline__ void stv(float* p, const float (&o)[V]) {
  if constexpr (V == 2) {
    *reinterpret_cast<f32x2*>(p) = f32x2{o[0], o[1]};
  } else if constexpr (V == 8) {
    *reinterpret_cast<f32x4*>(p) = f32x4{o[0], o[1], o[2], o[3]};
    *reinterpret_cast<f32x4*>(p + 4) = f32x4{o[4], o[5], o[6], o[7]};
  } else {
#pragma unroll
    for (int j = 0; j < V; ++j) p[j] = o[j];
  }
}

// Input d rows before token (t, channel c) of a chunk that starts at position `start` with the token
// at local index tl: the batch row t - d while tl - d >= 0, else the state tail row
// tl - d + (taps - 1) while the position start + tl - d >= 0, else zero (before the sequence).
// Weights are stored [taps, C] (tap-major), so V consecutive channels of one tap are one load.
template <typename T>
__device__ __forceinline__ float conv_input(const T* __restrict__ u, long stride, const T* __restrict__ st, int t,
                                            int tl, int pos, int d, int taps, int c, int C) {
  if (d > pos) return 0.f;
  if (d <= tl) return ldf(u + (size_t)(t - d) * stride + c);
  return ldf(st + (size_t)(tl - d + taps - 1) * C + c);
}

template <typename T, int V>
__device__ __forceinline__ bool conv_input_v(const T* __restrict__ u, long stride, const T* __restrict__ st, int t,
                                             int tl, int pos, int d, int taps, int c, int C, float (&o)[V]) {
  if (d > pos) return false;
  if (d <= tl) ldv<V>(u + (size_t)(t - d) * stride + c, o);
  else ldv<V>(st + (size_t)(tl - d + taps - 1) * C + c, o);
  return true;
}

#define SM_DISPATCH(f32, KERNEL, grid, block, lds, stream, ...)                                        \
  do {                                                                                                 \
    if (f32)                                                                                           \
      hipLaunchKernelGGL(HIP_KERNEL_NAME(KERNEL<float>), grid, block, lds, (hipStream_t)(stream), __VA_ARGS__); \
    else                                                                                               \
      hipLaunchKernelGGL(HIP_KERNEL_NAME(KERNEL<bf16>), grid, block, lds, (hipStream_t)(stream), __VA_ARGS__);  \
    DLLM_HIP_CHECK(hipGetLastError());                                                                 \
  } while (0)

#define SM_DISPATCH_V(f32, vec, KERNEL, grid, block, lds, stream, ...)                                          \
  do {                                                                                                          \
    hipStream_t s_ = (hipStream_t)(stream);                                                                     \
    if (f32) {                                                                                                  \
      if (vec) hipLaunchKernelGGL(HIP_KERNEL_NAME(KERNEL<float, 8>), grid, block, lds, s_, __VA_ARGS__);        \
      else hipLaunchKernelGGL(HIP_KERNEL_NAME(KERNEL<float, 1>), grid, block, lds, s_, __VA_ARGS__);            \
    } else {                                                                                                    \
      if (vec) hipLaunchKernelGGL(HIP_KERNEL_NAME(KERNEL<bf16, 8>), grid, block, lds, s_, __VA_ARGS__);         \
      else hipLaunchKernelGGL(HIP_KERNEL_NAME(KERNEL<bf16, 1>), grid, block, lds, s_, __VA_ARGS__);             \
    }                                                                                                           \
    DLLM_HIP_CHECK(hipGetLastError());                                                                          \
  } while (0)

}  // namespace dllm
