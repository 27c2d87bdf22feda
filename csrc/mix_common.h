// Helpers shared by the layer-list decoder kernels (mix_*.hip): every kernel
// is a template over the activation type A — u16 (bf16 bit pattern) when the
// engine serves in bf16, float when it serves in fp32 — and does its math in
// fp32 with full-precision expf/tanhf/sqrtf (no fast intrinsics: the fp32
// serving mode is held to fp32 accuracy end to end).
#pragma once

#include "common.h"

template <typename A> __device__ __forceinline__ float ldf(const A* p);
template <> __device__ __forceinline__ float ldf<u16>(const u16* p) {
  return bf2f(*p);
}
template <> __device__ __forceinline__ float ldf<float>(const float* p) {
  return *p;
}
template <typename A> __device__ __forceinline__ void stf(A* p, float v);
template <> __device__ __forceinline__ void stf<u16>(u16* p, float v) {
  *p = f2bf(v);
}
template <> __device__ __forceinline__ void stf<float>(float* p, float v) {
  *p = v;
}

__device__ __forceinline__ float sigmoid_f(float x) {
  return 1.f / (1.f + expf(-x));
}

__device__ __forceinline__ float softplus_f(float x) {
  return x > 20.f ? x : log1pf(expf(x));
}

// sum over a 256-thread block (4 waves); `red` is 4 floats of LDS. Callers
// must not reuse `red` before their next __syncthreads().
__device__ __forceinline__ float block_sum_256(float v, float* red) {
  v = wave_sum_f32(v);
  const int wid = threadIdx.x / WAVE;
  if ((threadIdx.x & (WAVE - 1)) == 0) red[wid] = v;
  __syncthreads();
  return red[0] + red[1] + red[2] + red[3];
}
