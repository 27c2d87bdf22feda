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

// sum over the R adjacent lanes of a column (R = 1, 2, 4, 8 or 16, aligned):
// DPP moves inside the VALU, no LDS round trip. quad_perm covers the xor-1
// and xor-2 steps; after them every lane of a quad holds the quad's sum, so
// the mirror steps (lane i <- lane 7-i, then 15-i) complete rows of 8 and 16.
template <int R>
__device__ __forceinline__ float group_sum(float v) {
  if (R >= 2)
    v += __int_as_float(__builtin_amdgcn_update_dpp(
        0, __float_as_int(v), 0xB1, 0xF, 0xF, true));   // quad_perm 1,0,3,2
  if (R >= 4)
    v += __int_as_float(__builtin_amdgcn_update_dpp(
        0, __float_as_int(v), 0x4E, 0xF, 0xF, true));   // quad_perm 2,3,0,1
  if (R >= 8)
    v += __int_as_float(__builtin_amdgcn_update_dpp(
        0, __float_as_int(v), 0x141, 0xF, 0xF, true));  // row_half_mirror
  if (R >= 16)
    v += __int_as_float(__builtin_amdgcn_update_dpp(
        0, __float_as_int(v), 0x140, 0xF, 0xF, true));  // row_mirror
  return v;
}
