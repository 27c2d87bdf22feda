// Row-wise pieces of layer-list decoders with an fp32 residual stream:
//   gelu_tanh_mul        act = gelu_tanh(gate) * up over two column sections
//   gated_norm_residual  x += m * g * n(y * sigmoid(gate)),  h = cast(x)
//   scalar_rmsnorm       out = g * n(x)
// n(z) = z / sqrt(mean(z^2) + eps); g is ONE number for all channels, read
// from device memory so no host sync is needed. Memory-bound: one block per
// row, the row is read once from HBM (second pass hits cache).
#include "mix_common.h"

template <typename A>
__global__ void gelu_tanh_mul_kernel(A* __restrict__ out,
                                     const A* __restrict__ proj, long ld,
                                     int gate_off, int up_off, long T, int F) {
  const long total = T * (long)F;
  for (long idx = (long)blockIdx.x * blockDim.x + threadIdx.x; idx < total;
       idx += (long)gridDim.x * blockDim.x) {
    const long row = idx / F;
    const int c = (int)(idx - row * F);
    const float g = ldf<A>(proj + row * ld + gate_off + c);
    const float u = ldf<A>(proj + row * ld + up_off + c);
    const float t =
        tanhf(0.7978845608028654f * (g + 0.044715f * g * g * g));
    stf<A>(out + idx, 0.5f * g * (1.f + t) * u);
  }
}

// 8 bf16 (or 4 fp32) per lane and step: 16-byte loads and stores. Needs F,
// both section offsets and the row stride to be multiples of the vector.
template <typename A, int V>
__global__ void gelu_tanh_mul_vec_kernel(A* __restrict__ out,
                                         const A* __restrict__ proj, long ld,
                                         int gate_off, int up_off, long T,
                                         int F) {
  typedef A vec_t __attribute__((ext_vector_type(V)));
  const int vpr = F / V;
  const long total = T * (long)vpr;
  for (long idx = (long)blockIdx.x * blockDim.x + threadIdx.x; idx < total;
       idx += (long)gridDim.x * blockDim.x) {
    const long row = idx / vpr;
    const int c = (int)(idx - row * vpr) * V;
    const vec_t g = *(const vec_t*)(proj + row * ld + gate_off + c);
    const vec_t u = *(const vec_t*)(proj + row * ld + up_off + c);
    vec_t o;
#pragma unroll
    for (int j = 0; j < V; ++j) {
      A gj = g[j], uj = u[j];
      const float gf = ldf<A>(&gj), uf = ldf<A>(&uj);
      const float t =
          tanhf(0.7978845608028654f * (gf + 0.044715f * gf * gf * gf));
      A r;
      stf<A>(&r, 0.5f * gf * (1.f + t) * uf);
      o[j] = r;
    }
    *(vec_t*)(out + row * F + c) = o;
  }
}

template <typename A>
__global__ void gated_norm_residual_kernel(
    float* __restrict__ x, const A* __restrict__ y, const A* __restrict__ proj,
    long ld, int gate_off, const float* __restrict__ gain, float eps,
    float mult, A* __restrict__ h_out, long T, int W) {
  __shared__ float red[4];
  const float g = gain[0] * mult;
  for (long row = blockIdx.x; row < T; row += gridDim.x) {
    const A* yr = y + row * W;
    const A* gr = proj + row * ld + gate_off;
    float ssq = 0.f;
    for (int c = threadIdx.x; c < W; c += blockDim.x) {
      const float z = ldf<A>(yr + c) * sigmoid_f(ldf<A>(gr + c));
      ssq += z * z;
    }
    const float tot = block_sum_256(ssq, red);
    const float inv = g / sqrtf(tot / (float)W + eps);
    float* xr = x + row * W;
    for (int c = threadIdx.x; c < W; c += blockDim.x) {
      const float z = ldf<A>(yr + c) * sigmoid_f(ldf<A>(gr + c));
      const float nx = xr[c] + z * inv;
      xr[c] = nx;
      if (h_out) stf<A>(h_out + row * W + c, nx);
    }
    __syncthreads();  // red[] is reused by the next row
  }
}

template <typename A>
__global__ void scalar_rmsnorm_kernel(A* __restrict__ out,
                                      const float* __restrict__ x,
                                      const float* __restrict__ gain,
                                      float eps, long T, int W) {
  __shared__ float red[4];
  const float g = gain[0];
  for (long row = blockIdx.x; row < T; row += gridDim.x) {
    const float* xr = x + row * W;
    float ssq = 0.f;
    for (int c = threadIdx.x; c < W; c += blockDim.x) ssq += xr[c] * xr[c];
    const float tot = block_sum_256(ssq, red);
    const float inv = g / sqrtf(tot / (float)W + eps);
    for (int c = threadIdx.x; c < W; c += blockDim.x)
      stf<A>(out + row * W + c, xr[c] * inv);
    __syncthreads();
  }
}

static inline int row_grid(long rows) {
  return (int)(rows < 4096 ? (rows > 0 ? rows : 1) : 4096);
}

extern "C" void mix_gelu_tanh_mul(void* out, const void* proj, long ld,
                                  int gate_off, int up_off, long T, int F,
                                  int f32, hipStream_t s) {
  const int V = f32 ? 4 : 8;
  if (F % V == 0 && gate_off % V == 0 && up_off % V == 0 && ld % V == 0) {
    long wantv = (T * (long)(F / V) + 255) / 256;
    int gridv = (int)(wantv < 8192 ? (wantv > 0 ? wantv : 1) : 8192);
    if (f32)
      hipLaunchKernelGGL((gelu_tanh_mul_vec_kernel<float, 4>), dim3(gridv),
                         dim3(256), 0, s, (float*)out, (const float*)proj, ld,
                         gate_off, up_off, T, F);
    else
      hipLaunchKernelGGL((gelu_tanh_mul_vec_kernel<u16, 8>), dim3(gridv),
                         dim3(256), 0, s, (u16*)out, (const u16*)proj, ld,
                         gate_off, up_off, T, F);
    return;
  }
  long want = (T * (long)F + 255) / 256;
  int grid = (int)(want < 4096 ? (want > 0 ? want : 1) : 4096);
  if (f32)
    hipLaunchKernelGGL(gelu_tanh_mul_kernel<float>, dim3(grid), dim3(256), 0,
                       s, (float*)out, (const float*)proj, ld, gate_off,
                       up_off, T, F);
  else
    hipLaunchKernelGGL(gelu_tanh_mul_kernel<u16>, dim3(grid), dim3(256), 0, s,
                       (u16*)out, (const u16*)proj, ld, gate_off, up_off, T,
                       F);
}

extern "C" void mix_gated_norm_residual(float* x, const void* y,
                                        const void* proj, long ld,
                                        int gate_off, const float* gain,
                                        float eps, float mult, void* h_out,
                                        long T, int W, int f32,
                                        hipStream_t s) {
  if (f32)
    hipLaunchKernelGGL(gated_norm_residual_kernel<float>, dim3(row_grid(T)),
                       dim3(256), 0, s, x, (const float*)y, (const float*)proj,
                       ld, gate_off, gain, eps, mult, (float*)h_out, T, W);
  else
    hipLaunchKernelGGL(gated_norm_residual_kernel<u16>, dim3(row_grid(T)),
                       dim3(256), 0, s, x, (const u16*)y, (const u16*)proj, ld,
                       gate_off, gain, eps, mult, (u16*)h_out, T, W);
}

extern "C" void mix_scalar_rmsnorm(void* out, const float* x,
                                   const float* gain, float eps, long T, int W,
                                   int f32, hipStream_t s) {
  if (f32)
    hipLaunchKernelGGL(scalar_rmsnorm_kernel<float>, dim3(row_grid(T)),
                       dim3(256), 0, s, (float*)out, x, gain, eps, T, W);
  else
    hipLaunchKernelGGL(scalar_rmsnorm_kernel<u16>, dim3(row_grid(T)),
                       dim3(256), 0, s, (u16*)out, x, gain, eps, T, W);
}
