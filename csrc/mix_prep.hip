// Projection post-processing of attention variants that norm a whole
// projection at once:
//   tied_attn_prep    q and k sections RMS-normed over ALL heads together
//                     (weights of the section's size); q times a temperature
//                     1 + coef * ln(floor((p + 1) / every) + 1) of its
//                     position p; normed k into the paged K cache and the RAW
//                     k section into the paged V cache (values are the keys)
//   section_rmsnorm   out[row(t)] = n(section of proj[t]) * w; row(t) = t, or
//                     an index list (scatter into cache pages: a latent)
//   sigmoid_gate_mul  v *= sigmoid(gate section), elementwise
// One 256-thread block a token (and section); fp32 math.
#include "mix_common.h"

template <typename A>
__global__ void tied_attn_prep_kernel(
    A* __restrict__ q_out, const A* __restrict__ proj, long ld, int q_off,
    int k_off, const float* __restrict__ q_w, const float* __restrict__ k_w,
    float eps, const long* __restrict__ pos, float temp_coef, int temp_every,
    const long* __restrict__ slots, A* __restrict__ k_cache,
    A* __restrict__ v_cache, int H, int G, int dk, int page) {
  __shared__ float red[4];
  const long t = blockIdx.x;
  const bool is_q = blockIdx.y == 0;
  const int n = (is_q ? H : G) * dk;
  const A* src = proj + t * ld + (is_q ? q_off : k_off);
  float ssq = 0.f;
  for (int c = threadIdx.x; c < n; c += blockDim.x) {
    const float v = ldf<A>(src + c);
    ssq += v * v;
  }
  float inv = 1.f / sqrtf(block_sum_256(ssq, red) / (float)n + eps);
  if (is_q) {
    if (temp_every > 0) {
      const long steps = (pos[t] + 1) / temp_every;
      inv *= 1.f + temp_coef * logf((float)steps + 1.f);
    }
    A* dst = q_out + t * (long)n;
    for (int c = threadIdx.x; c < n; c += blockDim.x)
      stf<A>(dst + c, ldf<A>(src + c) * q_w[c] * inv);
    return;
  }
  const long slot = slots[t];
  const long blk = slot / page, off = slot - blk * page;
  for (int c = threadIdx.x; c < n; c += blockDim.x) {
    const int g = c / dk, i = c - g * dk;
    const long at = ((blk * G + g) * page + off) * (long)dk + i;
    const float v = ldf<A>(src + c);
    stf<A>(k_cache + at, v * inv * k_w[c]);
    stf<A>(v_cache + at, v);
  }
}

template <typename A>
__global__ void section_rmsnorm_kernel(A* __restrict__ out, long ldo,
                                       const A* __restrict__ proj, long ld,
                                       int off, const float* __restrict__ w,
                                       float eps, const long* __restrict__ rows,
                                       int n) {
  __shared__ float red[4];
  const long t = blockIdx.x;
  const A* src = proj + t * ld + off;
  float ssq = 0.f;
  for (int c = threadIdx.x; c < n; c += blockDim.x) {
    const float v = ldf<A>(src + c);
    ssq += v * v;
  }
  const float inv = 1.f / sqrtf(block_sum_256(ssq, red) / (float)n + eps);
  A* dst = out + (rows ? rows[t] : t) * ldo;
  for (int c = threadIdx.x; c < n; c += blockDim.x)
    stf<A>(dst + c, ldf<A>(src + c) * inv * w[c]);
}

// 16-byte form: one vector a thread (sections up to 256 vectors long), the
// section is read once. Needs n, the offset and both row strides to be
// multiples of the vector (8 bf16 or 4 fp32).
template <typename A, int V>
__global__ void __launch_bounds__(256) section_rmsnorm_vec_kernel(
    A* __restrict__ out, long ldo, const A* __restrict__ proj, long ld,
    int off, const float* __restrict__ w, float eps,
    const long* __restrict__ rows, int n) {
  typedef A vec_t __attribute__((ext_vector_type(V)));
  __shared__ float red[4];
  const long t = blockIdx.x;
  const int c = threadIdx.x * V;
  float x[V];
  float ssq = 0.f;
  if (c < n) {
    const vec_t v = *(const vec_t*)(proj + t * ld + off + c);
#pragma unroll
    for (int e = 0; e < V; ++e) {
      A ve = v[e];
      x[e] = ldf<A>(&ve);
      ssq += x[e] * x[e];
    }
  }
  const float inv = 1.f / sqrtf(block_sum_256(ssq, red) / (float)n + eps);
  if (c < n) {
    vec_t o;
#pragma unroll
    for (int e = 0; e < V; ++e) {
      A oe;
      stf<A>(&oe, x[e] * inv * w[c + e]);
      o[e] = oe;
    }
    *(vec_t*)(out + (rows ? rows[t] : t) * ldo + c) = o;
  }
}

template <typename A>
__global__ void sigmoid_gate_mul_kernel(A* __restrict__ v, long ldv,
                                        const A* __restrict__ proj, long ld,
                                        int g_off, long T, int N) {
  const long total = T * (long)N;
  for (long idx = (long)blockIdx.x * blockDim.x + threadIdx.x; idx < total;
       idx += (long)gridDim.x * blockDim.x) {
    const long row = idx / N;
    const int c = (int)(idx - row * N);
    A* p = v + row * ldv + c;
    stf<A>(p, ldf<A>(p) * sigmoid_f(ldf<A>(proj + row * ld + g_off + c)));
  }
}

// 16-byte form: needs N, both row strides and the gate offset to be multiples
// of the vector (8 bf16 or 4 fp32)
template <typename A, int V>
__global__ void sigmoid_gate_mul_vec_kernel(A* __restrict__ v, long ldv,
                                            const A* __restrict__ proj,
                                            long ld, int g_off, long T, int N) {
  typedef A vec_t __attribute__((ext_vector_type(V)));
  const int vpr = N / V;
  const long total = T * (long)vpr;
  for (long idx = (long)blockIdx.x * blockDim.x + threadIdx.x; idx < total;
       idx += (long)gridDim.x * blockDim.x) {
    const long row = idx / vpr;
    const int c = (int)(idx - row * vpr) * V;
    vec_t* p = (vec_t*)(v + row * ldv + c);
    const vec_t x = *p;
    const vec_t g = *(const vec_t*)(proj + row * ld + g_off + c);
    vec_t o;
#pragma unroll
    for (int j = 0; j < V; ++j) {
      A xj = x[j], gj = g[j], r;
      stf<A>(&r, ldf<A>(&xj) * sigmoid_f(ldf<A>(&gj)));
      o[j] = r;
    }
    *p = o;
  }
}

extern "C" void mix_tied_attn_prep(void* q_out, const void* proj, long ld,
                                   int q_off, int k_off, const float* q_w,
                                   const float* k_w, float eps,
                                   const long* pos, float temp_coef,
                                   int temp_every, const long* slots,
                                   void* k_cache, void* v_cache, long T, int H,
                                   int G, int dk, int page, int f32,
                                   hipStream_t s) {
  if (T == 0) return;
  const dim3 grid((unsigned)T, 2);
  if (f32)
    hipLaunchKernelGGL(tied_attn_prep_kernel<float>, grid, dim3(256), 0, s,
                       (float*)q_out, (const float*)proj, ld, q_off, k_off,
                       q_w, k_w, eps, pos, temp_coef, temp_every, slots,
                       (float*)k_cache, (float*)v_cache, H, G, dk, page);
  else
    hipLaunchKernelGGL(tied_attn_prep_kernel<u16>, grid, dim3(256), 0, s,
                       (u16*)q_out, (const u16*)proj, ld, q_off, k_off, q_w,
                       k_w, eps, pos, temp_coef, temp_every, slots,
                       (u16*)k_cache, (u16*)v_cache, H, G, dk, page);
}

extern "C" void mix_section_rmsnorm(void* out, long ldo, const void* proj,
                                    long ld, int off, const float* w,
                                    float eps, const long* rows, long T, int n,
                                    int f32, hipStream_t s) {
  if (T == 0) return;
  const int V = f32 ? 4 : 8;
  if (n % V == 0 && n <= 256 * V && off % V == 0 && ld % V == 0 &&
      ldo % V == 0 && (size_t)out % 16 == 0 && (size_t)proj % 16 == 0) {
    if (f32)
      hipLaunchKernelGGL((section_rmsnorm_vec_kernel<float, 4>),
                         dim3((unsigned)T), dim3(256), 0, s, (float*)out, ldo,
                         (const float*)proj, ld, off, w, eps, rows, n);
    else
      hipLaunchKernelGGL((section_rmsnorm_vec_kernel<u16, 8>),
                         dim3((unsigned)T), dim3(256), 0, s, (u16*)out, ldo,
                         (const u16*)proj, ld, off, w, eps, rows, n);
    return;
  }
  if (f32)
    hipLaunchKernelGGL(section_rmsnorm_kernel<float>, dim3((unsigned)T),
                       dim3(256), 0, s, (float*)out, ldo, (const float*)proj,
                       ld, off, w, eps, rows, n);
  else
    hipLaunchKernelGGL(section_rmsnorm_kernel<u16>, dim3((unsigned)T),
                       dim3(256), 0, s, (u16*)out, ldo, (const u16*)proj, ld,
                       off, w, eps, rows, n);
}

extern "C" void mix_sigmoid_gate_mul(void* v, long ldv, const void* proj,
                                     long ld, int g_off, long T, int N,
                                     int f32, hipStream_t s) {
  const long total = T * (long)N;
  if (total == 0) return;
  const int V = f32 ? 4 : 8;
  if (N % V == 0 && ldv % V == 0 && ld % V == 0 && g_off % V == 0 &&
      (size_t)v % 16 == 0 && (size_t)proj % 16 == 0) {
    long vb = (total / V + 255) / 256;
    if (vb > 65536) vb = 65536;
    if (f32)
      hipLaunchKernelGGL((sigmoid_gate_mul_vec_kernel<float, 4>),
                         dim3((unsigned)vb), dim3(256), 0, s, (float*)v, ldv,
                         (const float*)proj, ld, g_off, T, N);
    else
      hipLaunchKernelGGL((sigmoid_gate_mul_vec_kernel<u16, 8>),
                         dim3((unsigned)vb), dim3(256), 0, s, (u16*)v, ldv,
                         (const u16*)proj, ld, g_off, T, N);
    return;
  }
  long blocks = (total + 255) / 256;
  if (blocks > 65536) blocks = 65536;
  if (f32)
    hipLaunchKernelGGL(sigmoid_gate_mul_kernel<float>, dim3((unsigned)blocks),
                       dim3(256), 0, s, (float*)v, ldv, (const float*)proj, ld,
                       g_off, T, N);
  else
    hipLaunchKernelGGL(sigmoid_gate_mul_kernel<u16>, dim3((unsigned)blocks),
                       dim3(256), 0, s, (u16*)v, ldv, (const u16*)proj, ld,
                       g_off, T, N);
}
