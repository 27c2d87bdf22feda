// mLSTM matrix memory (exponential input gate, sigmoid forget gate, running
// maximum as stabiliser), token by token, for every sequence of a batch.
//
//   mlstm_gates  per (sequence, head): log gates i = cap*tanh((a_i + b_i)/cap)
//                and f = logsigmoid(cap*tanh((a_f + b_f)/cap)) from the gate
//                sections of the merged projection, then the stabiliser
//                m_t = max(f_t + m_{t-1}, i_t) strictly in token order (the
//                one serial chain, two flops a token), then per token the
//                decay fa = exp(f + m_{t-1} - m_t), the input scale
//                ib = exp(i - m_t) and em = exp(-m_t).
//   mlstm_scan   C <- fa * C + (ib * k) [v, 1]^T ; o = C^T (q * dk^-1/2).
//                C is [dk, dv+1]: its last column is the normaliser n, so
//                o[dv] = n . q comes out of the same arithmetic.
//   mlstm_out    h = o[:dv] / (max(|o[dv]|, em) + 1e-6), per-head RMS norm,
//                norm weight, elementwise sigmoid gate, cast.
//
// mlstm_scan maps the state onto lanes by COLUMN, like the delta-rule scan: a
// column of C is owned by R adjacent lanes holding dk/R rows each in
// registers; one token costs one R-lane sum (DPP moves) and broadcast reads
// of the staged k and q rows. Blocks cover (sequence, head, group of value
// columns); a fifth wave of the first group's block carries the normaliser. A sequence whose first token (position 0) is in the batch starts
// from zero, whatever its slot held. Everything is fp32 except the
// projection sections, which arrive in the activation type.
#include "mix_common.h"

#define MTB 8   // tokens staged per step

__device__ __forceinline__ float logsigmoid_f(float x) {
  // -softplus(-x), stable on both sides
  return x >= 0.f ? -log1pf(expf(-x)) : x - log1pf(expf(x));
}

// one wave per (sequence, head)
template <typename A>
__global__ void mlstm_gates_kernel(
    float* __restrict__ fa, float* __restrict__ ib, float* __restrict__ em,
    const A* __restrict__ proj, long ld, int i_off, int f_off,
    const float* __restrict__ i_bias, const float* __restrict__ f_bias,
    float cap, float* __restrict__ mstate, const int* __restrict__ state_slots,
    const int* __restrict__ qlocs, const int* __restrict__ seq_lens, int S,
    int H) {
  const int lane = threadIdx.x & (WAVE - 1);
  const int u = blockIdx.x * (blockDim.x / WAVE) + threadIdx.x / WAVE;
  if (u >= S * H) return;  // wave-uniform
  const int s = u / H, h = u - s * H;
  const int q0 = qlocs[s], q1 = qlocs[s + 1];
  if (q1 <= q0) return;
  const int start = seq_lens[s] - (q1 - q0);
  float* mp = mstate + (long)state_slots[s] * H + h;
  float m = start > 0 ? *mp : 0.f;
  const float bi = i_bias[h], bf = f_bias[h];
  for (int t0 = q0; t0 < q1; t0 += WAVE) {
    const int t = t0 + lane;
    const bool live = t < q1;
    float ig = 0.f, fg = 0.f;
    if (live) {
      ig = cap * tanhf((ldf<A>(proj + (long)t * ld + i_off + h) + bi) / cap);
      fg = logsigmoid_f(
          cap * tanhf((ldf<A>(proj + (long)t * ld + f_off + h) + bf) / cap));
    }
    const int n = min((int)WAVE, q1 - t0);
    float m_prev = m, m_mine = m;
    for (int j = 0; j < n; ++j) {  // the serial chain, uniform over the wave
      const float fj = __shfl(fg, j, WAVE), ij = __shfl(ig, j, WAVE);
      const float mn = fmaxf(fj + m, ij);
      if (lane == j) {
        m_prev = m;
        m_mine = mn;
      }
      m = mn;
    }
    if (live) {
      fa[(long)t * H + h] = expf(fg + m_prev - m_mine);
      ib[(long)t * H + h] = expf(ig - m_mine);
      em[(long)t * H + h] = expf(-m_mine);
    }
  }
  if (lane == 0) *mp = m;
}

template <typename A, int R, int RPT>
__global__ void __launch_bounds__(320) mlstm_scan_kernel(
    float* __restrict__ o, const A* __restrict__ proj, long ld, int q_off,
    int k_off, int v_off, const float* __restrict__ fa,
    const float* __restrict__ ib, float* __restrict__ mem,
    const int* __restrict__ state_slots, const int* __restrict__ qlocs,
    const int* __restrict__ seq_lens, int H, int dk, int dv, int col_groups) {
  constexpr int DKP = R * RPT;
  constexpr int CPB = 256 / R;             // value columns per block
  constexpr int NK = 2 * MTB * DKP / 256;  // staged k|q floats per lane
  constexpr int NV = MTB * CPB / 256 > 0 ? MTB * CPB / 256 : 1;
  constexpr int TILE = 2 * MTB * DKP + MTB * CPB + MTB;
  __shared__ __attribute__((aligned(16))) float lds[2][TILE];

  int b = blockIdx.x;
  const int cg = b % col_groups; b /= col_groups;
  const int h = b % H;
  const int s = b / H;
  const int tid = threadIdx.x;
  // Waves 0-3 own the value columns of this group and stage the tiles. Wave
  // 4 exists for the normaliser (column dv of the state, whose "value" is
  // 1): its first R lanes own it in the first column group; everywhere else
  // the wave only keeps the barriers company. The value columns thus fill
  // whole groups (dv = 128 -> 4 groups, not 5 with one lane row in use).
  const bool extra = tid >= 256;
  const int r = tid % R;
  const int cl = (tid & 255) / R;          // column within the block
  const int dv1 = dv + 1;
  const int col = extra ? dv : cg * CPB + cl;
  const bool cv = extra ? (cg == 0 && tid - 256 < R) : col < dv;
  const int q0 = qlocs[s], q1 = qlocs[s + 1];
  if (q1 <= q0) return;
  const int start = seq_lens[s] - (q1 - q0);
  float* Cg = mem + (((long)state_slots[s] * H + h) * dk) * dv1;
  const float qscale = 1.f / sqrtf((float)dk);

  float C[RPT];
#pragma unroll
  for (int n = 0; n < RPT; ++n) {
    const int i = ((n >> 2) * R + r) * 4 + (n & 3);
    C[n] = (start > 0 && cv && i < dk) ? Cg[(long)i * dv1 + col] : 0.f;
  }

  // The prefetch only LOADS: raw elements and raw scale factors stay in
  // registers untouched until they are written to LDS one tile later, so no
  // wait for memory stands between the loads and the arithmetic of the
  // current tile.
  A rk[NK], rv[NV];
  float rs[NK], pf = 0.f;
  auto prefetch = [&](int t0) {
    if (extra) return;
#pragma unroll
    for (int n = 0; n < NK; ++n) {
      const int e = tid + n * 256;
      const int arr = e / (MTB * DKP), rem = e % (MTB * DKP);
      const int tok = rem / DKP, i = rem % DKP;
      const int t = t0 + tok;
      A x = (A)0;            // all-zero bits are 0.0 in both element types
      float sc = qscale;
      if (t < q1 && i < dk) {
        if (arr == 0) {
          x = proj[(long)t * ld + k_off + h * dk + i];
          sc = ib[(long)t * H + h];
        } else {
          x = proj[(long)t * ld + q_off + h * dk + i];
        }
      }
      rk[n] = x;
      rs[n] = sc;
    }
#pragma unroll
    for (int n = 0; n < NV; ++n) {
      const int e = tid + n * 256;
      const int tok = e / CPB, c = cg * CPB + e % CPB;
      const int t = t0 + tok;
      rv[n] = (e < MTB * CPB && t < q1 && c < dv)
                  ? proj[(long)t * ld + v_off + h * dv + c] : (A)0;
    }
    if (tid < MTB) pf = t0 + tid < q1 ? fa[(long)(t0 + tid) * H + h] : 1.f;
  };

  prefetch(q0);
  int buf = 0;
  for (int t0 = q0; t0 < q1; t0 += MTB, buf ^= 1) {
    float* L = lds[buf];
    if (!extra) {
#pragma unroll
      for (int n = 0; n < NK; ++n)
        L[tid + n * 256] = ldf<A>(&rk[n]) * rs[n];
#pragma unroll
      for (int n = 0; n < NV; ++n)
        if (tid + n * 256 < MTB * CPB)
          L[2 * MTB * DKP + tid + n * 256] = ldf<A>(&rv[n]);
      if (tid < MTB) L[2 * MTB * DKP + MTB * CPB + tid] = pf;
    }
    __syncthreads();
    if (t0 + MTB < q1) prefetch(t0 + MTB);
    if (!cv) continue;                     // wave-uniform except in wave 4
    const int nt = min(MTB, q1 - t0);
#pragma unroll
    for (int tok = 0; tok < MTB; ++tok) {
      if (tok >= nt) break;
      const f32x4* K4 = (const f32x4*)(L + tok * DKP);
      const f32x4* Q4 = (const f32x4*)(L + (MTB + tok) * DKP);
      const float vt = extra ? 1.f : L[2 * MTB * DKP + tok * CPB + cl];
      const float ft = L[2 * MTB * DKP + MTB * CPB + tok];
      float out = 0.f;
#pragma unroll
      for (int m = 0; m < RPT / 4; ++m) {
        const f32x4 k4 = K4[m * R + r], q4 = Q4[m * R + r];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          C[m * 4 + j] = ft * C[m * 4 + j] + k4[j] * vt;
          out += C[m * 4 + j] * q4[j];
        }
      }
      out = group_sum<R>(out);
      if (r == 0) o[((long)(t0 + tok) * H + h) * dv1 + col] = out;
    }
  }
  if (cv) {
#pragma unroll
    for (int n = 0; n < RPT; ++n) {
      const int i = ((n >> 2) * R + r) * 4 + (n & 3);
      if (i < dk) Cg[(long)i * dv1 + col] = C[n];
    }
  }
}

// one wave per (token, head)
template <typename A>
__global__ void mlstm_out_kernel(A* __restrict__ out, long ldo, int out_off,
                                 const float* __restrict__ o,
                                 const float* __restrict__ em,
                                 const float* __restrict__ norm_w,
                                 const A* __restrict__ proj, long ld,
                                 int g_off, float eps, long T, int H, int dv) {
  const int lane = threadIdx.x & (WAVE - 1);
  const long u = (long)blockIdx.x * (blockDim.x / WAVE) + threadIdx.x / WAVE;
  if (u >= T * H) return;  // wave-uniform
  const long t = u / H;
  const int h = (int)(u - t * H);
  const float* orow = o + u * (long)(dv + 1);
  const float den = fmaxf(fabsf(orow[dv]), em[u]) + 1e-6f;
  float ssq = 0.f;
  for (int c = lane; c < dv; c += WAVE) {
    const float v = orow[c] / den;
    ssq += v * v;
  }
  const float inv = 1.f / sqrtf(wave_sum_f32(ssq) / (float)dv + eps);
  for (int c = lane; c < dv; c += WAVE) {
    const int hc = h * dv + c;
    const float g = sigmoid_f(ldf<A>(proj + t * ld + g_off + hc));
    stf<A>(out + t * ldo + out_off + hc, orow[c] / den * inv * norm_w[hc] * g);
  }
}

extern "C" void mix_mlstm_scan(float* o, float* em, float* fa, float* ib,
                               const void* proj, long ld, int q_off, int k_off,
                               int v_off, int i_off, int f_off,
                               const float* i_bias, const float* f_bias,
                               float cap, float* mem, float* mstate,
                               const int* state_slots, const int* qlocs,
                               const int* seq_lens, int S, int H, int dk,
                               int dv, int f32, hipStream_t s) {
  if (S == 0) return;
  {
    const int waves = S * H;
    const int grid = (waves + 3) / 4;
    if (f32)
      hipLaunchKernelGGL(mlstm_gates_kernel<float>, dim3(grid), dim3(256), 0, s,
                         fa, ib, em, (const float*)proj, ld, i_off, f_off,
                         i_bias, f_bias, cap, mstate, state_slots, qlocs,
                         seq_lens, S, H);
    else
      hipLaunchKernelGGL(mlstm_gates_kernel<u16>, dim3(grid), dim3(256), 0, s,
                         fa, ib, em, (const u16*)proj, ld, i_off, f_off, i_bias,
                         f_bias, cap, mstate, state_slots, qlocs, seq_lens, S,
                         H);
  }
  int R = 1;
  while (R * 32 < dk) R <<= 1;  // dk <= 256 -> R <= 8 at 32 rows a lane
  int rpt = 32;
  {
    // few sequences x heads: 16 rows a lane doubles the waves in flight
    const long blocks32 = (long)S * H * ((dv + 256 / R - 1) / (256 / R));
    if (blocks32 < 512 && dk > 16) {
      rpt = 16;
      R = 2;
      while (R * 16 < dk) R <<= 1;  // R <= 16
    }
  }
  const int cols_pb = 256 / R;
  const int col_groups = (dv + cols_pb - 1) / cols_pb;
  const long grid = (long)S * H * col_groups;
#define LAUNCH_MS(AA, RR, PP)                                                 \
  hipLaunchKernelGGL((mlstm_scan_kernel<AA, RR, PP>), dim3((unsigned)grid),   \
                     dim3(320), 0, s, o, (const AA*)proj, ld, q_off, k_off,   \
                     v_off, fa, ib, mem, state_slots, qlocs, seq_lens, H, dk, \
                     dv, col_groups)
#define PICK_MS(AA)                                                      \
  if (rpt == 32) {                                                       \
    if (R == 1) LAUNCH_MS(AA, 1, 32);                                    \
    else if (R == 2) LAUNCH_MS(AA, 2, 32);                               \
    else if (R == 4) LAUNCH_MS(AA, 4, 32);                               \
    else LAUNCH_MS(AA, 8, 32);                                           \
  } else {                                                               \
    if (R == 2) LAUNCH_MS(AA, 2, 16);                                    \
    else if (R == 4) LAUNCH_MS(AA, 4, 16);                               \
    else if (R == 8) LAUNCH_MS(AA, 8, 16);                               \
    else LAUNCH_MS(AA, 16, 16);                                          \
  }
  if (f32) { PICK_MS(float) } else { PICK_MS(u16) }
#undef PICK_MS
#undef LAUNCH_MS
}

extern "C" void mix_mlstm_out(void* out, long ldo, int out_off, const float* o,
                              const float* em, const float* norm_w,
                              const void* proj, long ld, int g_off, float eps,
                              long T, int H, int dv, int f32, hipStream_t s) {
  const long units = T * H;
  if (units == 0) return;
  const int grid = (int)((units + 3) / 4);
  if (f32)
    hipLaunchKernelGGL(mlstm_out_kernel<float>, dim3(grid), dim3(256), 0, s,
                       (float*)out, ldo, out_off, o, em, norm_w,
                       (const float*)proj, ld, g_off, eps, T, H, dv);
  else
    hipLaunchKernelGGL(mlstm_out_kernel<u16>, dim3(grid), dim3(256), 0, s,
                       (u16*)out, ldo, out_off, o, em, norm_w,
                       (const u16*)proj, ld, g_off, eps, T, H, dv);
}
