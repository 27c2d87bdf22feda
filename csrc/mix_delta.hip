// Gated delta rule with one decay per head and key channel.
//
//   delta_prep         short causal depthwise filter + silu on the q|k|v
//                      channels, unit-norm q (times dk^-1/2) and k
//   delta_gates        beta = sigmoid, decay = exp(-exp(A_log) *
//                      softplus(a2 a1 + dt_bias)) per head and key channel
//   conv_state_update  keeps the last taps-1 raw filter inputs per sequence
//   delta_scan         S <- decay * S; u = beta (v - S^T k); S <- S + k u^T;
//                      o = S^T q, token by token, S [dk, dv] fp32 per head
//   delta_out          o / rms(o) * w * sigmoid(g2 g1), cast, into the
//                      output-projection input
//
// Everything the recurrence consumes is fp32. A sequence whose first token
// (position 0) is in the batch starts from zero filter history and zero S,
// whatever its state slot held before.
//
// delta_scan maps the state onto lanes by COLUMN: the dv columns of S never
// interact, so a column is owned by R adjacent lanes holding dk/R rows each
// in registers; one token costs two R-lane sums (DPP moves) and broadcast
// reads of the staged k, q and decay rows. Blocks cover (sequence, head,
// group of columns).
#include "mix_common.h"

#define WPB 4
#define PT 8   // tokens per wave in delta_prep

// merged channel c (q | k | v order) -> column of the projection buffer
__device__ __forceinline__ int chan_col(int c, int Cq, int q_off, int k_off,
                                        int v_off) {
  return c < Cq ? q_off + c : (c < 2 * Cq ? k_off + c - Cq : v_off + c - 2 * Cq);
}

template <typename A>
__global__ void delta_prep_kernel(
    float* __restrict__ qn, float* __restrict__ kn, float* __restrict__ vv,
    const A* __restrict__ proj, long ld, int q_off, int k_off, int v_off,
    const float* __restrict__ conv_w, int taps,
    const float* __restrict__ conv_state,
    const int* __restrict__ state_slots, const int* __restrict__ qlocs,
    const int* __restrict__ seq_lens, const int* __restrict__ token_seq,
    long T, int H, int G, int dk, int dv) {
  const int lane = threadIdx.x & (WAVE - 1);
  const int wid = threadIdx.x / WAVE;
  const int units = 2 * G + H;
  // a wave owns one head unit and PT consecutive tokens
  const long wv = (long)blockIdx.x * WPB + wid;
  const long tg = wv / units;
  const int j = (int)(wv - tg * units);
  const int Cq = G * dk, C = 2 * Cq + H * dv;
  for (long t = tg * PT; t < T && t < (tg + 1) * PT; ++t) {
  // filter + silu of one q, k or v head
  const int kind = j < G ? 0 : (j < 2 * G ? 1 : 2);
  const int head = kind == 0 ? j : (kind == 1 ? j - G : j - 2 * G);
  const int d = kind == 2 ? dv : dk;
  const int c0 = (kind == 0 ? 0 : (kind == 1 ? Cq : 2 * Cq)) + head * d;
  const int s = token_seq[t];
  const int q0 = qlocs[s], n = qlocs[s + 1] - q0;
  const int start = seq_lens[s] - n;      // position of the chunk's first token
  const int jl = (int)t - q0;             // local index in the chunk
  const float* hist = conv_state + (long)state_slots[s] * (taps - 1) * C;

  float y[4];  // d <= 256
  float ssq = 0.f;
  int k = 0;
  for (int i = lane; i < d; i += WAVE, ++k) {
    const int c = c0 + i;
    const int col = chan_col(c, Cq, q_off, k_off, v_off);
    float acc = 0.f;
    for (int back = 0; back < taps; ++back) {
      float x = 0.f;
      if (jl - back >= 0)
        x = ldf<A>(proj + (t - back) * ld + col);
      else if (start > 0)  // start + jl - back >= 0 is implied: the history
        x = hist[(long)(taps - 1 - back + jl) * C + c];  // holds zeros there
      acc += conv_w[(long)c * taps + (taps - 1 - back)] * x;
    }
    const float a = acc * sigmoid_f(acc);
    y[k] = a;
    ssq += a * a;
  }
  ssq = wave_sum_f32(ssq);
  float f = 1.f;
  if (kind != 2) {
    f = 1.f / sqrtf(ssq + 1e-6f);
    if (kind == 0) f *= 1.f / sqrtf((float)dk);
  }
  float* dst = kind == 0 ? qn + (t * G + head) * (long)dk
                         : (kind == 1 ? kn + (t * G + head) * (long)dk
                                      : vv + (t * H + head) * (long)dv);
  k = 0;
  for (int i = lane; i < d; i += WAVE, ++k) dst[i] = y[k] * f;
  }  // tokens of this wave
}

// bf16 fast path of delta_prep: a group of GS lanes owns one (token, head)
// unit, lane gl its 8-channel chunk (16-byte loads of the raw rows, float4
// loads of the transposed filter [taps, C] and of the history, float4
// stores). Needs dk, dv and all offsets to be multiples of 8.
template <int GS>
__global__ void delta_prep_vec_kernel(
    float* __restrict__ qn, float* __restrict__ kn, float* __restrict__ vv,
    const u16* __restrict__ proj, long ld, int q_off, int k_off, int v_off,
    const float* __restrict__ conv_wt, int taps,
    const float* __restrict__ conv_state,
    const int* __restrict__ state_slots, const int* __restrict__ qlocs,
    const int* __restrict__ seq_lens, const int* __restrict__ token_seq,
    long T, int H, int G, int dk, int dv) {
  constexpr int UPWV = 64 / GS;
  const int lane = threadIdx.x & (WAVE - 1);
  const int wid = threadIdx.x / WAVE;
  const int gi = lane / GS, gl = lane % GS;
  const int units = 2 * G + H;
  const long total = T * units;
  const long u = ((long)blockIdx.x * WPB + wid) * UPWV + gi;
  const bool valid = u < total;
  const long t = valid ? u / units : 0;
  const int j = valid ? (int)(u - t * units) : 0;
  const int Cq = G * dk, C = 2 * Cq + H * dv;
  const int kind = j < G ? 0 : (j < 2 * G ? 1 : 2);
  const int head = kind == 0 ? j : (kind == 1 ? j - G : j - 2 * G);
  const int d = kind == 2 ? dv : dk;
  const int c0 = gl * 8;
  const bool act = valid && c0 < d;
  const int c = (kind == 0 ? 0 : (kind == 1 ? Cq : 2 * Cq)) + head * d + c0;
  float acc[8];
#pragma unroll
  for (int e = 0; e < 8; ++e) acc[e] = 0.f;
  if (act) {
    const int col = chan_col(c, Cq, q_off, k_off, v_off);
    const int s = token_seq[t];
    const int q0 = qlocs[s], n = qlocs[s + 1] - q0;
    const int start = seq_lens[s] - n;
    const int jl = (int)t - q0;
    const float* hist = conv_state + (long)state_slots[s] * (taps - 1) * C;
    for (int back = 0; back < taps; ++back) {
      float x[8];
      if (jl - back >= 0) {
        bf8_to_f32(*(const u16x8*)(proj + (t - back) * ld + col), x);
      } else if (start > 0) {
        const float* hp = hist + (long)(taps - 1 - back + jl) * C + c;
        const f32x4 a = *(const f32x4*)hp, b = *(const f32x4*)(hp + 4);
#pragma unroll
        for (int e = 0; e < 4; ++e) { x[e] = a[e]; x[e + 4] = b[e]; }
      } else {
        continue;  // before the start of the sequence: zeros
      }
      const float* wp = conv_wt + (long)(taps - 1 - back) * C + c;
      const f32x4 w0 = *(const f32x4*)wp, w1 = *(const f32x4*)(wp + 4);
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        acc[e] += w0[e] * x[e];
        acc[e + 4] += w1[e] * x[e + 4];
      }
    }
  }
  float ssq = 0.f;
#pragma unroll
  for (int e = 0; e < 8; ++e) {
    acc[e] = acc[e] * sigmoid_f(acc[e]);
    ssq += acc[e] * acc[e];
  }
#pragma unroll
  for (int off = GS / 2; off > 0; off >>= 1) ssq += __shfl_xor(ssq, off, WAVE);
  if (!act) return;
  float f = 1.f;
  if (kind != 2) {
    f = 1.f / sqrtf(ssq + 1e-6f);
    if (kind == 0) f *= 1.f / sqrtf((float)dk);
  }
  float* dst = (kind == 0 ? qn + (t * G + head) * (long)dk
                          : (kind == 1 ? kn + (t * G + head) * (long)dk
                                       : vv + (t * H + head) * (long)dv)) + c0;
  f32x4 o0, o1;
#pragma unroll
  for (int e = 0; e < 4; ++e) { o0[e] = acc[e] * f; o1[e] = acc[e + 4] * f; }
  *(f32x4*)dst = o0;
  *(f32x4*)(dst + 4) = o1;
}

// ---- low-rank gates ---------------------------------------------------------
// Both gate kernels evaluate act(W2 (W1 h) + bias) where W1 h (`rank` numbers
// a token) is a section of the merged projection and W2 arrives transposed
// [rank, rows]. A wave owns GT consecutive tokens and one head: a lane keeps
// the W2 column of its output channel in registers across those tokens, the
// token's `rank` inputs sit one per lane and reach the FMAs through readlane
// (scalar operands), so the inner loop issues no loads at all.
#define GT 8     // tokens per wave
#define RMAX 32  // W2 rows held per pass

__device__ __forceinline__ float lane_bcast(float v, int src) {
  return __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), src));
}

// acc[tt] += sum_r w2t[(r0 + r) * stride + col] * in[t_base + tt][r0 + r]
template <typename A>
__device__ __forceinline__ void low_rank_acc(
    float (&acc)[GT], const float* __restrict__ w2t, long stride, long col,
    bool col_ok, int rank, const A* __restrict__ in, long ld, long t_base,
    long T, int lane) {
  for (int r0 = 0; r0 < rank; r0 += RMAX) {
    float w[RMAX];
#pragma unroll
    for (int r = 0; r < RMAX; ++r)
      w[r] = (col_ok && r0 + r < rank) ? w2t[(long)(r0 + r) * stride + col] : 0.f;
    float x[GT];  // lane r holds input r of token tt
#pragma unroll
    for (int tt = 0; tt < GT; ++tt)
      x[tt] = (t_base + tt < T && lane < RMAX && r0 + lane < rank)
                  ? ldf<A>(in + (t_base + tt) * ld + r0 + lane) : 0.f;
    // r outer, tokens inner: GT independent readlane + FMA chains
#pragma unroll
    for (int r = 0; r < RMAX; ++r)
#pragma unroll
      for (int tt = 0; tt < GT; ++tt) acc[tt] += w[r] * lane_bcast(x[tt], r);
  }
}

// decay[t,h,i] = exp(-exp(a_log[h]) * softplus(a2 a1 + dt_bias)), beta[t,h] =
// sigmoid(b section). grid (token groups, H).
template <typename A>
__global__ void delta_gates_kernel(
    float* __restrict__ decay, float* __restrict__ beta,
    const A* __restrict__ proj, long ld, int b_off, int a1_off,
    const float* __restrict__ a2t, int rank, const float* __restrict__ dt_bias,
    const float* __restrict__ a_log, long T, int H, int dk) {
  const int lane = threadIdx.x & (WAVE - 1);
  const int wid = __builtin_amdgcn_readfirstlane(threadIdx.x / WAVE);
  const int h = blockIdx.y;
  const long t_base = ((long)blockIdx.x * WPB + wid) * GT;
  if (t_base >= T) return;
  const float rate = expf(a_log[h]);
  const long HD = (long)H * dk;
  for (int k0 = 0; k0 < dk; k0 += WAVE) {
    const int i = k0 + lane;
    const bool in = i < dk;
    float acc[GT];
    const float bias = in ? dt_bias[h * dk + i] : 0.f;
#pragma unroll
    for (int tt = 0; tt < GT; ++tt) acc[tt] = bias;
    low_rank_acc<A>(acc, a2t, HD, (long)h * dk + i, in, rank, proj + a1_off, ld,
                    t_base, T, lane);
#pragma unroll
    for (int tt = 0; tt < GT; ++tt)
      if (in && t_base + tt < T)
        decay[((t_base + tt) * H + h) * (long)dk + i] =
            expf(-rate * softplus_f(acc[tt]));
  }
  if (lane < GT && t_base + lane < T)
    beta[(t_base + lane) * H + h] =
        sigmoid_f(ldf<A>(proj + (t_base + lane) * ld + b_off + h));
}

// one thread per (sequence, channel): new history = last taps-1 raw inputs
template <typename A>
__global__ void conv_state_update_kernel(
    float* __restrict__ conv_state, const A* __restrict__ proj, long ld,
    int q_off, int k_off, int v_off, int taps,
    const int* __restrict__ state_slots, const int* __restrict__ qlocs,
    const int* __restrict__ seq_lens, int S, int Cq, int C) {
  const long idx = (long)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= (long)S * C) return;
  const int s = (int)(idx / C), c = (int)(idx - (long)s * C);
  const int q0 = qlocs[s], n = qlocs[s + 1] - q0;
  if (n <= 0) return;
  const int start = seq_lens[s] - n;
  const int col = chan_col(c, Cq, q_off, k_off, v_off);
  float* hist = conv_state + (long)state_slots[s] * (taps - 1) * C + c;
  for (int i = 0; i < taps - 1; ++i) {
    const int tau = n - (taps - 1) + i;  // chunk-local time of history row i
    float x = 0.f;
    if (tau >= 0)
      x = ldf<A>(proj + (long)(q0 + tau) * ld + col);
    else if (start > 0 && i + n <= taps - 2)
      x = hist[(long)(i + n) * C];       // read before row i+n is rewritten
    hist[(long)i * C] = x;
  }
}

#define TB 8    // tokens staged per step

// Token-by-token scan. Block = (sequence, head, group of 256/R columns);
// lane (col, r) keeps rows {((n/4)*R + r)*4 + n%4 : n < RPT} of its column of
// S in registers (RPT = 32, or 16 to double the number of waves when a
// launch would leave SIMDs idle) (rows past dk stay zero: their k and q are staged as 0 and
// their decay as 1). k, q, decay, v and beta of TB tokens at a time are
// staged through a double-buffered LDS tile: the global loads of tile s+1
// are issued before the arithmetic of tile s and parked in registers. With
// this row mapping the R lanes of a column read consecutive float4s of a
// staged row, and all columns read the same addresses (LDS broadcast).
template <int R, int RPT>
__global__ void __launch_bounds__(256) delta_scan_kernel(
    float* __restrict__ o, const float* __restrict__ qn,
    const float* __restrict__ kn, const float* __restrict__ vv,
    const float* __restrict__ decay, const float* __restrict__ beta,
    float* __restrict__ ssm, const int* __restrict__ state_slots,
    const int* __restrict__ qlocs, const int* __restrict__ seq_lens, int H,
    int G, int dk, int dv, int col_groups) {
  constexpr int DKP = R * RPT;
  constexpr int CPB = 256 / R;            // columns per block
  constexpr int NK = 3 * TB * DKP / 256;  // staged k|q|decay floats per lane
  constexpr int NV = TB * CPB / 256 > 0 ? TB * CPB / 256 : 1;
  constexpr int TILE = 3 * TB * DKP + TB * CPB + TB;
  __shared__ __attribute__((aligned(16))) float lds[2][TILE];

  int b = blockIdx.x;
  const int cg = b % col_groups; b /= col_groups;
  const int h = b % H;
  const int s = b / H;
  const int tid = threadIdx.x;
  const int r = tid % R;
  const int cl = tid / R;                 // column within the block
  const int col = cg * CPB + cl;
  const bool cv = col < dv;
  const int g = h / (H / G);
  const int q0 = qlocs[s], q1 = qlocs[s + 1];
  if (q1 <= q0) return;
  const int start = seq_lens[s] - (q1 - q0);
  float* Sg = ssm + (((long)state_slots[s] * H + h) * dk) * dv;

  float S[RPT];
#pragma unroll
  for (int n = 0; n < RPT; ++n) {
    const int i = ((n >> 2) * R + r) * 4 + (n & 3);
    S[n] = (start > 0 && cv && i < dk) ? Sg[(long)i * dv + col] : 0.f;
  }

  float pk[NK], pv[NV], pb = 0.f;
  auto prefetch = [&](int t0) {
#pragma unroll
    for (int n = 0; n < NK; ++n) {
      const int e = tid + n * 256;
      const int arr = e / (TB * DKP), rem = e % (TB * DKP);
      const int tok = rem / DKP, i = rem % DKP;
      const int t = t0 + tok;
      float x = arr == 2 ? 1.f : 0.f;
      if (t < q1 && i < dk) {
        if (arr == 0) x = kn[((long)t * G + g) * dk + i];
        else if (arr == 1) x = qn[((long)t * G + g) * dk + i];
        else x = decay[((long)t * H + h) * dk + i];
      }
      pk[n] = x;
    }
#pragma unroll
    for (int n = 0; n < NV; ++n) {
      const int e = tid + n * 256;
      const int tok = e / CPB, c = cg * CPB + e % CPB;
      const int t = t0 + tok;
      pv[n] = (e < TB * CPB && t < q1 && c < dv)
                  ? vv[((long)t * H + h) * dv + c] : 0.f;
    }
    if (tid < TB) pb = t0 + tid < q1 ? beta[(long)(t0 + tid) * H + h] : 0.f;
  };

  prefetch(q0);
  int buf = 0;
  for (int t0 = q0; t0 < q1; t0 += TB, buf ^= 1) {
    float* L = lds[buf];
#pragma unroll
    for (int n = 0; n < NK; ++n) L[tid + n * 256] = pk[n];
#pragma unroll
    for (int n = 0; n < NV; ++n)
      if (tid + n * 256 < TB * CPB) L[3 * TB * DKP + tid + n * 256] = pv[n];
    if (tid < TB) L[3 * TB * DKP + TB * CPB + tid] = pb;
    __syncthreads();
    if (t0 + TB < q1) prefetch(t0 + TB);
    const int nt = min(TB, q1 - t0);
    for (int tok = 0; tok < nt; ++tok) {
      const f32x4* K4 = (const f32x4*)(L + tok * DKP);
      const f32x4* Q4 = (const f32x4*)(L + (TB + tok) * DKP);
      const f32x4* D4 = (const f32x4*)(L + (2 * TB + tok) * DKP);
      const float vt = L[3 * TB * DKP + tok * CPB + cl];
      const float bt = L[3 * TB * DKP + TB * CPB + tok];
      float kk[RPT];
      float dot = 0.f;
#pragma unroll
      for (int m = 0; m < RPT / 4; ++m) {
        const f32x4 k4 = K4[m * R + r], d4 = D4[m * R + r];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          kk[m * 4 + j] = k4[j];
          S[m * 4 + j] *= d4[j];
          dot += S[m * 4 + j] * k4[j];
        }
      }
      dot = group_sum<R>(dot);
      const float uu = bt * (vt - dot);
      float out = 0.f;
#pragma unroll
      for (int m = 0; m < RPT / 4; ++m) {
        const f32x4 q4 = Q4[m * R + r];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          S[m * 4 + j] += kk[m * 4 + j] * uu;
          out += S[m * 4 + j] * q4[j];
        }
      }
      out = group_sum<R>(out);
      if (r == 0 && cv) o[((long)(t0 + tok) * H + h) * dv + col] = out;
    }
  }
  if (cv) {
#pragma unroll
    for (int n = 0; n < RPT; ++n) {
      const int i = ((n >> 2) * R + r) * 4 + (n & 3);
      if (i < dk) Sg[(long)i * dv + col] = S[n];
    }
  }
}

// out[t, out_off + h*dv + c] = out_scale * o[t,h,c] / rms(o[t,h,:]) * w[c] *
// sigmoid(g2 g1)[h*dv + c]. grid (token groups, H); a wave owns GT tokens.
template <typename A>
__global__ void delta_out_kernel(A* __restrict__ out, long ldo, int out_off,
                                 const float* __restrict__ o,
                                 const float* __restrict__ norm_w,
                                 const A* __restrict__ proj, long ld,
                                 int g1_off, const float* __restrict__ g2t,
                                 int rank, float eps, float out_scale, long T,
                                 int H, int dv) {
  const int lane = threadIdx.x & (WAVE - 1);
  const int wid = __builtin_amdgcn_readfirstlane(threadIdx.x / WAVE);
  const int h = blockIdx.y;
  const long t_base = ((long)blockIdx.x * WPB + wid) * GT;
  if (t_base >= T) return;
  float inv[GT];
#pragma unroll
  for (int tt = 0; tt < GT; ++tt) {
    inv[tt] = 0.f;
    const long t = t_base + tt;
    if (t >= T) break;
    const float* orow = o + (t * H + h) * (long)dv;
    float ssq = 0.f;
    for (int c = lane; c < dv; c += WAVE) ssq += orow[c] * orow[c];
    ssq = wave_sum_f32(ssq);
    inv[tt] = out_scale / sqrtf(ssq / (float)dv + eps);
  }
  const long HV = (long)H * dv;
  for (int k0 = 0; k0 < dv; k0 += WAVE) {
    const int c = k0 + lane;
    const bool in = c < dv;
    float acc[GT];
#pragma unroll
    for (int tt = 0; tt < GT; ++tt) acc[tt] = 0.f;
    low_rank_acc<A>(acc, g2t, HV, (long)h * dv + c, in, rank, proj + g1_off, ld,
                    t_base, T, lane);
    const float wn = in ? norm_w[c] : 0.f;
#pragma unroll
    for (int tt = 0; tt < GT; ++tt) {
      const long t = t_base + tt;
      if (in && t < T)
        stf<A>(out + t * ldo + out_off + (long)h * dv + c,
               o[(t * H + h) * (long)dv + c] * inv[tt] * wn *
                   sigmoid_f(acc[tt]));
    }
  }
}

extern "C" void mix_delta_prep(
    float* qn, float* kn, float* vv, float* decay, float* beta,
    const void* proj, long ld, int q_off, int k_off, int v_off, int b_off,
    int a1_off, const float* conv_w, const float* conv_wt, int taps,
    const float* a2, int rank,
    const float* dt_bias, const float* a_log, float* conv_state,
    const int* state_slots, const int* qlocs, const int* seq_lens,
    const int* token_seq, long T, int S, int H, int G, int dk, int dv, int f32,
    hipStream_t s) {
  const long units = ((T + PT - 1) / PT) * (2 * G + H);
  const int grid = (int)((units + WPB - 1) / WPB);
  if (grid == 0) return;
  const dim3 ggrid((unsigned)((T + WPB * GT - 1) / (WPB * GT)), (unsigned)H);
  const int Cq = G * dk, C = 2 * Cq + H * dv;
  const long su = (long)S * C;
  const int sgrid = (int)((su + 255) / 256);
  const int dmax = dk > dv ? dk : dv;
  const int dm8 = (dmax + 7) / 8;
  const bool vec = !f32 && conv_wt && dk % 8 == 0 && dv % 8 == 0 &&
                   ld % 8 == 0 && q_off % 8 == 0 && k_off % 8 == 0 &&
                   v_off % 8 == 0 && dm8 <= 32;
  if (vec) {
    const int GS = dm8 <= 4 ? 4 : (dm8 <= 8 ? 8 : (dm8 <= 16 ? 16 : 32));
    const long tot = T * (2 * G + H);
    const long waves = (tot + 64 / GS - 1) / (64 / GS);
    const int vgrid = (int)((waves + WPB - 1) / WPB);
#define LAUNCH_DV(GG)                                                          \
  hipLaunchKernelGGL(delta_prep_vec_kernel<GG>, dim3(vgrid), dim3(WPB * WAVE), \
                     0, s, qn, kn, vv, (const u16*)proj, ld, q_off, k_off,     \
                     v_off, conv_wt, taps, conv_state, state_slots, qlocs,     \
                     seq_lens, token_seq, T, H, G, dk, dv)
    if (GS == 4) LAUNCH_DV(4);
    else if (GS == 8) LAUNCH_DV(8);
    else if (GS == 16) LAUNCH_DV(16);
    else LAUNCH_DV(32);
#undef LAUNCH_DV
    hipLaunchKernelGGL(delta_gates_kernel<u16>, ggrid, dim3(WPB * WAVE), 0, s,
                       decay, beta, (const u16*)proj, ld, b_off, a1_off, a2,
                       rank, dt_bias, a_log, T, H, dk);
    if (taps > 1)
      hipLaunchKernelGGL(conv_state_update_kernel<u16>, dim3(sgrid), dim3(256),
                         0, s, conv_state, (const u16*)proj, ld, q_off, k_off,
                         v_off, taps, state_slots, qlocs, seq_lens, S, Cq, C);
    return;
  }
  if (f32) {
    hipLaunchKernelGGL(delta_prep_kernel<float>, dim3(grid), dim3(WPB * WAVE),
                       0, s, qn, kn, vv, (const float*)proj, ld, q_off, k_off,
                       v_off, conv_w, taps, conv_state, state_slots, qlocs,
                       seq_lens, token_seq, T, H, G, dk, dv);
    hipLaunchKernelGGL(delta_gates_kernel<float>, ggrid, dim3(WPB * WAVE), 0, s,
                       decay, beta, (const float*)proj, ld, b_off, a1_off, a2,
                       rank, dt_bias, a_log, T, H, dk);
    if (taps > 1)
      hipLaunchKernelGGL(conv_state_update_kernel<float>, dim3(sgrid),
                         dim3(256), 0, s, conv_state, (const float*)proj, ld,
                         q_off, k_off, v_off, taps, state_slots, qlocs,
                         seq_lens, S, Cq, C);
  } else {
    hipLaunchKernelGGL(delta_prep_kernel<u16>, dim3(grid), dim3(WPB * WAVE), 0,
                       s, qn, kn, vv, (const u16*)proj, ld, q_off, k_off, v_off,
                       conv_w, taps, conv_state, state_slots, qlocs, seq_lens,
                       token_seq, T, H, G, dk, dv);
    hipLaunchKernelGGL(delta_gates_kernel<u16>, ggrid, dim3(WPB * WAVE), 0, s,
                       decay, beta, (const u16*)proj, ld, b_off, a1_off, a2,
                       rank, dt_bias, a_log, T, H, dk);
    if (taps > 1)
      hipLaunchKernelGGL(conv_state_update_kernel<u16>, dim3(sgrid), dim3(256),
                         0, s, conv_state, (const u16*)proj, ld, q_off, k_off,
                         v_off, taps, state_slots, qlocs, seq_lens, S, Cq, C);
  }
}

extern "C" void mix_delta_scan(float* o, const float* qn, const float* kn,
                               const float* vv, const float* decay,
                               const float* beta, float* ssm,
                               const int* state_slots, const int* qlocs,
                               const int* seq_lens, int S, int H, int G, int dk,
                               int dv, hipStream_t s) {
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
  if (grid == 0) return;
#define LAUNCH_SCAN(RR, PP)                                                  \
  hipLaunchKernelGGL((delta_scan_kernel<RR, PP>), dim3((unsigned)grid),      \
                     dim3(256), 0, s, o, qn, kn, vv, decay, beta, ssm,       \
                     state_slots, qlocs, seq_lens, H, G, dk, dv, col_groups)
  if (rpt == 32) {
    if (R == 1) LAUNCH_SCAN(1, 32);
    else if (R == 2) LAUNCH_SCAN(2, 32);
    else if (R == 4) LAUNCH_SCAN(4, 32);
    else LAUNCH_SCAN(8, 32);
  } else {
    if (R == 2) LAUNCH_SCAN(2, 16);
    else if (R == 4) LAUNCH_SCAN(4, 16);
    else if (R == 8) LAUNCH_SCAN(8, 16);
    else LAUNCH_SCAN(16, 16);
  }
#undef LAUNCH_SCAN
}

extern "C" void mix_delta_out(void* out, long ldo, int out_off, const float* o,
                              const float* norm_w, const void* proj, long ld,
                              int g1_off, const float* g2, int rank, float eps,
                              float out_scale, long T, int H, int dv, int f32,
                              hipStream_t s) {
  if (T == 0) return;
  const dim3 grid((unsigned)((T + WPB * GT - 1) / (WPB * GT)), (unsigned)H);
  if (f32)
    hipLaunchKernelGGL(delta_out_kernel<float>, grid, dim3(WPB * WAVE),
                       0, s, (float*)out, ldo, out_off, o, norm_w,
                       (const float*)proj, ld, g1_off, g2, rank, eps,
                       out_scale, T, H, dv);
  else
    hipLaunchKernelGGL(delta_out_kernel<u16>, grid, dim3(WPB * WAVE), 0,
                       s, (u16*)out, ldo, out_off, o, norm_w,
                       (const u16*)proj, ld, g1_off, g2, rank, eps, out_scale,
                       T, H, dv);
}
