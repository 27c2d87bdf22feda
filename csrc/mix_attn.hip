// Local (chunked / windowed) paged attention with split key and value sizes.
//
//   attn_prep        per-head RMS norm of q and k, rotation of a prefix of
//                    each head (rotate-half pairing; cos and sin of the fp32
//                    angle position * inv_freq[i] come in a [T, 2*half] table
//                    made once per step), K/V scatter into the paged caches,
//                    q out.
//   local_attention  softmax attention of every new token over the cached
//                    keys its mask lets it see, times a per-head sigmoid gate.
//
// Cache layout per layer: K [blocks, G, page, dk], V [blocks, G, page, dv].
// Mask of a query at position p: keys j in [lo, p],
//   lo = max(chunk ? (p / chunk) * chunk : 0, window ? p - window + 1 : 0).
// Positions count from the start of the sequence, so a chunk edge does not
// move when a prompt is processed in pieces.
//
// One wave per (token, head) for both kernels; all math fp32.
#include "mix_common.h"

#define WPB 4  // waves per block

template <typename A>
__global__ void attn_prep_kernel(
    A* __restrict__ q_out, const A* __restrict__ proj, long ld, int q_off,
    int k_off, int v_off, const float* __restrict__ q_w,
    const float* __restrict__ k_w, float eps,
    const float* __restrict__ cos_sin, int half,
    const long* __restrict__ slots, A* __restrict__ k_cache,
    A* __restrict__ v_cache, long T, int H, int G, int dk, int dv, int page) {
  extern __shared__ float sm[];  // WPB * dmax floats
  const int lane = threadIdx.x & (WAVE - 1);
  const int wid = threadIdx.x / WAVE;
  const int dmax = dk > dv ? dk : dv;
  float* buf = sm + wid * dmax;
  const int units = H + 2 * G;
  const long u = (long)blockIdx.x * WPB + wid;
  const bool valid = u < T * units;
  const long t = valid ? u / units : 0;
  const int j = valid ? (int)(u - t * units) : 0;
  // unit kind: 0 = q head, 1 = k head, 2 = v head
  const int kind = j < H ? 0 : (j < H + G ? 1 : 2);
  const int head = kind == 0 ? j : (kind == 1 ? j - H : j - H - G);
  const int d = kind == 2 ? dv : dk;
  const A* src = proj + t * ld +
                 (kind == 0 ? q_off : (kind == 1 ? k_off : v_off)) +
                 (long)head * d;
  const float* w = kind == 0 ? q_w : (kind == 1 ? k_w : nullptr);

  float ssq = 0.f;
  for (int i = lane; i < d; i += WAVE) {
    const float x = ldf<A>(src + i);
    buf[i] = x;
    ssq += x * x;
  }
  ssq = wave_sum_f32(ssq);
  const float inv = w ? 1.f / sqrtf(ssq / (float)d + eps) : 1.f;
  __syncthreads();
  const int hf = kind == 2 ? 0 : half;
  const float* cs = cos_sin + t * 2L * half;  // row t: cos[half] | sin[half]
  A* dst;
  if (kind == 0) {
    dst = q_out + (t * H + head) * (long)dk;
  } else {
    const long slot = slots[t];
    const long blk = slot / page, off = slot - blk * page;
    dst = (kind == 1 ? k_cache : v_cache) +
          ((blk * G + head) * page + off) * (long)d;
  }
  for (int i = lane; i < d; i += WAVE) {
    float x = buf[i] * inv * (w ? w[i] : 1.f);
    if (i < 2 * hf) {
      const int fi = i < hf ? i : i - hf;
      const int mate = i < hf ? i + hf : i - hf;
      const float y = buf[mate] * inv * (w ? w[mate] : 1.f);
      const float c = cs[fi], s = cs[half + fi];
      x = i < hf ? x * c - y * s : x * c + y * s;
    }
    if (valid) stf<A>(dst + i, x);
  }
}

// NV = value columns per lane (dv <= 64 * NV)
template <typename A, int NV>
__global__ void local_attention_kernel(
    A* __restrict__ out, long ldo, int out_off, const A* __restrict__ q,
    const A* __restrict__ k_cache, const A* __restrict__ v_cache,
    const int* __restrict__ bt, int bt_stride, const int* __restrict__ seq_lens,
    const int* __restrict__ qlocs, const int* __restrict__ token_seq,
    float scale, int chunk, int window, const A* __restrict__ proj, long ld,
    int gate_off, float out_scale, long t0, long T, int H, int G, int dk,
    int dv, int page) {
  extern __shared__ float sm[];  // WPB * dk floats: the wave's query
  const int lane = threadIdx.x & (WAVE - 1);
  const int wid = threadIdx.x / WAVE;
  float* qs = sm + wid * dk;
  const long u = (long)blockIdx.x * WPB + wid;
  const bool valid = u < T * H;
  const long t = t0 + (valid ? u / H : 0);  // rows [t0, t0 + T)
  const int h = valid ? (int)(u % H) : 0;
  const int g = h / (H / G);
  for (int i = lane; i < dk; i += WAVE)
    qs[i] = ldf<A>(q + (t * H + h) * (long)dk + i);
  __syncthreads();
  if (!valid) return;

  const int s = token_seq[t];
  const int p = seq_lens[s] - (qlocs[s + 1] - (int)t);  // position of token t
  int lo = 0;
  if (chunk > 0) lo = (p / chunk) * chunk;
  if (window > 0 && p - window + 1 > lo) lo = p - window + 1;
  const int* table = bt + (long)s * bt_stride;

  float m = -INFINITY, l = 0.f;
  float acc[NV];
#pragma unroll
  for (int c = 0; c < NV; ++c) acc[c] = 0.f;

  for (int base = lo; base <= p; base += WAVE) {
    const int j = base + lane;
    const bool live = j <= p;
    int row = 0;  // blk * page + offset of key j
    float sc = -INFINITY;
    if (live) {
      row = table[j / page] * page + j % page;
      const long blk = row / page, off = row - blk * page;
      const A* kr = k_cache + ((blk * G + g) * page + off) * (long)dk;
      float dot = 0.f;
      for (int i = 0; i < dk; ++i) dot += qs[i] * ldf<A>(kr + i);
      sc = dot * scale;
    }
    const float m_new = fmaxf(m, wave_max_f32(sc));
    const float pj = live ? expf(sc - m_new) : 0.f;
    const float corr = expf(m - m_new);  // m = -inf on the first tile -> 0
    l = l * corr + wave_sum_f32(pj);
#pragma unroll
    for (int c = 0; c < NV; ++c) acc[c] *= corr;
    m = m_new;
    const int n = (p - base + 1) < (int)WAVE ? (p - base + 1) : (int)WAVE;
    for (int jj = 0; jj < n; ++jj) {
      const float pw = __shfl(pj, jj, WAVE);
      const int r = __shfl(row, jj, WAVE);
      const long blk = r / page, off = r - blk * page;
      const A* vr = v_cache + ((blk * G + g) * page + off) * (long)dv;
#pragma unroll
      for (int c = 0; c < NV; ++c) {
        const int col = lane + c * (int)WAVE;
        if (col < dv) acc[c] += pw * ldf<A>(vr + col);
      }
    }
  }
  float gate = out_scale;
  if (gate_off >= 0) gate *= sigmoid_f(ldf<A>(proj + t * ld + gate_off + h));
  const float f = gate / l;
#pragma unroll
  for (int c = 0; c < NV; ++c) {
    const int col = lane + c * (int)WAVE;
    if (col < dv)
      stf<A>(out + t * ldo + out_off + (long)h * dv + col, acc[c] * f);
  }
}

extern "C" void mix_attn_prep(void* q_out, const void* proj, long ld,
                              int q_off, int k_off, int v_off,
                              const float* q_w, const float* k_w, float eps,
                              const float* cos_sin, int half,
                              const long* slots, void* k_cache, void* v_cache,
                              long T, int H, int G, int dk, int dv, int page,
                              int f32, hipStream_t s) {
  const long units = T * (H + 2 * G);
  const int grid = (int)((units + WPB - 1) / WPB);
  const int dmax = dk > dv ? dk : dv;
  const size_t smem = (size_t)WPB * dmax * sizeof(float);
  if (grid == 0) return;
  if (f32)
    hipLaunchKernelGGL(attn_prep_kernel<float>, dim3(grid), dim3(WPB * WAVE),
                       smem, s, (float*)q_out, (const float*)proj, ld, q_off,
                       k_off, v_off, q_w, k_w, eps, cos_sin, half, slots,
                       (float*)k_cache, (float*)v_cache, T, H, G, dk, dv, page);
  else
    hipLaunchKernelGGL(attn_prep_kernel<u16>, dim3(grid), dim3(WPB * WAVE),
                       smem, s, (u16*)q_out, (const u16*)proj, ld, q_off,
                       k_off, v_off, q_w, k_w, eps, cos_sin, half, slots,
                       (u16*)k_cache, (u16*)v_cache, T, H, G, dk, dv, page);
}

template <typename A>
static void launch_local_attention(
    void* out, long ldo, int out_off, const void* q, const void* k_cache,
    const void* v_cache, const int* bt, int bt_stride, const int* seq_lens,
    const int* qlocs, const int* token_seq, float scale, int chunk,
    int window, const void* proj, long ld, int gate_off, float out_scale,
    long t0, long T, int H, int G, int dk, int dv, int page, hipStream_t s) {
  const long units = T * H;
  const int grid = (int)((units + WPB - 1) / WPB);
  if (grid == 0) return;
  const size_t smem = (size_t)WPB * dk * sizeof(float);
#define LAUNCH_LA(NV)                                                        \
  hipLaunchKernelGGL((local_attention_kernel<A, NV>), dim3(grid),            \
                     dim3(WPB * WAVE), smem, s, (A*)out, ldo, out_off,       \
                     (const A*)q, (const A*)k_cache, (const A*)v_cache, bt,  \
                     bt_stride, seq_lens, qlocs, token_seq, scale, chunk,    \
                     window, (const A*)proj, ld, gate_off, out_scale, t0, T, \
                     H, G, dk, dv, page)
  if (dv <= 64) LAUNCH_LA(1);
  else if (dv <= 128) LAUNCH_LA(2);
  else LAUNCH_LA(4);
#undef LAUNCH_LA
}

extern "C" void mix_local_attention(
    void* out, long ldo, int out_off, const void* q, const void* k_cache,
    const void* v_cache, const int* bt, int bt_stride, const int* seq_lens,
    const int* qlocs, const int* token_seq, float scale, int chunk,
    int window, const void* proj, long ld, int gate_off, float out_scale,
    long t0, long T, int H, int G, int dk, int dv, int page, int f32,
    hipStream_t s) {
  if (f32)
    launch_local_attention<float>(out, ldo, out_off, q, k_cache, v_cache, bt,
                                  bt_stride, seq_lens, qlocs, token_seq, scale,
                                  chunk, window, proj, ld, gate_off, out_scale,
                                  t0, T, H, G, dk, dv, page, s);
  else
    launch_local_attention<u16>(out, ldo, out_off, q, k_cache, v_cache, bt,
                                bt_stride, seq_lens, qlocs, token_seq, scale,
                                chunk, window, proj, ld, gate_off, out_scale,
                                t0, T, H, G, dk, dv, page, s);
}
