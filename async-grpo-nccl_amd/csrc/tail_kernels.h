// Per-token GRPO objective, segmented reductions over cu_seqlens, per-group
// reward statistics, diagnostics, and the row soft-max kernels that serve
// callers holding materialised logits.  All of these are HBM-bound streaming
// kernels (tens of bytes per token); reductions are two-stage with a fixed
// order so that two runs on the same input are bit-identical.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include "lmhead_kernels.h"

namespace fgrpo {

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o);
  return v;
}
__device__ __forceinline__ double wave_sum_d(double v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o);
  return v;
}
__device__ __forceinline__ int wave_sum_i(int v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o);
  return v;
}

// Offsets read from device memory (cu_seqlens, group offsets) are clamped into [0, n] and made monotone before
// they index anything: a malformed vector then yields wrong numbers for its own rows, never an access outside
// the arrays.
__device__ __forceinline__ void clamp_range(int& b, int& e, int n) {
  b = b < 0 ? 0 : (b > n ? n : b);
  e = e < b ? b : (e > n ? n : e);
}

__global__ void fill_f32_kernel(float* dst, float v, int n) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) dst[i] = v;
}
__global__ void fill_i64_kernel(long long* dst, long long v, int n) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) dst[i] = v;
}

// ---------------------------------------------------------------------------
// Segment (sample) statistics over cu_seqlens: one wavefront per segment.
// ---------------------------------------------------------------------------
// cnt[s] = number of valid (label != -100) tokens of segment s; tokw[t] = 1/cnt
// of the token's segment (0 when the segment has no valid token).
__global__ void segment_valid_weight_kernel(const long long* labels, const int* cu, int nseq, int T, int* cnt, float* tokw) {
  const int s = blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
  const int lane = threadIdx.x & 63;
  if (s >= nseq) return;
  int b = cu[s], e = cu[s + 1];
  clamp_range(b, e, T);
  int c = 0;
  for (int t = b + lane; t < e; t += 64) c += (labels[t] != -100);
  c = wave_sum_i(c);
  if (lane == 0) cnt[s] = c;
  const float w = c > 0 ? 1.0f / (float)c : 0.f;
  for (int t = b + lane; t < e; t += 64) tokw[t] = w;
}

// out[t] = values[s] for every token of segment s
__global__ void segment_broadcast_kernel(const void* values, int values_f64, const int* cu, int nseq, int T, float* out) {
  const int s = blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
  const int lane = threadIdx.x & 63;
  if (s >= nseq) return;
  const float v = values_f64 ? (float)((const double*)values)[s] : ((const float*)values)[s];
  int b = cu[s], e = cu[s + 1];
  clamp_range(b, e, T);
  for (int t = b + lane; t < e; t += 64) out[t] = v;
}

// sum[s], and mean[s] = sum / count over the (optionally masked) tokens of segment s
__global__ void segment_reduce_kernel(const float* x, const long long* labels, const int* cu, int nseq, int T, float* sum,
                                      float* mean, int* count) {
  const int s = blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
  const int lane = threadIdx.x & 63;
  if (s >= nseq) return;
  float a = 0.f;
  int c = 0;
  int b = cu[s], e = cu[s + 1];
  clamp_range(b, e, T);
  for (int t = b + lane; t < e; t += 64) {
    const bool ok = labels ? (labels[t] != -100) : true;
    a += ok ? x[t] : 0.f;
    c += ok;
  }
  a = wave_sum(a);
  c = wave_sum_i(c);
  if (lane == 0) {
    if (sum) sum[s] = a;
    if (mean) mean[s] = c > 0 ? a / (float)c : 0.f;
    if (count) count[s] = c;
  }
}

// Positions of the logits that score each sample's generated tokens: sample i,
// packed at token offset tok_off[i], contributes
//   tok_off[i] + in_len[i] - 1 + j   for j in [0, out_len[i])
// written at out_off[i] + j.  One wavefront per sample.
__global__ void output_indices_kernel(const int* tok_off, const int* in_len, const int* out_off, int nsamples,
                                      int n_out, long long* out) {
  const int s = blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
  const int lane = threadIdx.x & 63;
  if (s >= nsamples) return;
  int b = out_off[s], e = out_off[s + 1];
  clamp_range(b, e, n_out);
  const long long first = (long long)tok_off[s] + in_len[s] - 1;
  for (int j = lane; j < e - b; j += 64) out[b + j] = first + j;
}

// Training labels of a packed batch: inside sample i (tokens tok_off[i] .. tok_off[i+1]) the generated span
// [in_len[i], in_len[i] + out_len[i]) keeps its token id, everything else is -100.  One wavefront per sample.
__global__ void build_labels_kernel(const long long* ids, const int* tok_off, const int* in_len, const int* out_len,
                                    int nsamples, int T, long long* labels) {
  const int s = blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
  const int lane = threadIdx.x & 63;
  if (s >= nsamples) return;
  int b = tok_off[s], e = tok_off[s + 1];
  clamp_range(b, e, T);
  const int lo = in_len[s], hi = lo + out_len[s];
  for (int t = b + lane; t < e; t += 64) {
    const int k = t - b;
    labels[t] = (k >= lo && k < hi) ? ids[t] : -100;
  }
}

// cu_seqlens from position ids: ordered list of the indices t with pos[t] == 0,
// followed by T.  A single work-group walks the array in order, eight
// consecutive tokens per thread and round; the rank of a hit is the prefix of
// the per-thread counts, so the output order is the token order.
// out has room for max_out entries; *count receives the number of boundaries
// found + 1 (even when it exceeds max_out, in which case the tail is dropped).
__global__ __launch_bounds__(1024) void segment_starts_kernel(const long long* pos, int T, int* out, int max_out,
                                                              int* count) {
  constexpr int kPer = 8;                    // consecutive tokens per thread and round
  __shared__ int wave_cnt[16];
  __shared__ int base;
  const int lane = threadIdx.x & 63, wv = threadIdx.x >> 6;
  if (threadIdx.x == 0) base = 0;
  __syncthreads();
  for (long long t0 = 0; t0 < T; t0 += 1024 * kPer) {
    const long long first = t0 + (long long)threadIdx.x * kPer;
    unsigned hits = 0;
#pragma unroll
    for (int i = 0; i < kPer; ++i)
      if (first + i < T && pos[first + i] == 0) hits |= 1u << i;
    const int mine = __popc(hits);
    // exclusive prefix of the per-thread counts inside the wavefront
    int incl = mine;
#pragma unroll
    for (int d = 1; d < 64; d <<= 1) {
      const int up = __shfl_up(incl, d, 64);
      if (lane >= d) incl += up;
    }
    if (lane == 63) wave_cnt[wv] = incl;
    __syncthreads();
    int off = base + incl - mine;
    for (int w = 0; w < wv; ++w) off += wave_cnt[w];
#pragma unroll
    for (int i = 0; i < kPer; ++i)
      if (hits & (1u << i)) {
        if (off < max_out) out[off] = (int)(first + i);
        ++off;
      }
    __syncthreads();
    if (threadIdx.x == 0) {
      int tot = 0;
      for (int w = 0; w < 16; ++w) tot += wave_cnt[w];
      base += tot;
    }
    __syncthreads();
  }
  if (threadIdx.x == 0) {
    if (base < max_out) out[base] = T;
    *count = base + 1;
  }
}

// adv[i] = (r[i] - mean_g) / (std_pop_g + eps) per group, double arithmetic
__global__ void group_advantage_kernel(const void* rewards, int rewards_f64, const int* goff, int ngroups, int n_rewards,
                                       double eps, float* out_f32, double* out_f64) {
  const int g = blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
  const int lane = threadIdx.x & 63;
  if (g >= ngroups) return;
  int b = goff[g], e = goff[g + 1];
  clamp_range(b, e, n_rewards);
  auto rd = [&](int i) -> double {
    return rewards_f64 ? ((const double*)rewards)[i] : (double)((const float*)rewards)[i];
  };
  double s = 0.0;
  for (int i = b + lane; i < e; i += 64) s += rd(i);
  s = wave_sum_d(s);
  const int n = e - b;
  const double mean = n > 0 ? s / (double)n : 0.0;
  double q = 0.0;
  for (int i = b + lane; i < e; i += 64) {
    const double d = rd(i) - mean;
    q += d * d;
  }
  q = wave_sum_d(q);
  const double sd = n > 0 ? sqrt(q / (double)n) : 0.0;
  const double inv = 1.0 / (sd + eps);
  for (int i = b + lane; i < e; i += 64) {
    const double a = (rd(i) - mean) * inv;
    if (out_f32) out_f32[i] = (float)a;
    if (out_f64) out_f64[i] = a;
  }
}

// ---------------------------------------------------------------------------
// GRPO per-token objective (dual clip, optional k3 KL to a reference policy)
// ---------------------------------------------------------------------------
struct LossParams {
  const float* lp;           // [T] policy logprob (0 on masked tokens)
  const float* old_lp;       // [T] or null (=> ratio 1)
  const float* ref_lp;       // [T] or null
  const float* adv;          // [T]
  const long long* labels;   // shifted labels [T]
  const float* tokw;         // [T] per-token weight (sample_mean) or null (token_mean)
  const int* seg_cnt;        // [nseq] valid tokens per segment (sample_mean) or null
  int nseq;
  int T;
  float clip_low, clip_high, clip_c, kl_beta;
  int agg_mode;              // 0 token_mean, 1 sample_mean
  double denom_override;     // > 0: use as normaliser (number of samples / tokens)
  float* g;                  // [T] d loss / d lp
  float* log_ratio;          // [T]
  float* clip1;              // [T]
  float* unclipped;          // [T]
  float* clipped;            // [T]
  double* partial;           // [2 * nblocks] : sum, count
  float* loss;               // scalar
  float* scal;               // [4] : normaliser, valid count, nonempty segments, raw sum
  // Normaliser known before the tokens are walked (grpo_loss_prepare_kernel): {denominator, valid tokens, non-empty
  // segments, 1 / denominator rounded to fp32}.  With it the token kernel writes g already normalised - the same
  // two fp32 products the finalize kernel would have made - so that a caller may walk the tokens in chunks and use
  // each chunk's g before the last chunk has been seen; the finalize kernel then only forms the loss.
  const double* pre;
};

constexpr int kLossThreads = 256;

__global__ __launch_bounds__(kLossThreads) void grpo_loss_tokens_kernel(const LossParams p) {
  __shared__ double sh[2][kLossThreads / 64];
  const int t = blockIdx.x * kLossThreads + threadIdx.x;
  float contrib = 0.f;
  int cnt = 0;
  if (t < p.T) {
    const bool valid = p.labels[t] != -100;
    const float lp = p.lp[t];
    const float old = p.old_lp ? p.old_lp[t] : lp;
    const float a = p.adv[t];
    const float lr = lp - old;
    const float r = expf(lr);
    const float lo = 1.0f - p.clip_low, hi = 1.0f + p.clip_high;
    const float l1 = -a * r;
    const float rc = fminf(fmaxf(r, lo), hi);
    const float l2 = -a * rc;
    const float c1 = fmaxf(l1, l2);
    const float c2 = fminf(c1, -a * p.clip_c);
    float tok = (a < 0.f) ? c2 : c1;
    const bool live = (a > 0.f && r <= hi) || (a < 0.f && r >= lo && r <= p.clip_c);
    float dtok = live ? -a * r : 0.f;
    if (p.ref_lp && p.kl_beta != 0.f) {
      const float d = p.ref_lp[t] - lp;
      const float ed = expf(d);
      tok += p.kl_beta * (ed - d - 1.0f);
      dtok += p.kl_beta * (1.0f - ed);
    }
    const float w = valid ? (p.tokw ? p.tokw[t] : 1.0f) : 0.f;
    float gv = w * dtok;
    if (p.pre) gv *= (float)p.pre[3];
    p.g[t] = gv;
    if (p.log_ratio) p.log_ratio[t] = lr;
    if (p.clip1) p.clip1[t] = c1;
    if (p.unclipped) p.unclipped[t] = l1;
    if (p.clipped) p.clipped[t] = l2;
    contrib = valid ? w * tok : 0.f;
    cnt = valid;
  }
  double s = wave_sum_d((double)contrib);
  int c = wave_sum_i(cnt);
  const int lane = threadIdx.x & 63, wv = threadIdx.x >> 6;
  if (lane == 0) {
    sh[0][wv] = s;
    sh[1][wv] = (double)c;
  }
  __syncthreads();
  if (threadIdx.x == 0) {
    double a = 0.0, b = 0.0;
    for (int i = 0; i < kLossThreads / 64; ++i) {
      a += sh[0][i];
      b += sh[1][i];
    }
    p.partial[2 * blockIdx.x] = a;
    p.partial[2 * blockIdx.x + 1] = b;
  }
}

// Every block re-derives the totals from the block partials in the same order,
// then scales its slices of g (a grid-stride walk: the launch holds at most
// kFinalizeBlocks blocks, so the partials are re-read that many times at most)
// by the normaliser; block 0 publishes the scalars.
constexpr int kFinalizeBlocks = 256;
__global__ __launch_bounds__(kLossThreads) void grpo_loss_finalize_kernel(const LossParams p, int nparts) {
  __shared__ double part[3][kLossThreads / 64];
  __shared__ double tot[3];
  {
    // all four wavefronts add their strided share, then one thread adds the four results: a fixed order
    double a = 0.0, b = 0.0, ne = 0.0;
    for (int i = threadIdx.x; i < nparts; i += kLossThreads) {
      a += p.partial[2 * i];
      b += p.partial[2 * i + 1];
    }
    if (p.seg_cnt)
      for (int i = threadIdx.x; i < p.nseq; i += kLossThreads) ne += (p.seg_cnt[i] > 0) ? 1.0 : 0.0;
    a = wave_sum_d(a);
    b = wave_sum_d(b);
    ne = wave_sum_d(ne);
    if ((threadIdx.x & 63) == 0) {
      part[0][threadIdx.x >> 6] = a;
      part[1][threadIdx.x >> 6] = b;
      part[2][threadIdx.x >> 6] = ne;
    }
    __syncthreads();
    if (threadIdx.x < 3) {
      double t = 0.0;
      for (int w = 0; w < kLossThreads / 64; ++w) t += part[threadIdx.x][w];
      tot[threadIdx.x] = t;
    }
  }
  __syncthreads();
  double den = (p.agg_mode == 0) ? tot[1] : tot[2];
  if (p.denom_override > 0.0) den = p.denom_override;
  if (den < 1.0) den = 1.0;
  double valid_n = tot[1], nonempty = tot[2];
  if (p.pre) {                       // the same numbers, formed from the labels before the tokens were walked
    den = p.pre[0];
    valid_n = p.pre[1];
    nonempty = p.pre[2];
  }
  const float norm = (float)(1.0 / den);
  if (!p.pre)
    for (long long t = (long long)blockIdx.x * kLossThreads + threadIdx.x; t < p.T; t += (long long)gridDim.x * kLossThreads)
      p.g[t] *= norm;
  if (blockIdx.x == 0 && threadIdx.x == 0) {
    *p.loss = (float)(tot[0] / den);
    if (p.scal) {
      p.scal[0] = norm;
      p.scal[1] = (float)valid_n;
      p.scal[2] = (float)nonempty;
      p.scal[3] = (float)tot[0];
    }
  }
}

// The normaliser of the objective depends on the labels and the segments only: valid tokens (token mean), segments
// with at least one valid token (sample mean), or the caller's override.  One work-group counts them before any
// logprob exists; pre = {denominator, valid tokens, non-empty segments, (double)(float)(1 / denominator)}.
__global__ __launch_bounds__(1024) void grpo_loss_prepare_kernel(const long long* labels, int T, const int* seg_cnt,
                                                                 int nseq, int agg_mode, double denom_override,
                                                                 double* pre) {
  __shared__ int sh[2][16];
  int c = 0, ne = 0;
  for (int t = threadIdx.x; t < T; t += 1024) c += (labels[t] != -100);
  if (seg_cnt)
    for (int i = threadIdx.x; i < nseq; i += 1024) ne += (seg_cnt[i] > 0);
  c = wave_sum_i(c);
  ne = wave_sum_i(ne);
  if ((threadIdx.x & 63) == 0) {
    sh[0][threadIdx.x >> 6] = c;
    sh[1][threadIdx.x >> 6] = ne;
  }
  __syncthreads();
  if (threadIdx.x == 0) {
    long long cs = 0, ns = 0;
    for (int w = 0; w < 16; ++w) {
      cs += sh[0][w];
      ns += sh[1][w];
    }
    double den = (agg_mode == 0) ? (double)cs : (double)ns;
    if (denom_override > 0.0) den = denom_override;
    if (den < 1.0) den = 1.0;
    pre[0] = den;
    pre[1] = (double)cs;
    pre[2] = (double)ns;
    pre[3] = (double)(float)(1.0 / den);
  }
}

// ---------------------------------------------------------------------------
// Diagnostics over the output-token index list, one launch, one result vector.
// ---------------------------------------------------------------------------
constexpr int kNumStats = 16;
struct MetricParams {
  const long long* idx;      // [n] positions
  int n;
  int T;
  const float* log_ratio;    // [T]
  const float* entropy;      // [T] or null
  const float* old_entropy;  // [T] or null
  const float* adv;          // [T]
  const float* unclipped;    // [T]
  const float* clipped;      // [T]
  float clip_low, clip_high;
  double* stats;             // [kNumStats] (one work-group) or [gridDim.x][kNumStats] partial sums
};
constexpr int kMetricBlocks = 128;     // most work-groups of the first stage

__global__ __launch_bounds__(1024) void grpo_metrics_kernel(const MetricParams p) {
  __shared__ double sh[kNumStats][16];
  double a[kNumStats];
#pragma unroll
  for (int k = 0; k < kNumStats; ++k) a[k] = 0.0;
  for (long long i = (long long)blockIdx.x * 1024 + threadIdx.x; i < p.n; i += (long long)gridDim.x * 1024) {
    long long t = p.idx[i];
    if (t < 0) t += p.T;  // python-style negative index
    if (t < 0 || t >= p.T) {
      a[15] += 1.0;  // out-of-range indices are counted, never dereferenced
      continue;
    }
    const float lr = p.log_ratio[t];
    const float r = expf(lr);
    const float ad = p.adv[t];
    a[0] += 1.0;
    a[1] += fabsf(lr);
    a[2] += lr;
    a[3] += (double)lr * lr;
    a[4] += (r - 1.0f - lr);
    a[5] += (r > 1.0f + p.clip_high) ? 1.0 : 0.0;
    a[6] += (r < 1.0f - p.clip_low) ? 1.0 : 0.0;
    a[7] += p.entropy ? p.entropy[t] : 0.f;
    a[8] += p.old_entropy ? p.old_entropy[t] : 0.f;
    a[9] += ad;
    a[10] += (double)ad * ad;
    a[11] += (ad > 0.f) ? 1.0 : 0.0;
    a[12] += (ad == 0.f) ? 1.0 : 0.0;
    a[13] += (p.clipped[t] > p.unclipped[t]) ? 1.0 : 0.0;
  }
  const int lane = threadIdx.x & 63, wv = threadIdx.x >> 6;
#pragma unroll
  for (int k = 0; k < kNumStats; ++k) {
    const double v = wave_sum_d(a[k]);
    if (lane == 0) sh[k][wv] = v;
  }
  __syncthreads();
  if (threadIdx.x < kNumStats) {
    double v = 0.0;
    for (int w = 0; w < 16; ++w) v += sh[threadIdx.x][w];
    p.stats[(long long)blockIdx.x * kNumStats + threadIdx.x] = v;
  }
}

// second stage: one wavefront per statistic; lane l adds the partial sums of work-groups l, l + 64, ... and the 64
// lanes are combined by the same butterfly every time (a fixed order: two runs agree bit for bit)
__global__ __launch_bounds__(64 * kNumStats) void grpo_metrics_reduce_kernel(const double* partial, int nblocks, double* stats) {
  const int k = threadIdx.x >> 6, lane = threadIdx.x & 63;
  double v = 0.0;
  for (int b = lane; b < nblocks; b += 64) v += partial[(long long)b * kNumStats + k];
  v = wave_sum_d(v);
  if (lane == 0) stats[k] = v;
}

// ---------------------------------------------------------------------------
// Row soft-max statistics on materialised logits [N x V] (bf16 or fp32):
// logprob of the label, entropy, lse; one work-group per row, one pass.
// ---------------------------------------------------------------------------
struct RowParams {
  const void* logits;
  int is_f32;
  long long ld;
  int N, V;
  const long long* labels;   // [N] or null; -100 (or `ignore`) = ignored
  long long ignore;
  int use_ignore;
  float* lp;                 // [N] or null
  float* ent;                // [N] or null
  float* lse;                // [N] or null
};

__device__ __forceinline__ float row_load(const RowParams& p, long long row, int v) {
  const long long o = row * p.ld + v;
  return p.is_f32 ? ((const float*)p.logits)[o] : bf16_to_f32(((const bf16_t*)p.logits)[o]);
}

// eight consecutive elements of a row as floats: one 16-byte load for bf16, two for fp32 (the row must start on a
// 16-byte boundary and c counts chunks of eight)
template <bool F32>
__device__ __forceinline__ void row_load8(const void* row_base, int c, float (&x)[8]) {
  if constexpr (F32) {
    const float4* b = (const float4*)row_base + 2 * (long long)c;
    const float4 lo = b[0], hi = b[1];
    x[0] = lo.x; x[1] = lo.y; x[2] = lo.z; x[3] = lo.w;
    x[4] = hi.x; x[5] = hi.y; x[6] = hi.z; x[7] = hi.w;
  } else {
    const uint4 q = ((const uint4*)row_base)[c];
    const uint32_t u[4] = {q.x, q.y, q.z, q.w};
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      x[2 * k] = __uint_as_float(u[k] << 16);
      x[2 * k + 1] = __uint_as_float(u[k] & 0xffff0000u);
    }
  }
}

// running (max, sum exp, sum exp * x) of one thread over the chunks c = first, first + 256, ... of a row
template <bool F32>
__device__ __forceinline__ void row_stats_chunks(const void* row_base, int nv, float& m, float& s, float& sx) {
  for (int c = threadIdx.x; c < nv; c += 256) {
    float x[8];
    row_load8<F32>(row_base, c, x);
    float mt = x[0];
#pragma unroll
    for (int k = 1; k < 8; ++k) mt = fmaxf(mt, x[k]);
    const float mn = fmaxf(m, mt);
    const float al = fast_exp2((m - mn) * kLog2e);
    s *= al;
    sx *= al;
#pragma unroll
    for (int k = 0; k < 8; ++k) {
      const float e = fast_exp2((x[k] - mn) * kLog2e);
      s += e;
      sx = __builtin_fmaf(e, x[k], sx);
    }
    m = mn;
  }
}

__device__ __forceinline__ bool row_vectorisable(const RowParams& p) {
  return (p.ld % 8 == 0) && ((((uintptr_t)p.logits) & 15) == 0);
}

__global__ __launch_bounds__(256) void logits_row_stats_kernel(const RowParams p) {
  __shared__ float sh[3][4];
  const long long row = blockIdx.x;
  float m = kNegBig, s = 0.f, sx = 0.f;
  int done = 0;                      // elements covered by the 16-byte loop
  if (row_vectorisable(p)) {
    const int nv = p.V / 8;
    if (p.is_f32)
      row_stats_chunks<true>((const float*)p.logits + row * p.ld, nv, m, s, sx);
    else
      row_stats_chunks<false>((const bf16_t*)p.logits + row * p.ld, nv, m, s, sx);
    done = nv * 8;
  }
  for (int v = done + threadIdx.x; v < p.V; v += 256) {
    const float x = row_load(p, row, v);
    lse_merge(m, s, sx, x, 1.f, x);
  }
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) {
    const float m2 = __shfl_xor(m, o), s2 = __shfl_xor(s, o), x2 = __shfl_xor(sx, o);
    lse_merge(m, s, sx, m2, s2, x2);
  }
  const int lane = threadIdx.x & 63, wv = threadIdx.x >> 6;
  if (lane == 0) {
    sh[0][wv] = m;
    sh[1][wv] = s;
    sh[2][wv] = sx;
  }
  __syncthreads();
  if (threadIdx.x == 0) {
    for (int w = 1; w < 4; ++w) lse_merge(m, s, sx, sh[0][w], sh[1][w], sh[2][w]);
    const float lse = m + logf(s);
    if (p.lse) p.lse[row] = lse;
    if (p.ent) p.ent[row] = lse - sx / s;
    if (p.lp) {
      long long lab = p.labels[row];
      const bool ign = p.use_ignore && lab == p.ignore;
      float out;
      if (ign)
        out = 0.f;
      else if (lab >= 0 && lab < p.V)
        out = row_load(p, row, (int)lab) - lse;
      else
        out = __uint_as_float(0x7fc00000u);
      p.lp[row] = out;
    }
  }
}

// dlogits[n, v] = g[n] * (1[v == y_n] - exp(x - lse[n])); ignored rows give 0
struct RowBwdParams {
  RowParams f;
  const float* g;       // [N] upstream gradient of lp
  const float* lse;     // [N]
  void* dlogits;        // [N x V] in the logits' dtype, rows ld_out elements apart
  long long ld_out;
};

__global__ __launch_bounds__(256) void logits_row_bwd_kernel(const RowBwdParams p) {
  const long long row = blockIdx.x;
  const long long lab = p.f.labels[row];
  const bool ign = p.f.use_ignore && lab == p.f.ignore;
  const float g = ign ? 0.f : p.g[row];
  const float l2 = p.lse[row] * kLog2e;
  int done = 0;
  if (row_vectorisable(p.f) && p.ld_out % 8 == 0 && ((((uintptr_t)p.dlogits) & 15) == 0)) {
    // eight elements per thread and step: 16-byte loads and stores (two each for fp32)
    const int nv = p.f.V / 8;
    const int lab_chunk = (lab >= 0 && lab < p.f.V) ? (int)(lab >> 3) : -1, lab_k = (int)(lab & 7);
    for (int c = threadIdx.x; c < nv; c += 256) {
      float x[8], d[8];
      if (ign) {
#pragma unroll
        for (int k = 0; k < 8; ++k) d[k] = 0.f;          // nothing to read: the row takes no gradient
      } else {
        if (p.f.is_f32)
          row_load8<true>((const float*)p.f.logits + row * p.f.ld, c, x);
        else
          row_load8<false>((const bf16_t*)p.f.logits + row * p.f.ld, c, x);
#pragma unroll
        for (int k = 0; k < 8; ++k) d[k] = -g * fast_exp2(__builtin_fmaf(x[k], kLog2e, -l2));
        if (c == lab_chunk) {
#pragma unroll
          for (int k = 0; k < 8; ++k) d[k] += (k == lab_k) ? g : 0.f;
        }
      }
      if (p.f.is_f32) {
        float4* o = (float4*)((float*)p.dlogits + row * p.ld_out) + 2 * (long long)c;
        o[0] = make_float4(d[0], d[1], d[2], d[3]);
        o[1] = make_float4(d[4], d[5], d[6], d[7]);
      } else {
        uint4 q;
        q.x = pack_bf16x2(d[0], d[1]);
        q.y = pack_bf16x2(d[2], d[3]);
        q.z = pack_bf16x2(d[4], d[5]);
        q.w = pack_bf16x2(d[6], d[7]);
        ((uint4*)((bf16_t*)p.dlogits + row * p.ld_out))[c] = q;
      }
    }
    done = nv * 8;
  }
  for (int v = done + threadIdx.x; v < p.f.V; v += 256) {
    const float x = row_load(p.f, row, v);
    float d = -g * fast_exp2(__builtin_fmaf(x, kLog2e, -l2));
    if (v == lab) d += g;
    const long long o = row * p.ld_out + v;
    if (p.f.is_f32)
      ((float*)p.dlogits)[o] = d;
    else
      ((bf16_t*)p.dlogits)[o] = f32_to_bf16_rn(d);
  }
}

}  // namespace fgrpo
