// Small non-template kernels around the LM-head tile kernels: the per-token merge of the vocabulary splits,
// operand staging (padding, transposition, bf16 hi/lo split of fp32 inputs) and the bias-gradient column sums.
// Included by exactly one translation unit (the kernels here are ordinary external functions).
#pragma once
#include "lmhead_kernels.h"

namespace fgrpo {

// One thread per token: merge the vocabulary splits, emit logprob / entropy / lse.
struct CombineParams {
  const float4* part;
  const float* xt;
  const long long* labels;
  int T, V, nsplit;
  float* lp;    // [T]
  float* ent;   // [T] or null
  float* lse;   // [T] or null
};

__global__ void lmhead_fwd_combine_kernel(const CombineParams p) {
  const int n = blockIdx.x * blockDim.x + threadIdx.x;
  if (n >= p.T) return;
  float4 a = p.part[n];
  float m = a.x, s = a.y, sx = a.z;
  for (int k = 1; k < p.nsplit; ++k) {
    const float4 b = p.part[(long long)k * p.T + n];
    lse_merge(m, s, sx, b.x, b.y, b.z);
  }
  const float lse = m + logf(s);
  if (p.lse) p.lse[n] = lse;
  const long long lab = p.labels[n];
  const bool valid = (lab != -100);
  float lp = 0.f, ent = 0.f;
  if (valid) {
    // a label outside [0, V) has no target logit: report NaN rather than a silent number
    lp = (lab >= 0 && lab < p.V) ? (p.xt[n] - lse) : __uint_as_float(0x7fc00000u);
    ent = lse - sx / s;
  }
  p.lp[n] = lp;
  if (p.ent) p.ent[n] = ent;
}

// ---------------------------------------------------------------------------
// Operand preparation: copy / transpose a [R x Cn] matrix (fp32 or bf16) into a
// zero-padded bf16 buffer, optionally also emitting the bf16 low half of an fp32
// source (x ~= hi + lo).  Destination is [Rpad x ld] (or [Cpad x ld] transposed).
// ---------------------------------------------------------------------------
struct ConvertParams {
  const void* src;
  int src_is_f32;
  long long ld_src;
  int R, Cn;          // logical source shape
  int Rpad, Cpad;     // padded extents written
  bf16_t* hi;
  bf16_t* lo;         // or null
  long long ld_dst;
  int transpose;
};

__global__ __launch_bounds__(256) void convert_pad_kernel(const ConvertParams p) {
  __shared__ float th[64][65];
  __shared__ float tl[64][65];
  const int r0 = blockIdx.y * 64, c0 = blockIdx.x * 64;
  const int tx = threadIdx.x & 63, ty = threadIdx.x >> 6;  // 64 x 4
  for (int rr = ty; rr < 64; rr += 4) {
    const int r = r0 + rr, c = c0 + tx;
    float v = 0.f;
    if (r < p.R && c < p.Cn) {
      const long long o = (long long)r * p.ld_src + c;
      v = p.src_is_f32 ? ((const float*)p.src)[o] : bf16_to_f32(((const bf16_t*)p.src)[o]);
    }
    const float h = bf16_to_f32(f32_to_bf16_rn(v));
    th[rr][tx] = h;
    tl[rr][tx] = v - h;
  }
  __syncthreads();
  if (!p.transpose) {
    for (int rr = ty; rr < 64; rr += 4) {
      const int r = r0 + rr, c = c0 + tx;
      if (r < p.Rpad && c < p.Cpad) {
        const long long o = (long long)r * p.ld_dst + c;
        p.hi[o] = f32_to_bf16_rn(th[rr][tx]);
        if (p.lo) p.lo[o] = f32_to_bf16_rn(tl[rr][tx]);
      }
    }
  } else {
    for (int cc = ty; cc < 64; cc += 4) {
      const int c = c0 + cc, r = r0 + tx;
      if (c < p.Cpad && r < p.Rpad) {
        const long long o = (long long)c * p.ld_dst + r;
        p.hi[o] = f32_to_bf16_rn(th[tx][cc]);
        if (p.lo) p.lo[o] = f32_to_bf16_rn(tl[tx][cc]);
      }
    }
  }
}

__global__ void to_f32_kernel(const void* src, int src_is_f32, float* dst, int n) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) dst[i] = src_is_f32 ? ((const float*)src)[i] : bf16_to_f32(((const bf16_t*)src)[i]);
}

// dbias from the [token][vocab] panel alone: out[v] = sum_t tv[t][v].  One block owns 64 columns; its four
// row groups are combined in a fixed order, so the result does not depend on scheduling.
__global__ void panel_col_sum_kernel(const bf16_t* tv_hi, const bf16_t* tv_lo, long long ld, long long blk, int rows_t,
                                     int cols, float* out_f32, bf16_t* out_bf16) {
  __shared__ float red[4][64];
  const int tx = threadIdx.x & 63, ty = threadIdx.x >> 6;
  const int c = blockIdx.x * 64 + tx;
  float s = 0.f;
  if (c < cols) {
    // blk != 0: 256-column blocks of row length 256 (block b at + b * blk)
    const long long base = blk ? (long long)(c >> 8) * blk + (c & 255) : (long long)c;
    const long long step = blk ? 256 : ld;
    for (int t = ty; t < rows_t; t += 4) {
      s += bf16_to_f32(tv_hi[base + (long long)t * step]);
      if (tv_lo) s += bf16_to_f32(tv_lo[base + (long long)t * step]);
    }
  }
  red[ty][tx] = s;
  __syncthreads();
  if (ty == 0 && c < cols) {
    const float r = (red[0][tx] + red[1][tx]) + (red[2][tx] + red[3][tx]);
    if (out_f32) out_f32[c] = r;
    if (out_bf16) out_bf16[c] = f32_to_bf16_rn(r);
  }
}

// bias gradient: db[v] = sum_t dS[v][t] over one [vocab][token] panel
__global__ void panel_row_sum_kernel(const bf16_t* vt_hi, const bf16_t* vt_lo, long long ld, int rows, int cols,
                                     float* out_f32, bf16_t* out_bf16) {
  const int row = blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
  const int lane = threadIdx.x & 63;
  if (row >= rows) return;
  float s = 0.f;
  for (int c = lane; c < cols; c += 64) {
    s += bf16_to_f32(vt_hi[(long long)row * ld + c]);
    if (vt_lo) s += bf16_to_f32(vt_lo[(long long)row * ld + c]);
  }
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) s += __shfl_xor(s, o);
  if (lane == 0) {
    if (out_f32) out_f32[row] = s;
    if (out_bf16) out_bf16[row] = f32_to_bf16_rn(s);
  }
}


// ---------------------------------------------------------------------------
// Kept soft-max numerators (forward KEEP kernel): the small kernels around them.
//
// keep_reference_kernel, before the forward: the per-token reference of the stored exponentials,
//   ref_t = max(x_t[y_t], max over a sample of the vocabulary of x_t[v]) / temperature + kKeepOffset
// (x_t[y_t] = W[y_t] . h_t + b[y_t], a dot product per token; the sample's maxima come from a run of the forward
// kernel over the first kKeepSampleRows rows of W, whose per-split partials this kernel merges), written as
// ref_t * log2(e); +huge for tokens with an ignored or invalid label (their rows are stored as zeros).
// Stored values are exp(x_tv/temperature - ref_t): finite in bf16 as long as the row's largest logit exceeds both
// the target's and the sample's by less than 88 + kKeepOffset = 128 nats (temperature applied) - i.e. always for a
// policy scoring tokens it could have sampled, and also for an untrained model with near-Gaussian logits; the
// forward kernel raises a flag otherwise.
//
// keep_backward_prep_kernel, before the gradient GEMMs: with s_t = exp(ref_t - lse_t) the probability is
// p_tv = E[t, v] * s_t, so dLogits[t, v] = c_t (1[v = y_t] - p_tv) = a_t * E'[t, v] with
//   a_t = -c_t * s_t,   E' = E except E'[t, y_t] = (p_y - 1) / s_t  (written in place, from the fp32 lse and target
//   logit, not from the stored bf16 value),   c_t = g_t * gout / temperature.
// dHidden = diag(a) (E' W): the row factor goes into the GEMM's epilogue; dW = E'^T (diag(a) hidden): the kernel
// writes the scaled copy of hidden.  One work-group of 256 threads per 4 tokens (a wavefront per token).
// ---------------------------------------------------------------------------
constexpr float kKeepOffset = 40.f;

struct KeepRefParams {
  const bf16_t* hidden;      // [T][H]
  const bf16_t* weight;      // [V][H]
  const float* bias;         // [V] fp32 or null
  const long long* labels;   // shifted labels [T]
  int T, H, V;
  float inv_temp;
  const float4* sample_part; // [sample_splits][T]: (max, ...) per split of the sample run, logit units
  int sample_splits;
  float* ref2;               // [T] out
  float* xy;                 // [T] out: the target's logit x_t[y_t] / temperature (0 for tokens without one)
  int* flag;                 // cleared here: nflags ints (one per forward launch that will raise it)
  int nflags;
};
constexpr int kKeepSampleRows = 512;

__global__ __launch_bounds__(256) void keep_reference_kernel(const KeepRefParams p) {
  const int t = blockIdx.x * 4 + (threadIdx.x >> 6), lane = threadIdx.x & 63;
  if (blockIdx.x == 0)
    for (int i = threadIdx.x; i < p.nflags; i += 256) p.flag[i] = 0;
  if (t >= p.T) return;
  const long long lab = p.labels[t];
  if (lab < 0 || lab >= p.V) {                 // ignored (-100) or invalid: no gradient, row stored as zeros
    if (lane == 0) {
      p.ref2[t] = -kNegBig;
      p.xy[t] = 0.f;
    }
    return;
  }
  const u32x4_t* h = (const u32x4_t*)(p.hidden + (long long)t * p.H);
  const u32x4_t* w = (const u32x4_t*)(p.weight + lab * p.H);
  float acc = 0.f;
  for (int c = lane; c < p.H / 8; c += 64) {   // H is a multiple of 8 (checked by the caller)
    const u32x4_t a = h[c], b = w[c];
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      acc = __builtin_fmaf(__uint_as_float(a[e] << 16), __uint_as_float(b[e] << 16), acc);
      acc = __builtin_fmaf(__uint_as_float(a[e] & 0xffff0000u), __uint_as_float(b[e] & 0xffff0000u), acc);
    }
  }
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) acc += __shfl_xor(acc, o);
  if (lane == 0) {
    float mx = (acc + (p.bias ? p.bias[lab] : 0.f)) * p.inv_temp;
    p.xy[t] = mx;
    for (int k = 0; k < p.sample_splits; ++k) mx = fmaxf(mx, p.sample_part[(long long)k * p.T + t].x);
    p.ref2[t] = (mx + kKeepOffset) * kLog2e;
  }
}

struct KeepPrepParams {
  bf16_t* e;                 // kept numerators, column-blocked (element (t, y_t) is patched)
  long long blk;             // elements between column blocks
  const float* ref2;         // [T]
  const float* xy;           // [T] target logits (from keep_reference_kernel)
  const long long* labels;   // shifted labels [T]
  const float* lse;          // [T]
  const float* gtok;         // [T]
  const float* gout;         // device scalar or null
  float inv_temp;
  const bf16_t* hidden;      // [T][H]
  int T, H, V;
  float* row_scale;          // [T] out: a_t
  // The forward's overflow flag, read here on the device (null = not consulted).  When it is set the kept values
  // are not to be trusted: the caller's next launch (lmhead_ds_kernel gated on the same flag) overwrites the whole
  // buffer with dLogits recomputed from the operands, and this kernel leaves the buffer alone and writes the row
  // factor as 1 for tokens with a gradient, 0 for the others - the gradient products that follow are the same
  // launches either way.
  const int* gate;
};

__global__ __launch_bounds__(256) void keep_backward_prep_kernel(const KeepPrepParams p) {
  const int t = blockIdx.x * 4 + (threadIdx.x >> 6), lane = threadIdx.x & 63;
  if (t >= p.T) return;
  const long long lab = p.labels[t];
  const bool recompute = p.gate != nullptr && *p.gate != 0;
  float a = 0.f;
  if (lab >= 0 && lab < p.V) {
    const float c = p.gtok[t] * (p.gout ? *p.gout : 1.f) * p.inv_temp;
    const float d2 = p.ref2[t] - p.lse[t] * kLog2e;        // log2 s_t
    a = recompute ? (c != 0.f ? 1.f : 0.f) : -c * fast_exp2(d2);
    if (lane == 0 && !recompute) {
      // p_y - 1 from the fp32 quantities: log p_y = x_y/temperature - lse
      const float pm1 = expm1f(p.xy[t] - p.lse[t]);
      p.e[(lab >> 8) * p.blk + (long long)t * 256 + (lab & 255)] = f32_to_bf16_rn(pm1 * fast_exp2(-d2));
    }
  }
  if (lane == 0) p.row_scale[t] = a;
}

// B operand of the dW product, contraction-contiguous: out[h][t] = a_t * hidden[t][h] for t < T, zero up to Tpad
// (the contraction runs over whole 64-token steps; the kept buffer's rows past T read as zero, and zero times a
// stale value must not be a NaN); rows of `out` are ld elements apart.  64 x 64 tiles through LDS; H % 64 == 0,
// Tpad % 64 == 0, ld >= Tpad, ld % 8 == 0.
__global__ __launch_bounds__(256) void keep_scaled_transpose_kernel(const bf16_t* hidden, const float* row_scale, int T,
                                                                    int H, int Tpad, long long ld, bf16_t* out) {
  __shared__ uint16_t tile[64][66];
  const int t0 = blockIdx.x * 64, h0 = blockIdx.y * 64;
  const int r = threadIdx.x >> 3, cidx = threadIdx.x & 7;
#pragma unroll
  for (int half = 0; half < 2; ++half) {
    const int tl = r + 32 * half, t = t0 + tl;
    u32x4_t v = {0u, 0u, 0u, 0u};
    float a = 0.f;
    if (t < T) {
      v = *(const u32x4_t*)(hidden + (long long)t * H + h0 + 8 * cidx);
      a = row_scale[t];
    }
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      const uint32_t pk = pack_bf16x2(a * __uint_as_float(v[e] << 16), a * __uint_as_float(v[e] & 0xffff0000u));
      tile[tl][8 * cidx + 2 * e] = (uint16_t)(pk & 0xffffu);
      tile[tl][8 * cidx + 2 * e + 1] = (uint16_t)(pk >> 16);
    }
  }
  __syncthreads();
#pragma unroll
  for (int half = 0; half < 2; ++half) {
    const int hl = r + 32 * half;
    u32x4_t o;
#pragma unroll
    for (int e = 0; e < 4; ++e)
      o[e] = (uint32_t)tile[8 * cidx + 2 * e][hl] | ((uint32_t)tile[8 * cidx + 2 * e + 1][hl] << 16);
    *(u32x4_t*)(out + (long long)(h0 + hl) * ld + t0 + 8 * cidx) = o;
  }
}

// Sum of the ksplit fp32 slices a split contraction wrote (fixed order: bit-reproducible), times the row factor,
// as bf16: out[m][n] = row_scale[m] * sum_ks part[ks][m][n].  Four columns per thread; ld % 4 == 0.
__global__ __launch_bounds__(256) void splitk_reduce_kernel(const float* part, int ksplit, long long slice, int M, int N,
                                                            long long ld, const float* row_scale, bf16_t* out) {
  const long long q = (long long)blockIdx.x * 256 + threadIdx.x;      // quad index
  const int nq = N / 4;
  if (q >= (long long)M * nq) return;
  const int m = (int)(q / nq), n = (int)(q - (long long)m * nq) * 4;
  const float* src = part + (long long)m * ld + n;
  float4 s = *(const float4*)src;
  for (int k = 1; k < ksplit; ++k) {
    const float4 v = *(const float4*)(src + (long long)k * slice);
    s.x += v.x;
    s.y += v.y;
    s.z += v.z;
    s.w += v.w;
  }
  const float a = row_scale ? row_scale[m] : 1.f;
  uint2 o;
  o.x = pack_bf16x2(s.x * a, s.y * a);
  o.y = pack_bf16x2(s.z * a, s.w * a);
  *(uint2*)(out + (long long)m * ld + n) = o;
}

// dbias from the kept numerators: out[v] = sum_t a_t * E'[t][v].  One block owns 64 columns; its four row groups
// are combined in a fixed order.
// acc_in (fp32 [V] or null) is added first; the sum goes to acc_out (fp32) and / or out_bf16, whichever is given:
// a caller that walks the tokens in chunks carries the sum in fp32 and takes bf16 from the last chunk.
__global__ void keep_col_sum_kernel(const bf16_t* e, long long blk, const float* row_scale, int T, int V,
                                    const float* acc_in, float* acc_out, bf16_t* out_bf16) {
  __shared__ float red[4][64];
  const int tx = threadIdx.x & 63, ty = threadIdx.x >> 6;
  const int c = blockIdx.x * 64 + tx;
  float s = 0.f;
  if (c < V) {
    const bf16_t* col = e + (long long)(c >> 8) * blk + (c & 255);
    for (int t = ty; t < T; t += 4) s = __builtin_fmaf(row_scale[t], bf16_to_f32(col[(long long)t * 256]), s);
  }
  red[ty][tx] = s;
  __syncthreads();
  if (ty == 0 && c < V) {
    float r = (red[0][tx] + red[1][tx]) + (red[2][tx] + red[3][tx]);
    if (acc_in) r += acc_in[c];
    if (acc_out) acc_out[c] = r;
    if (out_bf16) out_bf16[c] = f32_to_bf16_rn(r);
  }
}

// x[i] *= *scale for a bf16 or fp32 array, 16 bytes per thread and step (n: elements; the base is 16-byte aligned).
// A scale of exactly 1 leaves the array untouched: every work-group returns after reading the scalar.
__global__ __launch_bounds__(256) void scale_inplace_kernel(void* x, long long n, int is_f32, const float* scale) {
  const float s = *scale;
  if (s == 1.f) return;
  const long long per = is_f32 ? 4 : 8;
  const long long nv = n / per;
  for (long long i = (long long)blockIdx.x * 256 + threadIdx.x; i < nv; i += (long long)gridDim.x * 256) {
    if (is_f32) {
      float4 v = ((float4*)x)[i];
      v.x *= s, v.y *= s, v.z *= s, v.w *= s;
      ((float4*)x)[i] = v;
    } else {
      u32x4_t v = ((u32x4_t*)x)[i];
#pragma unroll
      for (int e = 0; e < 4; ++e)
        v[e] = pack_bf16x2(s * __uint_as_float(v[e] << 16), s * __uint_as_float(v[e] & 0xffff0000u));
      ((u32x4_t*)x)[i] = v;
    }
  }
  if (blockIdx.x == 0 && threadIdx.x == 0)
    for (long long i = nv * per; i < n; ++i) {
      if (is_f32)
        ((float*)x)[i] *= s;
      else
        ((bf16_t*)x)[i] = f32_to_bf16_rn(s * bf16_to_f32(((bf16_t*)x)[i]));
    }
}

// Which parts of the token axis carry a gradient at all (row factor a_t != 0): zero-advantage samples and ignored
// labels form long stretches of dead rows, which the gradient GEMMs skip - the dHidden product by 256-row tile
// (m_tile_live), the dW product, whose contraction runs over the tokens, by K step of 64 rows (k_runs: the list of
// live runs gemm_mainloop_km walks).  One work-group; thread i owns a contiguous piece of the 64-row chunks.
// If the rows alternate more often than the list can hold, k_runs[0] is written as one run over everything
// (the products are then merely not shortened).
struct KeepLiveParams {
  const float* row_scale;    // [T]
  int T;
  int n_chunks;              // ceil(T / 64), at most kLiveMaxChunks
  int k_steps;               // K steps of the dW product (round_up(T, 256) / 64)
  int* k_runs;               // [2 + 2 * kRunCap]
  int* m_tile_live;          // [ceil(T / 256)]
};
constexpr int kLiveMaxChunks = 32768;      // 2 M tokens: beyond that nothing is skipped (the lists say "all live")

__global__ __launch_bounds__(1024) void keep_live_runs_kernel(const KeepLiveParams p) {
  __shared__ unsigned char live[kLiveMaxChunks];
  __shared__ int starts_before[1024 + 1], live_before[1024 + 1];
  const int tid = threadIdx.x;
  // chunk flags: one wavefront per chunk, 64 rows each
  // (four chunks per wavefront and round, so that four loads are in flight at a time)
  for (int c4 = (tid >> 6) * 4; c4 < p.n_chunks; c4 += 64) {
    float v[4];
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      const int t = (c4 + k) * 64 + (tid & 63);
      v[k] = (c4 + k < p.n_chunks && t < p.T) ? p.row_scale[t] : 0.f;
    }
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      const bool any = __builtin_amdgcn_ballot_w64(v[k] != 0.f) != 0;
      if ((tid & 63) == 0 && c4 + k < p.n_chunks) live[c4 + k] = any ? 1 : 0;
    }
  }
  __syncthreads();
  for (int m = tid; m * 4 < p.n_chunks; m += 1024) {
    int any = 0;
    for (int c = m * 4; c < m * 4 + 4 && c < p.n_chunks; ++c) any |= live[c];
    p.m_tile_live[m] = any;
  }
  const int per = (p.n_chunks + 1023) / 1024;
  const int c0 = tid * per, c1 = (c0 + per < p.n_chunks ? c0 + per : p.n_chunks);
  int ns = 0, nl = 0;
  for (int c = c0; c < c1; ++c) {
    nl += live[c];
    ns += live[c] && (c == 0 || !live[c - 1]);
  }
  // inclusive prefix of (ns, nl) over the 1024 threads: shuffles inside the wavefront, the 16 wavefront totals in LDS
  {
    int is = ns, il = nl;
    const int lane = tid & 63, wv = tid >> 6;
#pragma unroll
    for (int d = 1; d < 64; d <<= 1) {
      const int us = __shfl_up(is, d, 64), ul = __shfl_up(il, d, 64);
      if (lane >= d) {
        is += us;
        il += ul;
      }
    }
    __shared__ int wave_s[16], wave_l[16];
    if (lane == 63) {
      wave_s[wv] = is;
      wave_l[wv] = il;
    }
    __syncthreads();
    int bs = 0, bl = 0;
    for (int w = 0; w < wv; ++w) {
      bs += wave_s[w];
      bl += wave_l[w];
    }
    starts_before[tid + 1] = bs + is;
    live_before[tid + 1] = bl + il;
    if (tid == 0) starts_before[0] = live_before[0] = 0;
  }
  __syncthreads();
  const int n_runs = starts_before[1024], n_live = live_before[1024];
  if (n_runs > kRunCap) {                  // too fragmented for the list: one run over every K step
    if (tid == 0) {
      p.k_runs[0] = 1;
      p.k_runs[1] = p.k_steps;
      p.k_runs[2] = 0;
      p.k_runs[2 + kRunCap] = p.k_steps;
    }
    return;
  }
  if (tid == 0) {
    p.k_runs[0] = n_runs;
    p.k_runs[1] = n_live;
  }
  int k = starts_before[tid];              // runs that start before this thread's piece
  for (int c = c0; c < c1; ++c) {
    if (!live[c]) continue;
    if (c == 0 || !live[c - 1]) p.k_runs[2 + k++] = c;                       // run k starts here
    if (c + 1 >= p.n_chunks || !live[c + 1]) p.k_runs[2 + kRunCap + k - 1] = c + 1;   // and the current run ends here
  }
}

}  // namespace fgrpo
