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
// Backward without recomputation: the forward kept x = W h + b (bf16, column-blocked [V/256][rows][256]); this
// kernel turns the buffer into dLogits in place,
//   dS[t, v] = c_t * (1[v == y_t] - exp(x_tv / temperature - lse_t)),  c_t = g_t * gout / temperature,
// which the two gradient GEMMs then read where it lies.  Rows with c_t == 0 (ignored labels, zero gradient, padding
// rows t >= T) are written as zeros without being read.  HBM-bound: 2 bytes read and 2 written per logit.
// One work-group = 64 token rows of one 256-column block (32 KiB, contiguous); a row is 32 lanes x 16 bytes.
// ---------------------------------------------------------------------------
struct KeptParams {
  bf16_t* x;                 // in: kept logits, out: dLogits
  long long blk;             // elements between column blocks (= rows * 256)
  int rows;                  // token rows per block (multiple of 64, >= T)
  int T, V;
  const long long* labels;   // shifted labels [T]
  const float* lse;          // [T]
  const float* gtok;         // [T]
  const float* gout;         // device scalar or null
  float inv_temp;
};

constexpr int kKeptRows = 64;

__global__ __launch_bounds__(256) void kept_logits_to_dlogits_kernel(const KeptParams p) {
  __shared__ float s_c[kKeptRows], s_l2[kKeptRows];
  __shared__ int s_y[kKeptRows];
  const int chunks = p.rows / kKeptRows;
  const int vb = blockIdx.x / chunks, t0 = (blockIdx.x - vb * chunks) * kKeptRows;
  const int tid = threadIdx.x;
  if (tid < kKeptRows) {
    const int t = t0 + tid;
    float c = 0.f, l2 = 0.f;
    int y = -1;
    if (t < p.T) {
      const long long lab = p.labels[t];
      if (lab != -100) {
        c = p.gtok[t] * (p.gout ? *p.gout : 1.f) * p.inv_temp;
        l2 = p.lse[t] * kLog2e;
        y = (lab >= 0 && lab < p.V) ? (int)lab - vb * 256 : -1;    // column inside this block, or out of range
      }
    }
    s_c[tid] = c;
    s_l2[tid] = l2;
    s_y[tid] = y;
  }
  __syncthreads();
  const float xs = p.inv_temp * kLog2e;
  const int r0 = tid >> 5, cpos = (tid & 31) * 8;          // row inside a pass of 8 rows, first column of the lane
  u32x4_t* base = (u32x4_t*)(p.x + (long long)vb * p.blk + (long long)t0 * 256) + tid;   // + pass * 256 pieces
  u32x4_t v[kKeptRows / 8];
#pragma unroll
  for (int ps = 0; ps < kKeptRows / 8; ++ps)
    if (s_c[ps * 8 + r0] != 0.f) v[ps] = __builtin_nontemporal_load(base + ps * 256);
#pragma unroll
  for (int ps = 0; ps < kKeptRows / 8; ++ps) {
    const int r = ps * 8 + r0;
    const float c = s_c[r];
    u32x4_t o = {0u, 0u, 0u, 0u};
    if (c != 0.f) {
      const float nc = -c, l2 = s_l2[r];
      const int yrel = s_y[r] - cpos;                       // 0..7 when the target sits in this lane's piece
      float d[8];
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const uint32_t w = v[ps][e];
        const float x0 = __uint_as_float(w << 16), x1 = __uint_as_float(w & 0xffff0000u);
        d[2 * e] = nc * fast_exp2(__builtin_fmaf(x0, xs, -l2));
        d[2 * e + 1] = nc * fast_exp2(__builtin_fmaf(x1, xs, -l2));
      }
      if (yrel >= 0 && yrel < 8) {
#pragma unroll
        for (int e = 0; e < 8; ++e) d[e] += (e == yrel) ? c : 0.f;
      }
#pragma unroll
      for (int e = 0; e < 4; ++e) o[e] = pack_bf16x2(d[2 * e], d[2 * e + 1]);
    }
    __builtin_nontemporal_store(o, base + ps * 256);
  }
}

}  // namespace fgrpo
