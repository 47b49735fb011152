// LM-head kernels built on the GEMM main loops: vocabulary statistics
// (forward), dLogits panels (backward recompute) and plain GEMM with a store
// epilogue (dHidden with K-contiguous operands, dW with contraction-major ones).  In the two LM-head kernels the MFMA "M" index is the
// vocabulary and "N" is the token, so one lane owns a single token per 32x32
// block and 16 vocabulary entries of it: the soft-max statistics reduce inside
// the lane and need one cross-lane step (lanes l and l^32) at the very end.
#pragma once
#include "gemm_core.h"
#include <type_traits>

namespace fgrpo {

constexpr float kNegBig = -1.0e30f;           // stand-in for -inf that keeps 0*x finite
constexpr float kLog2e = 1.4426950408889634f;

__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }

// fp32 -> bf16, round to nearest even, through the hardware conversion (v_cvt_pk_bf16_f32)
typedef __bf16 hwbf16x2_t __attribute__((ext_vector_type(2)));
typedef float f32x2_t __attribute__((ext_vector_type(2)));
__device__ __forceinline__ uint32_t pack_bf16x2(float lo, float hi) {
  const f32x2_t v = {lo, hi};
  return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, hwbf16x2_t));
}
__device__ __forceinline__ uint16_t f32_to_bf16_rn(float f) { return __builtin_bit_cast(uint16_t, (__bf16)f); }
__device__ __forceinline__ float bf16_to_f32(uint16_t h) { return __uint_as_float(((uint32_t)h) << 16); }

// (m1,s1,x1) (+) (m2,s2,x2) for sums of exp(v - m) and exp(v - m) * v.
// No contraction in here: a caller's m is often a product (raw maximum * 1/temperature), and fused into m - mn with
// mn == m that product's rounding residue would replace the exact zero - for the huge stand-in maximum of a slot
// that saw only masked rows a residue of ~1e22, whose exponential is 0 or +inf, and 0 * inf = NaN.
__device__ __forceinline__ void lse_merge(float& m, float& s, float& sx, float m2, float s2, float sx2) {
#pragma clang fp contract(off)
  const float mn = m > m2 ? m : m2;
  const float a1 = fast_exp2((m - mn) * kLog2e), a2 = fast_exp2((m2 - mn) * kLog2e);
  s = s * a1 + s2 * a2;
  sx = sx * a1 + sx2 * a2;
  m = mn;
}

// ---------------------------------------------------------------------------
// Forward: per token running (max, sum exp, sum exp*x) over a range of
// vocabulary tiles + the target logit.
// ---------------------------------------------------------------------------
struct FwdParams {
  GemmOperands g;            // A = W [V x K] (M = V), B = hidden [T x K] (N = T)
  const float* bias;         // [V] fp32 or null
  const long long* labels;   // shifted labels [T]; -100 = ignored
  float inv_temp;
  int tiles_v, tiles_t, nsplit, group_t;
  float4* part;              // [nsplit][T] : (m, s, sx, unused)
  float* xt;                 // [T] target logit (written only where a valid label exists)
  // KEEP kernels only: the soft-max numerators for the backward that does not recompute the logits,
  //   E[t, v] = exp(x_tv / temperature - ref_t)   (bf16; x = W h + b),
  // against a per-token reference chosen BEFORE the sweep (keep_ref2 = ref_t * log2(e); +huge for tokens that take no
  // gradient, whose rows are then stored as exact zeros).  The probability is E[t, v] * exp(ref_t - lse_t): one
  // factor per token, which the gradient GEMMs apply to their output rows / to the other operand, so the buffer
  // feeds them as it is.  Column-blocked [V/256][keep_rows][256]: element (t, v) at
  // (v / 256) * keep_blk + t * 256 + v % 256, keep_blk = keep_rows * 256, keep_rows = token tiles * BN.
  // keep_flag: set to 1 when some row's running maximum exceeds its reference by more than kKeepHeadroom2 (the stored
  // values may then have overflowed and the caller must recompute instead).
  bf16_t* keep;
  long long keep_blk;
  const float* keep_ref2;    // [T]
  int* keep_flag;
};

constexpr float kKeepHeadroom2 = 120.f;   // log2 units: exp2(120) * (values <= 1) stays finite in bf16 / fp32

// One 32-token x WTM-entry slab of bf16 values (the sub-tile column block j of a wavefront in the LM-head
// orientation: lane = token, 16 vocabulary rows per 32x32 block) written to a column-blocked buffer through the
// wavefront's private LDS patch: a lane's 8 bytes (4 vocabulary entries of one token) would be a 64-line scatter per
// store instruction; parked in the patch and read back as 16-byte pieces, PPT lanes per token row, every store
// instruction fills whole 128-byte lines.  Patch rows are unpadded; the 8-byte slots of row n are XOR-swizzled with
// n so that the 32 lanes of a write hit 32 different slots.  LDS traffic is inline assembly (the compiler would
// otherwise wait for the direct-to-LDS loads of the next tile that are in flight); LDS operations of one wavefront
// complete in order, so one wait before the stores is enough.  `out` points at (first token of the slab, first
// vocabulary entry of the wavefront's rows) in the block.
// patch_write_quad: entries i*32 + 8*q + 4*(lane/32) + 0..3 of this lane's token (8 bytes) into the patch;
// patch_flush: the whole slab out, after every quad of the slab has been written.
template <class C>
__device__ __forceinline__ void patch_write_quad(char* patch, int lane_v, int i, int q, uint2 v) {
  constexpr int ROWP = C::WTM * 2;                       // patch row: one token's WTM entries
  constexpr int NSLOT = ROWP / 8;                        // 8-byte slots per row
  const int slot = ((i * 32 + 8 * q) >> 2) + (lane_v >> 5);
  lds_write_b64_asm(lds_addr(patch) + (lane_v & 31) * ROWP + ((slot ^ (lane_v & (NSLOT - 1) & 31)) << 3), v.x, v.y);
}
// the same for the 16x16x32 accumulator layout: the lane's token is row 16*ch + lane%16 of the slab and the quad holds
// its entries i*32 + 16*rh + 4*(lane/16) + 0..3
template <class C>
__device__ __forceinline__ void patch_write_quad16(char* patch, int lane_v, int ch, int i, int rh, uint2 v) {
  constexpr int ROWP = C::WTM * 2;
  constexpr int NSLOT = ROWP / 8;
  const int tok = 16 * ch + (lane_v & 15);
  const int slot = ((i * 32 + 16 * rh) >> 2) + (lane_v >> 4);
  lds_write_b64_asm(lds_addr(patch) + tok * ROWP + ((slot ^ (tok & (NSLOT - 1) & 31)) << 3), v.x, v.y);
}
template <class C>
__device__ __forceinline__ void patch_flush(char* patch, bf16_t* out, int lane_v) {
  constexpr int ROWP = C::WTM * 2;
  constexpr int NSLOT = ROWP / 8;
  constexpr int PPT = ROWP / 16, TPP = 64 / PPT;         // 16-byte pieces per token, tokens per store instruction
  static_assert(64 % PPT == 0 && 32 % TPP == 0 && (NSLOT & (NSLOT - 1)) == 0, "epilogue patch");
  u32x4_t pv[32 / TPP];
#pragma unroll
  for (int r = 0; r < 32 / TPP; ++r) {
    const int tok = r * TPP + lane_v / PPT, piece = lane_v % PPT;
    const int m = tok & (NSLOT - 1);
    pv[r] = __builtin_bit_cast(u32x4_t, lds_read_b128_asm<0>(lds_addr(patch) + tok * ROWP + ((piece ^ (m >> 1)) << 4)));
  }
  wait_lgkm<0>();
  __builtin_amdgcn_sched_barrier(0);     // nothing that consumes pv may move above the wait
#pragma unroll
  for (int r = 0; r < 32 / TPP; ++r) {
    const int tok = r * TPP + lane_v / PPT, piece = lane_v % PPT;
    const int m = tok & (NSLOT - 1);
    u32x4_t v = pv[r];
    if (m & 1) v = u32x4_t{v[2], v[3], v[0], v[1]};       // odd rows hold the two slots of a piece swapped
    // non-temporal: the buffer is written once and read by a later launch; stored normally its 10 GB push the
    // operand tiles out of the L2s (forward kernel at T=32768, H=1536, V=151936: 14.46 ms, non-temporal 12.65)
    __builtin_nontemporal_store(v, (u32x4_t*)(out + (long long)tok * 256 + piece * 8));
  }
}

template <class C, bool KEEP = false>
__global__ __launch_bounds__(C::NT, C::OCC) void lmhead_fwd_kernel(const FwdParams p) {
  extern __shared__ __attribute__((aligned(16))) char smem[];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = wave / C::WN, wn = wave % C::WN;
  const int V = p.g.M, T = p.g.N;

  // block -> (token tile, vocabulary split); neighbours on one XCD share both
  const int lid = xcd_contiguous_id(blockIdx.x, gridDim.x);
  const int per_group = p.group_t * p.nsplit;
  const int grp = lid / per_group;
  const int first_t = grp * p.group_t;
  const int gsz = (p.tiles_t - first_t) < p.group_t ? (p.tiles_t - first_t) : p.group_t;
  const int w = lid - grp * per_group;
  const int tt = first_t + w % gsz;
  const int split = w / gsz;
  const int vt_begin = (int)((long long)split * p.tiles_v / p.nsplit);
  const int vt_end = (int)((long long)(split + 1) * p.tiles_v / p.nsplit);
  const int col0 = tt * C::BN;

  // 16x16x32 MFMAs (kMi16): a lane holds two token columns (ch = 0, 1) of every 32-column block j, 32 vocabulary
  // values of each per tile; otherwise one column and 64 values.  Slot jc = j * NCL + ch.
  constexpr bool MI16 = kMi16<C>;
  constexpr int NCL = MI16 ? 2 : 1, NS = C::TN * NCL;
  auto slot_col = [&](int jc) {      // column of slot jc inside the tile
    return MI16 ? wn * C::WTN + (jc >> 1) * 32 + 16 * (jc & 1) + (lane & 15) : acc_col<C>(wn, jc, lane);
  };
  float m_run[NS], s_run[NS], sx_run[NS];
  float ref2[NS];            // KEEP only
  int y[NS];
#pragma unroll
  for (int jc = 0; jc < NS; ++jc) {
    m_run[jc] = kNegBig;
    s_run[jc] = 0.f;
    sx_run[jc] = 0.f;
    const int n = col0 + slot_col(jc);
    long long lab = (n < T) ? p.labels[n] : -1;
    y[jc] = (lab >= 0 && lab < V) ? (int)lab : -1;
    if constexpr (KEEP) ref2[jc] = (n < T) ? p.keep_ref2[n] : -kNegBig;
  }

  // KEEP: the wavefront's patch lives behind LDS buffer 0, which the prefetch of the next tile may already be filling
  constexpr int KEEP_PATCH = C::NW * 32 * C::WTM * 2;
  static_assert(!KEEP || (kSplitPrologue<C> && C::BM == 256 && C::STAGE + KEEP_PATCH <= C::LDS_BYTES),
                "kept logits: 256-row tiles on the two-buffer direct-to-LDS loop");
  char* patch = smem + C::STAGE + wave * (32 * C::WTM * 2);

  // With the two-buffer direct-to-LDS loop the first K slice of the NEXT vocabulary tile is requested before this
  // tile's statistics are folded in, so its latency hides under that arithmetic.
  if constexpr (kSplitPrologue<C>) {
    if (vt_begin < vt_end) {
      f32x16_t none[C::TM][C::TN];
      gemm_mainloop_dma<C, 2, MI16>(p.g, vt_begin * C::BM, col0, smem, none);
    }
  }
  for (int vt = vt_begin; vt < vt_end; ++vt) {
    const int row0 = vt * C::BM;
    f32x16_t acc[C::TM][C::TN];
    zero_acc<C>(acc);
    if constexpr (kSplitPrologue<C>) {
      gemm_mainloop_dma<C, 1, MI16>(p.g, row0, col0, smem, acc);
      if (vt + 1 < vt_end) gemm_mainloop_dma<C, 2, MI16>(p.g, row0 + C::BM, col0, smem, acc);
    } else {
      run_mainloop<C>(p.g, row0, col0, smem, acc);
    }

    // Statistics are kept in units of the raw product (before the temperature): inv_temp > 0 commutes with
    // the maximum, enters the exponent through one fused multiply-add, and scales m and sum(e*x) once at the end.
    const bool edge = row0 + C::BM > V;
    if (p.bias != nullptr || edge) {
#pragma unroll
      for (int i = 0; i < C::TM; ++i)
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          if constexpr (MI16) {
            if ((r & 4) != 0) continue;                 // the row of element r does not depend on its column half
            const int v = row0 + acc16_row<C>(wm, i, r, lane);
            const float b = (p.bias != nullptr && v < V) ? p.bias[v] : 0.f;
#pragma unroll
            for (int j = 0; j < C::TN; ++j) {
              acc[i][j][r] = (v < V) ? acc[i][j][r] + b : kNegBig;
              acc[i][j][r + 4] = (v < V) ? acc[i][j][r + 4] + b : kNegBig;
            }
          } else {
            const int v = row0 + acc_row<C>(wm, i, r, lane);
            const float b = (p.bias != nullptr && v < V) ? p.bias[v] : 0.f;
#pragma unroll
            for (int j = 0; j < C::TN; ++j) acc[i][j][r] = (v < V) ? acc[i][j][r] + b : kNegBig;
          }
        }
    }

    const float xs = p.inv_temp * kLog2e;
    // Elements of slot jc: NQ quads of four consecutive vocabulary rows each.  Quad qq of slot jc is the registers
    // qreg(jc, qq) .. + 3 of block (qq / QPB, jc / NCL); its first row, relative to the lane's first row, is qrow(qq).
    constexpr int QPB = MI16 ? 2 : 4, NQ = C::TM * QPB;
    auto qreg = [&](int jc, int qq) { return MI16 ? 4 * (2 * (qq % QPB) + (jc & 1)) : 4 * (qq % QPB); };
    auto qrow = [&](int qq) { return MI16 ? (qq / QPB) * 32 + 16 * (qq % QPB) : (qq / QPB) * 32 + 8 * (qq % QPB); };
    const int lane_row0 = wm * C::WTM + 4 * (MI16 ? (lane >> 4) : (lane >> 5));
#pragma unroll
    for (int jc = 0; jc < NS; ++jc) {
      const int j = jc / NCL;
      float mt = kNegBig;
#pragma unroll
      for (int qq = 0; qq < NQ; ++qq)
#pragma unroll
        for (int c = 0; c < 4; ++c) mt = fmaxf(mt, acc[qq / QPB][j][qreg(jc, qq) + c]);
      const float mn = fmaxf(m_run[jc], mt);
      const float alpha = fast_exp2((m_run[jc] - mn) * xs);
      // a slot that has seen only masked rows keeps (m, s, sx) = (kNegBig, 0, 0):
      // x*xs - mb would otherwise be the rounding residue of two huge terms
      const float mb = (mn > 0.5f * kNegBig) ? mn * xs : 0.f;
      // target logit, if one of this lane's rows holds it: the lane's rows are quads 16 (8 with 32x32 blocks) apart,
      // so relative to its first row a row of its own has bits 2..3 (bit 2) clear; y = -1 gives a negative yrel
      const int yrel = y[jc] - row0 - lane_row0;
      constexpr int kRowGap = MI16 ? 12 : 4;
      if ((unsigned)yrel < (unsigned)C::WTM && (yrel & kRowGap) == 0) {
        float xv = 0.f;
#pragma unroll
        for (int qq = 0; qq < NQ; ++qq)
#pragma unroll
          for (int c = 0; c < 4; ++c) xv = (yrel == qrow(qq) + c) ? acc[qq / QPB][j][qreg(jc, qq) + c] : xv;
        p.xt[col0 + slot_col(jc)] = xv * p.inv_temp;
      }
      // KEEP: the exponential computed for the statistics (relative to the running maximum) times one factor per
      // token and tile re-bases it on the token's fixed reference; it replaces the accumulator it came from
      float kf = 0.f;
      if constexpr (KEEP) {
        const float d2 = mb - ref2[jc];
        kf = fast_exp2(d2);
        if (d2 > kKeepHeadroom2 && ref2[jc] < 0.5f * -kNegBig) *p.keep_flag = 1;
      }
      float s = s_run[jc] * alpha, sx = sx_run[jc] * alpha;
      // KEEP: the patch addresses are recomputed per tile on purpose (hoisted they would sit in registers across the
      // main loop); every quad goes to the patch as soon as its statistics are folded in
      int lane_v = lane;
      if constexpr (KEEP) asm volatile("" : "+v"(lane_v));
#pragma unroll
      for (int qq = 0; qq < NQ; ++qq) {
        float ek[4];
#pragma unroll
        for (int c = 0; c < 4; ++c) {
          const float x = acc[qq / QPB][j][qreg(jc, qq) + c];
          const float e = fast_exp2(__builtin_fmaf(x, xs, -mb));
          s += e;
          sx = __builtin_fmaf(e, x, sx);
          ek[c] = e * kf;
        }
        if constexpr (KEEP) {
          uint2 pk;
          pk.x = pack_bf16x2(ek[0], ek[1]);
          pk.y = pack_bf16x2(ek[2], ek[3]);
          if constexpr (MI16)
            patch_write_quad16<C>(patch, lane_v, jc & 1, qq / QPB, qq % QPB, pk);
          else
            patch_write_quad<C>(patch, lane_v, qq / QPB, qq % QPB, pk);
          // pin the running sums here: left alone the compiler first computes all the exponentials of the column
          // (to feed the patch writes) and folds them into the sums afterwards, which keeps all of them in registers
          asm volatile("" : "+v"(s), "+v"(sx));
        }
      }
      m_run[jc] = mn;
      s_run[jc] = s;
      sx_run[jc] = sx;
      if constexpr (KEEP) {
        if (jc % NCL == NCL - 1)          // the 32-token slab of block column j is complete
          patch_flush<C>(patch, p.keep + (long long)vt * p.keep_blk + (long long)(col0 + wn * C::WTN + j * 32) * 256 + wm * C::WTM,
                         lane_v);
      }
    }
  }

  // back to logit units (a masked-only slot keeps a huge negative maximum and zero sums)
#pragma unroll
  for (int jc = 0; jc < NS; ++jc) {
    m_run[jc] *= p.inv_temp;
    sx_run[jc] *= p.inv_temp;
    asm volatile("" : "+v"(m_run[jc]));      // a value from here on, not a product to fuse into the merges below
  }
  // lanes that hold the same tokens (different vocabulary rows): l ^ 32, and with 16x16 blocks also l ^ 16
#pragma unroll
  for (int jc = 0; jc < NS; ++jc) {
    if constexpr (MI16) {
      const float m1 = __shfl_xor(m_run[jc], 16), s1 = __shfl_xor(s_run[jc], 16), x1 = __shfl_xor(sx_run[jc], 16);
      lse_merge(m_run[jc], s_run[jc], sx_run[jc], m1, s1, x1);
    }
    const float m2 = __shfl_xor(m_run[jc], 32), s2 = __shfl_xor(s_run[jc], 32), x2 = __shfl_xor(sx_run[jc], 32);
    lse_merge(m_run[jc], s_run[jc], sx_run[jc], m2, s2, x2);
  }
  // wavefronts stacked along the vocabulary (same wn, different wm) meet in LDS
  float* red = (float*)smem;  // [WM][BN][3]
  if (lane < (MI16 ? 16 : 32)) {
#pragma unroll
    for (int jc = 0; jc < NS; ++jc) {
      float* d = red + ((wm * C::BN) + slot_col(jc)) * 3;
      d[0] = m_run[jc];
      d[1] = s_run[jc];
      d[2] = sx_run[jc];
    }
  }
  __syncthreads();
  for (int c = tid; c < C::BN; c += C::NT) {
    float m = red[c * 3], s = red[c * 3 + 1], sx = red[c * 3 + 2];
    for (int q = 1; q < C::WM; ++q) {
      const float* d = red + (q * C::BN + c) * 3;
      lse_merge(m, s, sx, d[0], d[1], d[2]);
    }
    const int n = col0 + c;
    if (n < T) p.part[(long long)split * T + n] = make_float4(m, s, sx, 0.f);
  }
}

// ---------------------------------------------------------------------------
// Backward recompute: dLogits for one vocabulary panel, written as bf16
//   * in-place mode (tv_blk != 0, vt_hi == null): once, as 256-column blocks [v/256][token][256], which both
//     gradient GEMMs read (dHidden K-contiguous, dW contraction-major);
//   * otherwise: in [token][vocab] and in [vocab][token] order (the contraction index of the GEMM that consumes
//     each copy is its contiguous index).
//   dS[t, v] = c_t * (1[v == y_t] - exp(x_tv - lse_t)),  c_t = g_t * gout / temperature
// Every element of the padded panel buffers is written (zeros outside T x V).
// ---------------------------------------------------------------------------
struct DsParams {
  GemmOperands g;            // A = W [V x K] (M = V), B = hidden [T x K] (N = T)
  const float* bias;
  const long long* labels;
  const float* lse;          // [T]
  const float* gtok;         // [T] d loss / d logprob
  const float* gout;         // device scalar (upstream gradient) or null
  float inv_temp;
  int v0;                    // first vocabulary row of the panel (multiple of BM)
  int tiles_v, tiles_t;      // tiles of the panel / of the tokens
  int nsplit, group_t;       // work-group = (token tile, 1/nsplit of the panel's vocabulary tiles); raster group
  bf16_t* tv_hi;             // [tiles_t*BN][ld_tv]
  bf16_t* tv_lo;             // low half for the fp32 path, or null
  long long ld_tv;
  long long tv_blk;          // != 0: [token][vocab] panel kept as 256-column blocks, block b at + b * tv_blk
                             //       with row length 256 (needs BM == 256); 0: plain rows of ld_tv
  bf16_t* vt_hi;             // [tiles_v*BM][ld_vt]
  bf16_t* vt_lo;
  long long ld_vt;
  const int* gate;           // optional device flag: the launch does nothing unless *gate != 0 (null: always runs)
};

template <class C, bool SPLIT>
__global__ __launch_bounds__(C::NT, C::OCC) void lmhead_ds_kernel(const DsParams p) {
  extern __shared__ __attribute__((aligned(16))) char smem[];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = wave / C::WN, wn = wave % C::WN;
  const int V = p.g.M, T = p.g.N;
  if (p.gate != nullptr && *p.gate == 0) return;     // work-group uniform: every wavefront leaves before any barrier

  // work-group -> (token tile, share of the panel's vocabulary tiles), rastered like the forward kernel: the
  // per-token inputs are read once and the next tile's first K slice is requested under this tile's epilogue
  const int lid = xcd_contiguous_id(blockIdx.x, gridDim.x);
  const int per_group = p.group_t * p.nsplit;
  const int grp = lid / per_group;
  const int first_t = grp * p.group_t;
  const int gsz = (p.tiles_t - first_t) < p.group_t ? (p.tiles_t - first_t) : p.group_t;
  const int w = lid - grp * per_group;
  const int tt = first_t + w % gsz;
  const int split = w / gsz;
  const int vt_begin = (int)((long long)split * p.tiles_v / p.nsplit);
  const int vt_end = (int)((long long)(split + 1) * p.tiles_v / p.nsplit);
  const int col0 = tt * C::BN;

  const float go = (p.gout ? *p.gout : 1.f) * p.inv_temp;
  const float xs = p.inv_temp * kLog2e;
  // 16x16x32 MFMAs (kMi16, not with SPLIT): two token columns per lane and 32-column block, see lmhead_fwd_kernel
  constexpr bool MI16 = kMi16<C> && !SPLIT;
  constexpr int NCL = MI16 ? 2 : 1, NS = C::TN * NCL;
  constexpr int QPB = MI16 ? 2 : 4, NQ = C::TM * QPB;
  auto slot_col = [&](int jc) {
    return MI16 ? wn * C::WTN + (jc >> 1) * 32 + 16 * (jc & 1) + (lane & 15) : acc_col<C>(wn, jc, lane);
  };
  auto qreg = [&](int jc, int qq) { return MI16 ? 4 * (2 * (qq % QPB) + (jc & 1)) : 4 * (qq % QPB); };
  auto qrow = [&](int qq) { return MI16 ? (qq / QPB) * 32 + 16 * (qq % QPB) : (qq / QPB) * 32 + 8 * (qq % QPB); };
  const int lane_row0 = wm * C::WTM + 4 * (MI16 ? (lane >> 4) : (lane >> 5));   // first row of this lane inside the tile
  float lse2[NS], cj[NS];
  int ylab[NS];
#pragma unroll
  for (int jc = 0; jc < NS; ++jc) {
    const int n = col0 + slot_col(jc);
    const bool tok_ok = n < T;
    lse2[jc] = tok_ok ? p.lse[n] * kLog2e : -kNegBig;         // padding columns: probability exactly 0
    const long long lab = tok_ok ? p.labels[n] : -100;
    cj[jc] = (lab != -100) ? p.gtok[n] * go : 0.f;            // ignored tokens carry no gradient
    ylab[jc] = (lab >= 0 && lab < V) ? (int)lab : (int)0xC0000000;  // far below any row: never matches
  }

  // Column-blocked panel: a lane's 8 bytes (4 vocabulary entries of one token) would be a 64-line scatter per
  // store instruction.  The wavefront instead parks 32 tokens x WTM entries in a private LDS patch and writes
  // them out as 16-byte pieces, PPT lanes per token row: every store instruction fills whole 128-byte lines.
  // Patch rows are unpadded; the 8-byte slots of row n are XOR-swizzled with n, so that the 32 lanes of a write
  // (one token each) hit 32 different slots.  The patch lives behind LDS buffer 0, which the prefetch of the next
  // tile may already be filling.
  constexpr int ROWP = C::WTM * 2;                       // patch row: one token's WTM entries
  constexpr int NSLOT = ROWP / 8;                        // 8-byte slots per row
  constexpr int PPT = ROWP / 16, TPP = 64 / PPT;         // 16-byte pieces per token, tokens per store instruction
  constexpr int PATCH = C::NW * 32 * ROWP;
  constexpr bool kPatchBehind = C::STAGE + PATCH <= C::LDS_BYTES;
  constexpr bool kPrefetch = kSplitPrologue<C> && kPatchBehind;
  static_assert(PATCH <= C::LDS_BYTES && 64 % PPT == 0 && 32 % TPP == 0 && (NSLOT & (NSLOT - 1)) == 0, "epilogue patch");
  char* patch = smem + (kPatchBehind ? C::STAGE : 0) + wave * (32 * ROWP);
  const bool through_lds = !SPLIT && p.tv_blk != 0;

  if constexpr (kPrefetch) {
    if (vt_begin < vt_end) {
      f32x16_t none[C::TM][C::TN];
      gemm_mainloop_dma<C, 2, MI16>(p.g, p.v0 + vt_begin * C::BM, col0, smem, none);
    }
  }
  for (int vt = vt_begin; vt < vt_end; ++vt) {
    const int prow0 = vt * C::BM;        // row inside the panel
    const int row0 = p.v0 + prow0;       // vocabulary row
    f32x16_t acc[C::TM][C::TN];
    zero_acc<C>(acc);
    if constexpr (kPrefetch) {
      gemm_mainloop_dma<C, 1, MI16>(p.g, row0, col0, smem, acc);
      if (vt + 1 < vt_end) gemm_mainloop_dma<C, 2, MI16>(p.g, row0 + C::BM, col0, smem, acc);
    } else {
      run_mainloop<C>(p.g, row0, col0, smem, acc);
    }

    // vocabulary rows past V get a logit that exponentiates to exactly 0; the bias joins the raw product
    if (p.bias != nullptr || row0 + C::BM > V) {
#pragma unroll
      for (int i = 0; i < C::TM; ++i)
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          if constexpr (MI16) {
            if ((r & 4) != 0) continue;                 // the row of element r does not depend on its column half
            const int v = row0 + acc16_row<C>(wm, i, r, lane);
            const float b = (p.bias != nullptr && v < V) ? p.bias[v] : 0.f;
#pragma unroll
            for (int j = 0; j < C::TN; ++j) {
              acc[i][j][r] = (v < V) ? acc[i][j][r] + b : kNegBig;
              acc[i][j][r + 4] = (v < V) ? acc[i][j][r + 4] + b : kNegBig;
            }
          } else {
            const int v = row0 + acc_row<C>(wm, i, r, lane);
            const float b = (p.bias != nullptr && v < V) ? p.bias[v] : 0.f;
#pragma unroll
            for (int j = 0; j < C::TN; ++j) acc[i][j][r] = (v < V) ? acc[i][j][r] + b : kNegBig;
          }
        }
    }
#pragma unroll
    for (int jc = 0; jc < NS; ++jc) {
      const int j = jc / NCL;
      const int n = col0 + slot_col(jc);
      const float c = cj[jc], nc = -c, l2 = lse2[jc];
      // target row relative to this lane's first row; out of range when not in this sub-tile
      const int yrel = ylab[jc] - row0 - lane_row0;
      // Few wavefronts hold a target row at all (64 tokens x WTM of V rows): the common case runs without
      // the per-element comparison.
      const bool any_y = __builtin_amdgcn_ballot_w64(yrel >= 0 && yrel < C::WTM) != 0;
      // The swizzled patch addresses are recomputed per tile on purpose: hoisted out of the vocabulary loop they
      // would occupy two dozen registers across the main loop.  The empty asm makes them loop-variant.
      int lane_v = lane;
      asm volatile("" : "+v"(lane_v));
      auto emit = [&](auto with_y, auto via_lds) {
        bf16_t *tv_hi = nullptr, *tv_lo = nullptr, *vt_hi = nullptr, *vt_lo = nullptr;
        if constexpr (!decltype(via_lds)::value) {      // direct stores: plain or blocked rows, optional [vocab][token] copy
          const long long tv_off = p.tv_blk ? (long long)vt * p.tv_blk + (long long)n * 256 + lane_row0
                                            : (long long)n * p.ld_tv + prow0 + lane_row0;
          tv_hi = p.tv_hi + tv_off;
          tv_lo = SPLIT ? p.tv_lo + tv_off : nullptr;
          vt_hi = p.vt_hi ? p.vt_hi + (long long)(prow0 + lane_row0) * p.ld_vt + n : nullptr;
          vt_lo = (SPLIT && p.vt_lo) ? p.vt_lo + (long long)(prow0 + lane_row0) * p.ld_vt + n : nullptr;
        }
#pragma unroll
        for (int qq = 0; qq < NQ; ++qq) {
          {
            const int rr0 = qrow(qq);        // row relative to the lane's first row
            float ds[4];
#pragma unroll
            for (int e = 0; e < 4; ++e) {
              const float pr = fast_exp2(__builtin_fmaf(acc[qq / QPB][j][qreg(jc, qq) + e], xs, -l2));
              if constexpr (decltype(with_y)::value)
                ds[e] = __builtin_fmaf(nc, pr, (rr0 + e == yrel) ? c : 0.f);
              else
                ds[e] = nc * pr;
            }
            // four consecutive vocabulary entries of one token = 8 bytes
            uint2 pk;
            pk.x = pack_bf16x2(ds[0], ds[1]);
            pk.y = pack_bf16x2(ds[2], ds[3]);
            if constexpr (decltype(via_lds)::value) {
              // 8-byte slot of the quad's first row in the token's patch row
              const int tok = MI16 ? 16 * (jc & 1) + (lane_v & 15) : (lane_v & 31);
              const int slot = (rr0 >> 2) + (MI16 ? (lane_v >> 4) : (lane_v >> 5));
              lds_write_b64_asm(lds_addr(patch) + tok * ROWP + ((slot ^ (tok & (NSLOT - 1) & 31)) << 3), pk.x, pk.y);
              continue;
            }
            *(uint2*)(tv_hi + rr0) = pk;
            uint2 pl;
            if (SPLIT) {
              pl.x = pack_bf16x2(ds[0] - __uint_as_float(pk.x << 16), ds[1] - __uint_as_float(pk.x & 0xffff0000u));
              pl.y = pack_bf16x2(ds[2] - __uint_as_float(pk.y << 16), ds[3] - __uint_as_float(pk.y & 0xffff0000u));
              *(uint2*)(tv_lo + rr0) = pl;
            }
            // [vocab][token] (only when the consumer GEMM wants that copy): lanes hold consecutive tokens
            if (vt_hi != nullptr) {
              vt_hi[(long long)(rr0 + 0) * p.ld_vt] = (uint16_t)(pk.x & 0xffffu);
              vt_hi[(long long)(rr0 + 1) * p.ld_vt] = (uint16_t)(pk.x >> 16);
              vt_hi[(long long)(rr0 + 2) * p.ld_vt] = (uint16_t)(pk.y & 0xffffu);
              vt_hi[(long long)(rr0 + 3) * p.ld_vt] = (uint16_t)(pk.y >> 16);
              if (SPLIT && vt_lo != nullptr) {
                vt_lo[(long long)(rr0 + 0) * p.ld_vt] = (uint16_t)(pl.x & 0xffffu);
                vt_lo[(long long)(rr0 + 1) * p.ld_vt] = (uint16_t)(pl.x >> 16);
                vt_lo[(long long)(rr0 + 2) * p.ld_vt] = (uint16_t)(pl.y & 0xffffu);
                vt_lo[(long long)(rr0 + 3) * p.ld_vt] = (uint16_t)(pl.y >> 16);
              }
            }
          }
        }
      };
      if (through_lds) {
        if (any_y)
          emit(std::true_type{}, std::true_type{});
        else
          emit(std::false_type{}, std::true_type{});
      } else {
        if (any_y)
          emit(std::true_type{}, std::false_type{});
        else
          emit(std::false_type{}, std::false_type{});
      }
      if (through_lds && jc % NCL == NCL - 1) {      // the 32-token slab of block column j is complete
        bf16_t* out = p.tv_hi + (long long)vt * p.tv_blk + (long long)(col0 + wn * C::WTN + j * 32) * 256 + wm * C::WTM;
        // inline-assembly LDS traffic (see lds_write_b64_asm): one wait for all reads, LDS operations of a
        // wavefront complete in order, so the reads see this wavefront's writes
        u32x4_t pv[32 / TPP];
#pragma unroll
        for (int r = 0; r < 32 / TPP; ++r) {
          const int tok = r * TPP + lane_v / PPT, piece = lane_v % PPT;
          const int m = tok & (NSLOT - 1);
          pv[r] = __builtin_bit_cast(u32x4_t, lds_read_b128_asm<0>(lds_addr(patch) + tok * ROWP + ((piece ^ (m >> 1)) << 4)));
        }
        wait_lgkm<0>();
        __builtin_amdgcn_sched_barrier(0);     // nothing that consumes pv may move above the wait
#pragma unroll
        for (int r = 0; r < 32 / TPP; ++r) {
          const int tok = r * TPP + lane_v / PPT, piece = lane_v % PPT;
          const int m = tok & (NSLOT - 1);
          u32x4_t v = pv[r];
          if (m & 1) v = u32x4_t{v[2], v[3], v[0], v[1]};       // odd rows hold the two slots of a piece swapped
          __builtin_nontemporal_store(v, (u32x4_t*)(out + (long long)tok * 256 + piece * 8));   // see patch_flush
        }
      }
    }
    if constexpr (!kPrefetch) __syncthreads();   // the patch (or the direct stores) are done before the buffers refill
  }
}

// ---------------------------------------------------------------------------
// Plain GEMM with store epilogue: C[m,n] = alpha * sum_k A[m,k] B[n,k] (+ C_in)
// ---------------------------------------------------------------------------
struct StoreParams {
  GemmOperands g;
  const float* c_in;     // optional fp32 addend, same ldc
  float* c_out_f32;      // exactly one of c_out_f32 / c_out_bf16 is set
  bf16_t* c_out_bf16;
  long long ldc;
  float alpha;
  const float* alpha_dev;  // optional device scalar multiplied into alpha
  int tiles_m, tiles_n, group_m;   // group_m == 0: row tiles dealt round-robin to the XCDs (see gemm_store_kernel)
  int nblocks;                     // work-groups to launch (set by the launcher's caller)
  int rr_rows, rr_cols;            // patch of the round-robin raster (group_m == 0): row tiles of the XCD x column tiles
  int wide_stores;         // ldc and the output / addend bases allow 16-byte pieces (set by the launcher)
  const float* row_scale;  // optional [M]: output row m is multiplied by row_scale[m] (after alpha, before c_in)
  const int* m_tile_live;  // optional [tiles_m] (BM = 256 rows per tile): 0 = every row of the tile has row_scale 0,
                           // the contraction is skipped and the tile is written as zeros (or as c_in)
  // Contraction split (gemm_store_kernel<..., SPLITK = true> only): work-group (tile, ks) contracts the K range
  // [ks * kchunk, (ks + 1) * kchunk) and writes its fp32 tile into slice ks of c_out_f32 (slices part_slice
  // elements apart); splitk_reduce_kernel adds the slices up in a fixed order.
  int ksplit, kchunk;      // kchunk: a multiple of 256
  long long part_slice;
};

// Output is either fp32 or bf16 (never both); rows/cols past M/N are skipped.
template <class C, bool HAS_IN, bool OUT_BF16, bool MI16 = false>
__device__ __forceinline__ void store_tile(const StoreParams& p, f32x16_t (&acc)[C::TM][C::TN], float alpha, int row0,
                                           int col0, int wm, int wn, int lane) {
  if constexpr (MI16) {           // 16x16 blocks: element e of block (i, j) at (acc16_row, acc16_col)
#pragma unroll
    for (int i = 0; i < C::TM; ++i)
#pragma unroll
      for (int j = 0; j < C::TN; ++j)
#pragma unroll
        for (int e = 0; e < 16; ++e) {
          const int m = row0 + acc16_row<C>(wm, i, e, lane), n = col0 + acc16_col<C>(wn, j, e, lane);
          if (m < p.g.M && n < p.g.N) {
            const long long o = (long long)m * p.ldc + n;
            float v = acc[i][j][e] * alpha;
            if (p.row_scale) v *= p.row_scale[m];
            if (HAS_IN) v += p.c_in[o];
            if (OUT_BF16)
              p.c_out_bf16[o] = f32_to_bf16_rn(v);
            else
              p.c_out_f32[o] = v;
          }
        }
    return;
  }
  const int mrem = p.g.M - (row0 + wm * C::WTM + 4 * (lane >> 5));  // rr < mrem <=> row valid
#pragma unroll
  for (int j = 0; j < C::TN; ++j) {
    const int n = col0 + acc_col<C>(wn, j, lane);
    if (n < p.g.N) {
      const long long o0 = (long long)(row0 + wm * C::WTM + 4 * (lane >> 5)) * p.ldc + n;
#pragma unroll
      for (int i = 0; i < C::TM; ++i)
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const int rr = i * 32 + 8 * (r >> 2) + (r & 3);
          if (rr < mrem) {
            const long long o = o0 + (long long)rr * p.ldc;
            float v = acc[i][j][r] * alpha;
            if (p.row_scale) v *= p.row_scale[row0 + wm * C::WTM + 4 * (lane >> 5) + rr];
            if (HAS_IN) v += p.c_in[o];
            if (OUT_BF16)
              p.c_out_bf16[o] = f32_to_bf16_rn(v);
            else
              p.c_out_f32[o] = v;
          }
        }
    }
  }
}

// The same stores made wide.  A lane's accumulator holds single elements of 32 different output columns, so direct
// stores are 2- or 4-byte scalars, 64-byte half lines per instruction.  Here every wavefront parks one 32-row slab of
// its sub-tile (fp32, already scaled) in a private LDS patch, row-major, and reads it back as 16-byte pieces along
// the output row: a store instruction then writes 8 consecutive bf16 (or 4 fp32) per lane and whole 128-byte lines per
// row; the optional addend is loaded the same way.  LDS operations of one wavefront complete in program order, so
// no barrier is needed between the slab's writes and reads, nor before the next slab overwrites the patch.
// Needs ldc and the bases such that every piece is 16-byte aligned (checked by the caller); pieces that cross N
// fall back to scalars.  `smem` must be free (the main loops end with a barrier).  Tiles whose accumulators fill the
// register file (128x128 per wavefront) keep the scalar stores: the patch addressing would push them into scratch.
template <class C>
constexpr bool kStoreViaLds = C::NW * 32 * C::WTN * 4 <= C::LDS_BYTES && C::WTN % 8 == 0 && 64 % (C::WTN / 8) == 0 &&
                              C::TM * C::TN <= 8;

template <class C, bool HAS_IN, bool OUT_BF16, bool MI16 = false>
__device__ __forceinline__ void store_tile_lds(const StoreParams& p, f32x16_t (&acc)[C::TM][C::TN], float alpha, int row0,
                                               int col0, int wm, int wn, int lane, int wave, char* smem) {
  constexpr int WTN = C::WTN;
  constexpr int PIECE = OUT_BF16 ? 8 : 4;                 // output elements per lane and store
  constexpr int LPR = WTN / PIECE;                        // lanes per patch row
  constexpr int RPP = 64 / LPR;                           // rows per store instruction
  static_assert(32 % RPP == 0, "patch rows per pass");
  float* patch = (float*)smem + wave * (32 * WTN);
  const int prow = lane / LPR, pcol = (lane % LPR) * PIECE;
  const int n0 = col0 + wn * WTN + pcol;                  // first output column of this lane's pieces
  const bool n_full = n0 + PIECE <= p.g.N;
  // The addend of slab i + 1 is requested before slab i is shuffled through the patch, so that its latency - the
  // one global round trip of this epilogue - passes under the LDS traffic and the stores of the slab before
  // (a dW sum carried in fp32 across token chunks pays this epilogue per tile and chunk: 18 us against 8 without).
  constexpr int NQ = 32 / RPP, NV = PIECE / 4;
  float4 cin[2][NQ][NV];
  auto load_cin = [&](int i, float4 (&dst)[NQ][NV]) {
#pragma unroll
    for (int q = 0; q < NQ; ++q) {
      const int m = row0 + wm * C::WTM + i * 32 + q * RPP + prow;
      const bool ok = n_full && m < p.g.M;
#pragma unroll
      for (int e = 0; e < NV; ++e)
        dst[q][e] = ok ? *(const float4*)(p.c_in + (long long)m * p.ldc + n0 + 4 * e) : make_float4(0.f, 0.f, 0.f, 0.f);
    }
  };
  if constexpr (HAS_IN) load_cin(0, cin[0]);
#pragma unroll
  for (int i = 0; i < C::TM; ++i) {
    if constexpr (HAS_IN) {
      if (i + 1 < C::TM) load_cin(i + 1, cin[(i + 1) & 1]);
      __builtin_amdgcn_sched_barrier(0);                  // the requests stay ahead of this slab's shuffle
    }
#pragma unroll
    for (int j = 0; j < C::TN; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        if constexpr (MI16)
          patch[(16 * (r >> 3) + 4 * (lane >> 4) + (r & 3)) * WTN + j * 32 + 16 * ((r >> 2) & 1) + (lane & 15)] = acc[i][j][r] * alpha;
        else
          patch[(8 * (r >> 2) + 4 * (lane >> 5) + (r & 3)) * WTN + j * 32 + (lane & 31)] = acc[i][j][r] * alpha;
      }
#pragma unroll
    for (int q = 0; q < NQ; ++q) {
      const int rr = q * RPP + prow;
      const int m = row0 + wm * C::WTM + i * 32 + rr;
      float v[PIECE];
#pragma unroll
      for (int e = 0; e < PIECE; e += 4) {
        const float4 t = *(const float4*)(patch + rr * WTN + pcol + e);
        v[e] = t.x, v[e + 1] = t.y, v[e + 2] = t.z, v[e + 3] = t.w;
      }
      if (m >= p.g.M || n0 >= p.g.N) continue;
      const long long o = (long long)m * p.ldc + n0;
      if (p.row_scale) {
        const float rs = p.row_scale[m];
#pragma unroll
        for (int e = 0; e < PIECE; ++e) v[e] *= rs;
      }
      if (n_full) {
        if constexpr (HAS_IN) {
#pragma unroll
          for (int e = 0; e < PIECE; e += 4) {
            const float4 t = cin[i & 1][q][e / 4];
            v[e] += t.x, v[e + 1] += t.y, v[e + 2] += t.z, v[e + 3] += t.w;
          }
        }
        if (OUT_BF16) {
          u32x4_t w = {pack_bf16x2(v[0], v[1]), pack_bf16x2(v[2], v[3]), pack_bf16x2(v[PIECE - 4], v[PIECE - 3]),
                       pack_bf16x2(v[PIECE - 2], v[PIECE - 1])};
          *(u32x4_t*)(p.c_out_bf16 + o) = w;
        } else {
          *(float4*)(p.c_out_f32 + o) = make_float4(v[0], v[1], v[2], v[3]);
        }
      } else {
        for (int e = 0; e < PIECE && n0 + e < p.g.N; ++e) {
          float x = v[e];
          if (HAS_IN) x += p.c_in[o + e];
          if (OUT_BF16)
            p.c_out_bf16[o + e] = f32_to_bf16_rn(x);
          else
            p.c_out_f32[o + e] = x;
        }
      }
    }
  }
}

// SPLITK (a K-contiguous, column-blocked A and a contraction-major B only): the tiles of a device round that would
// otherwise run nearly empty are contracted in ksplit pieces by ksplit work-groups each.
template <class C, bool AKM = false, bool BKM = false, bool SPLITK = false>
__global__ __launch_bounds__(C::NT, C::OCC) void gemm_store_kernel(const StoreParams p0) {
  extern __shared__ __attribute__((aligned(16))) char smem[];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = wave / C::WN, wn = wave % C::WN;

  if constexpr (SPLITK) {
    static_assert(!AKM && BKM && kMi16<C>, "split contraction: dHidden's layouts on the 16x16x32 tile");
    StoreParams p = p0;
    const int lid = xcd_contiguous_id(blockIdx.x, gridDim.x);
    const int tiles = p.tiles_m * p.tiles_n;
    // pieces of one K range side by side, and of them the column tiles of a row tile: they stream the same slice of
    // A, the big operand (rows fastest instead: 6.7 against 5.6 ms at T = 16384, H = 1536, V = 151936)
    const int ks = lid / tiles, w = lid - ks * tiles;
    const int tm = w / p.tiles_n, tn = w - tm * p.tiles_n;
    const int row0 = tm * C::BM, col0 = tn * C::BN;
    const int k0 = ks * p.kchunk;
    const int klen = (p.g.seg[0].K - k0) < p.kchunk ? (p.g.seg[0].K - k0) : p.kchunk;
    const int b_rows = (p.g.kb_valid > 0 ? p.g.kb_valid : p.g.seg[0].K) - k0;        // rows of B that exist from k0 on
    f32x16_t acc[C::TM][C::TN];
    zero_acc<C>(acc);
    const bool dead = (p.m_tile_live != nullptr && p.m_tile_live[tm] == 0) || klen <= 0 || b_rows <= 0;
    if (!dead) {
      p.g.seg[0].A += (long long)(k0 / 256) * p.g.a_blk;
      p.g.seg[0].B += (long long)k0 * p.g.ldb;
      p.g.seg[0].K = klen;
      p.g.kb_valid = b_rows;
      gemm_mainloop_km<C, false, true, true>(p.g, row0, col0, smem, acc);
    }
    p.c_out_f32 += (long long)ks * p.part_slice;
    if (p.wide_stores)
      store_tile_lds<C, false, false, true>(p, acc, 1.f, row0, col0, wm, wn, lane, wave, smem);
    else
      store_tile<C, false, false, true>(p, acc, 1.f, row0, col0, wm, wn, lane);
    return;
  }
  const StoreParams& p = p0;

  int tm, tn;
  if (p.group_m > 0) {
    // every XCD walks one contiguous range of tiles, group_m row tiles x all column tiles at a time
    const int lid = xcd_contiguous_id(blockIdx.x, gridDim.x);
    const int per_group = p.group_m * p.tiles_n;
    const int grp = lid / per_group;
    const int first_m = grp * p.group_m;
    const int gsz = (p.tiles_m - first_m) < p.group_m ? (p.tiles_m - first_m) : p.group_m;
    const int w = lid - grp * per_group;
    tm = first_m + w % gsz;
    tn = w / gsz;
  } else {
    // row tiles dealt round-robin to the XCDs (work-group b runs on XCD b % 8): neighbouring row tiles - which are
    // dead or alive together when whole samples carry no gradient - land on different XCDs, so skipped tiles thin
    // every XCD's share instead of emptying some.  Inside an XCD the tiles come in patches of rr_rows of its row
    // tiles x rr_cols column tiles (rr_rows * rr_cols = the XCD's 32 CUs; all column tiles when there are at most
    // 8), rows fastest: the 32 work-groups running side by side share rr_rows A slices and rr_cols B slices.
    const int xcd = blockIdx.x & 7, idx = blockIdx.x >> 3;
    const int rows_x = (p.tiles_m + 7) >> 3;                       // row tiles an XCD owns (the last ones may not exist)
    const int per_group = p.rr_rows * p.tiles_n;
    const int grp = idx / per_group;
    const int first = grp * p.rr_rows;
    const int gsz = (rows_x - first) < p.rr_rows ? (rows_x - first) : p.rr_rows;
    const int w = idx - grp * per_group;
    const int chunk = w / (gsz * p.rr_cols);                       // full column chunks before this one
    const int w2 = w - chunk * gsz * p.rr_cols;
    tm = (first + w2 % gsz) * 8 + xcd;
    tn = chunk * p.rr_cols + w2 / gsz;
    if (tm >= p.tiles_m) return;
  }
  const int row0 = tm * C::BM, col0 = tn * C::BN;

  constexpr bool MI16 = kMi16<C>;             // 16x16x32 MFMAs (and their accumulator layout) on the 8-wavefront tile
  f32x16_t acc[C::TM][C::TN];
  zero_acc<C>(acc);
  const bool dead = p.m_tile_live != nullptr && p.m_tile_live[tm] == 0;     // work-group uniform
  if (!dead) {
    if constexpr (AKM || BKM)
      gemm_mainloop_km<C, AKM, BKM, MI16>(p.g, row0, col0, smem, acc);
    else if constexpr (MI16)
      gemm_mainloop_dma<C, 0, true>(p.g, row0, col0, smem, acc);
    else
      run_mainloop<C>(p.g, row0, col0, smem, acc);
  }

  const float alpha = p.alpha * (p.alpha_dev ? *p.alpha_dev : 1.f);
  const int mode = (p.c_in ? 1 : 0) | (p.c_out_bf16 ? 2 : 0);
  if constexpr (kStoreViaLds<C>) {
    if (p.wide_stores) {
      switch (mode) {
        case 0: store_tile_lds<C, false, false, MI16>(p, acc, alpha, row0, col0, wm, wn, lane, wave, smem); break;
        case 1: store_tile_lds<C, true, false, MI16>(p, acc, alpha, row0, col0, wm, wn, lane, wave, smem); break;
        case 2: store_tile_lds<C, false, true, MI16>(p, acc, alpha, row0, col0, wm, wn, lane, wave, smem); break;
        default: store_tile_lds<C, true, true, MI16>(p, acc, alpha, row0, col0, wm, wn, lane, wave, smem); break;
      }
      return;
    }
  }
  switch (mode) {
    case 0: store_tile<C, false, false, MI16>(p, acc, alpha, row0, col0, wm, wn, lane); break;
    case 1: store_tile<C, true, false, MI16>(p, acc, alpha, row0, col0, wm, wn, lane); break;
    case 2: store_tile<C, false, true, MI16>(p, acc, alpha, row0, col0, wm, wn, lane); break;
    default: store_tile<C, true, true, MI16>(p, acc, alpha, row0, col0, wm, wn, lane); break;
  }
}

}  // namespace fgrpo
