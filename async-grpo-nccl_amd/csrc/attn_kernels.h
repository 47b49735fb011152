// Packed variable-length attention for gfx950 (head dimension 128 or 64, bf16 operands, fp32 softmax and accumulators):
// forward with log-sum-exp output, and the backward as two kernels (dQ by query tile, dK/dV by key tile).
// Replaces the flash-attn varlen call of the reference's packed path (gpu_process_worker.py:265-276) with the
// K/V head repeat of its grouped-query wrapper folded into the head index (gpu_process_worker.py:154-161).
//
// Tiling works on the PACKED token axis: a work-group owns 128 consecutive tokens whatever segments they
// belong to, and every score is masked with its query's own key range [seg_start[q], q] (causal) or
// [seg_start[q], seg_end[q]) - so no tile-to-segment map is needed and short segments share tiles.
// The query-side kernels have a second template argument HB (1, 2 or 4): the four wavefronts of a work-group
// take HB query heads of one K/V group over 128/HB consecutive tokens, so that one K/V tile in LDS serves several
// heads and short segments waste fewer masked pairs; HB = 1 is the shape for long segments.
//
// MFMA orientation (v_mfma_f32_32x32x16_bf16; operand lane l = row l%32, k values 8*(l/32)..+7; result lane l =
// column l%32, rows 8*(r/4) + 4*(l/32) + r%4 for r = 0..15):
//  * query-side kernels (forward, dQ) compute S^T = K Q^T, so that a lane owns ONE query (its column) and 32 of
//    the 64 keys of a step: the running max/sum, the rescale of the output accumulator (kept transposed,
//    O^T = V^T P^T) and the bf16 P all stay inside the lane - no cross-lane traffic but one 32-lane swap per
//    step for the row max.  The fp32 P values of a lane are, as they sit in the accumulator, exactly the k
//    values the next MFMA wants from that lane, up to a permutation of the keys that the other operand (V^T,
//    read with ds_read_b64_tr_b16 from the [key][d] tile) simply follows.
//  * the key-side kernel (dK/dV) computes S = Q K^T, so that a lane owns one key and P / dS feed the
//    dV = P^T dO and dK = dS^T Q products from registers in the same way.
// LDS tiles are [row][HD] bf16 with the 16-byte chunk index XOR-swizzled by the row (attn_swz): conflict-free both
// for 16-byte row reads (16 consecutive rows, one chunk) and for the transposing reads (4 consecutive rows x 64 B).
// Masks are applied only on steps that can hold a masked pair, and without branches (select before the exponential).
// Each of the three kernels exists in two forms with bit-identical results.  The first forms (varlen_attn_fwd_kernel,
// varlen_attn_dq_kernel, varlen_attn_dkv_kernel) move tiles global -> registers (bounds-checked buffer loads, issued
// one step ahead) -> LDS and leave the LDS reads to the compiler; the forward and dQ kernels fit 256 registers and
// run two wavefronts per SIMD, which is what overlaps one wavefront's softmax arithmetic with the other's MFMAs,
// while the dK/dV kernel holds two accumulator sets (128 registers) plus its K and V operands, runs one wavefront per
// SIMD and has its step software-pipelined by hand (one MFMA per softmax element); splitting it into a dV and a dK
// launch (two wavefronts per SIMD each, S computed twice) measured slower, as did a second LDS buffer.  The second
// forms, the defaults (varlen_attn_fwd2_kernel, varlen_attn_dq2_kernel, varlen_attn_dkv2_kernel, further down),
// move tiles global -> LDS directly and schedule every LDS access by hand; the dK/dV one deals a wavefront's
// work to a pair so that it, too, runs two wavefronts per SIMD.
// Launch order: work-groups start in the order of a device-built list, tiles with the most steps first (a third of
// a launch was tail before), and in the query-side kernels the query heads of one K/V group share an XCD.
#pragma once
#include "lmhead_kernels.h"

namespace fgrpo {

// Every kernel is a template on the head dimension HD (128 or 64): LDS rows of 2*HD bytes in HD/8 16-byte chunks,
// HD/16 MFMA k-steps per score, HD/32 output blocks of 32 columns.
constexpr int kAttnBQ = 128;         // tokens per work-group (32 per wavefront)
constexpr int kAttnBK = 64;          // tokens of the other side per step

struct AttnParams {
  const bf16_t* q;       // [T][Hq][HD] with element strides q_st (token), q_sh (head)
  const bf16_t* k;       // [T][Hkv][HD]
  const bf16_t* v;
  long long q_st, q_sh, k_st, k_sh, v_st, v_sh;
  const int* seg_start;  // [T] first token of the token's segment
  const int* seg_end;    // [T] one past the last token of the token's segment
  const int* order_q;    // query tiles (of the launch's tile size: 128, 64 or 32 tokens), most keys first
  const int* order_k;    // [ceil(T/128)] key tiles, most queries first
  int T, Hq, Hkv;
  float scale;
  int causal;
  bf16_t* out;           // [T][Hq][HD] contiguous
  float* lse;            // [Hq][T], natural log of the softmax denominator
  // backward
  const bf16_t* dout;    // [T][Hq][HD] contiguous
  float* delta;          // [Hq][T] rowsum(dO * O): written by the dQ kernel, read by the dK/dV kernel
  const bf16_t* out_fwd; // [T][Hq][HD] the forward's output (backward only)
  bf16_t* dq;            // [T][Hq][HD] contiguous
  bf16_t* dk;            // [T][Hkv][HD] contiguous
  bf16_t* dv;
};

typedef short i16x4_t __attribute__((ext_vector_type(4)));

// chunk-index XOR of an LDS row.  HD = 128 (16 chunks, one row = all 64 banks): (row&3)<<2 | (row>>2)&3.
// HD = 64 (8 chunks, two rows share the banks): (row>>1&1)<<2 | (row>>2)&3.  Both are conflict-free for 16-byte
// reads of 16 consecutive rows at one chunk and for the transposing reads (4 consecutive rows x 64 bytes).
template <int HD>
__device__ __forceinline__ int attn_swz(int row) {
  static_assert(HD == 128 || HD == 64, "head dimension");
  return HD == 128 ? (((row & 3) << 2) | ((row >> 2) & 3)) : ((((row >> 1) & 1) << 2) | ((row >> 2) & 3));
}

// Per-lane LDS byte offsets of the fragment reads, computed once: everything that varies inside the loops
// (tile, 32-row block, 16-row k block) is a compile-time offset added to one of these sixteen values.
template <int HD>
struct AttnLane {
  int rowc[HD / 16];    // K-contiguous fragment of row lane%32: chunk 2*st + lane/32, swizzled
  int tr[HD / 32][2];   // K-major fragment, column block nb: the two transposing reads (k rows 4h + j/4 and + 8)
};
template <int HD>
__device__ __forceinline__ AttnLane<HD> attn_lane(int lane) {
  AttnLane<HD> L;
  const int h = lane >> 5, g1 = (lane >> 4) & 1, j = lane & 15, r = lane & 31;
#pragma unroll
  for (int st = 0; st < HD / 16; ++st) L.rowc[st] = r * (HD * 2) + (((2 * st + h) ^ attn_swz<HD>(r)) << 4);
#pragma unroll
  for (int nb = 0; nb < HD / 32; ++nb)
#pragma unroll
    for (int rd = 0; rd < 2; ++rd) {
      const int row = 4 * h + (j >> 2) + 8 * rd;               // + kbase (a multiple of 16: same swizzle)
      const int chunk = 4 * nb + 2 * g1 + ((j & 3) >> 1);
      L.tr[nb][rd] = row * (HD * 2) + ((chunk ^ attn_swz<HD>(row)) << 4) + 8 * (j & 1);
    }
  return L;
}

// K-contiguous fragment: the 8 values [32*blk + lane%32][16*st + 8*(lane/32) .. +7]
template <int HD>
__device__ __forceinline__ bf16x8_t attn_frag(const char* tile, const AttnLane<HD>& L, int blk, int st) {
  return *(const bf16x8_t*)(tile + L.rowc[st] + blk * 32 * (HD * 2));
}

// K-major fragment: lane (n = lane%32, h = lane/32) receives Tile[kbase + 4h + 8*(j/4) + j%4][32*nb + n] for the
// eight slots j = 0..7 (kbase a multiple of 16) - the key order in which a result accumulator hands its values
// to the next MFMA.
template <int HD>
__device__ __forceinline__ bf16x8_t attn_frag_tr(const char* tile, const AttnLane<HD>& L, int kbase, int nb) {
  const char* p0 = tile + L.tr[nb][0] + kbase * (HD * 2);
  const char* p1 = tile + L.tr[nb][1] + kbase * (HD * 2);
  const i16x4_t lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) i16x4_t*)(p0));
  const i16x4_t hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) i16x4_t*)(p1));
  typedef short i16x8_t __attribute__((ext_vector_type(8)));
  const i16x8_t v = {lo.x, lo.y, lo.z, lo.w, hi.x, hi.y, hi.z, hi.w};
  return __builtin_bit_cast(bf16x8_t, v);
}

// eight consecutive accumulator values -> one bf16 operand
__device__ __forceinline__ bf16x8_t attn_pack8(const float* x) {
  const u32x4_t v = {pack_bf16x2(x[0], x[1]), pack_bf16x2(x[2], x[3]), pack_bf16x2(x[4], x[5]), pack_bf16x2(x[6], x[7])};
  return __builtin_bit_cast(bf16x8_t, v);
}

// 64 rows x 256 bytes of one head: global -> registers.  Buffer loads over a descriptor that starts at row `row0`
// (wavefront-uniform) and ends with row `row_end - 1`: rows from row_end on read as zero, and a load costs one
// instruction - the lane's byte offset inside the slab is a constant computed once per kernel.
template <int HD>
struct AttnFetch {
  uint32_t off[HD / 32];      // 64 rows x HD/8 chunks over 256 threads
};
template <int HD>
__device__ __forceinline__ AttnFetch<HD> attn_fetch_init(long long st) {
  AttnFetch<HD> f;
#pragma unroll
  for (int i = 0; i < HD / 32; ++i) {
    const int c = threadIdx.x + 256 * i;
    f.off[i] = (uint32_t)(((long long)(c / (HD / 8)) * st + (c % (HD / 8)) * 8) * 2);
  }
  return f;
}
template <int HD>
__device__ __forceinline__ void attn_fetch_rows(u32x4_t (&r)[HD / 32], const AttnFetch<HD>& f, const bf16_t* base, long long st,
                                                int row0, int row_end) {
  const long long rows = (long long)row_end - row0;
  long long bytes = rows > 0 ? (rows - 1) * st * 2 + HD * 2 : 0;
  if (bytes > 0xffffffffLL) bytes = 0xffffffffLL;
  const __amdgpu_buffer_rsrc_t rs = make_rsrc(base + (long long)row0 * st, (uint32_t)bytes);
#pragma unroll
  for (int i = 0; i < HD / 32; ++i)
    r[i] = __builtin_bit_cast(u32x4_t, __builtin_amdgcn_raw_buffer_load_b128(rs, (int)f.off[i], 0, 0));
}
// ... and registers -> swizzled LDS tile
template <int HD>
__device__ __forceinline__ void attn_put_rows(const u32x4_t (&r)[HD / 32], char* tile) {
#pragma unroll
  for (int i = 0; i < HD / 32; ++i) {
    const int c = threadIdx.x + 256 * i;
    const int row = c / (HD / 8);
    *(u32x4_t*)(tile + row * (HD * 2) + (((c % (HD / 8)) ^ attn_swz<HD>(row)) << 4)) = r[i];
  }
}

// the lane's own row of one head as an MFMA operand: chunks 2s + h, s = 0..7
template <int KS>
__device__ __forceinline__ void attn_row_operand(bf16x8_t (&f)[KS], const bf16_t* row_ptr, bool valid, int h) {
#pragma unroll
  for (int s = 0; s < KS; ++s) {
    const u32x4_t z = {0u, 0u, 0u, 0u};
    const u32x4_t x = valid ? *(const u32x4_t*)(row_ptr + (2 * s + h) * 8) : z;
    f[s] = __builtin_bit_cast(bf16x8_t, x);
  }
}

__device__ __forceinline__ float attn_swap32(float x) { return __shfl_xor(x, 32, 64); }
// The same exchange without the LDS round trip of a bpermute: on return `lo` holds, in every lane, the value lane % 32
// had and `hi` the value lane % 32 + 32 had (v_permlane32_swap: lanes 32..63 of the first operand <-> lanes 0..31 of
// the second).  fmaxf(lo, hi) and lo + hi are then what fmaxf(x, attn_swap32(x)) and x + attn_swap32(x) give.
__device__ __forceinline__ void attn_halves(float x, float& lo, float& hi) {
  lo = x, hi = x;
  asm volatile("s_nop 1\n\tv_permlane32_swap_b32 %0, %1" : "+v"(lo), "+v"(hi));
}

// transposed accumulator (4 blocks of 32 d x 32 tokens, the lane's token = its column) -> [token][head][128] bf16
template <int DB>
__device__ __forceinline__ void attn_store_rowmajor(const f32x16_t (&acc)[DB], float mul, bf16_t* row_ptr, int h) {
#pragma unroll
  for (int db = 0; db < DB; ++db)
#pragma unroll
    for (int g = 0; g < 4; ++g) {
      uint2 pk;
      pk.x = pack_bf16x2(acc[db][4 * g + 0] * mul, acc[db][4 * g + 1] * mul);
      pk.y = pack_bf16x2(acc[db][4 * g + 2] * mul, acc[db][4 * g + 3] * mul);
      *(uint2*)(row_ptr + 32 * db + 8 * g + 4 * h) = pk;
    }
}

// ---------------------------------------------------------------------------------------------------------
// Forward: 1-D grid of round_up(ceil(T/128) * Hkv, 8) * (Hq / Hkv) work-groups, 256 threads.
// ---------------------------------------------------------------------------------------------------------
template <int HD, int HB>
__global__ __launch_bounds__(256, 2) void varlen_attn_fwd_kernel(AttnParams p) {
  constexpr int KS = HD / 16, DB = HD / 32, kAttnTile = kAttnBK * HD * 2, kHD = HD;
  __shared__ __attribute__((aligned(16))) char smem[2 * kAttnTile];
  char* kt = smem;
  char* vt = smem + kAttnTile;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, h = lane >> 5;
  const AttnLane<HD> L = attn_lane<HD>(lane);
  // 1-D grid over (tile rank, K/V head, query head of the group), most work first.  Work-groups go to the 8 XCDs
  // round-robin (work-group b runs on XCD b % 8, each with its own L2): the query heads of one K/V group - which
  // stream the same K and V rows - are given consecutive slots of ONE XCD, and whole groups go round the XCDs.
  // HB query heads of the group share the work-group (4 / HB wavefronts = RB = 128 / HB tokens each): K and V tiles
  // are loaded once for all of them, and short tiles waste less on the diagonal and at segment boundaries.
  constexpr int WPH = 4 / HB, RB = 32 * WPH;
  const int G = p.Hq / p.Hkv, NB = (G + HB - 1) / HB;     // work-groups per (tile, K/V head)
  const int xcd = blockIdx.x & 7, slot = blockIdx.x >> 3;
  const int unit = (slot / NB) * 8 + xcd;                 // (tile rank, K/V head)
  const int ntile = (p.T + RB - 1) / RB;
  if (unit >= ntile * p.Hkv) return;
  const int hkv = unit % p.Hkv;
  const int head_g = (slot % NB) * HB + wave / WPH;       // this wavefront's query head inside the group
  const bool head_ok = head_g < G;
  const int hq = hkv * G + (head_ok ? head_g : G - 1);
  const int q0 = min(max(p.order_q[unit / p.Hkv], 0), ntile - 1) * RB;    // clamped: the list may come from the caller
  const int tq = q0 + 32 * (wave % WPH) + (lane & 31);
  const bool valid = head_ok && tq < p.T;
  const int lo = valid ? p.seg_start[tq] : 1;
  const int hi = valid ? (p.causal ? tq : p.seg_end[tq] - 1) : 0;
  const int last = (q0 + RB - 1 < p.T ? q0 + RB - 1 : p.T - 1);
  const int k_begin = max(__builtin_amdgcn_readfirstlane(p.seg_start[q0]), 0);   // wavefront-uniform loop bounds, inside [0, T]
  const int k_end = min(__builtin_amdgcn_readfirstlane(p.causal ? last + 1 : p.seg_end[last]), p.T);
  // this wavefront's own key range (whole steps outside it are skipped)
  const int wfirst = q0 + 32 * (wave % WPH), wlast = (wfirst + 31 < p.T ? wfirst + 31 : p.T - 1);
  const bool wave_on = head_ok && wfirst < p.T;
  const int w_lo = wave_on ? p.seg_start[wfirst] : 1;
  const int w_hi = wave_on ? (p.causal ? wlast : p.seg_end[wlast] - 1) : 0;
  // keys in [w_lo_max, w_hi_min] are visible to every query of the wavefront (only when all 32 rows exist)
  const bool wave_full = wave_on && wfirst + 31 < p.T;
  const int w_lo_max = wave_full ? p.seg_start[wlast] : 0x7fffffff;
  const int w_hi_min = wave_full ? (p.causal ? wfirst : p.seg_end[wfirst] - 1) : -1;

  bf16x8_t qf[KS];
  attn_row_operand(qf, p.q + (long long)(valid ? tq : 0) * p.q_st + (long long)hq * p.q_sh, valid, h);

  f32x16_t acc_o[DB];
#pragma unroll
  for (int db = 0; db < DB; ++db)
#pragma unroll
    for (int r = 0; r < 16; ++r) acc_o[db][r] = 0.f;
  float m_run = -INFINITY, l_run = 0.f;
  const float c = p.scale * kLog2e;

  const bf16_t* kbase = p.k + (long long)hkv * p.k_sh;
  const bf16_t* vbase = p.v + (long long)hkv * p.v_sh;
  u32x4_t rk[DB], rv[DB];
  const AttnFetch<HD> fk = attn_fetch_init<HD>(p.k_st), fv = attn_fetch_init<HD>(p.v_st);
  attn_fetch_rows(rk, fk, kbase, p.k_st, k_begin, k_end);
  attn_fetch_rows(rv, fv, vbase, p.v_st, k_begin, k_end);
  for (int kb = k_begin; kb < k_end; kb += kAttnBK) {
    attn_put_rows<HD>(rk, kt);
    attn_put_rows<HD>(rv, vt);
    __syncthreads();
    if (kb + kAttnBK < k_end) {   // next step's rows travel while this one is computed
      attn_fetch_rows(rk, fk, kbase, p.k_st, kb + kAttnBK, k_end);
      attn_fetch_rows(rv, fv, vbase, p.v_st, kb + kAttnBK, k_end);
    }
    if (wave_on && kb <= w_hi && kb + kAttnBK > w_lo) {
      f32x16_t s[2];
#pragma unroll
      for (int mb = 0; mb < 2; ++mb) {
#pragma unroll
        for (int r = 0; r < 16; ++r) s[mb][r] = 0.f;
#pragma unroll
        for (int st = 0; st < KS; ++st) s[mb] = FGRPO_MFMA(attn_frag(kt, L, mb, st), qf[st], s[mb]);
      }
      float mx = -INFINITY;
      if (kb >= w_lo_max && kb + kAttnBK - 1 <= w_hi_min) {   // every pair of this step is visible
#pragma unroll
        for (int mb = 0; mb < 2; ++mb)
#pragma unroll
          for (int r = 0; r < 16; ++r) mx = fmaxf(mx, s[mb][r]);
      } else {
#pragma unroll
        for (int mb = 0; mb < 2; ++mb)
#pragma unroll
          for (int r = 0; r < 16; ++r) {
            const int key = kb + 32 * mb + 8 * (r >> 2) + 4 * h + (r & 3);
            const float x = (key >= lo && key <= hi) ? s[mb][r] : -INFINITY;
            s[mb][r] = x;
            mx = fmaxf(mx, x);
          }
      }
      mx = fmaxf(mx, attn_swap32(mx));
      const float m_new = fmaxf(m_run, mx);
      const float m_use = (m_new == -INFINITY) ? 0.f : m_new;
      const float alpha = fast_exp2((m_run - m_use) * c);
      const float mc = m_use * c;
      float sum = 0.f;
#pragma unroll
      for (int mb = 0; mb < 2; ++mb)
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const float e = fast_exp2(__builtin_fmaf(s[mb][r], c, -mc));
          s[mb][r] = e;
          sum += e;
        }
      l_run = l_run * alpha + sum;
      m_run = m_new;
      if (__any(alpha != 1.f)) {      // once the running maxima have settled no lane rescales any more
#pragma unroll
        for (int db = 0; db < DB; ++db)
#pragma unroll
          for (int r = 0; r < 16; ++r) acc_o[db][r] *= alpha;
      }
#pragma unroll
      for (int mb = 0; mb < 2; ++mb)
#pragma unroll
        for (int s2 = 0; s2 < 2; ++s2) {
          float tmp[8];
#pragma unroll
          for (int j = 0; j < 8; ++j) tmp[j] = s[mb][8 * s2 + j];
          const bf16x8_t pf = attn_pack8(tmp);
#pragma unroll
          for (int db = 0; db < DB; ++db)
            acc_o[db] = FGRPO_MFMA(attn_frag_tr(vt, L, 32 * mb + 16 * s2, db), pf, acc_o[db]);
        }
    }
    __syncthreads();
  }
  const float l = l_run + attn_swap32(l_run);
  if (valid) {
    const float inv = l > 0.f ? 1.f / l : 0.f;
    attn_store_rowmajor(acc_o, inv, p.out + ((long long)tq * p.Hq + hq) * kHD, h);
    if (h == 0) p.lse[(long long)hq * p.T + tq] = l > 0.f ? m_run * p.scale + __logf(l) : -INFINITY;
  }
}

// ---------------------------------------------------------------------------------------------------------
// dQ: same grid as the forward, 256 threads.  Same walk as the forward; P is rebuilt from the saved log-sum-exp.
// Also produces delta[hq][t] = sum_d dO[t][hq][d] * O[t][hq][d] (each lane already holds its query's dO row).
// ---------------------------------------------------------------------------------------------------------
template <int HD, int HB>
__global__ __launch_bounds__(256, 2) void varlen_attn_dq_kernel(AttnParams p) {
  constexpr int KS = HD / 16, DB = HD / 32, kAttnTile = kAttnBK * HD * 2, kHD = HD;
  __shared__ __attribute__((aligned(16))) char smem[2 * kAttnTile];
  char* kt = smem;
  char* vt = smem + kAttnTile;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, h = lane >> 5;
  const AttnLane<HD> L = attn_lane<HD>(lane);
  // 1-D grid over (tile rank, K/V head, query head of the group), most work first.  Work-groups go to the 8 XCDs
  // round-robin (work-group b runs on XCD b % 8, each with its own L2): the query heads of one K/V group - which
  // stream the same K and V rows - are given consecutive slots of ONE XCD, and whole groups go round the XCDs.
  // HB query heads of the group share the work-group (4 / HB wavefronts = RB = 128 / HB tokens each): K and V tiles
  // are loaded once for all of them, and short tiles waste less on the diagonal and at segment boundaries.
  constexpr int WPH = 4 / HB, RB = 32 * WPH;
  const int G = p.Hq / p.Hkv, NB = (G + HB - 1) / HB;     // work-groups per (tile, K/V head)
  const int xcd = blockIdx.x & 7, slot = blockIdx.x >> 3;
  const int unit = (slot / NB) * 8 + xcd;                 // (tile rank, K/V head)
  const int ntile = (p.T + RB - 1) / RB;
  if (unit >= ntile * p.Hkv) return;
  const int hkv = unit % p.Hkv;
  const int head_g = (slot % NB) * HB + wave / WPH;       // this wavefront's query head inside the group
  const bool head_ok = head_g < G;
  const int hq = hkv * G + (head_ok ? head_g : G - 1);
  const int q0 = min(max(p.order_q[unit / p.Hkv], 0), ntile - 1) * RB;    // clamped: the list may come from the caller
  const int tq = q0 + 32 * (wave % WPH) + (lane & 31);
  const bool valid = head_ok && tq < p.T;
  const int lo = valid ? p.seg_start[tq] : 1;
  const int hi = valid ? (p.causal ? tq : p.seg_end[tq] - 1) : 0;
  const int last = (q0 + RB - 1 < p.T ? q0 + RB - 1 : p.T - 1);
  const int k_begin = max(__builtin_amdgcn_readfirstlane(p.seg_start[q0]), 0);   // wavefront-uniform loop bounds, inside [0, T]
  const int k_end = min(__builtin_amdgcn_readfirstlane(p.causal ? last + 1 : p.seg_end[last]), p.T);
  const int wfirst = q0 + 32 * (wave % WPH), wlast = (wfirst + 31 < p.T ? wfirst + 31 : p.T - 1);
  const bool wave_on = head_ok && wfirst < p.T;
  const int w_lo = wave_on ? p.seg_start[wfirst] : 1;
  const int w_hi = wave_on ? (p.causal ? wlast : p.seg_end[wlast] - 1) : 0;
  const bool wave_full = wave_on && wfirst + 31 < p.T;
  const int w_lo_max = wave_full ? p.seg_start[wlast] : 0x7fffffff;
  const int w_hi_min = wave_full ? (p.causal ? wfirst : p.seg_end[wfirst] - 1) : -1;

  bf16x8_t qf[KS], dof[KS];
  attn_row_operand(qf, p.q + (long long)(valid ? tq : 0) * p.q_st + (long long)hq * p.q_sh, valid, h);
  attn_row_operand(dof, p.dout + ((long long)(valid ? tq : 0) * p.Hq + hq) * kHD, valid, h);
  const float lse2 = valid ? p.lse[(long long)hq * p.T + tq] * kLog2e : 0.f;
  // delta = rowsum(dO * O) of the lane's query: each lane half holds alternate 8-element pieces of the row
  float dl = 0.f;
  {
    bf16x8_t of[KS];
    attn_row_operand(of, p.out_fwd + ((long long)(valid ? tq : 0) * p.Hq + hq) * kHD, valid, h);
#pragma unroll
    for (int st = 0; st < KS; ++st) {
      const u32x4_t x = __builtin_bit_cast(u32x4_t, dof[st]), y = __builtin_bit_cast(u32x4_t, of[st]);
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        dl += __uint_as_float(x[i] << 16) * __uint_as_float(y[i] << 16);
        dl += __uint_as_float(x[i] & 0xffff0000u) * __uint_as_float(y[i] & 0xffff0000u);
      }
    }
    dl += attn_swap32(dl);
    if (valid && h == 0) p.delta[(long long)hq * p.T + tq] = dl;    // for the dK/dV kernel, launched after this one
  }
  const float c = p.scale * kLog2e;

  f32x16_t acc[DB];
#pragma unroll
  for (int db = 0; db < DB; ++db)
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[db][r] = 0.f;

  const bf16_t* kbase = p.k + (long long)hkv * p.k_sh;
  const bf16_t* vbase = p.v + (long long)hkv * p.v_sh;
  u32x4_t rk[DB], rv[DB];
  const AttnFetch<HD> fk = attn_fetch_init<HD>(p.k_st), fv = attn_fetch_init<HD>(p.v_st);
  attn_fetch_rows(rk, fk, kbase, p.k_st, k_begin, k_end);
  attn_fetch_rows(rv, fv, vbase, p.v_st, k_begin, k_end);
  for (int kb = k_begin; kb < k_end; kb += kAttnBK) {
    attn_put_rows<HD>(rk, kt);
    attn_put_rows<HD>(rv, vt);
    __syncthreads();
    if (kb + kAttnBK < k_end) {
      attn_fetch_rows(rk, fk, kbase, p.k_st, kb + kAttnBK, k_end);
      attn_fetch_rows(rv, fv, vbase, p.v_st, kb + kAttnBK, k_end);
    }
    if (wave_on && kb <= w_hi && kb + kAttnBK > w_lo) {
#pragma unroll
      for (int mb = 0; mb < 2; ++mb) {
        f32x16_t s, dp;
#pragma unroll
        for (int r = 0; r < 16; ++r) s[r] = dp[r] = 0.f;
#pragma unroll
        for (int st = 0; st < KS; ++st) {
          s = FGRPO_MFMA(attn_frag(kt, L, mb, st), qf[st], s);
          dp = FGRPO_MFMA(attn_frag(vt, L, mb, st), dof[st], dp);
        }
        float ds[16];
        if (kb >= w_lo_max && kb + kAttnBK - 1 <= w_hi_min) {   // every pair of this step is visible
#pragma unroll
          for (int r = 0; r < 16; ++r) ds[r] = fast_exp2(__builtin_fmaf(s[r], c, -lse2)) * (dp[r] - dl);
        } else {
#pragma unroll
          for (int r = 0; r < 16; ++r) {
            const int key = kb + 32 * mb + 8 * (r >> 2) + 4 * h + (r & 3);
            const int vis = (int)(key >= lo) & (int)(key <= hi);
            const float pr = fast_exp2(vis ? __builtin_fmaf(s[r], c, -lse2) : -INFINITY);
            ds[r] = pr * (dp[r] - dl);
          }
        }
#pragma unroll
        for (int s2 = 0; s2 < 2; ++s2) {
          const bf16x8_t dsf = attn_pack8(ds + 8 * s2);
#pragma unroll
          for (int db = 0; db < DB; ++db)
            acc[db] = FGRPO_MFMA(attn_frag_tr(kt, L, 32 * mb + 16 * s2, db), dsf, acc[db]);
        }
      }
    }
    __syncthreads();
  }
  if (valid) attn_store_rowmajor(acc, p.scale, p.dq + ((long long)tq * p.Hq + hq) * kHD, h);   // dS was kept / scale
}

// ---------------------------------------------------------------------------------------------------------
// dK, dV: grid (Hkv, ceil(T/128)), 256 threads; a wavefront owns 32 keys (one per lane pair) and walks the
// queries that can see them, for every query head of the group.
// ---------------------------------------------------------------------------------------------------------
template <int HD>
__global__ __launch_bounds__(256) void varlen_attn_dkv_kernel(AttnParams p) {
  constexpr int KS = HD / 16, DB = HD / 32, kAttnTile = kAttnBK * HD * 2, kHD = HD;
  __shared__ __attribute__((aligned(16))) char smem[2 * kAttnTile];
  __shared__ __attribute__((aligned(16))) float row_lse2[kAttnBK];
  __shared__ __attribute__((aligned(16))) float row_dl[kAttnBK];
  __shared__ __attribute__((aligned(16))) int row_lo[kAttnBK];
  __shared__ __attribute__((aligned(16))) int row_hi[kAttnBK];
  char* qt = smem;
  char* dot = smem + kAttnTile;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, h = lane >> 5;
  const AttnLane<HD> L = attn_lane<HD>(lane);
  const int hkv = blockIdx.x, G = p.Hq / p.Hkv;
  const int k0 = min(max(p.order_k[blockIdx.y], 0), (int)gridDim.y - 1) * kAttnBQ;   // clamped: the list may come from the caller
  const int key = k0 + 32 * wave + (lane & 31);
  const bool valid = key < p.T;
  const int last = (k0 + kAttnBQ - 1 < p.T ? k0 + kAttnBQ - 1 : p.T - 1);
  // queries that can see a key of this tile
  const int q_begin = max(__builtin_amdgcn_readfirstlane(p.causal ? k0 : p.seg_start[k0]), 0);   // wavefront-uniform loop bounds, inside [0, T]
  const int q_end = min(__builtin_amdgcn_readfirstlane(p.seg_end[last]), p.T);
  const int wfirst = k0 + 32 * wave, wlast = (wfirst + 31 < p.T ? wfirst + 31 : p.T - 1);
  const bool wave_on = wfirst < p.T;
  const int wq_lo = wave_on ? (p.causal ? wfirst : p.seg_start[wfirst]) : 1;   // first / last query of interest
  const int wq_hi = wave_on ? p.seg_end[wlast] - 1 : 0;

  bf16x8_t kf[KS], vf[KS];
  attn_row_operand(kf, p.k + (long long)(valid ? key : 0) * p.k_st + (long long)hkv * p.k_sh, valid, h);
  attn_row_operand(vf, p.v + (long long)(valid ? key : 0) * p.v_st + (long long)hkv * p.v_sh, valid, h);
  const float c = p.scale * kLog2e;

  f32x16_t acc_k[DB], acc_v[DB];
#pragma unroll
  for (int nb = 0; nb < DB; ++nb)
#pragma unroll
    for (int r = 0; r < 16; ++r) acc_k[nb][r] = acc_v[nb][r] = 0.f;

  const AttnFetch<HD> fq_ = attn_fetch_init<HD>(p.q_st), fd_ = attn_fetch_init<HD>((long long)p.Hq * kHD);
  for (int g = 0; g < G; ++g) {
    const int hq = hkv * G + g;
    const bf16_t* qbase = p.q + (long long)hq * p.q_sh;
    const bf16_t* dobase = p.dout + (long long)hq * kHD;
    const long long do_st = (long long)p.Hq * kHD;
    u32x4_t rq[DB], rd[DB];
    // per-query scalars of a step travel with its rows: fetched one step ahead, never waited for inside a step
    float n_lse = 0.f, n_dl = 0.f;
    int n_lo = 1, n_hi = 0;
    auto fetch_row_scalars = [&](int qb) {
      if (threadIdx.x < kAttnBK) {
        const int t = qb + threadIdx.x;
        const bool ok = t < q_end;
        n_lse = ok ? p.lse[(long long)hq * p.T + t] * kLog2e : 0.f;
        n_dl = ok ? p.delta[(long long)hq * p.T + t] : 0.f;
        n_lo = ok ? p.seg_start[t] : 1;
        n_hi = ok ? (p.causal ? t : p.seg_end[t] - 1) : 0;
      }
    };
    attn_fetch_rows(rq, fq_, qbase, p.q_st, q_begin, q_end);
    attn_fetch_rows(rd, fd_, dobase, do_st, q_begin, q_end);
    fetch_row_scalars(q_begin);
    for (int qb = q_begin; qb < q_end; qb += kAttnBK) {
      attn_put_rows<HD>(rq, qt);
      attn_put_rows<HD>(rd, dot);
      if (threadIdx.x < kAttnBK) {
        row_lse2[threadIdx.x] = n_lse;
        row_dl[threadIdx.x] = n_dl;
        row_lo[threadIdx.x] = n_lo;
        row_hi[threadIdx.x] = n_hi;
      }
      __syncthreads();
      if (qb + kAttnBK < q_end) {
        attn_fetch_rows(rq, fq_, qbase, p.q_st, qb + kAttnBK, q_end);
        attn_fetch_rows(rd, fd_, dobase, do_st, qb + kAttnBK, q_end);
        fetch_row_scalars(qb + kAttnBK);
      }
      if (wave_on && qb <= wq_hi && qb + kAttnBK > wq_lo) {
        // every (query, key) pair of this step visible: all 64 queries exist, the last one's segment starts at or
        // before the wavefront's first key, the first one sees the wavefront's last key
        const bool all_visible = wfirst + 31 < p.T && qb + kAttnBK <= q_end && row_lo[kAttnBK - 1] <= wfirst && row_hi[0] >= wlast;
        // One wavefront per SIMD: only this wavefront's own instruction order can overlap the softmax arithmetic
        // with the matrix pipe (an MFMA occupies the pipe for 32 cycles but issues in 4).  The step's two 32-query
        // sub-blocks are therefore software-pipelined by hand, one MFMA per softmax element:
        //   S,dP(0) | S,dP(1) + softmax(0) | dV,dK(0) + softmax(1) | dV,dK(1)
        // and LDS fragments are requested a phase before the MFMAs that use them.
        bf16x8_t qa[KS], da[KS], fdo[2][DB], fq[2][DB], pf[2][2], dsf[2][2];
        f32x16_t s[2], dp[2];
        auto load_rows = [&](int mq) {
#pragma unroll
          for (int st = 0; st < KS; ++st) {
            qa[st] = attn_frag(qt, L, mq, st);
            da[st] = attn_frag(dot, L, mq, st);
          }
        };
        auto load_tr = [&](int mq) {
#pragma unroll
          for (int s2 = 0; s2 < 2; ++s2)
#pragma unroll
            for (int nb = 0; nb < DB; ++nb) {
              fdo[s2][nb] = attn_frag_tr(dot, L, 32 * mq + 16 * s2, nb);
              fq[s2][nb] = attn_frag_tr(qt, L, 32 * mq + 16 * s2, nb);
            }
        };
        constexpr int NM = 2 * KS;                  // MFMAs of a phase (16 for HD = 128): one per 16 / NM softmax elements
        auto score_mfma = [&](int mq, int m) {      // MFMA m of NM: two chains (S, dP) of KS
          if (m & 1) dp[mq] = FGRPO_MFMA(da[m >> 1], vf[m >> 1], dp[mq]);
          else s[mq] = FGRPO_MFMA(qa[m >> 1], kf[m >> 1], s[mq]);
        };
        auto grad_mfma = [&](int mq, int m) {       // MFMA m of NM: 2 * DB accumulators, two 16-query halves
          const int s2 = (m >> 1) / DB, nb = (m >> 1) % DB;
          if (m & 1) acc_k[nb] = FGRPO_MFMA(dsf[mq][s2], fq[s2][nb], acc_k[nb]);
          else acc_v[nb] = FGRPO_MFMA(pf[mq][s2], fdo[s2][nb], acc_v[nb]);
        };
        // softmax element r of sub-block mq: P and dS / scale (the scale is applied once, to the dK accumulators)
        float pr[16], ds[16];
        // per-query scalars of a register group (four queries), read one group ahead of their use
        float4 l4s[2], d4s[2];
        int4 lo4s[2] = {{0, 0, 0, 0}, {0, 0, 0, 0}}, hi4s[2] = {{0, 0, 0, 0}, {0, 0, 0, 0}};
        auto read_group = [&](int mq, int grp, bool masked) {     // -> set grp % 2
          const int row = 32 * mq + 8 * grp + 4 * h;
          l4s[grp & 1] = *(const float4*)(row_lse2 + row);
          d4s[grp & 1] = *(const float4*)(row_dl + row);
          if (masked) {
            lo4s[grp & 1] = *(const int4*)(row_lo + row);
            hi4s[grp & 1] = *(const int4*)(row_hi + row);
          }
        };
        auto element = [&](int mq, int r, bool masked) {
          if ((r & 3) == 0) {
            if (r + 4 < 16) read_group(mq, (r >> 2) + 1, masked);
            else if (mq == 0) read_group(1, 0, masked);          // first group of the other sub-block
          }
          const int e = r & 3, st = (r >> 2) & 1;
          const float4 l4 = l4s[st], d4 = d4s[st];
          const int4 lo4 = lo4s[st], hi4 = hi4s[st];
          const float ls = e == 0 ? l4.x : e == 1 ? l4.y : e == 2 ? l4.z : l4.w;
          const float dd = e == 0 ? d4.x : e == 1 ? d4.y : e == 2 ? d4.z : d4.w;
          float x = __builtin_fmaf(s[mq][r], c, -ls);
          if (masked) {
            const int lo = e == 0 ? lo4.x : e == 1 ? lo4.y : e == 2 ? lo4.z : lo4.w;
            const int hi = e == 0 ? hi4.x : e == 1 ? hi4.y : e == 2 ? hi4.z : hi4.w;
            // select before the exponential: a masked pair becomes exp2(-inf) = 0 without a branch
            x = ((int)(key >= lo) & (int)(key <= hi)) ? x : -INFINITY;
          }
          const float pv = fast_exp2(x);
          pr[r] = pv;
          ds[r] = pv * (dp[mq][r] - dd);
        };
        auto pack = [&](int mq) {
#pragma unroll
          for (int s2 = 0; s2 < 2; ++s2) {
            pf[mq][s2] = attn_pack8(pr + 8 * s2);
            dsf[mq][s2] = attn_pack8(ds + 8 * s2);
          }
        };
#pragma unroll
        for (int mq = 0; mq < 2; ++mq)
#pragma unroll
          for (int r = 0; r < 16; ++r) s[mq][r] = dp[mq][r] = 0.f;

        load_rows(0);
        load_tr(0);
        read_group(0, 0, !all_visible);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int m = 0; m < NM; ++m) score_mfma(0, m);
        load_rows(1);
        __builtin_amdgcn_sched_barrier(0);
        if (all_visible) {
#pragma unroll
          for (int j = 0; j < 16; ++j) {
            if (j % (16 / NM) == 0) score_mfma(1, j / (16 / NM));
            element(0, j, false);
            __builtin_amdgcn_sched_barrier(0);
          }
          pack(0);
          __builtin_amdgcn_sched_barrier(0);
#pragma unroll
          for (int j = 0; j < 16; ++j) {
            if (j % (16 / NM) == 0) grad_mfma(0, j / (16 / NM));
            element(1, j, false);
            __builtin_amdgcn_sched_barrier(0);
          }
        } else {
#pragma unroll
          for (int j = 0; j < 16; ++j) {
            if (j % (16 / NM) == 0) score_mfma(1, j / (16 / NM));
            element(0, j, true);
            __builtin_amdgcn_sched_barrier(0);
          }
          pack(0);
          __builtin_amdgcn_sched_barrier(0);
#pragma unroll
          for (int j = 0; j < 16; ++j) {
            if (j % (16 / NM) == 0) grad_mfma(0, j / (16 / NM));
            element(1, j, true);
            __builtin_amdgcn_sched_barrier(0);
          }
        }
        pack(1);
        load_tr(1);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int m = 0; m < NM; ++m) grad_mfma(1, m);
      }
      __syncthreads();
    }
  }
  // result lane = column d, rows = keys of this wavefront
#pragma unroll
  for (int nb = 0; nb < DB; ++nb)
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      const int kk = k0 + 32 * wave + 8 * (r >> 2) + 4 * h + (r & 3);
      if (kk < p.T) {
        const long long o = ((long long)kk * p.Hkv + hkv) * kHD + 32 * nb + (lane & 31);
        p.dk[o] = f32_to_bf16_rn(acc_k[nb][r] * p.scale);
        p.dv[o] = f32_to_bf16_rn(acc_v[nb][r]);
      }
    }
}

// ---------------------------------------------------------------------------------------------------------
// dK, dV with two wavefronts per SIMD: grid (Hkv, ceil(T/128)), 512 threads.  The same walk and the same arithmetic,
// in the same order, as varlen_attn_dkv_kernel (results are bit-identical); the work of a 32-key wavefront is
// dealt to a PAIR of wavefronts (w, w + 4: one SIMD) so that each fits 256 registers:
//   role A (w < 4) holds the K rows:  S = Q K^T, P = exp(S * scale - lse)        -> P (fp32) to its partner through LDS
//   role B         holds the V rows:  dP = dO V^T, dS = P * (dP - delta) / scale  -> dS (bf16 operand) to its partner
// and each owns one half of the head dimension of BOTH accumulators (dV += P^T dO, dK += dS^T Q), so no product is
// computed twice and the Q / dO tiles are read from LDS exactly as often as by the single wavefront.
// The sub-blocks of 32 queries (all steps of all query heads of the group, one sequence n = 0, 1, ..) run as a
// software pipeline with ONE barrier per sub-block; between barriers n - 1 and n
//   A:  S(n) and dK_A(n - 2) interleaved (dS(n - 2) came from the partner an interval ago);  P(n) -> LDS;  dV_A(n)
//   B:  P(n - 1) from LDS, dS(n - 1) -> LDS;  dV_B(n - 1), dK_B(n - 1) and dP(n) interleaved
// so that each wavefront has 16 matrix instructions and its share of the softmax arithmetic in every interval, A
// starting with the former and B with the latter: the partner's matrix instructions run under a wavefront's vector
// arithmetic, which a lone wavefront per SIMD cannot have.  P and dS have two LDS slots each (written for one
// sub-block while the previous one is read); the Q / dO tiles and the per-query scalars have three buffers (the
// tile before the current one is still read, the next one is being written).
// Tiles travel global -> LDS directly (buffer_load ... lds, rows past the end of the queries read as zero), a step
// ahead; every LDS access of the loop is inline assembly with its own counted waits (the compiler would otherwise
// wait for the tile loads in flight at each LDS access it can see, and streams fragments one per matrix
// instruction when left to schedule them).  The barriers are bare s_barrier instructions behind a wait for the
// wavefront's own LDS traffic.  Every wavefront passes every barrier (steps outside a pair's query range skip the
// arithmetic only).
// ---------------------------------------------------------------------------------------------------------
template <int HD>
constexpr int kAttnDkv2Lds = 3 * 2 * kAttnBK * HD * 2 + 2 * 4 * 64 * 64 + 2 * 4 * 64 * 32 + 3 * 4 * kAttnBK * 4;

template <int OFF>
__device__ __forceinline__ u32x4_t lds_read_u128_asm(uint32_t addr) {
  static_assert(OFF >= 0 && OFF < 65536, "DS offset field");
  u32x4_t v;
  asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(v) : "v"(addr), "i"(OFF));
  return v;
}
template <int OFF>
__device__ __forceinline__ void lds_write_u128_asm(uint32_t addr, u32x4_t v) {
  static_assert(OFF >= 0 && OFF < 65536, "DS offset field");
  asm volatile("ds_write_b128 %0, %1 offset:%2" : : "v"(addr), "v"(v), "i"(OFF) : "memory");
}
template <int OFF>
__device__ __forceinline__ void lds_write_u32_asm(uint32_t addr, uint32_t v) {
  static_assert(OFF >= 0 && OFF < 65536, "DS offset field");
  asm volatile("ds_write_b32 %0, %1 offset:%2" : : "v"(addr), "v"(v), "i"(OFF) : "memory");
}

template <int HD>
__global__ __launch_bounds__(512) void varlen_attn_dkv2_kernel(AttnParams p) {
  constexpr int KS = HD / 16, DB = HD / 32, DH = DB / 2, kAttnTile = kAttnBK * HD * 2, kHD = HD;
  constexpr int RPI = 1024 / (HD * 2);                 // tile rows one direct-to-LDS instruction fills (64 lanes x 16 bytes)
  constexpr int NLD = kAttnBK / RPI / 8;               // such instructions per wavefront and tile
  constexpr int kRows = 4 * kAttnBK * 4;               // bytes of a buffer of per-query scalars: lse2 | delta | lo | hi
  constexpr int kXp = 3 * 2 * kAttnTile;               // P, fp32: [slot][pair][4][64 lanes] x 16 bytes
  constexpr int kXd = kXp + 2 * 4 * 64 * 64;           // dS, bf16 operands: [slot][pair][2][64 lanes] x 16 bytes
  constexpr int kRw = kXd + 2 * 4 * 64 * 32;           // [buffer][lse2 | delta | lo | hi][64]
  static_assert(kRw + 3 * kRows == kAttnDkv2Lds<HD>, "LDS layout");
  extern __shared__ __attribute__((aligned(16))) char smem[];
  const uint32_t lds0 = lds_addr(smem);
  const int lane = threadIdx.x & 63, h = lane >> 5;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int pw = wave & 3;                             // the pair's 32 keys
  const bool role_a = wave < 4;
  const int dh = role_a ? 0 : DH;                      // first 32-column block of this wavefront's half
  const int hkv = blockIdx.x, G = p.Hq / p.Hkv;
  const int k0 = min(max(p.order_k[blockIdx.y], 0), (int)gridDim.y - 1) * kAttnBQ;   // clamped: the list may come from the caller
  const int key = k0 + 32 * pw + (lane & 31);
  const bool valid = key < p.T;
  const int last = (k0 + kAttnBQ - 1 < p.T ? k0 + kAttnBQ - 1 : p.T - 1);
  const int q_begin = max(__builtin_amdgcn_readfirstlane(p.causal ? k0 : p.seg_start[k0]), 0);   // work-group-uniform loop bounds, inside [0, T]
  const int q_end = min(__builtin_amdgcn_readfirstlane(p.seg_end[last]), p.T);
  const int wfirst = k0 + 32 * pw, wlast = (wfirst + 31 < p.T ? wfirst + 31 : p.T - 1);
  const bool wave_on = wfirst < p.T;
  const int wq_lo = wave_on ? (p.causal ? wfirst : p.seg_start[wfirst]) : 1;   // first / last query of interest
  const int wq_hi = wave_on ? p.seg_end[wlast] - 1 : 0;

  // per-lane LDS offsets: row fragments as in attn_lane, transposing fragments for this wavefront's half only
  uint32_t rowc[KS], trh[DH][2];
  {
    const int g1 = (lane >> 4) & 1, j = lane & 15, r = lane & 31;
#pragma unroll
    for (int st = 0; st < KS; ++st) rowc[st] = r * (HD * 2) + (((2 * st + h) ^ attn_swz<HD>(r)) << 4);
#pragma unroll
    for (int nb = 0; nb < DH; ++nb)
#pragma unroll
      for (int rd = 0; rd < 2; ++rd) {
        const int row = 4 * h + (j >> 2) + 8 * rd;
        const int chunk = 4 * (dh + nb) + 2 * g1 + ((j & 3) >> 1);
        trh[nb][rd] = row * (HD * 2) + ((chunk ^ attn_swz<HD>(row)) << 4) + 8 * (j & 1);
      }
  }
  const uint32_t xp = lds0 + kXp + pw * (64 * 64) + lane * 16;      // + slot * 16384 + grp * 1024
  const uint32_t xd = lds0 + kXd + pw * (64 * 32) + lane * 16;      // + slot * 8192 + s2 * 1024
  const uint32_t rwl = lds0 + kRw + h * 16;                         // + buffer * kRows + array * 256 + (32 mq + 8 grp) * 4

  // the lane's own K row (role A) or V row (role B) as the operand of the score products
  bf16x8_t of[KS];
  attn_row_operand(of, role_a ? p.k + (long long)(valid ? key : 0) * p.k_st + (long long)hkv * p.k_sh
                              : p.v + (long long)(valid ? key : 0) * p.v_st + (long long)hkv * p.v_sh, valid, h);
  const float c = p.scale * kLog2e;

  f32x16_t acc_k[DH], acc_v[DH];
#pragma unroll
  for (int nb = 0; nb < DH; ++nb)
#pragma unroll
    for (int r = 0; r < 16; ++r) acc_k[nb][r] = acc_v[nb][r] = 0.f;

  // tile fetch, global -> LDS: instruction i of this wavefront fills tile rows (8 i + wave) * RPI .. + RPI - 1; lane l
  // lands at 16 l of that KiB, i.e. row l / (HD/8), chunk slot l % (HD/8) - so it fetches the chunk the swizzle
  // puts there
  const long long do_st = (long long)p.Hq * kHD;
  uint32_t foq[NLD], fod[NLD];
#pragma unroll
  for (int i = 0; i < NLD; ++i) {
    const int row = (8 * i + wave) * RPI + lane / (HD / 8), ch = (lane % (HD / 8)) ^ attn_swz<HD>(row);
    foq[i] = (uint32_t)(((long long)row * p.q_st + ch * 8) * 2);
    fod[i] = (uint32_t)(((long long)row * do_st + ch * 8) * 2);
  }

  // tiles in walking order: query head g = 0 .. G-1, inside it the 64-query steps from q_begin to q_end
  const int nsteps = q_end > q_begin ? (q_end - q_begin + kAttnBK - 1) / kAttnBK : 0;
  const int NT = nsteps * G;
  int f_g = 0, f_qb = q_begin;                 // the tile the next fetch brings
  // raw values of the tile's per-query scalars, as fetched (nothing is computed from them until publish(): an
  // instruction that touches them would wait for the tile loads issued before them too - the memory counter retires in order)
  float r_lse = 0.f, r_dl = 0.f;
  int r_lo = 0, r_end = 0, r_t = 0;
  // The descriptors of the next tile move by additions (down a head's queries 64 at a time) and are formed from
  // scratch only when the walk starts the next head: every wavefront does this scalar work at the same moment, at the
  // top of a tile's first interval, before its first LDS request.
  const char *f_qp = nullptr, *f_dp = nullptr;                   // first row of the next tile
  long long f_qbytes = 0, f_dbytes = 0;                          // from there to the end of the head's last query row
  const float *f_lse = nullptr, *f_delta = nullptr;              // the head's per-query scalars
  const long long f_qstep = (long long)kAttnBK * p.q_st * 2, f_dstep = (long long)kAttnBK * do_st * 2;
  auto fetch_head = [&]() {                    // the walk is at the first tile of head f_g
    const int hq = hkv * G + f_g;
    f_qp = (const char*)(p.q + (long long)hq * p.q_sh + (long long)q_begin * p.q_st);
    f_dp = (const char*)(p.dout + (long long)hq * kHD + (long long)q_begin * do_st);
    f_qbytes = ((long long)q_end - q_begin - 1) * p.q_st * 2 + HD * 2;      // strides >= HD: not positive past the end
    f_dbytes = ((long long)q_end - q_begin - 1) * do_st * 2 + HD * 2;
    f_lse = p.lse + (long long)hq * p.T;
    f_delta = p.delta + (long long)hq * p.T;
  };
  auto fetch_next = [&](int buf) {             // tile -> LDS buffer buf (in flight until publish()), its scalars -> registers
    if (f_qb == q_begin) fetch_head();
    long long bq = f_qbytes > 0 ? f_qbytes : 0, bd = f_dbytes > 0 ? f_dbytes : 0;
    if (bq > 0xffffffffLL) bq = 0xffffffffLL;
    if (bd > 0xffffffffLL) bd = 0xffffffffLL;
    const __amdgpu_buffer_rsrc_t rsq = make_rsrc(f_qp, (uint32_t)bq);
    const __amdgpu_buffer_rsrc_t rsd = make_rsrc(f_dp, (uint32_t)bd);
    char* qt = smem + buf * 2 * kAttnTile + wave * 1024;
#pragma unroll
    for (int i = 0; i < NLD; ++i) {
      __builtin_amdgcn_raw_ptr_buffer_load_lds(rsq, FGRPO_LDS_PTR(qt + i * 8192), 16, (int)foq[i], 0, 0, 0);
      __builtin_amdgcn_raw_ptr_buffer_load_lds(rsd, FGRPO_LDS_PTR(qt + kAttnTile + i * 8192), 16, (int)fod[i], 0, 0, 0);
    }
    if (threadIdx.x < kAttnBK) {
      r_t = f_qb + threadIdx.x;
      const int tc = r_t < q_end ? r_t : q_end - 1;       // q_end > q_begin here: a row that exists
      r_lse = f_lse[tc];
      r_dl = f_delta[tc];
      r_lo = p.seg_start[tc];
      r_end = p.seg_end[tc];
    }
    f_qb += kAttnBK;
    f_qp += f_qstep, f_dp += f_dstep, f_qbytes -= f_qstep, f_dbytes -= f_dstep;
    if (f_qb >= q_end) f_qb = q_begin, ++f_g;
  };
  auto publish = [&](int buf) {                // before the barrier that opens the tile's first interval
    if (threadIdx.x < kAttnBK) {
      const bool ok = r_t < q_end;
      const uint32_t rw = lds0 + kRw + buf * kRows + threadIdx.x * 4;
      lds_write_u32_asm<0>(rw, __float_as_uint(ok ? r_lse * kLog2e : 0.f));
      lds_write_u32_asm<kAttnBK * 4>(rw, __float_as_uint(ok ? r_dl : 0.f));
      lds_write_u32_asm<2 * kAttnBK * 4>(rw, (uint32_t)(ok ? r_lo : 1));
      lds_write_u32_asm<3 * kAttnBK * 4>(rw, (uint32_t)(ok ? (p.causal ? r_t : r_end - 1) : 0));
    }
  };
  auto barrier = [&]() {
    wait_lgkm<0>();           // this wavefront's LDS traffic has landed
    wg_barrier();
  };
  // the K / V operand rows are complete here: nothing in the loop may wait for them behind the tile loads it keeps
  // in flight (the memory counter retires in order)
#pragma unroll
  for (int st = 0; st < KS; ++st) asm volatile("" : "+v"(of[st]));

  // all of LDS starts as zeros (see the loop)
  for (int o = threadIdx.x * 16; o < kAttnDkv2Lds<HD>; o += 512 * 16) lds_write_u128_asm<0>(lds0 + o, u32x4_t{0u, 0u, 0u, 0u});
  barrier();
  if (NT > 0) {
    fetch_next(0);
    publish(0);
  }
  FGRPO_WAIT_VMCNT(0);
  barrier();
  // Fragment requests are inline assembly: the value is there after the matching wait, and NOTHING may read the
  // registers before it.  The compiler does not know that (to it the request defines them), so every value goes
  // through settle() right after its wait: an empty volatile asm that redefines the registers, which pins every
  // use behind the wait (volatile asm statements and the wait keep their order; a plain use could otherwise be
  // hoisted above the wait, e.g. out of both arms of a branch).
  struct TrFrag {
    u32x2_t lo, hi;
  };
  auto rd_tr = [&](uint32_t tile, auto kbc, int nb) {   // K-major fragment of 16 k rows from kbase, column block dh + nb
    constexpr int kb = decltype(kbc)::value;
    TrFrag f;
    asm volatile("ds_read_b64_tr_b16 %0, %1 offset:%2" : "=v"(f.lo) : "v"(tile + trh[nb][0]), "i"(kb * HD * 2));
    asm volatile("ds_read_b64_tr_b16 %0, %1 offset:%2" : "=v"(f.hi) : "v"(tile + trh[nb][1]), "i"(kb * HD * 2));
    return f;
  };
  auto settle_tr = [](TrFrag& f) {
    asm volatile("" : "+v"(f.lo), "+v"(f.hi));
    return u32x4_t{f.lo.x, f.lo.y, f.hi.x, f.hi.y};
  };
  auto settle = [](u32x4_t& v) { asm volatile("" : "+v"(v)); };
  auto mfma = [](u32x4_t a, u32x4_t b, f32x16_t acc) {
    return FGRPO_MFMA(__builtin_bit_cast(bf16x8_t, a), __builtin_bit_cast(bf16x8_t, b), acc);
  };
  auto fence = []() { __builtin_amdgcn_sched_barrier(0); };
  constexpr int kTr = 4 * DH;                  // LDS instructions of the transposing fragments of one product's sub-block

  // The loop exists once per role (the roles keep different values across intervals).  An interval is straight-line
  // code: the requests of a later group are in flight under the matrix instructions of an earlier one, every wait is
  // counted.  Stages that have nothing to do - the ramps of the pipeline at the ends of a pair's query range, tiles
  // between them that no key of the pair can see - are not branched around: A's P comes out as exact zeros (every
  // pair masked), and each role clears what it takes from the partner's slot when that sub-block is not the
  // pair's (the slot may then hold an older sub-block's values).  All of LDS starts as zeros, so that what such a
  // stage multiplies by zero is never a NaN pattern.  An interval in which neither stage has work is skipped whole.
  auto pipeline = [&](auto rolec) {
    constexpr bool ROLE_A = decltype(rolec)::value;
    int b_prev = 2, b_cur = 0, b_next = 1;       // LDS buffers of tiles t - 1, t, t + 1
    int qb_cur = q_begin;
    bool act_prev = false;
    float dpd[16];                               // role B: dP - delta of the sub-block before the current one
#pragma unroll
    for (int r = 0; r < 16; ++r) dpd[r] = 0.f;
    for (int t = 0; t <= NT; ++t) {              // the last round only drains the pipeline
      const uint32_t qt = lds0 + b_cur * 2 * kAttnTile, dot = qt + kAttnTile;
      const uint32_t qt_prev = lds0 + b_prev * 2 * kAttnTile, dot_prev = qt_prev + kAttnTile;
      const uint32_t rw = rwl + b_cur * kRows;
      const bool act_cur = t < NT && wave_on && qb_cur <= wq_hi && qb_cur + kAttnBK > wq_lo;   // the same for both wavefronts of a pair
      // every (query, key) pair of this step visible: all 64 queries exist, the last one's segment starts at or
      // before the pair's first key, the first one sees its last key
      bool all_visible = false;
      if (ROLE_A && act_cur) {
        int lo_last, hi_first;
        asm volatile("ds_read_b32 %0, %2 offset:%3\n\tds_read_b32 %1, %2 offset:%4\n\ts_waitcnt lgkmcnt(0)"
                     : "=&v"(lo_last), "=&v"(hi_first)
                     : "v"(lds0 + kRw + b_cur * kRows), "i"(2 * kAttnBK * 4 + (kAttnBK - 1) * 4), "i"(3 * kAttnBK * 4));
        all_visible = wfirst + 31 < p.T && qb_cur + kAttnBK <= q_end && __builtin_amdgcn_readfirstlane(lo_last) <= wfirst &&
                      __builtin_amdgcn_readfirstlane(hi_first) >= wlast;
      }
      // The next tile is fetched (descriptors, loads, wave 0's scalars) from inside the tile's first interval, behind
      // the first run of matrix instructions: at the top of the loop every wavefront would do that work at the same
      // moment, right behind the barrier, before its first LDS request.  b_next was last read two intervals ago (as
      // the tile before the previous one).
      const bool do_fetch = t + 1 < NT;

      // ---- role A: [Q rows | dS, Q^T of the tile before] S(first half) [dO^T, lse] S(second half) x dK; exp; P out; dV
      auto run_a = [&](auto mqc) {
        constexpr int mq = decltype(mqc)::value;
        u32x4_t fa[KS], dsf[2], l4[4];
        TrFrag fqk_[2][DH], fdo_[2][DH];
        f32x16_t sc;
        static_for<KS>([&](auto stc) { fa[decltype(stc)::value] = lds_read_u128_asm<mq * 32 * HD * 2>(qt + rowc[decltype(stc)::value]); });
        static_for<2>([&](auto s2c) {
          constexpr int s2 = decltype(s2c)::value;
          dsf[s2] = lds_read_u128_asm<mq * 8192 + s2 * 1024>(xd);
#pragma unroll
          for (int nb = 0; nb < DH; ++nb) fqk_[s2][nb] = rd_tr(qt_prev, std::integral_constant<int, 32 * mq + 16 * s2>{}, nb);
        });
        wait_lgkm<2 + kTr>();                               // the Q rows are there (requested first; LDS returns in order)
        fence();
        // a wavefront in a run of matrix instructions goes first at the SIMD's issue port: its partner's vector
        // arithmetic fills the cycles the matrix pipe leaves, not the other way round (-4 % on the kernel)
        __builtin_amdgcn_s_setprio(2);
#pragma unroll
        for (int st = 0; st < KS; ++st) settle(fa[st]);
#pragma unroll
        for (int r = 0; r < 16; ++r) sc[r] = 0.f;
#pragma unroll
        for (int st = 0; st < KS / 2; ++st) sc = mfma(fa[st], __builtin_bit_cast(u32x4_t, of[st]), sc);
        fence();
        if constexpr (mq == 0) {
          if (do_fetch) fetch_next(b_next);
          fence();
        }
        static_for<2>([&](auto s2c) {
          constexpr int s2 = decltype(s2c)::value;
#pragma unroll
          for (int nb = 0; nb < DH; ++nb) fdo_[s2][nb] = rd_tr(dot, std::integral_constant<int, 32 * mq + 16 * s2>{}, nb);
        });
        static_for<4>([&](auto gc) { l4[decltype(gc)::value] = lds_read_u128_asm<(32 * mq + 8 * decltype(gc)::value) * 4>(rw); });
        wait_lgkm<kTr + 4>();                               // dS and the Q^T fragments are there
        fence();
        u32x4_t fqk[2][DH];
#pragma unroll
        for (int s2 = 0; s2 < 2; ++s2) {
          settle(dsf[s2]);
          if (!act_prev) dsf[s2] = u32x4_t{0u, 0u, 0u, 0u};     // the slot holds an older sub-block's dS
#pragma unroll
          for (int nb = 0; nb < DH; ++nb) fqk[s2][nb] = settle_tr(fqk_[s2][nb]);
        }
        // second half of the S chain and the dK products, alternating
        static_for<(KS / 2 < 2 * DH ? 2 * DH : KS / 2)>([&](auto ic) {
          constexpr int i = decltype(ic)::value;
          if constexpr (i < KS / 2) sc = mfma(fa[KS / 2 + i], __builtin_bit_cast(u32x4_t, of[KS / 2 + i]), sc);
          if constexpr (i < 2 * DH) acc_k[i % DH] = mfma(dsf[i / DH], fqk[i / DH][i % DH], acc_k[i % DH]);
        });
        fence();
        __builtin_amdgcn_s_setprio(0);
        wait_lgkm<0>();                                     // the dO^T fragments and lse are there
        fence();
        u32x4_t fdo[2][DH];
#pragma unroll
        for (int s2 = 0; s2 < 2; ++s2)
#pragma unroll
          for (int nb = 0; nb < DH; ++nb) fdo[s2][nb] = settle_tr(fdo_[s2][nb]);
#pragma unroll
        for (int grp = 0; grp < 4; ++grp) settle(l4[grp]);
        float pr[16];
        if (all_visible) {
#pragma unroll
          for (int grp = 0; grp < 4; ++grp)
#pragma unroll
            for (int e = 0; e < 4; ++e) pr[4 * grp + e] = fast_exp2(__builtin_fmaf(sc[4 * grp + e], c, -__uint_as_float(l4[grp][e])));
        } else {
          // the key ranges of the queries: only now, when the registers of the Q fragments are free
          u32x4_t lo4[4], hi4[4];
          static_for<4>([&](auto gc) {
            lo4[decltype(gc)::value] = lds_read_u128_asm<2 * kAttnBK * 4 + (32 * mq + 8 * decltype(gc)::value) * 4>(rw);
            hi4[decltype(gc)::value] = lds_read_u128_asm<3 * kAttnBK * 4 + (32 * mq + 8 * decltype(gc)::value) * 4>(rw);
          });
          wait_lgkm<0>();
          fence();
#pragma unroll
          for (int grp = 0; grp < 4; ++grp) settle(lo4[grp]), settle(hi4[grp]);
#pragma unroll
          for (int grp = 0; grp < 4; ++grp)
#pragma unroll
            for (int e = 0; e < 4; ++e) {
              float x = __builtin_fmaf(sc[4 * grp + e], c, -__uint_as_float(l4[grp][e]));
              // select before the exponential: a masked pair becomes exp2(-inf) = 0 without a branch; a tile that is not
              // the pair's (or not there at all: the draining round) has every pair masked
              x = ((int)(key >= (int)lo4[grp][e]) & (int)(key <= (int)hi4[grp][e]) & (int)act_cur) ? x : -INFINITY;
              pr[4 * grp + e] = fast_exp2(x);
            }
        }
        static_for<4>([&](auto gc) {
          constexpr int grp = decltype(gc)::value;
          lds_write_u128_asm<mq * 16384 + grp * 1024>(xp, u32x4_t{__float_as_uint(pr[4 * grp]), __float_as_uint(pr[4 * grp + 1]),
                                                                    __float_as_uint(pr[4 * grp + 2]), __float_as_uint(pr[4 * grp + 3])});
        });
#pragma unroll
        for (int s2 = 0; s2 < 2; ++s2) {
          const u32x4_t pf = __builtin_bit_cast(u32x4_t, attn_pack8(pr + 8 * s2));
#pragma unroll
          for (int nb = 0; nb < DH; ++nb) acc_v[nb] = mfma(pf, fdo[s2][nb], acc_v[nb]);
        }
      };
      // ---- role B: [P | dO^T, Q^T of sub-block n - 1, first 16 queries] dS, dS out [first dO rows | the other 16 queries]
      //      dV, dK (first halves) [other dO rows] dP x (second halves) [delta] dP
      auto run_b = [&](auto mqc, bool act1) {
        constexpr int mq = decltype(mqc)::value, mq1 = 1 - mq;
        // the sub-block before this one: the other half of this tile (mq = 1) or the second half of the previous tile
        const uint32_t qt1 = mq == 0 ? qt_prev : qt, dot1 = mq == 0 ? dot_prev : dot;
        u32x4_t fa[KS], p4[4], d4[4], dsf[2], pf[2];
        TrFrag fq1_[2][DH], fdo1_[2][DH];
        static_for<4>([&](auto gc) { p4[decltype(gc)::value] = lds_read_u128_asm<mq1 * 16384 + decltype(gc)::value * 1024>(xp); });
#pragma unroll
        for (int nb = 0; nb < DH; ++nb) {
          fdo1_[0][nb] = rd_tr(dot1, std::integral_constant<int, 32 * mq1>{}, nb);
          fq1_[0][nb] = rd_tr(qt1, std::integral_constant<int, 32 * mq1>{}, nb);
        }
        wait_lgkm<kTr>();                                   // P is there (requested first; LDS returns in order)
        fence();
        {
          float ds[16], pr[16];
#pragma unroll
          for (int grp = 0; grp < 4; ++grp) {
            settle(p4[grp]);
#pragma unroll
            for (int e = 0; e < 4; ++e) {
              pr[4 * grp + e] = act1 ? __uint_as_float(p4[grp][e]) : 0.f;      // else the slot holds an older sub-block's P
              ds[4 * grp + e] = pr[4 * grp + e] * dpd[4 * grp + e];
            }
          }
#pragma unroll
          for (int s2 = 0; s2 < 2; ++s2) {
            dsf[s2] = __builtin_bit_cast(u32x4_t, attn_pack8(ds + 8 * s2));
            pf[s2] = __builtin_bit_cast(u32x4_t, attn_pack8(pr + 8 * s2));
          }
        }
        fence();
        lds_write_u128_asm<mq1 * 8192>(xd, dsf[0]);
        lds_write_u128_asm<mq1 * 8192 + 1024>(xd, dsf[1]);
        static_for<KS / 2>([&](auto stc) { fa[decltype(stc)::value] = lds_read_u128_asm<mq * 32 * HD * 2>(dot + rowc[decltype(stc)::value]); });
#pragma unroll
        for (int nb = 0; nb < DH; ++nb) {
          fdo1_[1][nb] = rd_tr(dot1, std::integral_constant<int, 32 * mq1 + 16>{}, nb);
          fq1_[1][nb] = rd_tr(qt1, std::integral_constant<int, 32 * mq1 + 16>{}, nb);
        }
        wait_lgkm<2 + KS / 2 + kTr>();                      // the first transposed fragments are there
        fence();
        __builtin_amdgcn_s_setprio(2);
#pragma unroll
        for (int nb = 0; nb < DH; ++nb) acc_v[nb] = mfma(pf[0], settle_tr(fdo1_[0][nb]), acc_v[nb]);
#pragma unroll
        for (int nb = 0; nb < DH; ++nb) acc_k[nb] = mfma(dsf[0], settle_tr(fq1_[0][nb]), acc_k[nb]);
        fence();
        if constexpr (mq == 0) {
          if (do_fetch) fetch_next(b_next);
          fence();
        }
        static_for<KS / 2>([&](auto stc) {
          fa[KS / 2 + decltype(stc)::value] = lds_read_u128_asm<mq * 32 * HD * 2>(dot + rowc[KS / 2 + decltype(stc)::value]);
        });
        wait_lgkm<KS / 2>();                                // the first dO rows and the other transposed fragments are there
        fence();
        u32x4_t fdo1[DH], fq1[DH];
#pragma unroll
        for (int nb = 0; nb < DH; ++nb) fdo1[nb] = settle_tr(fdo1_[1][nb]), fq1[nb] = settle_tr(fq1_[1][nb]);
#pragma unroll
        for (int st = 0; st < KS / 2; ++st) settle(fa[st]);
        f32x16_t sc;
#pragma unroll
        for (int r = 0; r < 16; ++r) sc[r] = 0.f;
        static_for<(KS / 2 < 2 * DH ? 2 * DH : KS / 2)>([&](auto ic) {
          constexpr int i = decltype(ic)::value;
          if constexpr (i < KS / 2) sc = mfma(fa[i], __builtin_bit_cast(u32x4_t, of[i]), sc);
          if constexpr (i < DH) acc_v[i] = mfma(pf[1], fdo1[i], acc_v[i]);
          else if constexpr (i < 2 * DH) acc_k[i - DH] = mfma(dsf[1], fq1[i - DH], acc_k[i - DH]);
        });
        fence();
        static_for<4>([&](auto gc) { d4[decltype(gc)::value] = lds_read_u128_asm<kAttnBK * 4 + (32 * mq + 8 * decltype(gc)::value) * 4>(rw); });
        wait_lgkm<4>();                                     // the other dO rows are there (delta on its way)
        fence();
#pragma unroll
        for (int st = KS / 2; st < KS; ++st) {
          settle(fa[st]);
          sc = mfma(fa[st], __builtin_bit_cast(u32x4_t, of[st]), sc);
        }
        fence();
        __builtin_amdgcn_s_setprio(0);
        wait_lgkm<0>();
        fence();
#pragma unroll
        for (int grp = 0; grp < 4; ++grp) {
          settle(d4[grp]);
#pragma unroll
          for (int e = 0; e < 4; ++e) dpd[4 * grp + e] = sc[4 * grp + e] - __uint_as_float(d4[grp][e]);
        }
      };
      static_for<2>([&](auto mqc) {
        constexpr int mq = decltype(mqc)::value;
        if constexpr (ROLE_A) {
          if (act_cur || act_prev) run_a(mqc);
          else if (mq == 0 && do_fetch) fetch_next(b_next);
        } else {
          const bool act1 = mq == 0 ? act_prev : act_cur;
          if (act1 || act_cur) run_b(mqc, act1);
          else if (mq == 0 && do_fetch) fetch_next(b_next);
        }
        if constexpr (mq == 1) {
          if (t + 1 < NT) publish(b_next);
          // this wavefront's part of the next tile is in LDS.  Unconditional, so that no fetch counts as pending at
          // the top of the loop (where the next one is issued and every wait would be for both).
          FGRPO_WAIT_VMCNT(0);
        }
        barrier();
      });
      const int bb = b_prev;
      b_prev = b_cur, b_cur = b_next, b_next = bb;
      act_prev = act_cur;
      qb_cur += kAttnBK;
      if (qb_cur >= q_end) qb_cur = q_begin;
    }
  };
  if (role_a) pipeline(std::true_type{}); else pipeline(std::false_type{});
  // result lane = column d, rows = keys of this pair
#pragma unroll
  for (int nb = 0; nb < DH; ++nb)
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      const int kk = k0 + 32 * pw + 8 * (r >> 2) + 4 * h + (r & 3);
      if (kk < p.T) {
        const long long o = ((long long)kk * p.Hkv + hkv) * kHD + 32 * (dh + nb) + (lane & 31);
        p.dk[o] = f32_to_bf16_rn(acc_k[nb][r] * p.scale);
        p.dv[o] = f32_to_bf16_rn(acc_v[nb][r]);
      }
    }
}

// ---------------------------------------------------------------------------------------------------------
// Query-side kernels, second form: the same walk and the same arithmetic in the same order as
// varlen_attn_fwd_kernel / varlen_attn_dq_kernel (bit-identical results), with the memory side done by hand:
//  * K / V tiles travel global -> LDS directly (buffer_load ... lds; rows past the end of the keys read as zero) into
//    two buffers, a step ahead: no staging registers, one barrier per 64-key step instead of two;
//  * every LDS fragment read is inline assembly, requested in groups a group ahead of the matrix instructions that
//    use it, with counted waits (left to the compiler, each matrix instruction waits for a fragment requested one
//    instruction earlier: an LDS round trip per 32-cycle instruction); the dO^T / V^T fragments of the second
//    product are on their way while the softmax arithmetic runs.
// Every value an asm read delivers passes through attn_settle() right after its wait (see varlen_attn_dkv2_kernel).
// ---------------------------------------------------------------------------------------------------------
struct AttnTr {
  u32x2_t lo, hi;
};
template <int OFF>
__device__ __forceinline__ AttnTr attn_rd_tr_asm(uint32_t a0, uint32_t a1) {
  static_assert(OFF >= 0 && OFF < 65536, "DS offset field");
  AttnTr f;
  asm volatile("ds_read_b64_tr_b16 %0, %1 offset:%2" : "=v"(f.lo) : "v"(a0), "i"(OFF));
  asm volatile("ds_read_b64_tr_b16 %0, %1 offset:%2" : "=v"(f.hi) : "v"(a1), "i"(OFF));
  return f;
}
__device__ __forceinline__ u32x4_t attn_settle_tr(AttnTr& f) {
  asm volatile("" : "+v"(f.lo), "+v"(f.hi));
  return u32x4_t{f.lo.x, f.lo.y, f.hi.x, f.hi.y};
}
__device__ __forceinline__ void attn_settle(u32x4_t& v) { asm volatile("" : "+v"(v)); }
__device__ __forceinline__ f32x16_t attn_mfma(u32x4_t a, u32x4_t b, f32x16_t acc) {
  return FGRPO_MFMA(__builtin_bit_cast(bf16x8_t, a), __builtin_bit_cast(bf16x8_t, b), acc);
}

// Direct-to-LDS fetch of 64-row tiles by a 256-thread work-group: instruction i of wavefront w fills the KiB
// (4 i + w) of the tile, i.e. rows (4 i + w) * RPI .. with RPI = 1024 / (2 HD); lane l lands at 16 l of that KiB - row
// l / (HD/8), chunk slot l % (HD/8) - and therefore fetches the chunk the swizzle puts there.  The swizzle of a row
// depends on the lane and the wavefront only (not on i), so one per-lane byte offset serves every instruction and
// the step from one to the next is a scalar.
template <int HD>
__device__ __forceinline__ uint32_t attn_dma_lane_offset(int wave, int lane, long long st) {
  constexpr int RPI = 1024 / (HD * 2);
  const int row = wave * RPI + lane / (HD / 8), ch = (lane % (HD / 8)) ^ attn_swz<HD>(row);
  return (uint32_t)(((long long)row * st + ch * 8) * 2);
}
template <int HD>
__device__ __forceinline__ void attn_dma_tile(const bf16_t* base, long long st, int row0, int row_end, uint32_t lane_off,
                                              char* tile_w /* tile + wave * 1024 */) {
  constexpr int RPI = 1024 / (HD * 2), NLD = kAttnBK / RPI / 4;
  const long long rows = (long long)row_end - row0;
  long long bytes = rows > 0 ? (rows - 1) * st * 2 + HD * 2 : 0;
  if (bytes > 0xffffffffLL) bytes = 0xffffffffLL;
  const __amdgpu_buffer_rsrc_t rs = make_rsrc(base + (long long)row0 * st, (uint32_t)bytes);
#pragma unroll
  for (int i = 0; i < NLD; ++i)
    __builtin_amdgcn_raw_ptr_buffer_load_lds(rs, FGRPO_LDS_PTR(tile_w + i * 4096), 16, (int)lane_off, (int)(i * 4 * RPI * st * 2), 0, 0);
}

// The descriptor of the next 64-row tile, kept up to date by additions: the walk goes down the rows 64 at a time,
// and forming `base + row0 * st` and the byte count from scratch costs four 64-bit multiplications a tile - scalar
// work at the top of a step, which every wavefront of the work-group does at the same moment, right behind the
// barrier, before its first LDS request.  bytes = distance from the tile's first row to the end of the last row there
// is (row_end - 1); zero or less when the walk has passed the end: the loads then write zeros.
template <int HD>
struct AttnTileCursor {
  const char* ptr;
  long long bytes, step;
  __device__ __forceinline__ void init(const bf16_t* base, long long st, int row0, int row_end) {
    ptr = (const char*)(base + (long long)row0 * st);
    bytes = ((long long)row_end - row0 - 1) * st * 2 + HD * 2;      // st >= HD: not positive from row0 = row_end on
    step = (long long)kAttnBK * st * 2;
  }
  __device__ __forceinline__ void next() { ptr += step, bytes -= step; }
  // loads of the tile at the cursor, by a 256-thread work-group (see attn_dma_tile)
  __device__ __forceinline__ void load(long long st, uint32_t lane_off, char* tile_w) const {
    constexpr int RPI = 1024 / (HD * 2), NLD = kAttnBK / RPI / 4;
    long long b = bytes > 0 ? bytes : 0;
    if (b > 0xffffffffLL) b = 0xffffffffLL;
    const __amdgpu_buffer_rsrc_t rs = make_rsrc(ptr, (uint32_t)b);
#pragma unroll
    for (int i = 0; i < NLD; ++i)
      __builtin_amdgcn_raw_ptr_buffer_load_lds(rs, FGRPO_LDS_PTR(tile_w + i * 4096), 16, (int)lane_off, (int)(i * 4 * RPI * st * 2), 0, 0);
  }
};

template <int HD, int HB>
__global__ __launch_bounds__(256, 2) void varlen_attn_fwd2_kernel(AttnParams p) {
  constexpr int KS = HD / 16, DB = HD / 32, kAttnTile = kAttnBK * HD * 2, kHD = HD, G4 = KS / 2;
  __shared__ __attribute__((aligned(16))) char smem[4 * kAttnTile];      // [buffer][K | V]
  const uint32_t lds0 = lds_addr(smem);
  const int lane = threadIdx.x & 63, h = lane >> 5;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  AttnLane<HD> L = attn_lane<HD>(lane);      // + the LDS base: a fragment address is one of these plus a constant
#pragma unroll
  for (int st = 0; st < KS; ++st) L.rowc[st] += (int)lds0;
#pragma unroll
  for (int db = 0; db < DB; ++db) L.tr[db][0] += (int)lds0, L.tr[db][1] += (int)lds0;
  // work-group -> (tile, K/V head, query heads): as in varlen_attn_fwd_kernel
  constexpr int WPH = 4 / HB, RB = 32 * WPH;
  const int G = p.Hq / p.Hkv, NB = (G + HB - 1) / HB;
  const int xcd = blockIdx.x & 7, slot = blockIdx.x >> 3;
  const int unit = (slot / NB) * 8 + xcd;
  const int ntile = (p.T + RB - 1) / RB;
  if (unit >= ntile * p.Hkv) return;
  const int hkv = unit % p.Hkv;
  const int head_g = (slot % NB) * HB + wave / WPH;
  const bool head_ok = head_g < G;
  const int hq = hkv * G + (head_ok ? head_g : G - 1);
  const int q0 = min(max(p.order_q[unit / p.Hkv], 0), ntile - 1) * RB;
  const int tq = q0 + 32 * (wave % WPH) + (lane & 31);
  const bool valid = head_ok && tq < p.T;
  const int lo = valid ? p.seg_start[tq] : 1;
  const int hi = valid ? (p.causal ? tq : p.seg_end[tq] - 1) : 0;
  const int last = (q0 + RB - 1 < p.T ? q0 + RB - 1 : p.T - 1);
  const int k_begin = max(__builtin_amdgcn_readfirstlane(p.seg_start[q0]), 0);
  const int k_end = min(__builtin_amdgcn_readfirstlane(p.causal ? last + 1 : p.seg_end[last]), p.T);
  const int wfirst = q0 + 32 * (wave % WPH), wlast = (wfirst + 31 < p.T ? wfirst + 31 : p.T - 1);
  const bool wave_on = head_ok && wfirst < p.T;
  const int w_lo = wave_on ? p.seg_start[wfirst] : 1;
  const int w_hi = wave_on ? (p.causal ? wlast : p.seg_end[wlast] - 1) : 0;
  const bool wave_full = wave_on && wfirst + 31 < p.T;
  const int w_lo_max = wave_full ? p.seg_start[wlast] : 0x7fffffff;
  const int w_hi_min = wave_full ? (p.causal ? wfirst : p.seg_end[wfirst] - 1) : -1;

  bf16x8_t qf[KS];
  attn_row_operand(qf, p.q + (long long)(valid ? tq : 0) * p.q_st + (long long)hq * p.q_sh, valid, h);
#pragma unroll
  for (int st = 0; st < KS; ++st) asm volatile("" : "+v"(qf[st]));     // complete before the loop: nothing in it waits for them behind a tile load

  f32x16_t acc_o[DB];
#pragma unroll
  for (int db = 0; db < DB; ++db)
#pragma unroll
    for (int r = 0; r < 16; ++r) acc_o[db][r] = 0.f;
  float m_run = -INFINITY, l_run = 0.f;
  const float c = p.scale * kLog2e;

  const bf16_t* kbase = p.k + (long long)hkv * p.k_sh;
  const bf16_t* vbase = p.v + (long long)hkv * p.v_sh;
  const uint32_t fko = attn_dma_lane_offset<HD>(wave, lane, p.k_st), fvo = attn_dma_lane_offset<HD>(wave, lane, p.v_st);
  AttnTileCursor<HD> ck, cv;               // the tile the next fetch brings: the steps are fetched in order
  ck.init(kbase, p.k_st, k_begin, k_end);
  cv.init(vbase, p.v_st, k_begin, k_end);
  auto fetch = [&](int buf) {
    char* t = smem + buf * 2 * kAttnTile + wave * 1024;
    ck.load(p.k_st, fko, t);
    cv.load(p.v_st, fvo, t + kAttnTile);
    ck.next();
    cv.next();
  };
  if (k_begin < k_end) fetch(0);
  FGRPO_WAIT_VMCNT(0);
  wg_barrier();
  // a step on LDS buffer `cur`, a compile-time constant: buffer, tile and block are the instruction's offset field
  auto step = [&](auto curc, int kb) {
    constexpr int cur = decltype(curc)::value, kt = cur * 2 * kAttnTile, vt = kt + kAttnTile;
    if (kb + kAttnBK < k_end) fetch(cur ^ 1);     // the next step's tiles; that buffer was last read a step ago, before the barrier
    if (wave_on && kb <= w_hi && kb + kAttnBK > w_lo) {
      // ---- S^T = K Q^T: four groups of G4 K fragments (key block mb = g / 2, k steps G4 (g % 2) ..), two groups in flight
      u32x4_t kf[2][G4];
      AttnTr vq[2][DB];
      f32x16_t s[2];
#pragma unroll
      for (int mb = 0; mb < 2; ++mb)
#pragma unroll
        for (int r = 0; r < 16; ++r) s[mb][r] = 0.f;
      auto req_k = [&](auto gc) {
        constexpr int g = decltype(gc)::value;
        static_for<G4>([&](auto ic) {
          constexpr int i = decltype(ic)::value, st = G4 * (g % 2) + i;
          kf[g % 2][i] = lds_read_u128_asm<kt + (g / 2) * 32 * HD * 2>((uint32_t)L.rowc[st]);
        });
      };
      auto req_v = [&](auto qc) {          // V^T fragments of keys 16 q .. 16 q + 15, every 32-column block
        constexpr int q = decltype(qc)::value;
        static_for<DB>([&](auto dc) {
          constexpr int db = decltype(dc)::value;
          vq[q % 2][db] = attn_rd_tr_asm<vt + 16 * q * HD * 2>((uint32_t)L.tr[db][0], (uint32_t)L.tr[db][1]);
        });
      };
      auto mma_k = [&](auto gc) {
        constexpr int g = decltype(gc)::value;
#pragma unroll
        for (int i = 0; i < G4; ++i) {
          attn_settle(kf[g % 2][i]);
          s[g / 2] = attn_mfma(kf[g % 2][i], __builtin_bit_cast(u32x4_t, qf[G4 * (g % 2) + i]), s[g / 2]);
        }
      };
      using I0 = std::integral_constant<int, 0>;
      using I1 = std::integral_constant<int, 1>;
      using I2 = std::integral_constant<int, 2>;
      using I3 = std::integral_constant<int, 3>;
      req_k(I0{});
      req_k(I1{});
      wait_lgkm<G4>();
      __builtin_amdgcn_sched_barrier(0);
      mma_k(I0{});
      __builtin_amdgcn_sched_barrier(0);
      req_k(I2{});
      wait_lgkm<G4>();
      __builtin_amdgcn_sched_barrier(0);
      mma_k(I1{});
      __builtin_amdgcn_sched_barrier(0);
      req_k(I3{});
      req_v(I0{});                          // on its way while the softmax arithmetic runs
      wait_lgkm<G4 + 2 * DB>();
      __builtin_amdgcn_sched_barrier(0);
      mma_k(I2{});
      __builtin_amdgcn_sched_barrier(0);
      wait_lgkm<2 * DB>();
      __builtin_amdgcn_sched_barrier(0);
      mma_k(I3{});
      __builtin_amdgcn_sched_barrier(0);

      float mx = -INFINITY;
      if (kb >= w_lo_max && kb + kAttnBK - 1 <= w_hi_min) {   // every pair of this step is visible
#pragma unroll
        for (int mb = 0; mb < 2; ++mb)
#pragma unroll
          for (int r = 0; r < 16; ++r) mx = fmaxf(mx, s[mb][r]);
      } else {
#pragma unroll
        for (int mb = 0; mb < 2; ++mb)
#pragma unroll
          for (int r = 0; r < 16; ++r) {
            const int key = kb + 32 * mb + 8 * (r >> 2) + 4 * h + (r & 3);
            const float x = (key >= lo && key <= hi) ? s[mb][r] : -INFINITY;
            s[mb][r] = x;
            mx = fmaxf(mx, x);
          }
      }
      {
        float mlo, mhi;
        attn_halves(mx, mlo, mhi);
        mx = fmaxf(mlo, mhi);
      }
      const float m_new = fmaxf(m_run, mx);
      const float m_use = (m_new == -INFINITY) ? 0.f : m_new;
      const float alpha = fast_exp2((m_run - m_use) * c);
      const float mc = m_use * c;
      float sum = 0.f;
#pragma unroll
      for (int mb = 0; mb < 2; ++mb)
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const float e = fast_exp2(__builtin_fmaf(s[mb][r], c, -mc));
          s[mb][r] = e;
          sum += e;
        }
      l_run = l_run * alpha + sum;
      m_run = m_new;
      if (__any(alpha != 1.f)) {      // once the running maxima have settled no lane rescales any more
#pragma unroll
        for (int db = 0; db < DB; ++db)
#pragma unroll
          for (int r = 0; r < 16; ++r) acc_o[db][r] *= alpha;
      }
      __builtin_amdgcn_sched_barrier(0);
      // ---- O^T += V^T P^T: four groups of 16 keys, the next group's fragments requested before this one's products
      static_for<4>([&](auto qc) {
        constexpr int q = decltype(qc)::value, mb = q / 2, s2 = q % 2;
        if constexpr (q < 3) req_v(std::integral_constant<int, q + 1>{});
        wait_lgkm<(q < 3 ? 2 * DB : 0)>();
        __builtin_amdgcn_sched_barrier(0);
        float tmp[8];
#pragma unroll
        for (int j = 0; j < 8; ++j) tmp[j] = s[mb][8 * s2 + j];
        const u32x4_t pf = __builtin_bit_cast(u32x4_t, attn_pack8(tmp));
#pragma unroll
        for (int db = 0; db < DB; ++db) acc_o[db] = attn_mfma(attn_settle_tr(vq[q % 2][db]), pf, acc_o[db]);
        __builtin_amdgcn_sched_barrier(0);
      });
    }
    FGRPO_WAIT_VMCNT(0);            // this wavefront's part of the next tile is in LDS
    wait_lgkm<0>();
    wg_barrier();
  };
  for (int kb = k_begin; kb < k_end; kb += 2 * kAttnBK) {
    step(std::integral_constant<int, 0>{}, kb);
    if (kb + kAttnBK < k_end) step(std::integral_constant<int, 1>{}, kb + kAttnBK);
  }
  float l_lo, l_hi;
  attn_halves(l_run, l_lo, l_hi);
  const float l = l_lo + l_hi;
  if (valid) {
    const float inv = l > 0.f ? 1.f / l : 0.f;
    attn_store_rowmajor(acc_o, inv, p.out + ((long long)tq * p.Hq + hq) * kHD, h);
    if (h == 0) p.lse[(long long)hq * p.T + tq] = l > 0.f ? m_run * p.scale + __logf(l) : -INFINITY;
  }
}

// dQ in the same form (see varlen_attn_fwd2_kernel).  A 64-key step runs as six phases of eight matrix instructions
// with the vector arithmetic of one 32-key half placed behind the matrix instructions of the other (see the step);
// row fragments arrive in groups of four k steps, two groups in flight, the K^T fragments of the dQ products a
// phase ahead.
template <int HD, int HB>
__global__ __launch_bounds__(256, 2) void varlen_attn_dq2_kernel(AttnParams p) {
  constexpr int KS = HD / 16, DB = HD / 32, kAttnTile = kAttnBK * HD * 2, kHD = HD;
  __shared__ __attribute__((aligned(16))) char smem[4 * kAttnTile];      // [buffer][K | V]
  const uint32_t lds0 = lds_addr(smem);
  const int lane = threadIdx.x & 63, h = lane >> 5;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  AttnLane<HD> L = attn_lane<HD>(lane);      // + the LDS base: a fragment address is one of these plus a constant
#pragma unroll
  for (int st = 0; st < KS; ++st) L.rowc[st] += (int)lds0;
#pragma unroll
  for (int db = 0; db < DB; ++db) L.tr[db][0] += (int)lds0, L.tr[db][1] += (int)lds0;
  // work-group -> (tile, K/V head, query heads): as in varlen_attn_dq_kernel
  constexpr int WPH = 4 / HB, RB = 32 * WPH;
  const int G = p.Hq / p.Hkv, NB = (G + HB - 1) / HB;
  const int xcd = blockIdx.x & 7, slot = blockIdx.x >> 3;
  const int unit = (slot / NB) * 8 + xcd;
  const int ntile = (p.T + RB - 1) / RB;
  if (unit >= ntile * p.Hkv) return;
  const int hkv = unit % p.Hkv;
  const int head_g = (slot % NB) * HB + wave / WPH;
  const bool head_ok = head_g < G;
  const int hq = hkv * G + (head_ok ? head_g : G - 1);
  const int q0 = min(max(p.order_q[unit / p.Hkv], 0), ntile - 1) * RB;
  const int tq = q0 + 32 * (wave % WPH) + (lane & 31);
  const bool valid = head_ok && tq < p.T;
  const int lo = valid ? p.seg_start[tq] : 1;
  const int hi = valid ? (p.causal ? tq : p.seg_end[tq] - 1) : 0;
  const int last = (q0 + RB - 1 < p.T ? q0 + RB - 1 : p.T - 1);
  const int k_begin = max(__builtin_amdgcn_readfirstlane(p.seg_start[q0]), 0);
  const int k_end = min(__builtin_amdgcn_readfirstlane(p.causal ? last + 1 : p.seg_end[last]), p.T);
  const int wfirst = q0 + 32 * (wave % WPH), wlast = (wfirst + 31 < p.T ? wfirst + 31 : p.T - 1);
  const bool wave_on = head_ok && wfirst < p.T;
  const int w_lo = wave_on ? p.seg_start[wfirst] : 1;
  const int w_hi = wave_on ? (p.causal ? wlast : p.seg_end[wlast] - 1) : 0;
  const bool wave_full = wave_on && wfirst + 31 < p.T;
  const int w_lo_max = wave_full ? p.seg_start[wlast] : 0x7fffffff;
  const int w_hi_min = wave_full ? (p.causal ? wfirst : p.seg_end[wfirst] - 1) : -1;

  bf16x8_t qf[KS], dof[KS];
  attn_row_operand(qf, p.q + (long long)(valid ? tq : 0) * p.q_st + (long long)hq * p.q_sh, valid, h);
  attn_row_operand(dof, p.dout + ((long long)(valid ? tq : 0) * p.Hq + hq) * kHD, valid, h);
  const float lse2 = valid ? p.lse[(long long)hq * p.T + tq] * kLog2e : 0.f;
  // delta = rowsum(dO * O) of the lane's query: each lane half holds alternate 8-element pieces of the row
  float dl = 0.f;
  {
    bf16x8_t of[KS];
    attn_row_operand(of, p.out_fwd + ((long long)(valid ? tq : 0) * p.Hq + hq) * kHD, valid, h);
#pragma unroll
    for (int st = 0; st < KS; ++st) {
      const u32x4_t x = __builtin_bit_cast(u32x4_t, dof[st]), y = __builtin_bit_cast(u32x4_t, of[st]);
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        dl += __uint_as_float(x[i] << 16) * __uint_as_float(y[i] << 16);
        dl += __uint_as_float(x[i] & 0xffff0000u) * __uint_as_float(y[i] & 0xffff0000u);
      }
    }
    dl += attn_swap32(dl);
    if (valid && h == 0) p.delta[(long long)hq * p.T + tq] = dl;    // for the dK/dV kernel, launched after this one
  }
  const float c = p.scale * kLog2e;
#pragma unroll
  for (int st = 0; st < KS; ++st) asm volatile("" : "+v"(qf[st]), "+v"(dof[st]));     // complete before the loop
  // finite also for a query that sees no key at all (lse = -inf; every pair of such a query is hidden and gets its
  // zero from the score, see hide() below): -inf * c + inf would be a NaN
  float lse2_v = lse2 == -INFINITY ? 0.f : lse2;
  asm volatile("" : "+v"(lse2_v));

  f32x16_t acc[DB];
#pragma unroll
  for (int db = 0; db < DB; ++db)
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[db][r] = 0.f;

  const bf16_t* kbase = p.k + (long long)hkv * p.k_sh;
  const bf16_t* vbase = p.v + (long long)hkv * p.v_sh;
  const uint32_t fko = attn_dma_lane_offset<HD>(wave, lane, p.k_st), fvo = attn_dma_lane_offset<HD>(wave, lane, p.v_st);
  AttnTileCursor<HD> ck, cv;               // the tile the next fetch brings: the steps are fetched in order
  ck.init(kbase, p.k_st, k_begin, k_end);
  cv.init(vbase, p.v_st, k_begin, k_end);
  auto fetch = [&](int buf) {
    char* t = smem + buf * 2 * kAttnTile + wave * 1024;
    ck.load(p.k_st, fko, t);
    cv.load(p.v_st, fvo, t + kAttnTile);
    ck.next();
    cv.next();
  };
  if (k_begin < k_end) fetch(0);
  FGRPO_WAIT_VMCNT(0);
  wg_barrier();
  // a step on LDS buffer `cur`, a compile-time constant: buffer, tile and block are the instruction's offset field
  auto step = [&](auto curc, int kb) {
    constexpr int cur = decltype(curc)::value, kt = cur * 2 * kAttnTile, vt = kt + kAttnTile;
    if (kb + kAttnBK < k_end) fetch(cur ^ 1);     // the next step's tiles; that buffer was last read a step ago, before the barrier
    if (wave_on && kb <= w_hi && kb + kAttnBK > w_lo) {
      const bool all_vis = kb >= w_lo_max && kb + kAttnBK - 1 <= w_hi_min;       // every pair of this step is visible
      // The two 32-key halves of the step as a software pipeline in which the vector arithmetic of a half runs in
      // the shadow of matrix instructions (a 32x32x16 instruction keeps the matrix pipe busy for 32 cycles and the
      // issue port for about 8: four or five vector instructions fit behind each one for free, whereas a wavefront
      // that alternates long runs of the two kinds leaves the pipe idle during its arithmetic).  Eight matrix
      // instructions a phase:
      //   S(0) | dP(0) + E(0) | S(1) + F(0) | dP(1) + E(1) | Z(0) + F(1) | Z(1)
      // S, dP = the score products of a half, E = P = exp2(S c - lse) of its 16 elements, F = dS = P (dP - delta)
      // and the bf16 operand, Z = dQ += dS K.  Every product and every sum is the one the half-by-half order
      // computes, in the same order.
      {
        constexpr int GR = KS / 2;            // k steps (= LDS reads) of a group of row fragments: two groups a product, two in flight
        u32x4_t fr[2][GR];
        AttnTr kq[2][DB];
        f32x16_t sc[2], dp[2];
#pragma unroll
        for (int mb = 0; mb < 2; ++mb)
#pragma unroll
          for (int r = 0; r < 16; ++r) sc[mb][r] = dp[mb][r] = 0.f;
        auto fence = []() { __builtin_amdgcn_sched_barrier(0); };
        // group n = 0 .. 7 of the row fragments: product n / 2 (S(0), dP(0), S(1), dP(1)), k steps GR (n % 2) ..
        auto req_g = [&](auto nc) {
          constexpr int n = decltype(nc)::value, prod = n / 2, mb = prod / 2, tile = (prod % 2 == 0 ? kt : vt);
          static_for<GR>([&](auto ic) {
            constexpr int i = decltype(ic)::value, st = GR * (n % 2) + i;
            fr[n % 2][i] = lds_read_u128_asm<tile + mb * 32 * HD * 2>((uint32_t)L.rowc[st]);
          });
        };
        auto req_t = [&](auto mbc, auto s2c) {          // K^T fragments of keys 32 mb + 16 s2 .., every 32-column block
          constexpr int mb = decltype(mbc)::value, s2 = decltype(s2c)::value;
          static_for<DB>([&](auto dc) {
            constexpr int db = decltype(dc)::value;
            kq[s2][db] = attn_rd_tr_asm<kt + (32 * mb + 16 * s2) * HD * 2>((uint32_t)L.tr[db][0], (uint32_t)L.tr[db][1]);
          });
        };
        auto e_el = [&](auto mbc, auto rc) {             // P in place of S
          constexpr int mb = decltype(mbc)::value, r = decltype(rc)::value;
          sc[mb][r] = fast_exp2(__builtin_fmaf(sc[mb][r], c, -lse2_v));
          asm volatile("" : "+v"(sc[mb][r]));      // computed here, behind its matrix instruction: not where the value is next used
        };
        // a step with hidden pairs: their scores become -inf between the S and the E phase (exp2 then gives the
        // exact zero the select in front of the exponential gives: lse2_v is finite and the scale positive, which the
        // host checks).  A branch of its own around
        // sixteen selects: one around a whole phase costs copies of the accumulators it merges.
        auto hide = [&](auto mbc) {
          constexpr int mb = decltype(mbc)::value;
#pragma unroll
          for (int r = 0; r < 16; ++r) {
            const int key = kb + 32 * mb + 8 * (r >> 2) + 4 * h + (r & 3);
            sc[mb][r] = ((int)(key >= lo) & (int)(key <= hi)) ? sc[mb][r] : -INFINITY;
          }
        };
        auto f_el = [&](auto mbc, auto rc) {             // dS in place of P
          constexpr int mb = decltype(mbc)::value, r = decltype(rc)::value;
          sc[mb][r] = sc[mb][r] * (dp[mb][r] - dl);
          asm volatile("" : "+v"(sc[mb][r]));
        };
        u32x4_t dsf[2][2];
        auto pack = [&](auto mbc, auto s2c) {
          constexpr int mb = decltype(mbc)::value, s2 = decltype(s2c)::value;
          float tmp[8];
#pragma unroll
          for (int j = 0; j < 8; ++j) tmp[j] = sc[mb][8 * s2 + j];
          dsf[mb][s2] = __builtin_bit_cast(u32x4_t, attn_pack8(tmp));
        };
        // the GR matrix instructions of group n; behind instruction i the vector work side(i)
        auto mma_g = [&](auto nc, auto&& side) {
          constexpr int n = decltype(nc)::value, prod = n / 2, mb = prod / 2;
          static_for<GR>([&](auto ic) {
            constexpr int i = decltype(ic)::value, st = GR * (n % 2) + i;
            attn_settle(fr[n % 2][i]);
            if constexpr (prod % 2 == 0) sc[mb] = attn_mfma(fr[n % 2][i], __builtin_bit_cast(u32x4_t, qf[st]), sc[mb]);
            else dp[mb] = attn_mfma(fr[n % 2][i], __builtin_bit_cast(u32x4_t, dof[st]), dp[mb]);
            fence();       // the matrix instruction first: the vector work then runs while the pipe is busy
            side(ic);
            fence();
          });
        };
        using I0 = std::integral_constant<int, 0>;
        using I1 = std::integral_constant<int, 1>;
        constexpr int EPI = 8 / GR;            // elements behind one matrix instruction: a group covers eight
        auto none = [](auto) {};
        auto side_e = [&](auto mbc, auto halfc) {        // E of elements 8 half .. 8 half + 7
          return [&, mbc, halfc](auto ic) {
            static_for<EPI>([&](auto jc) { e_el(mbc, std::integral_constant<int, 8 * decltype(halfc)::value + EPI * decltype(ic)::value + decltype(jc)::value>{}); });
          };
        };
        auto side_f = [&](auto mbc, auto halfc) {
          return [&, mbc, halfc](auto ic) {
            static_for<EPI>([&](auto jc) { f_el(mbc, std::integral_constant<int, 8 * decltype(halfc)::value + EPI * decltype(ic)::value + decltype(jc)::value>{}); });
          };
        };
        // ---- S(0)
        req_g(std::integral_constant<int, 0>{});
        req_g(std::integral_constant<int, 1>{});
        wait_lgkm<GR>();
        fence();
        mma_g(std::integral_constant<int, 0>{}, none);
        req_g(std::integral_constant<int, 2>{});
        wait_lgkm<GR>();
        fence();
        mma_g(std::integral_constant<int, 1>{}, none);
        // ---- dP(0) + E(0)
        req_g(std::integral_constant<int, 3>{});
        if (!all_vis) hide(I0{});
        wait_lgkm<GR>();
        fence();
        mma_g(std::integral_constant<int, 2>{}, side_e(I0{}, I0{}));
        req_g(std::integral_constant<int, 4>{});
        wait_lgkm<GR>();
        fence();
        mma_g(std::integral_constant<int, 3>{}, side_e(I0{}, I1{}));
        // ---- S(1) + F(0)
        req_g(std::integral_constant<int, 5>{});
        wait_lgkm<GR>();
        fence();
        mma_g(std::integral_constant<int, 4>{}, side_f(I0{}, I0{}));
        pack(I0{}, I0{});
        req_g(std::integral_constant<int, 6>{});
        wait_lgkm<GR>();
        fence();
        mma_g(std::integral_constant<int, 5>{}, side_f(I0{}, I1{}));
        pack(I0{}, I1{});
        // ---- dP(1) + E(1)
        req_g(std::integral_constant<int, 7>{});
        if (!all_vis) hide(I1{});
        wait_lgkm<GR>();
        fence();
        mma_g(std::integral_constant<int, 6>{}, side_e(I1{}, I0{}));
        req_t(I0{}, I0{});
        wait_lgkm<2 * DB>();
        fence();
        mma_g(std::integral_constant<int, 7>{}, side_e(I1{}, I1{}));
        // ---- Z(0) + F(1): two elements behind each matrix instruction
        req_t(I0{}, I1{});
        static_for<2>([&](auto s2c) {
          constexpr int s2 = decltype(s2c)::value;
          wait_lgkm<(s2 == 0 ? 2 * DB : 0)>();
          fence();
          static_for<DB>([&](auto dc) {
            constexpr int db = decltype(dc)::value;
            acc[db] = attn_mfma(attn_settle_tr(kq[s2][db]), dsf[0][s2], acc[db]);
            fence();
            static_for<8 / DB>([&](auto jc) { f_el(I1{}, std::integral_constant<int, 8 * s2 + (8 / DB) * db + decltype(jc)::value>{}); });
            fence();
          });
          pack(I1{}, s2c);
          req_t(I1{}, s2c);
        });
        // ---- Z(1)
        static_for<2>([&](auto s2c) {
          constexpr int s2 = decltype(s2c)::value;
          wait_lgkm<(s2 == 0 ? 2 * DB : 0)>();
          fence();
#pragma unroll
          for (int db = 0; db < DB; ++db) acc[db] = attn_mfma(attn_settle_tr(kq[s2][db]), dsf[1][s2], acc[db]);
          fence();
        });
      }
    }
    FGRPO_WAIT_VMCNT(0);            // this wavefront's part of the next tile is in LDS
    wait_lgkm<0>();
    wg_barrier();
  };
  for (int kb = k_begin; kb < k_end; kb += 2 * kAttnBK) {
    step(std::integral_constant<int, 0>{}, kb);
    if (kb + kAttnBK < k_end) step(std::integral_constant<int, 1>{}, kb + kAttnBK);
  }
  if (valid) attn_store_rowmajor(acc, p.scale, p.dq + ((long long)tq * p.Hq + hq) * kHD, h);   // dS was kept / scale
}

// seg_start[t], seg_end[t] from cu_seqlens (tokens outside every segment stand alone)
__global__ void segment_bounds_kernel(const int* cu, int nseq, int T, int* seg_start, int* seg_end) {
  const int t = blockIdx.x * blockDim.x + threadIdx.x;
  if (t >= T) return;
  // largest i with cu[i] <= t
  int a = 0, b = nseq;   // invariant: answer in [a, b] if cu[0] <= t
  if (nseq <= 0 || t < cu[0] || t >= cu[nseq]) {
    seg_start[t] = t;
    seg_end[t] = t + 1;
    return;
  }
  while (a < b) {
    const int mid = (a + b + 1) >> 1;
    if (cu[mid] <= t) a = mid; else b = mid - 1;
  }
  // cu[a] <= t < cu[a+1] (empty segments share a start and are skipped by taking the largest i)
  int e = a + 1;
  while (e < nseq && cu[e] <= t) ++e;
  seg_start[t] = cu[a] > 0 ? cu[a] : 0;
  seg_end[t] = cu[e] < T ? cu[e] : T;
}

// Work-group start order: tiles sorted by the number of steps they will walk, most first (ties by index), so that
// the long tiles of long segments do not end up alone at the tail of the launch.  Four lists, one work-group of
// 1024 threads per eighth of a list: key tiles of 128 tokens, query tiles of 128, 64 and 32 tokens.  Rank by counting
// (n <= kAttnMaxSorted tiles), otherwise the plain guess (late query tiles / early key tiles first).
// Layout behind the 2*T per-token bounds: order_k [c128], order_q128 [c128], order_q64 [c64], order_q32 [c32],
// cX = ceil(T / X).
constexpr int kAttnMaxSorted = 2048;
__host__ __device__ inline long long attn_order_offset(int T, int list) {     // list 0: keys; 1, 2, 3: queries 128 / 64 / 32
  const long long c128 = (T + 127) / 128, c64 = (T + 63) / 64;
  return 2LL * T + (list == 0 ? 0 : list == 1 ? c128 : list == 2 ? 2 * c128 : 2 * c128 + c64);
}
__host__ __device__ inline long long attn_bounds_elems(int T) { return attn_order_offset(T, 3) + (T + 31) / 32; }

constexpr int kAttnOrderSlices = 8;      // work-groups per list: each ranks 1/8 of the list's tiles
__global__ void attn_tile_order_kernel(const int* seg_start, const int* seg_end, int T, int causal, int* ws) {
  __shared__ int wk[kAttnMaxSorted], rk[kAttnMaxSorted / kAttnOrderSlices];
  const int list = blockIdx.x;                       // 0: keys; 1, 2, 3: queries 128 / 64 / 32
  const bool keys = list == 0;
  const int ts = list <= 1 ? 128 : list == 2 ? 64 : 32;
  int* order = ws + attn_order_offset(T, list);
  const int n = (T + ts - 1) / ts;
  const int per = (n + kAttnOrderSlices - 1) / kAttnOrderSlices;
  const int t0 = blockIdx.y * per, t1 = (t0 + per < n ? t0 + per : n), m = t1 - t0;
  if (m <= 0) return;
  if (n > kAttnMaxSorted) {
    for (int t = t0 + threadIdx.x; t < t1; t += blockDim.x) order[t] = keys ? t : n - 1 - t;
    return;
  }
  for (int t = threadIdx.x; t < n; t += blockDim.x) {
    const int first = t * ts, last = (first + ts - 1 < T ? first + ts - 1 : T - 1);
    wk[t] = keys ? seg_end[last] - (causal ? first : seg_start[first])            // queries a key tile walks
                 : (causal ? last + 1 : seg_end[last]) - seg_start[first];        // keys a query tile walks
  }
  for (int t = threadIdx.x; t < m; t += blockDim.x) rk[t] = 0;
  __syncthreads();
  // rank by counting, `parts` threads per tile of this slice, each scanning 1/parts of the whole list
  const int parts = (int)blockDim.x / m > 1 ? (int)blockDim.x / m : 1;
  const int span = (n + parts - 1) / parts;
  for (int w = threadIdx.x; w < m * parts; w += blockDim.x) {
    const int t = t0 + w / parts, u0 = (w % parts) * span, u1 = (u0 + span < n ? u0 + span : n);
    const int a = wk[t];
    int r = 0;
    for (int u = u0; u < u1; ++u) {
      const int x = wk[u];
      r += (x > a) | ((x == a) & (u < t));
    }
    atomicAdd(&rk[t - t0], r);       // integer counts: the order of the additions does not matter
  }
  __syncthreads();
  for (int t = threadIdx.x; t < m; t += blockDim.x) order[rk[t]] = t0 + t;
}

}  // namespace fgrpo
