// bf16 "NT" GEMM main loop for gfx950 (CDNA4): D[m,n] = sum_k A[m,k] * B[n,k].
//
// Both operands are row-major with the contraction index contiguous, which is
// the layout v_mfma_f32_32x32x16_bf16 wants from a 16-byte LDS read: lane l
// supplies row (l % 32) and the eight k values 8*(l/32) .. 8*(l/32)+7.
//
// Work-group tile BM x BN, K step BK, WM x WN wavefronts (64 lanes each), every
// wavefront owning a (BM/WM) x (BN/WN) sub-tile made of 32x32 MFMA blocks kept
// in fp32 accumulators.  Global -> register -> LDS staging with NSTAGE LDS
// buffers: the loads of K step kt+1 are in flight while step kt is multiplied.
// LDS rows are padded by 16 bytes so that the 16-byte fragment reads of 8 or 16
// consecutive rows fall into distinct bank groups.
//
// A contraction may be the sum of up to three (A_s, B_s, K_s) segments sharing
// the leading dimensions; the fp32 path uses that for the bf16 hi/lo split
// a*b ~= a_hi*b_hi + a_hi*b_lo + a_lo*b_hi.
//
// Contract checked by the host launchers: every K_s is a positive multiple of
// BK, every operand base is 16-byte aligned, lda/ldb are multiples of 8
// elements, rows past M (or N) are never read (row indices are clamped) and a
// tile's rows span less than 4 GiB.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace fgrpo {

typedef uint16_t bf16_t;  // storage type of a bfloat16
typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8_t;
typedef __attribute__((__vector_size__(16 * sizeof(float)))) float f32x16_t;
typedef __attribute__((__vector_size__(4 * sizeof(uint32_t)))) uint32_t u32x4_t;  // one 16-byte chunk

struct GemmSeg {
  const bf16_t* A;
  const bf16_t* B;
  int K;
};

struct GemmOperands {
  GemmSeg seg[3];
  int nseg;
  long long lda, ldb;  // elements
  int M, N;
};

template <int BM_, int BN_, int BK_, int WM_, int WN_, int OCC_>
struct TileCfg {
  static constexpr int BM = BM_, BN = BN_, BK = BK_, WM = WM_, WN = WN_, OCC = OCC_;
  static constexpr int NT = WM * WN * 64;       // threads per work-group
  static constexpr int WTM = BM / WM;           // wavefront tile rows
  static constexpr int WTN = BN / WN;           // wavefront tile cols
  static constexpr int TM = WTM / 32;           // 32x32 blocks per wavefront, rows
  static constexpr int TN = WTN / 32;           // 32x32 blocks per wavefront, cols
  static constexpr int CPR = BK / 8;            // 16-byte chunks per tile row
  static constexpr int RPP = NT / CPR;          // tile rows covered by one load pass
  static constexpr int PA = BM / RPP;           // load passes for A
  static constexpr int PB = BN / RPP;           // load passes for B
  static constexpr int ROWB = BK * 2 + 16;      // padded LDS row, bytes
  static constexpr int STAGE = (BM + BN) * ROWB;
  static constexpr int NSTAGE = 2;
  static constexpr int LDS_BYTES = STAGE * NSTAGE;
  static_assert(BM % (WM * 32) == 0 && BN % (WN * 32) == 0, "tile/wave shape");
  static_assert(BK % 16 == 0 && NT % CPR == 0 && BM % RPP == 0 && BN % RPP == 0, "loader shape");
};

// Accumulator element (i, j, r) of lane `lane` in wavefront (wm, wn) sits at
//   row = wm*WTM + i*32 + 8*(r/4) + 4*(lane/32) + (r%4)
//   col = wn*WTN + j*32 + (lane%32)
// relative to the tile origin.
template <class C>
__device__ __forceinline__ int acc_row(int wm, int i, int r, int lane) {
  return wm * C::WTM + i * 32 + 8 * (r >> 2) + 4 * (lane >> 5) + (r & 3);
}
template <class C>
__device__ __forceinline__ int acc_col(int wn, int j, int lane) {
  return wn * C::WTN + j * 32 + (lane & 31);
}

template <class C>
__device__ __forceinline__ void zero_acc(f32x16_t (&acc)[C::TM][C::TN]) {
#pragma unroll
  for (int i = 0; i < C::TM; ++i)
#pragma unroll
    for (int j = 0; j < C::TN; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;
}

// acc += A[row0 : row0+BM, :] * B[col0 : col0+BN, :]^T over all segments.
// Must be called by every thread of the work-group (it contains barriers).  On
// return all LDS reads have completed and a barrier has been passed, so the
// caller may reuse `smem`.
template <class C>
__device__ __forceinline__ void gemm_mainloop(const GemmOperands& g, int row0, int col0, char* smem,
                                              f32x16_t (&acc)[C::TM][C::TN]) {
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int wm = wave / C::WN, wn = wave % C::WN;
  const int lrow = tid / C::CPR, lchk = tid % C::CPR;

  uint32_t aoff[C::PA], boff[C::PB];
  const int amax = g.M - 1 - row0, bmax = g.N - 1 - col0;
#pragma unroll
  for (int i = 0; i < C::PA; ++i) {
    int r = lrow + i * C::RPP;
    r = r < amax ? r : amax;
    aoff[i] = (uint32_t)((long long)r * g.lda * 2 + lchk * 16);
  }
#pragma unroll
  for (int i = 0; i < C::PB; ++i) {
    int r = lrow + i * C::RPP;
    r = r < bmax ? r : bmax;
    boff[i] = (uint32_t)((long long)r * g.ldb * 2 + lchk * 16);
  }
  // LDS byte offsets of this thread's staging stores and fragment reads.
  const int st_a = lrow * C::ROWB + lchk * 16;
  const int st_b = C::BM * C::ROWB + st_a;
  const int fr_a = (wm * C::WTM + (lane & 31)) * C::ROWB + (lane >> 5) * 16;
  const int fr_b = C::BM * C::ROWB + (wn * C::WTN + (lane & 31)) * C::ROWB + (lane >> 5) * 16;

  for (int s = 0; s < g.nseg; ++s) {
    const char* Ab = (const char*)(g.seg[s].A + (long long)row0 * g.lda);
    const char* Bb = (const char*)(g.seg[s].B + (long long)col0 * g.ldb);
    const int nk = g.seg[s].K / C::BK;

    u32x4_t ra[C::PA], rb[C::PB];
#pragma unroll
    for (int i = 0; i < C::PA; ++i) ra[i] = *(const u32x4_t*)(Ab + aoff[i]);
#pragma unroll
    for (int i = 0; i < C::PB; ++i) rb[i] = *(const u32x4_t*)(Bb + boff[i]);
#pragma unroll
    for (int i = 0; i < C::PA; ++i) *(u32x4_t*)(smem + st_a + i * C::RPP * C::ROWB) = ra[i];
#pragma unroll
    for (int i = 0; i < C::PB; ++i) *(u32x4_t*)(smem + st_b + i * C::RPP * C::ROWB) = rb[i];
    __syncthreads();

    for (int kt = 0; kt < nk; ++kt) {
      const int cur = (kt & 1) * C::STAGE;
      const bool more = (kt + 1 < nk);
      if (more) {
        Ab += C::BK * 2;
        Bb += C::BK * 2;
#pragma unroll
        for (int i = 0; i < C::PA; ++i) ra[i] = *(const u32x4_t*)(Ab + aoff[i]);
#pragma unroll
        for (int i = 0; i < C::PB; ++i) rb[i] = *(const u32x4_t*)(Bb + boff[i]);
      }
#pragma unroll
      for (int kk = 0; kk < C::BK / 16; ++kk) {
        bf16x8_t af[C::TM], bf[C::TN];
#pragma unroll
        for (int i = 0; i < C::TM; ++i)
          af[i] = *(const bf16x8_t*)(smem + cur + fr_a + i * 32 * C::ROWB + kk * 32);
#pragma unroll
        for (int j = 0; j < C::TN; ++j)
          bf[j] = *(const bf16x8_t*)(smem + cur + fr_b + j * 32 * C::ROWB + kk * 32);
#pragma unroll
        for (int i = 0; i < C::TM; ++i)
#pragma unroll
          for (int j = 0; j < C::TN; ++j)
            acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(af[i], bf[j], acc[i][j], 0, 0, 0);
      }
      if (more) {
        const int nxt = C::STAGE - cur;
#pragma unroll
        for (int i = 0; i < C::PA; ++i) *(u32x4_t*)(smem + nxt + st_a + i * C::RPP * C::ROWB) = ra[i];
#pragma unroll
        for (int i = 0; i < C::PB; ++i) *(u32x4_t*)(smem + nxt + st_b + i * C::RPP * C::ROWB) = rb[i];
      }
      __syncthreads();
    }
  }
}

// Work-groups are handed to the 8 XCDs round-robin (block b runs on XCD b % 8)
// and each XCD has a private L2.  Remap so that every XCD walks one contiguous
// range of logical tile ids; neighbouring logical ids share operand panels.
__device__ __forceinline__ int xcd_contiguous_id(int bid, int nblocks) {
  const int q = nblocks >> 3, rem = nblocks & 7;
  const int xcd = bid & 7, idx = bid >> 3;
  return xcd * q + (xcd < rem ? xcd : rem) + idx;
}

}  // namespace fgrpo
