// bf16 GEMM main loops for gfx950 (CDNA4): D[m,n] = sum_k A[m,k] * B[n,k] on v_mfma_f32_32x32x16_bf16
// (lane l supplies row l % 32 and the eight k values 8*(l/32) .. 8*(l/32)+7 of each operand) or, on the
// 8-wavefront 256x256x64 tile every large problem takes (kMi16 below), on v_mfma_f32_16x16x32_bf16
// (lane l supplies row l % 16 and the eight k values 8*(l/16) .. 8*(l/16)+7).
//
// Work-group tile BM x BN, K step BK, WM x WN wavefronts (64 lanes each), every wavefront owning a
// (BM/WM) x (BN/WN) sub-tile made of 32x32 MFMA blocks kept in fp32 accumulators.  Four loops, chosen by the
// tile configuration (run_mainloop) or by the caller:
//   gemm_mainloop      global -> registers -> LDS, padded LDS rows, two buffers (small tiles, fp32 split path);
//   gemm_mainloop_dma  global -> LDS directly (buffer_load ... lds), swizzled LDS rows; with two buffers it runs
//                      the early-barrier schedule below (the default for large problems), with three a plain
//                      prefetch loop;
//   gemm_mainloop_la   direct-to-LDS with four or more BK=32 buffers and one K step of fragment look-ahead;
//   gemm_mainloop_km   operands whose contraction index is the ROW index as stored (read through
//                      ds_read_b64_tr_b16), early-barrier schedule.
// Operands are K-contiguous (X[m][k]) unless a loop says otherwise.
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
#include <type_traits>
#include <utility>

// Every fragment read must stay consumed by an MFMA: the two-buffer loops issue their LDS reads as inline
// assembly, and a read whose result is dead lets the register allocator reuse its destination while the
// data is still in flight (a build that dropped the MFMAs corrupted load addresses that way).
#define FGRPO_MFMA(a, b, c) __builtin_amdgcn_mfma_f32_32x32x16_bf16((a), (b), (c), 0, 0, 0)

#define FGRPO_LDFRAG(ptr) (*(const bf16x8_t*)(ptr))

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
  // K-major operands only (gemm_mainloop_km): rows k >= ka_valid / kb_valid do not exist in memory
  // and read as zero (buffer bounds).  0 = every row of K exists.
  int ka_valid, kb_valid;
  // Column-blocked A (direct-to-LDS two/three-buffer loops and gemm_mainloop_km only): when a_blk != 0 the
  // logical matrix X[r][c] (r = row as stored, c = contiguous index) is kept as 256-column blocks,
  // X[r][c] at A + (c / 256) * a_blk + r * 256 + (c % 256) elements (lda must be 256).  A tile that walks
  // down the rows of one block (K-major use) then reads one sequential stream, and a tile that walks along
  // the columns (K-contiguous use) reads 128 KiB contiguous pieces.
  long long a_blk;
  // gemm_mainloop_km with a K-major A only: the contraction may skip whole K steps (64 rows each) that
  // are known to contribute nothing.  k_runs (device memory, written by an earlier launch on the stream) =
  // {number of runs R, K steps in all runs, start_0 .. start_{kRunCap-1}, end_0 .. end_{kRunCap-1}}: run r covers
  // the K steps start_r <= k < end_r, runs ascending and disjoint.  Null = every K step.
  const int* k_runs;
};
constexpr int kRunCap = 4096;   // runs a k_runs list can hold (more live/dead alternations than that: pass null)

template <int BM_, int BN_, int BK_, int WM_, int WN_, int OCC_, int NST_ = 2, bool DMA_ = false>
struct TileCfg {
  static constexpr int BM = BM_, BN = BN_, BK = BK_, WM = WM_, WN = WN_, OCC = OCC_;
  static constexpr bool DMA = DMA_;             // global -> LDS directly (no register staging)
  static constexpr int NW = WM * WN;            // wavefronts per work-group
  static constexpr int NT = NW * 64;            // threads per work-group
  static constexpr int WTM = BM / WM;           // wavefront tile rows
  static constexpr int WTN = BN / WN;           // wavefront tile cols
  static constexpr int TM = WTM / 32;           // 32x32 blocks per wavefront, rows
  static constexpr int TN = WTN / 32;           // 32x32 blocks per wavefront, cols
  static constexpr int CPR = BK / 8;            // 16-byte chunks per tile row
  static constexpr int RPP = NT / CPR;          // tile rows covered by one load pass of the work-group
  static constexpr int PA = BM / RPP;           // load passes for A (per thread)
  static constexpr int PB = BN / RPP;           // load passes for B (per thread)
  static constexpr int RPI = 64 / CPR;          // tile rows covered by one wavefront-wide 16-byte load
  static constexpr int ROWB = DMA ? BK * 2 : BK * 2 + 16;  // LDS row bytes (register path pads, DMA path swizzles)
  static constexpr int STAGE = (BM + BN) * ROWB;
  static constexpr int NSTAGE = NST_;
  static constexpr int LDS_BYTES = STAGE * NSTAGE;
  static_assert(BM % (WM * 32) == 0 && BN % (WN * 32) == 0, "tile/wave shape");
  static_assert(BK % 16 == 0 && NT % CPR == 0 && BM % RPP == 0 && BN % RPP == 0, "loader shape");
  static_assert(!DMA || (CPR == 4 || CPR == 8), "DMA path supports BK = 32 or 64");
  static_assert(LDS_BYTES <= 160 * 1024, "LDS budget");
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

// The 256x256x64 two-buffer direct-to-LDS loops of the 8-wavefront tile can run on v_mfma_f32_16x16x32_bf16 instead
// of 32x32x16 (kMi16): same flops per cycle, half the fp32 accumulator registers read and written per flop - on this
// power-limited part the same kernels run 5 % faster with it.  A 32x32 block (i, j) of a wavefront is then four
// 16x16 blocks (rh, ch), each one MFMA per 32-wide K slice, and the block's sixteen accumulator registers are
//   element e = 4*(2*rh + ch) + r :  row = wm*WTM + i*32 + 16*rh + 4*(lane/16) + r
//                                   col = wn*WTN + j*32 + 16*ch + (lane%16)
// relative to the tile origin.
template <class C>
constexpr bool kMi16 = C::DMA && C::NSTAGE == 2 && C::NW == 8 && C::BK == 64 && C::TM == 4 && C::TN == 2;
template <class C>
__device__ __forceinline__ int acc16_row(int wm, int i, int e, int lane) {
  return wm * C::WTM + i * 32 + 16 * (e >> 3) + 4 * (lane >> 4) + (e & 3);
}
template <class C>
__device__ __forceinline__ int acc16_col(int wn, int j, int e, int lane) {
  return wn * C::WTN + j * 32 + 16 * ((e >> 2) & 1) + (lane & 15);
}
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float f32x4_t;
// acc<registers 4Q .. 4Q+3> += a (16 rows x 32 k) * b (16 columns x 32 k)
template <int Q>
__device__ __forceinline__ void mfma16_slice(bf16x8_t a, bf16x8_t b, f32x16_t& c) {
  f32x4_t t = __builtin_shufflevector(c, c, 4 * Q, 4 * Q + 1, 4 * Q + 2, 4 * Q + 3);
  t = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, t, 0, 0, 0);
  c[4 * Q] = t[0];
  c[4 * Q + 1] = t[1];
  c[4 * Q + 2] = t[2];
  c[4 * Q + 3] = t[3];
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
            acc[i][j] = FGRPO_MFMA(af[i], bf[j], acc[i][j]);
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

// ---------------------------------------------------------------------------
// Direct-to-LDS variant.  global_load_lds_dwordx4 writes lane l's 16 bytes at
// (wave-uniform LDS base) + 16*l, so one wavefront-wide load fills RPI whole
// tile rows of BK*2 bytes without padding.  Bank conflicts of the fragment
// reads are avoided by an XOR swizzle of the 16-byte chunk index with a
// function of the row, applied on the *global* side (each lane fetches the
// chunk that belongs at its LDS slot).  NSTAGE LDS buffers keep NSTAGE-1 K
// steps of loads in flight; completion is tracked with explicit vmcnt waits and
// one s_barrier per K step.
// ---------------------------------------------------------------------------
#define FGRPO_DMA_AUX 0   // cache-policy bits of the direct-to-LDS loads
#define FGRPO_GLOBAL_PTR(p) ((const __attribute__((address_space(1))) void*)(p))
#define FGRPO_LDS_PTR(p) ((__attribute__((address_space(3))) void*)(p))

// Raw buffer descriptor over [base, base + bytes): offsets past `bytes` read as zero.
__device__ __forceinline__ __amdgpu_buffer_rsrc_t make_rsrc(const void* base, uint32_t bytes) {
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(base), 0, (int)bytes, 0x00020000);
}

// s_waitcnt that waits only for the vector-memory counter to drop to n (n < 64).
#define FGRPO_WAIT_VMCNT(n) __builtin_amdgcn_s_waitcnt(((n) & 15) | (7 << 4) | (15 << 8) | (((n) >> 4) << 14))
// same, and also wait for every outstanding LDS read (lgkmcnt = 0)
#define FGRPO_WAIT_VMCNT_LGKM0(n) __builtin_amdgcn_s_waitcnt(((n) & 15) | (7 << 4) | (0 << 8) | (((n) >> 4) << 14))

template <class C, bool MI16 = false>
__device__ __forceinline__ int lds_swizzle(int row) {
  // Chosen with SQ_LDS_BANK_CONFLICT on the real kernels and a read-rate microbenchmark.  32x32x16 fragment read:
  // lane l -> row l%32, chunk l/32 + 2*kk.  16x16x32 fragment read: lane l -> row l%16, chunk l/16 + 4*k2; under the
  // 32-row swizzle these reads run at half rate (two-way conflicts), under row%8 at the full rate.
  if constexpr (C::CPR == 4)
    return (row >> 2) & 3;                       // 64-byte rows
  else if constexpr (MI16)
    return row & 7;                              // 128-byte rows, 16-row fragments
  else
    return (row + ((row >> 3) & 1)) & 7;         // 128-byte rows, 32-row fragments
}

__device__ __forceinline__ void wg_barrier() {
  asm volatile("" ::: "memory");
  __builtin_amdgcn_s_barrier();
  asm volatile("" ::: "memory");
}

// The fragment reads of the two-buffer direct-to-LDS loops are written as inline assembly: for an LDS access it can see, the
// compiler waits (vmcnt) for every direct-to-LDS load in flight, which would serialise the prefetch of the
// next K step behind each fragment read.  The price: the compiler does not count these reads either, so
// the loop waits for them itself (s_waitcnt lgkmcnt(n); LDS operations return in order).
typedef uint32_t u32x2_t __attribute__((ext_vector_type(2)));

__device__ __forceinline__ uint32_t lds_addr(const char* p) {
  return (uint32_t)(uintptr_t)(__attribute__((address_space(3))) const char*)p;
}
template <int OFF0, int OFF1>
__device__ __forceinline__ bf16x8_t lds_read_tr_pair(uint32_t addr) {
  static_assert(OFF0 >= 0 && OFF1 < 65536, "DS offset field");
  u32x2_t lo, hi;
  asm volatile("ds_read_b64_tr_b16 %0, %2 offset:%3\n\tds_read_b64_tr_b16 %1, %2 offset:%4"
               : "=&v"(lo), "=&v"(hi)
               : "v"(addr), "i"(OFF0), "i"(OFF1));
  const u32x4_t v = {lo.x, lo.y, hi.x, hi.y};
  return __builtin_bit_cast(bf16x8_t, v);
}
// 8-byte LDS store the compiler does not see either (an epilogue patch written while direct-to-LDS loads of the
// next tile are in flight would otherwise wait for them)
__device__ __forceinline__ void lds_write_b64_asm(uint32_t addr, uint32_t lo, uint32_t hi) {
  const u32x2_t v = {lo, hi};
  asm volatile("ds_write_b64 %0, %1" : : "v"(addr), "v"(v) : "memory");
}
template <int OFF>
__device__ __forceinline__ bf16x8_t lds_read_b128_asm(uint32_t addr) {
  static_assert(OFF >= 0 && OFF < 65536, "DS offset field");
  u32x4_t v;
  asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(v) : "v"(addr), "i"(OFF));
  return __builtin_bit_cast(bf16x8_t, v);
}

// ---------------------------------------------------------------------------
// Two-buffer schedule shared by the direct-to-LDS loops ("barrier one sub-step early").
// The barrier of step kt sits before its LAST 16-wide sub-step: by then every
// wavefront has its last fragments of buffer `cur` in registers and the loads of
// step kt+1 have landed, so (a) the first fragments of step kt+1 are fetched right
// after the barrier and arrive under the MFMAs of the last sub-step (no LDS
// latency is exposed), and (b) buffer `cur` is free from that point: the loads of
// step kt+2 start into it at once, spread one by one over the MFMA groups of the
// next EB_PHASES sub-steps, which leaves them the rest of the step to land.
//   issue_one(stage, idx): load idx (0 .. LPT-1) of the next K step into `stage`;
//                          idx == LPT-1 also advances the source cursor.
//   load_a/load_b(stage_ptr, block, kk): one MFMA operand from LDS.
// On entry the loads of step 0 have been issued into buffer 0 (if nk_total > 0).
// ---------------------------------------------------------------------------
constexpr int kLoadPhases = 2;   // sub-steps over which one K step's loads are issued (1 and 3 measured slower)
// compile-time loop: f(std::integral_constant<int, 0>{}) ... f(std::integral_constant<int, N-1>{})
template <class F, int... Is>
__device__ __forceinline__ void static_for_impl(F&& f, std::integer_sequence<int, Is...>) {
  (f(std::integral_constant<int, Is>{}), ...);
}
template <int N, class F>
__device__ __forceinline__ void static_for(F&& f) {
  static_for_impl(f, std::make_integer_sequence<int, N>{});
}

//   load_a/load_b(stage_ptr, I, KK): one MFMA operand from LDS (I, KK are std::integral_constant), issued as
//   RA / RB inline-assembly LDS instructions that the compiler does not count: this function places every
//   s_waitcnt lgkmcnt(n) itself (LDS operations return in order).
// The fragments of the following sub-step are requested between the MFMA row groups of the current one, in the
// order a0, b0 .. b(TN-1), a1 .. a(TM-1) (row group 0 needs a0 and every b), so that the LDS sees a steady
// trickle of reads next to the direct-to-LDS stream instead of a burst per sub-step (a burst measured equal or
// slower).
template <int N>
__device__ __forceinline__ void wait_lgkm() {
  static_assert(N >= 0, "wait count");
  __builtin_amdgcn_s_waitcnt(0xC07F | ((N > 15 ? 15 : N) << 8));   // vmcnt / expcnt untouched
}

template <class C, int LPT, int RA, int RB, class IssueOne, class LoadA, class LoadB>
__device__ __forceinline__ void early_barrier_pipeline(int nk_total, char* smem, f32x16_t (&acc)[C::TM][C::TN],
                                                       IssueOne&& issue_one, LoadA&& load_a, LoadB&& load_b) {
  constexpr int KK = C::BK / 16;
  constexpr int TM = C::TM, TN = C::TN, NR = TM + TN;
  static_assert(KK % 2 == 0 && KK >= kLoadPhases + 1, "sub-steps per K step");
  constexpr int NSLOT = kLoadPhases * TM;         // MFMA groups over which one step's loads are spread
  // fragment order and bookkeeping (all compile time)
  struct Ord {
    static constexpr int cum(int i) { return (i * NR + TM - 1) / TM; }  // entries requested before row group i ends.. starts
    static constexpr int instrs(int n) {              // LDS instructions of the first n entries
      int c = 0;
      for (int e = 0; e < n; ++e) c += (e == 0 || e > TN) ? RA : RB;
      return c;
    }
    static constexpr int need(int i) { return i == 0 ? TN : TN + i; }   // last entry row group i waits for
    // instructions that may still be outstanding when row group i starts
    static constexpr int allowed(int i, bool issuing) {
      return instrs(NR) - instrs(need(i) + 1) + (issuing ? instrs(cum(i)) : 0);
    }
  };
  FGRPO_WAIT_VMCNT(0);
  wg_barrier();                                       // step 0 is in buffer 0
  int steps_issued = nk_total > 0 ? 1 : 0;
  bool active = steps_issued < nk_total;              // a step is being loaded
  int tgt = 1;                                        // ... into this buffer
  if (active) {
    ++steps_issued;
    static_for<LPT>([&](auto q) {
      if constexpr (decltype(q)::value * NSLOT / LPT < TM) issue_one(1, decltype(q)::value);  // phase 0's share
    });
  }
  bf16x8_t af[2][TM], bf[2][TN];
  // entry e of the request order, for sub-step KN of the buffer at `base`, into register buffer BUF
  auto request = [&](const char* base, auto ec, auto knc, auto bufc) {
    constexpr int e = decltype(ec)::value, buf = decltype(bufc)::value;
    if constexpr (e == 0)
      af[buf][0] = load_a(base, std::integral_constant<int, 0>{}, knc);
    else if constexpr (e <= TN)
      bf[buf][e - 1] = load_b(base, std::integral_constant<int, e - 1>{}, knc);
    else
      af[buf][e - TN] = load_a(base, std::integral_constant<int, e - TN>{}, knc);
  };
  static_for<NR>([&](auto e) { request(smem, e, std::integral_constant<int, 0>{}, std::integral_constant<int, 0>{}); });
  int cur = 0;
  // One K step.  STEADY: at least two more steps follow, so a next step exists and a further one is always
  // there to be loaded; the body then carries no conditionals at all.
  auto step = [&](int kt, auto steady_c) {
    constexpr bool STEADY = decltype(steady_c)::value;
    const char* st = smem + cur * C::STAGE;
    const char* sn = smem + (cur ^ 1) * C::STAGE;
    const bool next = STEADY || kt + 1 < nk_total;
    static_for<KK>([&](auto kkc) {
      constexpr int kk = decltype(kkc)::value;
      constexpr bool last = (kk == KK - 1);
      constexpr int kn = last ? 0 : kk + 1, nbuf = (kk + 1) & 1;
      const char* src = last ? sn : st;
      const bool issuing = STEADY || !last || next;
      if constexpr (last) {
        if (next) {
          FGRPO_WAIT_VMCNT_LGKM0(0);                  // my loads of step kt+1 landed; my reads of `cur` returned
          wg_barrier();
          active = STEADY || steps_issued < nk_total; // loads of step kt+2 go into the buffer just freed
          tgt = cur;
          if (active) ++steps_issued;
        }
      }
      // phase of the load spreading this sub-step belongs to: 0 = last sub-step, then 1, 2 .. from the top
      constexpr int phase = last ? 0 : kk + 1;
      const bool loads_here = STEADY || (active && phase < kLoadPhases && (phase > 0 || next));
      __builtin_amdgcn_sched_barrier(0);
      static_for<TM>([&](auto ic) {
        constexpr int i = decltype(ic)::value;
        if constexpr (!last) {
          wait_lgkm<Ord::allowed(i, true)>();
        } else {
          if (next) wait_lgkm<Ord::allowed(i, true)>(); else wait_lgkm<Ord::allowed(i, false)>();
        }
        __builtin_amdgcn_sched_barrier(0);
        {
          // the group's fragment requests and loads go BETWEEN its MFMAs (after MFMA j the extras x with
          // x*TN/X == j): an MFMA keeps the matrix pipe busy for 32 cycles but issues in 4, so whatever is
          // issued right behind it is free - what is issued after the last one delays the next group.
          constexpr int R = Ord::cum(i + 1) - Ord::cum(i);
          constexpr int slot = phase * TM + i;
          constexpr int q_lo = (phase < kLoadPhases) ? (slot * LPT + NSLOT - 1) / NSLOT : 0;
          constexpr int q_hi = (phase < kLoadPhases) ? ((slot + 1) * LPT + NSLOT - 1) / NSLOT : 0;   // loads q_lo .. q_hi-1
          constexpr int X = R + (q_hi - q_lo);
          static_for<TN>([&](auto jc) {
            constexpr int j = decltype(jc)::value;
            acc[i][j] = FGRPO_MFMA(af[kk & 1][i], bf[kk & 1][j], acc[i][j]);
            static_for<X>([&](auto xc) {
              constexpr int x = decltype(xc)::value;
              if constexpr (x * TN / (X > 0 ? X : 1) == j) {
                if constexpr (x < R) {
                  if (issuing)
                    request(src, std::integral_constant<int, Ord::cum(i) + x>{}, std::integral_constant<int, kn>{},
                            std::integral_constant<int, nbuf>{});
                } else {
                  if (loads_here) issue_one(tgt, q_lo + (x - R));
                }
              }
            });
            __builtin_amdgcn_sched_barrier(0);
          });
        }
      });
    });
    cur ^= 1;
  };
  int kt = 0;
  for (; kt + 2 < nk_total; ++kt) step(kt, std::true_type{});
  for (; kt < nk_total; ++kt) step(kt, std::false_type{});
  wg_barrier();                                       // LDS may be reused by the caller
}

// The same schedule on 16x16x32 MFMAs (kMi16 tiles: TM = 4, TN = 2, BK = 64).  A K step is still four sub-steps of
// equal length: sub-step kk works on the 32-wide K slice k2 = kk/2 and on the row half rh = kk%2 of every 32x32
// block - 16 MFMAs: for each block row i the fragment a(i, rh) (16 rows x 32 k) against the four fragments
// b(j, ch) (16 columns x 32 k) of the slice.  The b fragments of a slice are fetched once, before its first
// sub-step, and serve both; so the fragment requests alternate between 4 (a only, before an odd sub-step) and
// 8 (a0, the four b, a1 .. a3, before an even one).
//   load_a(stage_ptr, I, KK): fragment a(I, KK % 2) of slice KK / 2;  load_b(stage_ptr, JC, K2): fragment b(JC/2, JC%2).
template <class C, int LPT, int RA, int RB, class IssueOne, class LoadA, class LoadB>
__device__ __forceinline__ void early_barrier_pipeline16(int nk_total, char* smem, f32x16_t (&acc)[C::TM][C::TN],
                                                         IssueOne&& issue_one, LoadA&& load_a, LoadB&& load_b) {
  constexpr int KK = 4;
  constexpr int TM = C::TM, NB = 2 * C::TN;           // a fragments per sub-step, b fragments per K slice
  static_assert(kMi16<C> && C::BK == 64, "16x16x32 schedule: 8-wavefront 256x256x64 tile");
  constexpr int NSLOT = kLoadPhases * TM;
  // request list of a sub-step by its parity P (0: a0, b0 .. b(NB-1), a1 ..; 1: a0 .. a(TM-1)), all compile time
  struct Ord {
    static constexpr int nr(int P) { return P == 0 ? TM + NB : TM; }
    static constexpr int cost(int P, int e) { return P == 0 ? ((e == 0 || e > NB) ? RA : RB) : RA; }
    static constexpr int instrs(int P, int n) {
      int c = 0;
      for (int e = 0; e < n; ++e) c += cost(P, e);
      return c;
    }
    static constexpr int cum(int P, int i) { return (i * nr(P) + TM - 1) / TM; }     // entries requested before row group i starts
    static constexpr int need(int P, int i) { return P == 0 ? (i == 0 ? NB : NB + i) : i; }   // last entry row group i waits for
    // LDS instructions that may still be outstanding when row group i of a sub-step of parity P starts
    static constexpr int allowed(int P, int i, bool issuing) {
      return instrs(P, nr(P)) - instrs(P, need(P, i) + 1) + (issuing ? instrs(1 - P, cum(1 - P, i)) : 0);
    }
  };
  FGRPO_WAIT_VMCNT(0);
  wg_barrier();                                       // step 0 is in buffer 0
  int steps_issued = nk_total > 0 ? 1 : 0;
  bool active = steps_issued < nk_total;              // a step is being loaded
  int tgt = 1;                                        // ... into this buffer
  if (active) {
    ++steps_issued;
    static_for<LPT>([&](auto q) {
      if constexpr (decltype(q)::value * NSLOT / LPT < TM) issue_one(1, decltype(q)::value);  // phase 0's share
    });
  }
  bf16x8_t af[2][TM], bfr[2][NB];
  // entry e of the request list of sub-step KN, read from the buffer at `base`
  auto request = [&](const char* base, auto ec, auto knc) {
    constexpr int e = decltype(ec)::value, kn = decltype(knc)::value;
    if constexpr ((kn & 1) == 1) {
      af[1][e] = load_a(base, ec, knc);
    } else if constexpr (e == 0) {
      af[0][0] = load_a(base, std::integral_constant<int, 0>{}, knc);
    } else if constexpr (e <= NB) {
      bfr[(kn >> 1) & 1][e - 1] = load_b(base, std::integral_constant<int, e - 1>{}, std::integral_constant<int, (kn >> 1)>{});
    } else {
      af[0][e - NB] = load_a(base, std::integral_constant<int, e - NB>{}, knc);
    }
  };
  static_for<Ord::nr(0)>([&](auto e) { request(smem, e, std::integral_constant<int, 0>{}); });
  int cur = 0;
  auto step = [&](int kt, auto steady_c) {
    constexpr bool STEADY = decltype(steady_c)::value;
    const char* st = smem + cur * C::STAGE;
    const char* sn = smem + (cur ^ 1) * C::STAGE;
    const bool next = STEADY || kt + 1 < nk_total;
    static_for<KK>([&](auto kkc) {
      constexpr int kk = decltype(kkc)::value;
      constexpr bool last = (kk == KK - 1);
      constexpr int kn = last ? 0 : kk + 1;
      constexpr int P = kk & 1, k2 = kk >> 1;
      const char* src = last ? sn : st;
      const bool issuing = STEADY || !last || next;
      if constexpr (last) {
        if (next) {
          FGRPO_WAIT_VMCNT_LGKM0(0);                  // my loads of step kt+1 landed; my reads of `cur` returned
          wg_barrier();
          active = STEADY || steps_issued < nk_total; // loads of step kt+2 go into the buffer just freed
          tgt = cur;
          if (active) ++steps_issued;
        }
      }
      constexpr int phase = last ? 0 : kk + 1;
      const bool loads_here = STEADY || (active && phase < kLoadPhases && (phase > 0 || next));
      __builtin_amdgcn_sched_barrier(0);
      static_for<TM>([&](auto ic) {
        constexpr int i = decltype(ic)::value;
        if constexpr (!last) {
          wait_lgkm<Ord::allowed(P, i, true)>();
        } else {
          if (next) wait_lgkm<Ord::allowed(P, i, true)>(); else wait_lgkm<Ord::allowed(P, i, false)>();
        }
        __builtin_amdgcn_sched_barrier(0);
        {
          constexpr int R = Ord::cum(1 - P, i + 1) - Ord::cum(1 - P, i);
          constexpr int slot = phase * TM + i;
          constexpr int q_lo = (phase < kLoadPhases) ? (slot * LPT + NSLOT - 1) / NSLOT : 0;
          constexpr int q_hi = (phase < kLoadPhases) ? ((slot + 1) * LPT + NSLOT - 1) / NSLOT : 0;   // loads q_lo .. q_hi-1
          constexpr int X = R + (q_hi - q_lo);
          static_for<NB>([&](auto jcc) {
            constexpr int jc = decltype(jcc)::value;       // b fragment (j, ch) = (jc / 2, jc % 2)
            mfma16_slice<2 * P + (jc & 1)>(af[P][i], bfr[k2 & 1][jc], acc[i][jc >> 1]);
            static_for<X>([&](auto xc) {
              constexpr int x = decltype(xc)::value;
              if constexpr (x * NB / (X > 0 ? X : 1) == jc) {
                if constexpr (x < R) {
                  if (issuing) request(src, std::integral_constant<int, Ord::cum(1 - P, i) + x>{}, std::integral_constant<int, kn>{});
                } else {
                  if (loads_here) issue_one(tgt, q_lo + (x - R));
                }
              }
            });
            __builtin_amdgcn_sched_barrier(0);
          });
        }
      });
    });
    cur ^= 1;
  };
  int kt = 0;
  for (; kt + 2 < nk_total; ++kt) step(kt, std::true_type{});
  for (; kt < nk_total; ++kt) step(kt, std::false_type{});
  wg_barrier();                                       // LDS may be reused by the caller
}

// MODE 0: the whole contraction.  MODE 2: only issue the loads of K step 0 into buffer 0 and return (the caller
// does something else, e.g. the epilogue of the previous tile, while they fly); MODE 1: the contraction, given that
// a MODE 2 call for the same tile has been made since the last MODE 0/1 call returned.  Modes 1 and 2 exist for
// the two-buffer schedule only (kSplitPrologue).
template <class C>
constexpr bool kSplitPrologue = C::DMA && C::NSTAGE == 2 && (C::BK / 16) % 2 == 0;

template <class C, int MODE = 0, bool MI16 = false>
__device__ __forceinline__ void gemm_mainloop_dma(const GemmOperands& g, int row0, int col0, char* smem,
                                                  f32x16_t (&acc)[C::TM][C::TN]) {
  static_assert(MODE == 0 || kSplitPrologue<C>, "split prologue needs the two-buffer schedule");
  static_assert(!MI16 || kMi16<C>, "16x16x32 MFMAs: 8-wavefront 256x256x64 two-buffer tile only");
  constexpr int D = C::NSTAGE - 1;              // K steps of loads in flight
  constexpr int LPT = C::PA + C::PB;            // loads per thread per K step
  static_assert(D >= 1 && D <= 4 && LPT * (D - 1) < 64, "pipeline depth");
  // The per-lane offsets below are cheap to derive and expensive to keep: a caller that runs this loop once per
  // tile with an epilogue in between would otherwise carry two dozen loop-invariant registers through that
  // epilogue.  The empty asm makes the thread id opaque, so they are recomputed per call.
  int tid = threadIdx.x;
  asm volatile("" : "+v"(tid));
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);   // wavefront-uniform: LDS targets stay scalar
  const int wm = wave / C::WN, wn = wave % C::WN;

  // loader: instruction i of this wavefront covers tile rows (i*NW + wave)*RPI ..
  const int lrow = lane / C::CPR, lpc = lane % C::CPR;
  uint32_t aoff[C::PA], boff[C::PB];
  const int amax = g.M - 1 - row0, bmax = g.N - 1 - col0;
#pragma unroll
  for (int i = 0; i < C::PA; ++i) {
    const int rt = (i * C::NW + wave) * C::RPI + lrow;            // row inside the tile (decides the swizzle)
    const int r = rt < amax ? rt : amax;                          // row actually read
    aoff[i] = (uint32_t)((long long)r * g.lda * 2 + ((lpc ^ lds_swizzle<C, MI16>(rt)) * 16));
  }
#pragma unroll
  for (int i = 0; i < C::PB; ++i) {
    const int rt = (i * C::NW + wave) * C::RPI + lrow;
    const int r = rt < bmax ? rt : bmax;
    boff[i] = (uint32_t)((long long)r * g.ldb * 2 + ((lpc ^ lds_swizzle<C, MI16>(rt)) * 16));
  }
  const int dst_a = wave * C::RPI * C::ROWB;                      // + i * NW*RPI*ROWB, wave-uniform
  const int dst_b = C::BM * C::ROWB + dst_a;
  // fragment reads
  const int sw = lds_swizzle<C>(lane & 31);
  const int fr_a = (wm * C::WTM + (lane & 31)) * C::ROWB;
  const int fr_b = C::BM * C::ROWB + (wn * C::WTN + (lane & 31)) * C::ROWB;
  int fr_c[C::BK / 16];
#pragma unroll
  for (int kk = 0; kk < C::BK / 16; ++kk) fr_c[kk] = ((kk * 2 + (lane >> 5)) ^ sw) * 16;

  int nk_total = 0;
  for (int s = 0; s < g.nseg; ++s) nk_total += g.seg[s].K / C::BK;

  // Issue cursor over (segment, k).  The loads are buffer loads: a 128-bit descriptor per operand (base = first
  // row of the tile in the current segment / column block), the lane's constant byte offset in a VGPR and the
  // running K offset in an SGPR, so that issuing a load costs two scalar instructions and no vector arithmetic.
  int iseg = 0, ileft = g.seg[0].K / C::BK;
  const char* Abase = (const char*)(g.seg[0].A + (long long)row0 * g.lda);
  const char* Bbase = (const char*)(g.seg[0].B + (long long)col0 * g.ldb);
  __amdgpu_buffer_rsrc_t rsa = make_rsrc(Abase, 0xffffffffu);
  __amdgpu_buffer_rsrc_t rsb = make_rsrc(Bbase, 0xffffffffu);
  uint32_t ka = 0, kb = 0;                            // byte offset of the K slice being issued
  // after the last load of a K step: next K slice, next 256-column block of a blocked A, next segment
  constexpr int kStepsPerBlk = 256 / C::BK;
  const long long a_blk_bytes = g.a_blk * 2;
  int ablk_left = kStepsPerBlk;
  auto advance = [&]() {
    ka += C::BK * 2;
    kb += C::BK * 2;
    if (--ablk_left == 0) {
      ablk_left = kStepsPerBlk;
      if (a_blk_bytes != 0) {                          // next column block of A: re-base the descriptor
        Abase += a_blk_bytes;
        rsa = make_rsrc(Abase, 0xffffffffu);
        ka = 0;
      }
    }
    if (--ileft == 0 && iseg + 1 < g.nseg) {
      ++iseg;
      ileft = g.seg[iseg].K / C::BK;
      Abase = (const char*)(g.seg[iseg].A + (long long)row0 * g.lda);
      Bbase = (const char*)(g.seg[iseg].B + (long long)col0 * g.ldb);
      rsa = make_rsrc(Abase, 0xffffffffu);
      rsb = make_rsrc(Bbase, 0xffffffffu);
      ka = kb = 0;
      ablk_left = kStepsPerBlk;
    }
  };
  // One load of the current issue step (idx < PA: operand A, else B); the last one advances the cursor.
  auto issue_one = [&](int stage, int idx) {
    char* base = smem + stage * C::STAGE;
    if (idx < C::PA)
      __builtin_amdgcn_raw_ptr_buffer_load_lds(rsa, FGRPO_LDS_PTR(base + dst_a + idx * C::NW * C::RPI * C::ROWB), 16,
                                               (int)aoff[idx], (int)ka, 0, FGRPO_DMA_AUX);
    else
      __builtin_amdgcn_raw_ptr_buffer_load_lds(rsb, FGRPO_LDS_PTR(base + dst_b + (idx - C::PA) * C::NW * C::RPI * C::ROWB),
                                               16, (int)boff[idx - C::PA], (int)kb, 0, FGRPO_DMA_AUX);
    if (idx == LPT - 1) advance();
  };
  auto issue = [&](int stage) {
#pragma unroll
    for (int i = 0; i < LPT; ++i) issue_one(stage, i);
  };

  int issued = 0;
  if constexpr (MODE == 1) {                    // step 0 is already on its way into buffer 0
    if (nk_total > 0) {
      advance();
      issued = 1;
    }
  } else {
    // loads issued before this call (by the caller's epilogue) must not be mistaken for ours
    FGRPO_WAIT_VMCNT(0);
    for (; issued < D && issued < nk_total; ++issued) issue(issued);
    if constexpr (MODE == 2) return;
  }

  if constexpr (MI16) {
    // 16x16x32 fragments: lane l reads row (l % 16) of a 16-row block and the 16-byte chunk 4*k2 + l/16 of its
    // 64-wide K slice (16 consecutive rows at one chunk index: conflict-free under the same swizzle)
    const int sw16 = lds_swizzle<C, MI16>(lane & 15);
    const int fa16 = (wm * C::WTM + (lane & 15)) * C::ROWB, fb16 = C::BM * C::ROWB + (wn * C::WTN + (lane & 15)) * C::ROWB;
    int fc16[2];
#pragma unroll
    for (int k2 = 0; k2 < 2; ++k2) fc16[k2] = ((4 * k2 + (lane >> 4)) ^ sw16) * 16;
    early_barrier_pipeline16<C, LPT, 1, 1>(
        nk_total, smem, acc, issue_one,
        [&](const char* st, auto i, auto kk) {
          constexpr int kkv = decltype(kk)::value;
          return lds_read_b128_asm<(decltype(i)::value * 32 + 16 * (kkv & 1)) * C::ROWB>(lds_addr(st) + fa16 + fc16[kkv >> 1]);
        },
        [&](const char* st, auto jc, auto k2) {
          constexpr int jcv = decltype(jc)::value;
          return lds_read_b128_asm<((jcv >> 1) * 32 + 16 * (jcv & 1)) * C::ROWB>(lds_addr(st) + fb16 + fc16[decltype(k2)::value]);
        });
    return;
  }
  if constexpr (C::NSTAGE == 2 && (C::BK / 16) % 2 == 0) {
    early_barrier_pipeline<C, LPT, 1, 1>(
        nk_total, smem, acc, issue_one,
        [&](const char* st, auto i, auto kk) {
          return lds_read_b128_asm<decltype(i)::value * 32 * C::ROWB>(lds_addr(st) + fr_a + fr_c[decltype(kk)::value]);
        },
        [&](const char* st, auto j, auto kk) {
          return lds_read_b128_asm<decltype(j)::value * 32 * C::ROWB>(lds_addr(st) + fr_b + fr_c[decltype(kk)::value]);
        });
    return;
  }

  // The loads of a step are interleaved with its MFMAs (a burst right after the barrier would keep
  // every wavefront busy issuing addresses, about 40 cycles per load, before its first MFMA).
  // With three or more LDS buffers they are spread over the whole step; with two buffers over the
  // first half, so that the last one still has half a step to land.
  constexpr int kGroups = (C::BK / 16) * C::TM;                                  // MFMA groups (TN MFMAs each) per step
  constexpr int kSpreadG = (C::NSTAGE >= 3) ? kGroups : (kGroups / 2 > 0 ? kGroups / 2 : 1);
  constexpr int kPer = (LPT + kSpreadG - 1) / kSpreadG;                          // loads after each group
  constexpr bool kSpread = true;
  constexpr int KK = C::BK / 16;

  int cur = 0, nxt = D % C::NSTAGE;
  for (int kt = 0; kt < nk_total; ++kt) {
    const int rem = nk_total - 1 - kt;          // K steps after this one
    // wait until this step's loads have landed: at most min(rem, D-1) younger steps may stay in flight
    if (rem >= D - 1) {
      FGRPO_WAIT_VMCNT(LPT * (D - 1));
    } else if (D >= 3 && rem == 2) {
      FGRPO_WAIT_VMCNT(LPT * 2);
    } else if (D >= 2 && rem == 1) {
      FGRPO_WAIT_VMCNT(LPT * 1);
    } else {
      FGRPO_WAIT_VMCNT(0);
    }
    wg_barrier();   // everyone's part of step kt is in LDS; everyone is done reading step kt-1
    const bool more = issued < nk_total;
    if (more) ++issued;
    if (!kSpread && more) issue(nxt);
    const char* st = smem + cur * C::STAGE;
    bf16x8_t af[2][C::TM], bf[2][C::TN];
#pragma unroll
    for (int i = 0; i < C::TM; ++i) af[0][i] = FGRPO_LDFRAG(st + fr_a + i * 32 * C::ROWB + fr_c[0]);
#pragma unroll
    for (int j = 0; j < C::TN; ++j) bf[0][j] = FGRPO_LDFRAG(st + fr_b + j * 32 * C::ROWB + fr_c[0]);
#pragma unroll
    for (int kk = 0; kk < KK; ++kk) {
      if (kk + 1 < KK) {   // next sub-step's fragments fly while this one multiplies
#pragma unroll
        for (int i = 0; i < C::TM; ++i)
          af[(kk + 1) & 1][i] = FGRPO_LDFRAG(st + fr_a + i * 32 * C::ROWB + fr_c[kk + 1]);
#pragma unroll
        for (int j = 0; j < C::TN; ++j)
          bf[(kk + 1) & 1][j] = FGRPO_LDFRAG(st + fr_b + j * 32 * C::ROWB + fr_c[kk + 1]);
      }
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int i = 0; i < C::TM; ++i) {
#pragma unroll
        for (int j = 0; j < C::TN; ++j) acc[i][j] = FGRPO_MFMA(af[kk & 1][i], bf[kk & 1][j], acc[i][j]);
        if (kSpread && more) {
#pragma unroll
          for (int q = 0; q < kPer; ++q)
            if ((kk * C::TM + i) * kPer + q < LPT) issue_one(nxt, (kk * C::TM + i) * kPer + q);
        }
        __builtin_amdgcn_sched_barrier(0);
      }
    }
    cur = (cur + 1 == C::NSTAGE) ? 0 : cur + 1;
    nxt = (nxt + 1 == C::NSTAGE) ? 0 : nxt + 1;
  }
  wg_barrier();   // LDS may be reused by the caller
}

// ---------------------------------------------------------------------------
// Direct-to-LDS main loop with one K step of look-ahead (NSTAGE >= 4).
// The barrier that opens step kt also guarantees that step kt+1 is complete in
// LDS, so the first fragments of step kt+1 are read *before* the next barrier,
// while the last MFMAs of step kt run: no LDS latency is exposed after a
// barrier.  Per step: fragments double-buffered in registers, the loads of step
// kt+NSTAGE-1 spread one per TN MFMAs, one vmcnt wait + one s_barrier.
// ---------------------------------------------------------------------------
template <class C>
__device__ __forceinline__ void gemm_mainloop_la(const GemmOperands& g, int row0, int col0, char* smem,
                                                 f32x16_t (&acc)[C::TM][C::TN]) {
  constexpr int NST = C::NSTAGE;
  constexpr int LPT = C::PA + C::PB;            // loads per thread per K step
  constexpr int KK = C::BK / 16;
  static_assert(NST >= 4 && NST <= 6, "look-ahead pipeline needs 4..6 LDS buffers");
  static_assert(LPT <= KK * C::TM, "one load slot per TN MFMAs");
  static_assert(LPT * (NST - 3) < 64, "vmcnt range");
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int wm = wave / C::WN, wn = wave % C::WN;

  const int lrow = lane / C::CPR, lpc = lane % C::CPR;
  uint32_t aoff[C::PA], boff[C::PB];
  const int amax = g.M - 1 - row0, bmax = g.N - 1 - col0;
#pragma unroll
  for (int i = 0; i < C::PA; ++i) {
    const int rt = (i * C::NW + wave) * C::RPI + lrow;
    const int r = rt < amax ? rt : amax;
    aoff[i] = (uint32_t)((long long)r * g.lda * 2 + ((lpc ^ lds_swizzle<C>(rt)) * 16));
  }
#pragma unroll
  for (int i = 0; i < C::PB; ++i) {
    const int rt = (i * C::NW + wave) * C::RPI + lrow;
    const int r = rt < bmax ? rt : bmax;
    boff[i] = (uint32_t)((long long)r * g.ldb * 2 + ((lpc ^ lds_swizzle<C>(rt)) * 16));
  }
  const int dst_a = wave * C::RPI * C::ROWB;
  const int dst_b = C::BM * C::ROWB + dst_a;
  const int sw = lds_swizzle<C>(lane & 31);
  const int fr_a = (wm * C::WTM + (lane & 31)) * C::ROWB;
  const int fr_b = C::BM * C::ROWB + (wn * C::WTN + (lane & 31)) * C::ROWB;
  int fr_c[KK];
#pragma unroll
  for (int kk = 0; kk < KK; ++kk) fr_c[kk] = ((kk * 2 + (lane >> 5)) ^ sw) * 16;

  // segment table in registers (no scalar memory traffic inside the loop)
  const char* segA[3];
  const char* segB[3];
  int segN[3];
  int nk_total = 0;
#pragma unroll
  for (int s = 0; s < 3; ++s) {
    const bool on = s < g.nseg;
    segA[s] = on ? (const char*)(g.seg[s].A + (long long)row0 * g.lda) : nullptr;
    segB[s] = on ? (const char*)(g.seg[s].B + (long long)col0 * g.ldb) : nullptr;
    segN[s] = on ? g.seg[s].K / C::BK : 0;
    nk_total += segN[s];
  }
  int iseg = 0, ileft = segN[0];
  const char* Ai = segA[0];
  const char* Bi = segB[0];
  auto issue_one = [&](int stage, int idx) {
    char* base = smem + stage * C::STAGE;
    if (idx < C::PA)
      __builtin_amdgcn_global_load_lds(FGRPO_GLOBAL_PTR(Ai + aoff[idx]),
                                       FGRPO_LDS_PTR(base + dst_a + idx * C::NW * C::RPI * C::ROWB), 16, 0, FGRPO_DMA_AUX);
    else
      __builtin_amdgcn_global_load_lds(FGRPO_GLOBAL_PTR(Bi + boff[idx - C::PA]),
                                       FGRPO_LDS_PTR(base + dst_b + (idx - C::PA) * C::NW * C::RPI * C::ROWB), 16, 0,
                                       FGRPO_DMA_AUX);
    if (idx == LPT - 1) {
      Ai += C::BK * 2;
      Bi += C::BK * 2;
      if (--ileft == 0) {
        ++iseg;
        const bool s1 = (iseg == 1);
        ileft = s1 ? segN[1] : segN[2];
        Ai = s1 ? segA[1] : segA[2];
        Bi = s1 ? segB[1] : segB[2];
      }
    }
  };
  // At most `tiles` K steps of this thread's loads stay in flight.  The look-ahead fragment reads
  // issued half a step earlier are certainly back by now; saying so (lgkmcnt 0) lets the compiler
  // start the next step's MFMAs without waiting for the reads it issues at the top of that step.
  auto wait_allow = [&](int tiles) {
    if (tiles >= NST - 3) {
      FGRPO_WAIT_VMCNT_LGKM0(LPT * (NST - 3));
    } else if (NST >= 6 && tiles == 2) {
      FGRPO_WAIT_VMCNT_LGKM0(LPT * 2);
    } else if (NST >= 5 && tiles == 1) {
      FGRPO_WAIT_VMCNT_LGKM0(LPT * 1);
    } else {
      FGRPO_WAIT_VMCNT_LGKM0(0);
    }
  };

  FGRPO_WAIT_VMCNT(0);   // the caller's own loads must not be mistaken for ours
  int issued = 0;
  for (; issued < NST - 1 && issued < nk_total; ++issued) {
#pragma unroll
    for (int idx = 0; idx < LPT; ++idx) issue_one(issued, idx);
  }
  // steps 0 and 1 must be in LDS before the first barrier
  {
    int allow = issued - 2;
    wait_allow(allow < 0 ? 0 : allow);
  }
  wg_barrier();

  bf16x8_t af[2][C::TM], bf[2][C::TN];
#pragma unroll
  for (int i = 0; i < C::TM; ++i) af[0][i] = FGRPO_LDFRAG(smem + fr_a + i * 32 * C::ROWB + fr_c[0]);
#pragma unroll
  for (int j = 0; j < C::TN; ++j) bf[0][j] = FGRPO_LDFRAG(smem + fr_b + j * 32 * C::ROWB + fr_c[0]);
  __builtin_amdgcn_s_waitcnt(0xC07F);   // lgkmcnt(0): enter the loop with these fragments in registers

  int cur = 0;                 // stage of step kt
  int nst = (NST - 1) % NST;   // stage that the loads issued during step kt go to (= stage of step kt-1)
  for (int kt = 0; kt < nk_total; ++kt) {
    const bool more = issued < nk_total;       // a step to issue during this one
    const bool has_next = kt + 1 < nk_total;
    const char* st = smem + cur * C::STAGE;
    const int nx = (cur + 1 == NST) ? 0 : cur + 1;
    const char* sn = smem + nx * C::STAGE;
#pragma unroll
    for (int kk = 0; kk < KK; ++kk) {
      const int b = kk & 1;
      // fragments of the next sub-step (or of the next K step's first sub-step) fly under these MFMAs
      if (kk + 1 < KK) {
#pragma unroll
        for (int i = 0; i < C::TM; ++i) af[b ^ 1][i] = FGRPO_LDFRAG(st + fr_a + i * 32 * C::ROWB + fr_c[kk + 1]);
#pragma unroll
        for (int j = 0; j < C::TN; ++j) bf[b ^ 1][j] = FGRPO_LDFRAG(st + fr_b + j * 32 * C::ROWB + fr_c[kk + 1]);
      } else if (has_next) {
#pragma unroll
        for (int i = 0; i < C::TM; ++i) af[b ^ 1][i] = FGRPO_LDFRAG(sn + fr_a + i * 32 * C::ROWB + fr_c[0]);
#pragma unroll
        for (int j = 0; j < C::TN; ++j) bf[b ^ 1][j] = FGRPO_LDFRAG(sn + fr_b + j * 32 * C::ROWB + fr_c[0]);
      }
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int i = 0; i < C::TM; ++i) {
#pragma unroll
        for (int j = 0; j < C::TN; ++j) acc[i][j] = FGRPO_MFMA(af[b][i], bf[b][j], acc[i][j]);
        if (kk * C::TM + i < LPT) {
          if (more) issue_one(nst, kk * C::TM + i);
        }
        __builtin_amdgcn_sched_barrier(0);
      }
    }
    static_assert(KK % 2 == 0, "fragment buffer parity must return to 0 every K step");
    if (more) ++issued;
    // before the next step starts, step kt+2 must be complete (step kt+1 already is)
    {
      int allow = issued - (kt + 3);
      wait_allow(allow < 0 ? 0 : allow);
    }
    wg_barrier();
    cur = nx;
    nst = (nst + 1 == NST) ? 0 : nst + 1;
  }
}

// ---------------------------------------------------------------------------
// Main loop for operands stored "K-major" (the contraction index is the ROW
// index: X[k][m], m contiguous), as dLogits [token][vocab], hidden [token][H] and
// W [vocab][H] are when the contraction runs over tokens or vocabulary.  No
// transposed copy is made: the tile goes to LDS as it lies in memory (two k rows
// of 256 columns per wavefront-wide direct-to-LDS load) and the MFMA operand is
// assembled by ds_read_b64_tr_b16, which hands lane i of every 16-lane group the
// i-th column of a 4 (k) x 16 (m) block whose rows are addressed by lanes
// 4e .. 4e+3.  Two such reads give the eight consecutive k values of a
// 32x32x16 operand.  16-byte chunks of a row are XOR-swizzled with 4*(k%4) so
// that the four rows one read touches fall into different banks.
// Either operand may instead be K-contiguous (X[m][k]) and is then handled as in
// gemm_mainloop_dma.  One segment, BM = BN = 256, BK = 64, two LDS buffers.
// ---------------------------------------------------------------------------
// Chunk-index XOR of k row `kr` of a K-major LDS tile (512-byte rows).  The transposing reads of a 32x32x16 operand
// take rows k .. k+3 per 16-lane group with the two groups of a pass 32 bytes apart in the row: 4*(k%4) spreads the
// four rows.  A 16x16x32 operand's groups of a pass read the same columns of rows k and k + 8: bit 3 of k moves
// them another 32 bytes apart.
template <bool MI16>
__device__ __forceinline__ int km_swizzle(int kr) {
  return MI16 ? (((kr & 3) << 2) | (((kr >> 3) & 1) << 1)) : ((kr & 3) << 2);
}
template <class C, bool AKM, bool BKM, bool MI16 = false>
__device__ __forceinline__ void gemm_mainloop_km(const GemmOperands& g, int row0, int col0, char* smem,
                                                 f32x16_t (&acc)[C::TM][C::TN]) {
  static_assert(C::DMA && C::NSTAGE == 2 && C::BM == 256 && C::BN == 256 && C::BK == 64, "K-major loop: 256x256x64, 2 buffers");
  static_assert(!MI16 || kMi16<C>, "16x16x32 MFMAs: 8-wavefront tile only");
  constexpr int LPT = C::PA + C::PB;
  constexpr int KK = C::BK / 16;
  constexpr int KROWB = 512;                    // bytes of one k row of a K-major tile (256 columns)
  constexpr int REG = C::BM * C::ROWB;          // bytes of one operand region (32 KiB either way)
  static_assert(C::ROWB == 128 && REG == C::BK * KROWB, "region size");
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);   // wavefront-uniform
  const int wm = wave / C::WN, wn = wave % C::WN;

  // ---- loader ------------------------------------------------------------------------------
  uint32_t aoff[C::PA], boff[C::PB];            // per-lane byte offset of each load inside the step's slice
  {
    const int lrow = lane / C::CPR, lpc = lane % C::CPR;
    const int amax = g.M - 1 - row0, bmax = g.N - 1 - col0;
#pragma unroll
    for (int i = 0; i < C::PA; ++i) {
      if constexpr (AKM) {
        const int kr = (i * C::NW + wave) * 2 + (lane >> 5);
        aoff[i] = (uint32_t)((long long)kr * g.lda * 2) + (uint32_t)((((lane & 31) ^ km_swizzle<MI16>(kr))) * 16);
      } else {
        const int rt = (i * C::NW + wave) * C::RPI + lrow;
        const int r = rt < amax ? rt : amax;
        aoff[i] = (uint32_t)((long long)r * g.lda * 2 + ((lpc ^ lds_swizzle<C, MI16>(rt)) * 16));
      }
    }
#pragma unroll
    for (int i = 0; i < C::PB; ++i) {
      if constexpr (BKM) {
        const int kr = (i * C::NW + wave) * 2 + (lane >> 5);
        boff[i] = (uint32_t)((long long)kr * g.ldb * 2) + (uint32_t)((((lane & 31) ^ km_swizzle<MI16>(kr))) * 16);
      } else {
        const int rt = (i * C::NW + wave) * C::RPI + lrow;
        const int r = rt < bmax ? rt : bmax;
        boff[i] = (uint32_t)((long long)r * g.ldb * 2 + ((lpc ^ lds_swizzle<C, MI16>(rt)) * 16));
      }
    }
  }
  // Buffer loads: the lane's constant byte offset travels in a VGPR, everything that moves is scalar.
  //  * K-contiguous operand: descriptor on the tile's first row, K offset in an SGPR (re-based per 256-column
  //    block when A is column-blocked);
  //  * K-major operand: descriptor re-based on the first k row of every step, with num_records = the bytes of
  //    the k rows that exist from there on, so rows past the end of the contraction read as zero.
  // K-major A kept in 256-column blocks: tile column block row0/256 is one [K][256] matrix of its own
  const char* Ap = AKM ? (const char*)(g.seg[0].A + (g.a_blk ? (long long)(row0 >> 8) * g.a_blk : (long long)row0))
                       : (const char*)(g.seg[0].A + (long long)row0 * g.lda);
  const char* Bp = BKM ? (const char*)(g.seg[0].B + col0) : (const char*)(g.seg[0].B + (long long)col0 * g.ldb);
  const long long lda2 = g.lda * 2, ldb2 = g.ldb * 2;
  long long a_rem = (AKM && g.ka_valid > 0) ? g.ka_valid : (1LL << 40);   // k rows of A that exist from Ap on
  long long b_rem = (BKM && g.kb_valid > 0) ? g.kb_valid : (1LL << 40);
  // bytes from a descriptor's base (first k row of the step, first column of the tile) to the end of the operand:
  // `rows` k rows of ld2 bytes, less the tile's column offset - the last tile of a row width that is not a multiple
  // of 256 reads past the end of every row, which must not carry past the end of the last one
  auto bytes_of = [](long long rows, long long ld2, long long col_bytes) -> uint32_t {
    if (rows <= 0) return 0u;
    const long long bts = rows * ld2 - col_bytes;
    if (bts <= 0) return 0u;
    return (rows > (1LL << 31) || bts > 0xffffffffLL) ? 0xffffffffu : (uint32_t)bts;
  };
  const long long a_col = (AKM && g.a_blk == 0) ? (long long)row0 * 2 : 0, b_col = BKM ? (long long)col0 * 2 : 0;
  __amdgpu_buffer_rsrc_t rsa = make_rsrc(Ap, AKM ? bytes_of(a_rem, lda2, a_col) : 0xffffffffu);
  __amdgpu_buffer_rsrc_t rsb = make_rsrc(Bp, BKM ? bytes_of(b_rem, ldb2, b_col) : 0xffffffffu);
  uint32_t ka = 0, kb = 0;                      // running K byte offset of a K-contiguous operand
  const int dst_w = wave * 1024;                // both layouts: one load fills 1 KiB, loads i are NW KiB apart

  // run list (A K-major; B either way): the issue cursor walks the listed K steps; the compute side never
  // knows, it consumes LDS buffers in the order they were filled
  const int* runs = AKM ? g.k_runs : nullptr;
  const int n_runs = runs ? runs[0] : 0;
  const int nk_total = runs ? runs[1] : g.seg[0].K / C::BK;
  int run_idx = 0, run_left = 0, cur_step = 0;
  if (runs != nullptr && n_runs > 0) {
    cur_step = runs[2];
    run_left = runs[2 + kRunCap] - cur_step;
    Ap += (long long)cur_step * C::BK * lda2;
    a_rem -= (long long)cur_step * C::BK;
    rsa = make_rsrc(Ap, bytes_of(a_rem, lda2, a_col));
    if constexpr (BKM) {
      Bp += (long long)cur_step * C::BK * ldb2;
      b_rem -= (long long)cur_step * C::BK;
      rsb = make_rsrc(Bp, bytes_of(b_rem, ldb2, b_col));
    } else {
      kb = (uint32_t)cur_step * C::BK * 2;
    }
  }
  const long long a_blk_bytes = (!AKM) ? g.a_blk * 2 : 0;
  int ablk_left = 256 / C::BK;
  auto issue_one = [&](int stage, int idx) {
    char* base = smem + stage * C::STAGE;
    if (idx < C::PA)
      __builtin_amdgcn_raw_ptr_buffer_load_lds(rsa, FGRPO_LDS_PTR(base + dst_w + idx * C::NW * 1024), 16, (int)aoff[idx],
                                               (int)ka, 0, FGRPO_DMA_AUX);
    else
      __builtin_amdgcn_raw_ptr_buffer_load_lds(rsb, FGRPO_LDS_PTR(base + REG + dst_w + (idx - C::PA) * C::NW * 1024), 16,
                                               (int)boff[idx - C::PA], (int)kb, 0, FGRPO_DMA_AUX);
    if (idx == LPT - 1) {                        // next K step
      long long jump = 1;                        // K steps from this one to the next one to fetch
      if constexpr (AKM) {
        if (runs != nullptr && --run_left == 0 && run_idx + 1 < n_runs) {   // this run is done: on to the next
          ++run_idx;
          const int s = runs[2 + run_idx];
          jump = s - cur_step;
          run_left = runs[2 + kRunCap + run_idx] - s;
        }
        cur_step += (int)jump;
      }
      if constexpr (AKM) {
        Ap += jump * C::BK * lda2;
        a_rem -= jump * C::BK;
        rsa = make_rsrc(Ap, bytes_of(a_rem, lda2, a_col));
      } else {
        ka += C::BK * 2;
        if (--ablk_left == 0) {
          ablk_left = 256 / C::BK;
          if (a_blk_bytes != 0) {                // K-contiguous A kept in 256-column blocks: next block
            Ap += a_blk_bytes;
            rsa = make_rsrc(Ap, 0xffffffffu);
            ka = 0;
          }
        }
      }
      if constexpr (BKM) {
        Bp += jump * C::BK * ldb2;
        b_rem -= jump * C::BK;
        rsb = make_rsrc(Bp, bytes_of(b_rem, ldb2, b_col));
      } else {
        kb += (uint32_t)jump * C::BK * 2;
      }
    }
  };

  // ---- fragment addressing -------------------------------------------------------------------
  // K-contiguous operand: row (lane%32), chunk (2*kk + lane/32) ^ swizzle(row)
  const int swn = lds_swizzle<C>(lane & 31);
  int frn_c[KK];
#pragma unroll
  for (int kk = 0; kk < KK; ++kk) frn_c[kk] = ((kk * 2 + (lane >> 5)) ^ swn) * 16;
  const int frn_a = (wm * C::WTM + (lane & 31)) * C::ROWB;
  const int frn_b = REG + (wn * C::WTN + (lane & 31)) * C::ROWB;
  // K-major operand: lane l = 16*g + j supplies row k = 16*kk + 8*(g/2) + 4*r + j/4 and the 8 bytes at
  // column (g%2)*16 + 4*(j%4) of the 32-column block; chunk index XOR 4*(k%4) = 4*(j/4)
  const int j4 = (lane & 15) >> 2;
  const int frk_row = (8 * (lane >> 5) + j4) * KROWB;                         // + (16*kk + 4*r) * KROWB
  const int frk_sw = j4 << 2;
  const int frk_cl = (((lane >> 4) & 1) * 16 + 4 * (lane & 3)) >> 3;          // chunk of the lane's column inside a block
  const int frk_half = (lane & 1) * 8;
  auto km_off = [&](int block_col0) {            // byte offset of this lane's 8 bytes inside a k row
    return ((((block_col0 >> 3) + frk_cl) ^ frk_sw) << 4) + frk_half;
  };
  int fka[C::TM], fkb[C::TN];
#pragma unroll
  for (int i = 0; i < C::TM; ++i) fka[i] = frk_row + km_off(wm * C::WTM + i * 32);
#pragma unroll
  for (int j = 0; j < C::TN; ++j) fkb[j] = REG + frk_row + km_off(wn * C::WTN + j * 32);

  auto load_a = [&](const char* st, auto ic, auto kc) -> bf16x8_t {
    constexpr int i = decltype(ic)::value, kk = decltype(kc)::value;
    if constexpr (AKM)
      return lds_read_tr_pair<(16 * kk) * KROWB, (16 * kk + 4) * KROWB>(lds_addr(st) + fka[i]);
    else
      return lds_read_b128_asm<i * 32 * C::ROWB>(lds_addr(st) + frn_a + frn_c[kk]);
  };
  auto load_b = [&](const char* st, auto jc, auto kc) -> bf16x8_t {
    constexpr int j = decltype(jc)::value, kk = decltype(kc)::value;
    if constexpr (BKM)
      return lds_read_tr_pair<(16 * kk) * KROWB, (16 * kk + 4) * KROWB>(lds_addr(st) + fkb[j]);
    else
      return lds_read_b128_asm<j * 32 * C::ROWB>(lds_addr(st) + frn_b + frn_c[kk]);
  };
  // ---- pipeline: two buffers, barrier one sub-step early ----
  FGRPO_WAIT_VMCNT(0);
  if (nk_total > 0) {
#pragma unroll
    for (int idx = 0; idx < LPT; ++idx) issue_one(0, idx);
  }
  if constexpr (MI16) {
    // 16x16x32 fragments.  K-contiguous operand: row l % 16 of a 16-row block, chunk 4*k2 + l/16.  K-major operand:
    // lane l = 16*g + j supplies row k = 32*k2 + 8*g + 4*r + j/4 (r = 0, 1: the two transposing reads) and the 8 bytes
    // at column 4*(j%4) of the 16-column block; every 16-lane group gets its own eight k values of the slice.
    const int sw16 = lds_swizzle<C, MI16>(lane & 15);
    const int fa16 = (wm * C::WTM + (lane & 15)) * C::ROWB, fb16 = REG + (wn * C::WTN + (lane & 15)) * C::ROWB;
    int fc16[2];
#pragma unroll
    for (int k2 = 0; k2 < 2; ++k2) fc16[k2] = ((4 * k2 + (lane >> 4)) ^ sw16) * 16;
    const int g16 = lane >> 4;
    const int k16_row = (8 * g16 + j4) * KROWB;                      // + (32*k2 + 4*r) * KROWB
    const int k16_sw = (j4 << 2) | ((g16 & 1) << 1);                 // km_swizzle of the lane's rows
    const int k16_cl = (lane & 3) >> 1;                              // chunk of the lane's column inside a 16-column block
    auto km16_off = [&](int block_col0) { return ((((block_col0 >> 3) + k16_cl) ^ k16_sw) << 4) + frk_half; };
    int fka16[C::TM][2], fkb16[2 * C::TN];
#pragma unroll
    for (int i = 0; i < C::TM; ++i)
#pragma unroll
      for (int rh = 0; rh < 2; ++rh) fka16[i][rh] = k16_row + km16_off(wm * C::WTM + i * 32 + 16 * rh);
#pragma unroll
    for (int jc = 0; jc < 2 * C::TN; ++jc) fkb16[jc] = REG + k16_row + km16_off(wn * C::WTN + (jc >> 1) * 32 + 16 * (jc & 1));
    early_barrier_pipeline16<C, LPT, AKM ? 2 : 1, BKM ? 2 : 1>(
        nk_total, smem, acc, issue_one,
        [&](const char* st, auto ic, auto kc) -> bf16x8_t {
          constexpr int i = decltype(ic)::value, kk = decltype(kc)::value, k2 = kk >> 1, rh = kk & 1;
          if constexpr (AKM)
            return lds_read_tr_pair<(32 * k2) * KROWB, (32 * k2 + 4) * KROWB>(lds_addr(st) + fka16[i][rh]);
          else
            return lds_read_b128_asm<(i * 32 + 16 * rh) * C::ROWB>(lds_addr(st) + fa16 + fc16[k2]);
        },
        [&](const char* st, auto jcc, auto k2c) -> bf16x8_t {
          constexpr int jc = decltype(jcc)::value, k2 = decltype(k2c)::value;
          if constexpr (BKM)
            return lds_read_tr_pair<(32 * k2) * KROWB, (32 * k2 + 4) * KROWB>(lds_addr(st) + fkb16[jc]);
          else
            return lds_read_b128_asm<((jc >> 1) * 32 + 16 * (jc & 1)) * C::ROWB>(lds_addr(st) + fb16 + fc16[k2]);
        });
    return;
  }
  early_barrier_pipeline<C, LPT, AKM ? 2 : 1, BKM ? 2 : 1>(nk_total, smem, acc, issue_one, load_a, load_b);
}

template <class C>
__device__ __forceinline__ void run_mainloop(const GemmOperands& g, int row0, int col0, char* smem,
                                             f32x16_t (&acc)[C::TM][C::TN]) {
  if constexpr (C::DMA && C::NSTAGE >= 4)
    gemm_mainloop_la<C>(g, row0, col0, smem, acc);
  else if constexpr (C::DMA)
    gemm_mainloop_dma<C>(g, row0, col0, smem, acc);
  else
    gemm_mainloop<C>(g, row0, col0, smem, acc);
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
