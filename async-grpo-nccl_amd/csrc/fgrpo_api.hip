// C ABI of the fused logprob + GRPO path: argument checking, workspace layout
// and kernel launches.  Declarations and the reference interfaces they replace
// are in include/fgrpo.h.
#include <hip/hip_runtime.h>
#include <stdarg.h>
#include <stdio.h>
#include <string.h>
#include <initializer_list>
#include <mutex>
#include <string>
#include <vector>

#include "host_common.h"
#include "prep_kernels.h"
#include "tail_kernels.h"

using namespace fgrpo;

// Device memory that fgrpo_logprob_fwd_static uses in place of a caller workspace.  Every GPU the library runs
// on holds its own copy until the process ends.  In host code this name is only a handle for
// hipGetSymbolAddress: kernels, fills and copies take the per-device address kept in g_static_scratch.
static_assert(FGRPO_STATIC_SCRATCH_BYTES % 256 == 0, "scratch size");
static __device__ __align__(256) unsigned char scratch[FGRPO_STATIC_SCRATCH_BYTES];

namespace fgrpo {

namespace {
thread_local std::string g_err;
}

int fail(int code, const char* fmt, ...) {
  char buf[512];
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(buf, sizeof(buf), fmt, ap);
  va_end(ap);
  g_err = buf;
  return code;
}

Tuning g_tune;

int num_cus() {
  static int n = 0;
  if (n == 0) {
    int dev = 0;
    hipDeviceProp_t prop;
    if (hipGetDevice(&dev) == hipSuccess && hipGetDeviceProperties(&prop, dev) == hipSuccess)
      n = prop.multiProcessorCount;
    if (n <= 0) n = 256;
  }
  return n;
}

}  // namespace fgrpo

namespace {

// Optional per-phase event brackets of the backward (fgrpo_phase_timing_begin / _end).  One timer per process:
// the backward usually runs on another thread (autograd's) than the one that asked for the timing.
struct PhaseTimer {
  bool on = false, created = false;
  int n = 0, dropped = 0;
  hipEvent_t ev[2 * FGRPO_MAX_TIMED_PHASES];
  int kind[FGRPO_MAX_TIMED_PHASES];
};
PhaseTimer g_phase;
std::mutex g_phase_mu;

struct PhaseScope {
  hipStream_t st;
  int slot = -1;
  PhaseScope(int kind, hipStream_t s) : st(s) {
    PhaseTimer& t = g_phase;
    if (!t.on) return;                            // unlocked peek: timing is off in every production call
    std::lock_guard<std::mutex> lock(g_phase_mu);
    if (!t.on) return;
    if (t.n >= FGRPO_MAX_TIMED_PHASES) {
      ++t.dropped;
      return;
    }
    slot = t.n++;
    t.kind[slot] = kind;
    (void)hipEventRecord(t.ev[2 * slot], st);
  }
  ~PhaseScope() {
    if (slot >= 0) (void)hipEventRecord(g_phase.ev[2 * slot + 1], st);
  }
};
enum { kPhaseDlogits = 0, kPhaseDh = 1, kPhaseDw = 2, kPhaseOther = 3, kPhaseFwd = 4 };


int* tuning_slot(const char* key) {
  if (!key) return nullptr;
  if (!strcmp(key, "fwd_variant")) return &g_tune.fwd_variant;
  if (!strcmp(key, "ds_variant")) return &g_tune.ds_variant;
  if (!strcmp(key, "gemm_variant")) return &g_tune.gemm_variant;
  if (!strcmp(key, "fwd_nsplit")) return &g_tune.fwd_nsplit;
  if (!strcmp(key, "fwd_group_t")) return &g_tune.fwd_group_t;
  if (!strcmp(key, "ds_nsplit")) return &g_tune.ds_nsplit;
  if (!strcmp(key, "ds_group_t")) return &g_tune.ds_group_t;
  if (!strcmp(key, "dh_group_m")) return &g_tune.dh_group_m;
  if (!strcmp(key, "dw_group_m")) return &g_tune.dw_group_m;
  if (!strcmp(key, "gemm_group_m")) return &g_tune.gemm_group_m;
  if (!strcmp(key, "panel_cols")) return &g_tune.panel_cols;
  if (!strcmp(key, "small_variant")) return &g_tune.small_variant;
  if (!strcmp(key, "bwd_kmajor")) return &g_tune.bwd_kmajor;
  if (!strcmp(key, "attn_heads")) return &g_tune.attn_heads;
  if (!strcmp(key, "attn_dkv")) return &g_tune.attn_dkv;
  if (!strcmp(key, "attn_qside")) return &g_tune.attn_qside;
  if (!strcmp(key, "wide_stores")) return &g_tune.wide_stores;
  if (!strcmp(key, "keep_panels")) return &g_tune.keep_panels;
  if (!strcmp(key, "keep_skip_dead")) return &g_tune.keep_skip_dead;
  if (!strcmp(key, "tail_split")) return &g_tune.tail_split;
  return nullptr;
}

int check_operands(const GemmOperands& g, int bk) {
  if (g.nseg < 1 || g.nseg > 3) return fail(FGRPO_ERR_BAD_ARG, "gemm: nseg=%d", g.nseg);
  if (g.M <= 0 || g.N <= 0) return fail(FGRPO_ERR_BAD_ARG, "gemm: M=%d N=%d", g.M, g.N);
  if (g.lda % 8 || g.ldb % 8) return fail(FGRPO_ERR_ALIGN, "gemm: lda=%lld ldb=%lld not multiples of 8", g.lda, g.ldb);
  for (int s = 0; s < g.nseg; ++s) {
    if (!g.seg[s].A || !g.seg[s].B) return fail(FGRPO_ERR_BAD_ARG, "gemm: null operand in segment %d", s);
    if (!aligned16(g.seg[s].A) || !aligned16(g.seg[s].B)) return fail(FGRPO_ERR_ALIGN, "gemm: operand of segment %d not 16-byte aligned", s);
    if (g.seg[s].K <= 0 || g.seg[s].K % bk) return fail(FGRPO_ERR_UNSUPPORTED, "gemm: K=%d of segment %d not a positive multiple of %d", g.seg[s].K, s, bk);
    if ((g.a_blk == 0 && g.seg[s].K > g.lda) || g.seg[s].K > g.ldb)
      return fail(FGRPO_ERR_BAD_ARG, "gemm: K=%d exceeds a leading dimension", g.seg[s].K);
  }
  // a tile's rows must be addressable with 32-bit byte offsets
  if (256LL * g.lda * 2 >= (1LL << 32) || 256LL * g.ldb * 2 >= (1LL << 32))
    return fail(FGRPO_ERR_UNSUPPORTED, "gemm: leading dimension too large");
  if (g.a_blk != 0 && (g.lda != 256 || g.nseg != 1 || g.a_blk % 8 || g.a_blk < 256LL * g.M))
    return fail(FGRPO_ERR_BAD_ARG, "gemm: column-blocked A needs lda = 256, one segment and blocks of at least M rows");
  return 0;
}

int launch_convert(const void* src, int src_is_f32, long long ld_src, int R, int Cn, int Rpad, int Cpad, bf16_t* hi,
                   bf16_t* lo, long long ld_dst, int transpose, hipStream_t st) {
  ConvertParams p{src, src_is_f32, ld_src, R, Cn, Rpad, Cpad, hi, lo, ld_dst, transpose};
  dim3 grid((unsigned)((Cpad + 63) / 64), (unsigned)((Rpad + 63) / 64));
  if (transpose ? (Rpad > ld_dst) : (Cpad > ld_dst)) return fail(FGRPO_ERR_BAD_ARG, "convert: padded extent exceeds ld");
  hipLaunchKernelGGL(convert_pad_kernel, grid, dim3(256), 0, st, p);
  HIP_TRY(hipGetLastError());
  return 0;
}

// ---- workspace carving -------------------------------------------------------------
struct Carver {
  char* base;
  size_t off = 0;
  explicit Carver(void* b) : base((char*)b) {}
  template <class T>
  T* take(size_t count) {
    off = (size_t)round_up((long long)off, 256);
    T* p = base ? (T*)(base + off) : nullptr;
    off += count * sizeof(T);
    return p;
  }
  size_t total() const { return (size_t)round_up((long long)off, 256); }
};

int pick_variant(const Tuning& tn, int requested, long long M, long long N) {
  int v = requested;
  if (v < 0 || v >= kNumCfg) v = 0;
  // small problems: a big tile would leave most CUs idle
  const long long tiles = ((M + kCfg[v].bm - 1) / kCfg[v].bm) * ((N + kCfg[v].bn - 1) / kCfg[v].bn);
  if (tiles < num_cus() / 2 && tn.small_variant >= 0 && tn.small_variant < kNumCfg) v = tn.small_variant;
  return v;
}

// ---- forward plan -------------------------------------------------------------------
struct FwdPlan {
  int variant, tiles_v, tiles_t, nsplit;
  // Token regions: the first t_main tokens (whole device rounds of token tiles at `nsplit` vocabulary splits) and, when
  // t_main < T, the rest with a split count of their own (`nsplit_rem`), launched right behind them.
  int t_main, nsplit_rem;
  float4* part_rem;
  int Hp;            // padded contraction length
  bool copy_ops;     // operands are staged (fp32 split or padding) instead of used in place
  bf16_t *w_hi, *w_lo, *h_hi, *h_lo;
  float* bias32;
  float4* part;
  float* xt;
  size_t bytes;
};

// Device rounds x vocabulary tiles per work-group: the time of a launch in tile units.
long long split_cost(int tiles_t, int tiles_v, int slots, int s) {
  const long long blocks = (long long)tiles_t * s;
  const long long rounds = (blocks + slots - 1) / slots;
  const long long per = (tiles_v + s - 1) / s;
  return rounds * per;
}

int choose_nsplit(int tiles_t, int tiles_v, int slots, int forced, int prefer = 4, int max_split = 64) {
  if (forced > 0) return forced < tiles_v ? forced : tiles_v;
  int best = 1;
  long long best_cost = -1;
  const int cap = tiles_v < max_split ? tiles_v : max_split;
  auto cost_of = [&](int s) { return split_cost(tiles_t, tiles_v, slots, s); };
  for (int s = 1; s <= cap; ++s) {
    const long long cost = cost_of(s);
    if (best_cost < 0 || cost < best_cost) {
      best_cost = cost;
      best = s;
    }
  }
  // Four splits x eight token tiles (the default raster group) put 32 work-groups = one XCD on an 8 x 4
  // patch of (token tile, vocabulary range): every W slice fetched into that XCD's L2 serves 8 work-groups and
  // every hidden slice 4.  With fewer splits the hidden tiles, which do not fit a 4 MiB L2, are re-fetched per
  // work-group (measured: 0.94 -> 1.14 PFLOP/s at T=65536, H=3584; a 66-tile panel at one split instead of four:
  // +6 % on the whole backward).  Take it when it costs at most 6% in rounds: rounding a share of 16 or more
  // tiles up to a multiple of four never costs more.
  // The dLogits kernel, which also writes its tile, measures 1-2 % better on the whole backward with eight splits
  // and two token tiles per group (`prefer` = 8); it falls back to four, then to the cheapest.
  if (prefer != 4 && cap >= prefer && cost_of(prefer) * 100 <= best_cost * 106) return prefer;
  if (cap >= 4 && cost_of(4) * 100 <= best_cost * 106) best = 4;
  return best;
}

void plan_fwd(const Tuning& tn, FwdPlan& pl, void* ws, int T, int H, int V, int dtype, bool has_bias) {
  pl.variant = pick_variant(tn, tn.fwd_variant, V, T);
  const CfgInfo& c = kCfg[pl.variant];
  pl.tiles_v = (V + c.bm - 1) / c.bm;
  pl.tiles_t = (T + c.bn - 1) / c.bn;
  // A work-group keeps its token tile and re-reads that tile's hidden slab for every vocabulary tile it walks; with
  // four splits the device works on 8 XCDs x 8 token tiles = 16384 rows of hidden at a time.  From H = 6144 on that is
  // more than 192 MB and no longer stays in the 256 MB cache in front of HBM next to the W stream: eight splits
  // (4 token tiles per XCD) halve it (T=16384, H=8192, V=128256: 28.9 -> 24.9 ms; H=5120 and 3584 measure equal
  // or better with four).
  const int prefer = (16384LL * H * 2 > (192LL << 20)) ? 8 : 4;
  const int slots = num_cus() * c.wgs_per_cu;
  pl.nsplit = choose_nsplit(pl.tiles_t, pl.tiles_v, slots, tn.fwd_nsplit, prefer);
  pl.t_main = T;
  pl.nsplit_rem = 0;
  // A token count that is not a whole number of device rounds (slots / prefer token tiles each) leaves the choice
  // above between a last round that is nearly empty and a split count that fits the rounds but breaks up the 32
  // work-group patches an XCD shares its operands in (T = 33000 instead of 32768: 14.7 instead of 12.8 ms).  Give the
  // whole rounds the preferred split and the remaining token tiles a launch of their own, split as finely as it
  // takes to spread them over the device, unless the tile count says that is more than 10 % dearer (the count knows
  // nothing of the patches: by it alone 33 splits of 129 token tiles cost 306 tile times against 303 for the two
  // regions, measured they are 15 % apart).
  if (tn.fwd_nsplit <= 0 && tn.tail_split != 0 && pl.tiles_v >= prefer && slots % prefer == 0) {
    const int per_round = slots / prefer;                       // token tiles of one full round
    const int main_tiles = pl.tiles_t / per_round * per_round;
    if (main_tiles > 0 && main_tiles < pl.tiles_t) {
      const int rem_tiles = pl.tiles_t - main_tiles;
      const int ns_rem = choose_nsplit(rem_tiles, pl.tiles_v, slots, 0, prefer, 128);
      const long long two = split_cost(main_tiles, pl.tiles_v, slots, prefer) + split_cost(rem_tiles, pl.tiles_v, slots, ns_rem);
      if (two * 100 <= split_cost(pl.tiles_t, pl.tiles_v, slots, pl.nsplit) * 110) {
        pl.nsplit = prefer;
        pl.t_main = main_tiles * c.bn;
        pl.nsplit_rem = ns_rem;
      }
    }
  }
  pl.Hp = (int)round_up(H, 64);
  pl.copy_ops = (dtype == FGRPO_F32) || (H % 64 != 0);
  Carver cv(ws);
  pl.w_hi = pl.w_lo = pl.h_hi = pl.h_lo = nullptr;
  if (pl.copy_ops) {
    pl.w_hi = cv.take<bf16_t>((size_t)V * pl.Hp);
    pl.h_hi = cv.take<bf16_t>((size_t)T * pl.Hp);
    if (dtype == FGRPO_F32) {
      pl.w_lo = cv.take<bf16_t>((size_t)V * pl.Hp);
      pl.h_lo = cv.take<bf16_t>((size_t)T * pl.Hp);
    }
  }
  pl.bias32 = has_bias ? cv.take<float>((size_t)V) : nullptr;
  pl.part = cv.take<float4>((size_t)pl.nsplit * T);
  pl.part_rem = pl.t_main < T ? cv.take<float4>((size_t)pl.nsplit_rem * (T - pl.t_main)) : nullptr;
  pl.xt = cv.take<float>((size_t)T);
  pl.bytes = cv.total();
}

// Fill the operands of the logits contraction: A = weight side, B = hidden side.
int stage_logit_operands(GemmOperands& g, const void* hidden, const void* weight, int T, int H, int V, int dtype,
                         bool copy_ops, int Hp, bf16_t* w_hi, bf16_t* w_lo, bf16_t* h_hi, bf16_t* h_lo, hipStream_t st) {
  g.M = V;
  g.N = T;
  if (!copy_ops) {
    g.nseg = 1;
    g.seg[0] = GemmSeg{(const bf16_t*)weight, (const bf16_t*)hidden, H};
    g.lda = g.ldb = H;
    return 0;
  }
  const int f32 = (dtype == FGRPO_F32);
  int rc = launch_convert(weight, f32, H, V, H, V, Hp, w_hi, f32 ? w_lo : nullptr, Hp, 0, st);
  if (rc) return rc;
  rc = launch_convert(hidden, f32, H, T, H, T, Hp, h_hi, f32 ? h_lo : nullptr, Hp, 0, st);
  if (rc) return rc;
  g.lda = g.ldb = Hp;
  if (f32) {
    g.nseg = 3;
    g.seg[0] = GemmSeg{w_hi, h_hi, Hp};
    g.seg[1] = GemmSeg{w_hi, h_lo, Hp};
    g.seg[2] = GemmSeg{w_lo, h_hi, Hp};
  } else {
    g.nseg = 1;
    g.seg[0] = GemmSeg{w_hi, h_hi, Hp};
  }
  return 0;
}

// 16-byte epilogue pieces need every row of the output (and of the addend) to start on a 16-byte boundary.
bool can_store_wide(const Tuning& tn, const StoreParams& p) {
  if (!tn.wide_stores) return false;
  const long long per16 = p.c_out_bf16 ? 8 : 4;
  if (p.ldc % per16) return false;
  if (p.c_out_bf16 && !aligned16(p.c_out_bf16)) return false;
  if (p.c_out_f32 && !aligned16(p.c_out_f32)) return false;
  if (p.c_in && (!aligned16(p.c_in) || p.ldc % 4)) return false;
  return true;
}

// Gradient GEMMs whose contraction index is the row index of an operand as it lies in memory.
// akm/bkm: that operand is [K][M] (resp. [K][N]) with leading dimension lda (ldb); the other is [M][K] ([N][K]).
int run_store_gemm_kmajor(const Tuning& tn, StoreParams p, bool akm, bool bkm, hipStream_t st, int group_m_auto = 0) {
  const GemmOperands& g = p.g;
  if (g.nseg != 1 || !g.seg[0].A || !g.seg[0].B) return fail(FGRPO_ERR_BAD_ARG, "gemm(k-major): one segment expected");
  if (g.M <= 0 || g.N <= 0 || g.seg[0].K <= 0 || g.seg[0].K % Cfg8::BK)
    return fail(FGRPO_ERR_UNSUPPORTED, "gemm(k-major): M=%d N=%d K=%d", g.M, g.N, g.seg[0].K);
  if (g.lda % 8 || g.ldb % 8 || !aligned16(g.seg[0].A) || !aligned16(g.seg[0].B))
    return fail(FGRPO_ERR_ALIGN, "gemm(k-major): operands must be 16-byte aligned with ld %% 8 == 0");
  p.tiles_m = (g.M + Cfg8::BM - 1) / Cfg8::BM;
  p.tiles_n = (g.N + Cfg8::BN - 1) / Cfg8::BN;
  // a K-major tile is read 256 columns wide without clamping: the rows must hold them
  if (g.a_blk != 0 && (g.lda != 256 || g.a_blk % 8 || g.a_blk < 256LL * (akm ? g.seg[0].K : g.M)))
    return fail(FGRPO_ERR_BAD_ARG, "gemm(k-major): column-blocked A needs lda = 256 and blocks that hold every row");
  // A K-major tile is read 256 columns wide without clamping.  Rows shorter than the padded width are fine: the
  // excess columns of a row are the start of the next one (values that only reach output columns past M / N, which
  // are never stored) and, past the last existing row, zeros from the buffer descriptor's bound.  The rows must
  // hold the logical width, though.
  if (akm && g.a_blk == 0 && g.M > g.lda) return fail(FGRPO_ERR_BAD_ARG, "gemm(k-major): lda < M");
  if (bkm && g.N > g.ldb) return fail(FGRPO_ERR_BAD_ARG, "gemm(k-major): ldb < N");
  // the kernel bounds its reads by the rows that exist: "all of them" must be said as a number
  if (akm && p.g.ka_valid <= 0) p.g.ka_valid = g.seg[0].K;
  if (bkm && p.g.kb_valid <= 0) p.g.kb_valid = g.seg[0].K;
  if (256LL * g.lda * 2 >= (1LL << 32) || 256LL * g.ldb * 2 >= (1LL << 32))
    return fail(FGRPO_ERR_UNSUPPORTED, "gemm(k-major): leading dimension too large");
  {
    // group_m_auto: > 0 that many row tiles per raster group, < 0 row tiles dealt round-robin to the XCDs,
    // 0 the tuning default; a tuning key set for this GEMM overrides it
    // Either way the 32 work-groups an XCD runs side by side should form a patch of row tiles x column tiles that is
    // not a sliver: with more than 8 column tiles (H > 2048) a single row tile's columns would fill the XCD and
    // every work-group would fetch a B slice of its own (measured at T=16384, H=8192, V=128256: 139 / 143 GB past
    // the L2s for dHidden / dW against 53-66 GB for the vendor library's kernels), so 4 row tiles x 8 columns then.
    const int own = akm ? tn.dw_group_m : tn.dh_group_m;
    const int wide = p.tiles_n > 8;
    if (group_m_auto > 0 && wide) group_m_auto = 4;
    p.group_m = own > 0 ? own : group_m_auto > 0 ? group_m_auto : group_m_auto < 0 ? 0 : (tn.gemm_group_m > 0 ? tn.gemm_group_m : (wide ? 4 : 1));
    p.rr_cols = wide ? 8 : p.tiles_n;
    p.rr_rows = wide ? 4 : 1;
  }
  p.wide_stores = can_store_wide(tn, p);
  p.nblocks = p.group_m > 0 ? p.tiles_m * p.tiles_n : 8 * ((p.tiles_m + 7) / 8) * p.tiles_n;
  return launch_store_kmajor(akm, bkm, p, st);
}

int run_store_gemm(const Tuning& tn, StoreParams p, int variant, hipStream_t st) {
  variant = pick_variant(tn, variant, p.g.M, p.g.N);
  if (p.g.a_blk != 0 && variant != 6 && variant != 7 && variant != 8) variant = 8;  // loops that know the layout
  const CfgInfo& c = kCfg[variant];
  int rc = check_operands(p.g, c.bk);
  if (rc) return rc;
  p.tiles_m = (p.g.M + c.bm - 1) / c.bm;
  p.tiles_n = (p.g.N + c.bn - 1) / c.bn;
  p.group_m = tn.gemm_group_m > 0 ? tn.gemm_group_m : 1;
  p.wide_stores = can_store_wide(tn, p);
  p.nblocks = p.tiles_m * p.tiles_n;
  return launch_store_variant(variant, p, st);
}

// ---- backward plan ------------------------------------------------------------------
struct BwdPlan {
  int variant;            // of the dS kernel
  int bm, bn;
  int Hp, Tpad, Vpad;     // Tpad, Vpad: multiples of 256
  int panel, npanels;     // vocabulary rows per panel (multiple of 256)
  int tiles_t;
  bool copy_ops, f32;
  bool kmajor;            // dW GEMM reads dLogits [token][vocab] and hidden in place: no [vocab][token] copy
  bool kmajor_dh;         // dH GEMM reads W in place: no transposed weight copy
  bf16_t *w_hi, *w_lo, *h_hi, *h_lo;          // straight operands (staged only when copy_ops)
  bf16_t *wT_hi, *wT_lo, *hT_hi, *hT_lo;      // transposed copies [H x Vpad], [H x Tpad]
  bf16_t *tv_hi, *tv_lo, *vt_hi, *vt_lo;      // dS panels
  float* bias32;
  float* dh_acc;                              // [T x H] fp32 when more than one panel
  size_t bytes;
};

// Panel budget when the caller gives none: a quarter of the [T x V] matrix, at least 2^25 and at most 2^30 elements
// (2 GiB of bf16) - the whole matrix is only ever held when it is small.
long long default_panel_elems(int T, int V) {
  long long e = (long long)T * V / 4;
  if (e < (1LL << 25)) e = 1LL << 25;
  if (e > (1LL << 30)) e = 1LL << 30;
  return e;
}

// Panels: at least `np_min` (the memory bound).  Of np_min .. np_min + 3, the count whose dW GEMMs (one tile per
// 256 vocabulary rows x 256 hidden columns, contraction over all T tokens - the one GEMM of the backward whose
// tile count depends on the panel width) waste the fewest rounds of the device, plus a fixed cost per panel
// (three launches' tails and one pass over the fp32 dH accumulator, measured at about 0.15 of such a round).
// Measured at T=32768, H=1536, V=151936: 8 panels (450 tiles, 1.76 rounds each) 39.1 ms, 7 panels (510 tiles) 38.2.
int fit_panel_count(int np_min, int H, int V) {
  const int cus = num_cus(), hT = (H + 255) / 256, max_np = (V + 255) / 256;
  if ((long long)((V + np_min - 1) / np_min + 255) / 256 * hT < cus / 2) return np_min;   // small problems: the small-tile path
  int best = np_min;
  long long best_cost = -1;
  for (int np = np_min; np <= np_min + 3 && np <= max_np; ++np) {
    const int panel = (int)round_up((V + np - 1) / np, 256);
    long long cost = 0;
    for (int v0 = 0; v0 < V; v0 += panel) {
      const int rows = (V - v0) < panel ? (V - v0) : panel;
      cost += 100LL * ((((long long)(rows + 255) / 256) * hT + cus - 1) / cus) + 15;
    }
    if (best_cost < 0 || cost < best_cost) {
      best_cost = cost;
      best = np;
    }
  }
  return best;
}

void plan_bwd(const Tuning& tn, BwdPlan& pl, void* ws, int T, int H, int V, int dtype, long long hint, bool has_bias,
              bool want_dh, bool want_dw) {
  pl.f32 = (dtype == FGRPO_F32);
  pl.variant = pl.f32 ? 4 : pick_variant(tn, tn.ds_variant, V, T);
  pl.bm = kCfg[pl.variant].bm;
  pl.bn = kCfg[pl.variant].bn;
  pl.Hp = (int)round_up(H, 64);
  pl.Tpad = (int)round_up(T, 256);
  pl.Vpad = (int)round_up(V, 256);
  pl.tiles_t = (T + pl.bn - 1) / pl.bn;
  long long cols = tn.panel_cols > 0 ? tn.panel_cols : default_panel_elems(T, V) / (T > 0 ? T : 1);
  if (hint > 0) cols = hint / (T > 0 ? T : 1);
  if (cols < 256) cols = 256;
  int np = (int)((V + cols - 1) / cols);
  if (np < 1) np = 1;
  if (!pl.f32 && H % 64 == 0) np = fit_panel_count(np, H, V);
  pl.panel = (int)round_up((V + np - 1) / np, 256);
  pl.npanels = (V + pl.panel - 1) / pl.panel;
  pl.copy_ops = pl.f32 || (H % 64 != 0);
  Carver cv(ws);
  pl.w_hi = pl.w_lo = pl.h_hi = pl.h_lo = nullptr;
  if (pl.copy_ops) {
    pl.w_hi = cv.take<bf16_t>((size_t)V * pl.Hp);
    pl.h_hi = cv.take<bf16_t>((size_t)T * pl.Hp);
    if (pl.f32) {
      pl.w_lo = cv.take<bf16_t>((size_t)V * pl.Hp);
      pl.h_lo = cv.take<bf16_t>((size_t)T * pl.Hp);
    }
  }
  // In-place (K-major) gradient GEMMs: bf16 operands used as they are, H a multiple of the tile width, and
  // enough tiles to fill the device (small problems keep the small-tile path).
  {
    // (H need not be a multiple of the 256-column tile: the last tile reads past the end of each row into the next
    // one - inside the buffer descriptor, zeros beyond it - and those output columns are never stored)
    const long long th = (long long)((T + 255) / 256) * ((H + 255) / 256);
    const long long vh = (long long)(((V < pl.panel ? V : pl.panel) + 255) / 256) * ((H + 255) / 256);
    pl.kmajor = tn.bwd_kmajor && !pl.copy_ops && H % 64 == 0 && pl.bm == 256 && pl.bn % 64 == 0 &&
                th >= num_cus() / 2 && vh >= num_cus() / 2;
    pl.kmajor_dh = pl.kmajor && tn.bwd_kmajor >= 2;
  }
  pl.wT_hi = pl.wT_lo = pl.hT_hi = pl.hT_lo = nullptr;
  if (want_dh && !pl.kmajor_dh) {
    pl.wT_hi = cv.take<bf16_t>((size_t)H * pl.Vpad);
    if (pl.f32) pl.wT_lo = cv.take<bf16_t>((size_t)H * pl.Vpad);
  }
  if (want_dw && !pl.kmajor) {
    pl.hT_hi = cv.take<bf16_t>((size_t)H * pl.Tpad);
    if (pl.f32) pl.hT_lo = cv.take<bf16_t>((size_t)H * pl.Tpad);
  }
  const size_t pe = (size_t)pl.Tpad * pl.panel;
  pl.tv_hi = cv.take<bf16_t>(pe);
  pl.vt_hi = pl.kmajor ? nullptr : cv.take<bf16_t>(pe);
  pl.tv_lo = pl.vt_lo = nullptr;
  if (pl.f32) {
    pl.tv_lo = cv.take<bf16_t>(pe);
    pl.vt_lo = cv.take<bf16_t>(pe);
  }
  pl.bias32 = has_bias ? cv.take<float>((size_t)V) : nullptr;
  pl.dh_acc = (want_dh && pl.npanels > 1 && !pl.f32) ? cv.take<float>((size_t)T * H) : nullptr;
  pl.bytes = cv.total();
}

}  // namespace

namespace {
// Conditions of the kept-logits pair: the forward on the 256x256x64 two-buffer tile with operands used in place,
// both gradient GEMMs on operands read where they lie.
bool keep_supported(const Tuning& tn, int T, int H, int V, int dtype) {
  if (dtype != FGRPO_BF16 || T <= 0 || V <= 0 || H <= 0 || H % 64 != 0) return false;
  if (pick_variant(tn, 8, V, T) != 8) return false;
  // dW's tiles (vocabulary x hidden) must fill at least half the device; dHidden's (tokens x hidden) need not: few
  // of them are contracted in pieces (plan_dh_split), and the forward splits the vocabulary as finely as it takes.
  // Measured at H = 1536, V = 151936 against the recomputing pair: T = 512 1.14 against 4.02 ms, 4096 4.78 against 8.61.
  const long long vh = (long long)((V + 255) / 256) * ((H + 255) / 256);
  return vh >= num_cus() / 2;
}
// Layout of the kept buffer: the column-blocked bf16 numerators, then the per-token references and target logits
// (fp32 each), then the overflow flag (one int in its own 256 bytes).
size_t keep_block_bytes(int T, int V) { return (size_t)round_up(V, 256) * (size_t)round_up(T, 256) * sizeof(bf16_t); }
size_t keep_bytes(int T, int V) { return keep_block_bytes(T, V) + 2 * (size_t)round_up(T, 256) * sizeof(float) + 256; }
float* keep_ref2_of(void* keep, int T, int V) { return (float*)((char*)keep + keep_block_bytes(T, V)); }
float* keep_xy_of(void* keep, int T, int V) { return keep_ref2_of(keep, T, V) + round_up(T, 256); }
int* keep_flag_of(void* keep, int T, int V) {
  return (int*)((char*)keep + keep_block_bytes(T, V) + 2 * (size_t)round_up(T, 256) * sizeof(float));
}

// Per-token references and target logits of a kept buffer, and its overflow flag.  They lie behind the numerators
// in the buffer itself - unless the caller has formed them already, for the tokens of many launches at once
// (ready: the forward then skips its own pre-pass, and the flag was cleared with them).
struct KeepAux {
  float* ref2;
  float* xy;
  int* flag;
  bool ready;
};
KeepAux keep_aux_of(void* keep, int T, int V) {
  return KeepAux{keep_ref2_of(keep, T, V), keep_xy_of(keep, T, V), keep_flag_of(keep, T, V), false};
}

// The pre-pass of the kept forward: the reference's sample of the vocabulary - the plain forward kernel over the
// first rows of W; only the maxima of its per-split partials are used - then one dot product per token.
// `p`: the forward's parameters for these tokens (operands staged, bias, labels, temperature); part: scratch for
// min(2, nsplit) x T partials.
int keep_prepass(const FwdParams& p, const void* hidden, const void* weight, const int64_t* labels, int T, int H, int V,
                 int nsplit, float4* part, const KeepAux& aux, int nflags, hipStream_t st) {
  FwdParams sp = p;
  const int vs = V < kKeepSampleRows ? V : kKeepSampleRows;
  sp.g.M = vs;
  sp.g.N = T;
  sp.tiles_v = (vs + kCfg[8].bm - 1) / kCfg[8].bm;
  sp.tiles_t = (T + kCfg[8].bn - 1) / kCfg[8].bn;
  sp.nsplit = sp.tiles_v < nsplit ? sp.tiles_v : nsplit;
  sp.part = part;
  sp.keep = nullptr;
  int rc = launch_fwd_variant(8, sp, st);
  if (rc) return rc;
  KeepRefParams r{(const bf16_t*)hidden, (const bf16_t*)weight, p.bias, (const long long*)labels, T, H, V, p.inv_temp,
                  part, sp.nsplit, aux.ref2, aux.xy, aux.flag, nflags};
  hipLaunchKernelGGL(keep_reference_kernel, dim3((T + 3) / 4), dim3(256), 0, st, r);
  HIP_TRY(hipGetLastError());
  return 0;
}

int logprob_fwd_impl(const void* hidden, const void* weight, const void* bias, const int64_t* labels, float inv_temp,
                      int T, int H, int V, int dtype, float* lp_out, float* ent_out, float* lse_out, void* ws,
                      size_t ws_bytes, void* stream, void* keep = nullptr, const Tuning* snapshot = nullptr,
                      const KeepAux* aux_in = nullptr) {
  hipStream_t st = (hipStream_t)stream;
  if (!hidden || !weight || !labels || !lp_out) return fail(FGRPO_ERR_BAD_ARG, "logprob_fwd: null argument");
  if (T <= 0 || H <= 0 || V <= 0) return fail(FGRPO_ERR_BAD_ARG, "logprob_fwd: T=%d H=%d V=%d", T, H, V);
  if (dtype != FGRPO_BF16 && dtype != FGRPO_F32) return fail(FGRPO_ERR_BAD_ARG, "logprob_fwd: dtype=%d", dtype);
  if (!(inv_temp > 0.f)) return fail(FGRPO_ERR_BAD_ARG, "logprob_fwd: inv_temperature must be positive");
  if (!ws || !aligned16(ws)) return fail(FGRPO_ERR_WORKSPACE, "logprob_fwd: workspace null or misaligned");
  if (!aligned16(hidden) || !aligned16(weight)) return fail(FGRPO_ERR_ALIGN, "logprob_fwd: hidden/weight must be 16-byte aligned");
  Tuning tn = snapshot ? *snapshot : g_tune;   // one reading of the tuning state per call
  if (keep) tn.fwd_variant = 8;
  FwdPlan pl;
  plan_fwd(tn, pl, ws, T, H, V, dtype, bias != nullptr);
  if (keep && (pl.variant != 8 || pl.copy_ops)) return fail(FGRPO_ERR_UNSUPPORTED, "logprob_fwd_keep: shape not supported");
  if (pl.bytes > ws_bytes) return fail(FGRPO_ERR_WORKSPACE, "logprob_fwd: workspace %zu < %zu bytes", ws_bytes, pl.bytes);

  FwdParams p;
  memset(&p, 0, sizeof(p));
  int rc = stage_logit_operands(p.g, hidden, weight, T, H, V, dtype, pl.copy_ops, pl.Hp, pl.w_hi, pl.w_lo, pl.h_hi,
                                pl.h_lo, st);
  if (rc) return rc;
  rc = check_operands(p.g, kCfg[pl.variant].bk);
  if (rc) return rc;
  if (bias) {
    hipLaunchKernelGGL(to_f32_kernel, dim3((V + 255) / 256), dim3(256), 0, st, bias, dtype == FGRPO_F32, pl.bias32, V);
    HIP_TRY(hipGetLastError());
  }
  p.bias = bias ? pl.bias32 : nullptr;
  p.labels = (const long long*)labels;
  p.inv_temp = inv_temp;
  p.tiles_v = pl.tiles_v;
  p.tiles_t = pl.tiles_t;
  p.nsplit = pl.nsplit;
  p.group_t = tn.fwd_group_t > 0 ? tn.fwd_group_t : 1;
  if (pl.nsplit >= 8 && p.group_t * pl.nsplit > 32) p.group_t = 32 / pl.nsplit > 0 ? 32 / pl.nsplit : 1;   // one XCD's 32 work-groups per patch
  const int c_bn = kCfg[pl.variant].bn;
  p.part = pl.part;
  p.xt = pl.xt;
  if (keep) {
    p.keep = (bf16_t*)keep;
    p.keep_blk = (long long)pl.tiles_t * kCfg[8].bn * 256;
    const KeepAux aux = aux_in ? *aux_in : keep_aux_of(keep, T, V);
    if (!aux.ready) {     // (the main launch below overwrites the sample's partials afterwards)
      rc = keep_prepass(p, hidden, weight, labels, T, H, V, pl.nsplit, pl.part, aux, 1, st);
      if (rc) return rc;
    }
    p.keep_ref2 = aux.ref2;
    p.keep_flag = aux.flag;
  }
  // One launch per token region: tokens [t0, t0 + count) with `nsplit` vocabulary splits, then their merge.
  auto run_region = [&](int t0, int count, int nsplit, float4* part) -> int {
    FwdParams q = p;
    q.g.N = count;
    for (int sg = 0; sg < q.g.nseg; ++sg) q.g.seg[sg].B += (long long)t0 * q.g.ldb;
    q.labels += t0;
    q.tiles_t = (count + c_bn - 1) / c_bn;
    q.nsplit = nsplit;
    q.group_t = tn.fwd_group_t > 0 ? tn.fwd_group_t : 1;
    if (nsplit >= 8 && q.group_t * nsplit > 32) q.group_t = 32 / nsplit > 0 ? 32 / nsplit : 1;   // one XCD's 32 work-groups per patch
    q.part = part;
    q.xt += t0;
    if (keep) {
      q.keep += (long long)t0 * 256;           // token t0 of every 256-column block
      q.keep_ref2 += t0;
    }
    const int rc2 = keep ? launch_fwd_keep(q, st) : launch_fwd_variant(pl.variant, q, st);
    if (rc2) return rc2;
    CombineParams c{part, pl.xt + t0, (const long long*)labels + t0, count, V, nsplit, lp_out + t0,
                    ent_out ? ent_out + t0 : nullptr, lse_out ? lse_out + t0 : nullptr};
    hipLaunchKernelGGL(lmhead_fwd_combine_kernel, dim3((count + 255) / 256), dim3(256), 0, st, c);
    HIP_TRY(hipGetLastError());
    return 0;
  };
  rc = run_region(0, pl.t_main, pl.nsplit, pl.part);
  if (rc) return rc;
  if (pl.t_main < T) rc = run_region(pl.t_main, T - pl.t_main, pl.nsplit_rem, pl.part_rem);
  return rc;
}

// Per-device address of `scratch`, resolved once per device with that device current.
std::mutex g_static_mu;
void* g_static_scratch[64] = {nullptr};

int static_scratch_ptr(void** out) {
  int dev = 0;
  HIP_TRY(hipGetDevice(&dev));
  if (dev < 0 || dev >= 64) return fail(FGRPO_ERR_UNSUPPORTED, "static scratch: device index %d out of range", dev);
  std::lock_guard<std::mutex> lock(g_static_mu);
  if (!g_static_scratch[dev]) {
    void* ptr = nullptr;
    HIP_TRY(hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch)));
    if (!ptr) return fail(FGRPO_ERR_HIP, "static scratch: hipGetSymbolAddress returned a null address");
    g_static_scratch[dev] = ptr;
  }
  *out = g_static_scratch[dev];
  return 0;
}
}  // namespace

extern "C" {

int fgrpo_version(void) { return 100; }
const char* fgrpo_last_error(void) { return g_err.c_str(); }

int fgrpo_set_tuning(const char* key, int value) {
  int* s = tuning_slot(key);
  if (!s) return fail(FGRPO_ERR_BAD_ARG, "unknown tuning key '%s'", key ? key : "(null)");
  *s = value;
  return 0;
}
int fgrpo_get_tuning(const char* key) {
  int* s = tuning_slot(key);
  if (!s) return fail(FGRPO_ERR_BAD_ARG, "unknown tuning key '%s'", key ? key : "(null)");
  return *s;
}

size_t fgrpo_logprob_fwd_workspace(int T, int H, int V, int dtype) {
  if (T <= 0 || H <= 0 || V <= 0) return 0;
  FwdPlan pl;
  plan_fwd(g_tune, pl, nullptr, T, H, V, dtype, true);
  return pl.bytes;
}

int fgrpo_logprob_fwd(const void* hidden, const void* weight, const void* bias, const int64_t* labels, float inv_temp,
                      int T, int H, int V, int dtype, float* lp_out, float* ent_out, float* lse_out, void* ws,
                      size_t ws_bytes, void* stream) {
  return logprob_fwd_impl(hidden, weight, bias, labels, inv_temp, T, H, V, dtype, lp_out, ent_out, lse_out, ws, ws_bytes,
                          stream);
}

int fgrpo_logprob_fwd_static(const void* hidden, const void* weight, const void* bias, const int64_t* labels,
                             float inv_temp, int T, int H, int V, int dtype, float* lp_out, float* ent_out,
                             float* lse_out, void* stream) {
  if (T <= 0 || H <= 0 || V <= 0) return fail(FGRPO_ERR_BAD_ARG, "logprob_fwd_static: T=%d H=%d V=%d", T, H, V);
  if (dtype != FGRPO_BF16 && dtype != FGRPO_F32) return fail(FGRPO_ERR_BAD_ARG, "logprob_fwd_static: dtype=%d", dtype);
  FwdPlan pl;
  plan_fwd(g_tune, pl, nullptr, T, H, V, dtype, bias != nullptr);
  if (pl.bytes > FGRPO_STATIC_SCRATCH_BYTES)
    return fail(FGRPO_ERR_WORKSPACE,
                "logprob_fwd_static: this call needs %zu bytes of scratch, the built-in buffer holds %u "
                "(use fgrpo_logprob_fwd with a caller workspace)", pl.bytes, (unsigned)FGRPO_STATIC_SCRATCH_BYTES);
  void* ptr = nullptr;
  int rc = static_scratch_ptr(&ptr);
  if (rc) return rc;
  return logprob_fwd_impl(hidden, weight, bias, labels, inv_temp, T, H, V, dtype, lp_out, ent_out, lse_out, ptr,
                          FGRPO_STATIC_SCRATCH_BYTES, stream);
}

size_t fgrpo_lmhead_bwd_workspace(int T, int H, int V, int dtype, long long hint) {
  if (T <= 0 || H <= 0 || V <= 0) return 0;
  BwdPlan pl;
  plan_bwd(g_tune, pl, nullptr, T, H, V, dtype, hint, true, true, true);
  return pl.bytes;
}

int fgrpo_lmhead_bwd_panel_cols(int T, int H, int V, int dtype, long long hint) {
  if (T <= 0 || H <= 0 || V <= 0) return fail(FGRPO_ERR_BAD_ARG, "lmhead_bwd_panel_cols: T=%d H=%d V=%d", T, H, V);
  BwdPlan pl;
  plan_bwd(g_tune, pl, nullptr, T, H, V, dtype, hint, true, true, true);
  return pl.panel;
}

int fgrpo_lmhead_bwd(const void* hidden, const void* weight, const void* bias, const int64_t* labels, const float* lse,
                     const float* g, const float* gout_dev, float inv_temp, int T, int H, int V, int dtype,
                     void* dH_out, void* dW_out, void* dbias_out, long long hint, void* ws, size_t ws_bytes,
                     void* stream) {
  hipStream_t st = (hipStream_t)stream;
  if (!hidden || !weight || !labels || !lse || !g) return fail(FGRPO_ERR_BAD_ARG, "lmhead_bwd: null argument");
  if (T <= 0 || H <= 0 || V <= 0) return fail(FGRPO_ERR_BAD_ARG, "lmhead_bwd: T=%d H=%d V=%d", T, H, V);
  if (dtype != FGRPO_BF16 && dtype != FGRPO_F32) return fail(FGRPO_ERR_BAD_ARG, "lmhead_bwd: dtype=%d", dtype);
  if (!(inv_temp > 0.f)) return fail(FGRPO_ERR_BAD_ARG, "lmhead_bwd: inv_temperature must be positive");
  if (!dH_out && !dW_out && !dbias_out) return 0;
  if (!ws || !aligned16(ws)) return fail(FGRPO_ERR_WORKSPACE, "lmhead_bwd: workspace null or misaligned");
  if (dbias_out && !bias) return fail(FGRPO_ERR_BAD_ARG, "lmhead_bwd: dbias requested without a bias");
  if (!aligned16(hidden) || !aligned16(weight)) return fail(FGRPO_ERR_ALIGN, "lmhead_bwd: hidden/weight must be 16-byte aligned");
  const bool want_dh = dH_out != nullptr, want_dw = dW_out != nullptr;
  const Tuning tn = g_tune;   // one reading of the tuning state per call
  BwdPlan pl;
  plan_bwd(tn, pl, ws, T, H, V, dtype, hint, bias != nullptr, want_dh, want_dw);
  if (pl.bytes > ws_bytes) return fail(FGRPO_ERR_WORKSPACE, "lmhead_bwd: workspace %zu < %zu bytes", ws_bytes, pl.bytes);
  const int f32 = pl.f32;

  DsParams d;
  memset(&d, 0, sizeof(d));
  int rc = stage_logit_operands(d.g, hidden, weight, T, H, V, dtype, pl.copy_ops, pl.Hp, pl.w_hi, pl.w_lo, pl.h_hi,
                                pl.h_lo, st);
  if (rc) return rc;
  rc = check_operands(d.g, kCfg[pl.variant].bk);
  if (rc) return rc;
  if (bias) {
    hipLaunchKernelGGL(to_f32_kernel, dim3((V + 255) / 256), dim3(256), 0, st, bias, f32, pl.bias32, V);
    HIP_TRY(hipGetLastError());
  }
  // contraction-major copies for the two gradient GEMMs
  if (want_dh && !pl.kmajor_dh) {
    rc = launch_convert(weight, f32, H, V, H, pl.Vpad, H, pl.wT_hi, pl.wT_lo, pl.Vpad, 1, st);
    if (rc) return rc;
  }
  if (want_dw && !pl.kmajor) {
    rc = launch_convert(hidden, f32, H, T, H, pl.Tpad, H, pl.hT_hi, pl.hT_lo, pl.Tpad, 1, st);
    if (rc) return rc;
  }
  d.bias = bias ? pl.bias32 : nullptr;
  d.labels = (const long long*)labels;
  d.lse = lse;
  d.gtok = g;
  d.gout = gout_dev;
  d.inv_temp = inv_temp;
  d.tiles_t = pl.tiles_t;
  d.group_t = tn.ds_group_t > 0 ? tn.ds_group_t : (tn.fwd_group_t > 0 ? tn.fwd_group_t : 1);
  d.tv_hi = pl.tv_hi;
  d.tv_lo = pl.tv_lo;
  d.vt_hi = pl.vt_hi;
  d.vt_lo = pl.vt_lo;
  d.ld_tv = pl.panel;
  d.ld_vt = pl.Tpad;
  // in-place mode keeps the [token][vocab] panel as 256-column blocks: the dW GEMM then streams each block
  // top to bottom, and the dH GEMM reads 128 KiB contiguous pieces
  const long long tv_blk = pl.kmajor ? (long long)pl.Tpad * 256 : 0;
  d.tv_blk = tv_blk;

  for (int pi = 0; pi < pl.npanels; ++pi) {
    const int v0 = pi * pl.panel;
    const int rows = (V - v0) < pl.panel ? (V - v0) : pl.panel;
    d.v0 = v0;
    d.tiles_v = (rows + pl.bm - 1) / pl.bm;
    d.nsplit = choose_nsplit(pl.tiles_t, d.tiles_v, num_cus() * kCfg[pl.variant].wgs_per_cu,
                             tn.ds_nsplit > 0 ? tn.ds_nsplit : tn.fwd_nsplit, 8);
    d.group_t = tn.ds_group_t > 0 ? tn.ds_group_t
                : d.nsplit == 8        ? 2       // 2 token tiles x 8 splits: half an XCD's work-groups per patch
                : tn.fwd_group_t > 0 ? tn.fwd_group_t : 1;
    const int kv = d.tiles_v * pl.bm;        // written panel width
    const int kt = pl.tiles_t * pl.bn;       // written token extent
    {
      PhaseScope ph(kPhaseDlogits, st);
      rc = launch_ds_variant(pl.variant, f32 != 0, d, st);
    }
    if (rc) return rc;

    if (want_dh) {  // dH[T x H] (+)= dS_tv[T x kv] * W^T[H x kv]^T
      StoreParams s;
      memset(&s, 0, sizeof(s));
      s.g.M = T;
      s.g.N = H;
      s.g.lda = tv_blk ? 256 : pl.panel;
      s.g.a_blk = tv_blk;
      s.g.ldb = pl.Vpad;
      if (pl.kmajor_dh) {  // B = W[v0 + k][h] read in place; vocabulary rows past V do not exist
        s.g.nseg = 1;
        s.g.seg[0] = GemmSeg{pl.tv_hi, (const bf16_t*)weight + (size_t)v0 * H, kv};
        s.g.ldb = H;
        s.g.kb_valid = rows;
      } else if (f32) {
        s.g.nseg = 3;
        s.g.seg[0] = GemmSeg{pl.tv_hi, pl.wT_hi + v0, kv};
        s.g.seg[1] = GemmSeg{pl.tv_hi, pl.wT_lo + v0, kv};
        s.g.seg[2] = GemmSeg{pl.tv_lo, pl.wT_hi + v0, kv};
      } else {
        s.g.nseg = 1;
        s.g.seg[0] = GemmSeg{pl.tv_hi, pl.wT_hi + v0, kv};
      }
      s.ldc = H;
      s.alpha = 1.f;
      const bool first = (pi == 0), last = (pi == pl.npanels - 1);
      if (f32) {  // accumulate in the fp32 output itself
        s.c_in = first ? nullptr : (const float*)dH_out;
        s.c_out_f32 = (float*)dH_out;
      } else if (pl.npanels == 1) {
        s.c_out_bf16 = (bf16_t*)dH_out;
      } else {
        s.c_in = first ? nullptr : pl.dh_acc;
        if (last)
          s.c_out_bf16 = (bf16_t*)dH_out;
        else
          s.c_out_f32 = pl.dh_acc;
      }
      {
        PhaseScope ph(kPhaseDh, st);
        rc = pl.kmajor_dh ? run_store_gemm_kmajor(tn, s, false, true, st) : run_store_gemm(tn, s, tn.gemm_variant, st);
      }
      if (rc) return rc;
    }
    if (want_dw) {  // dW[v0 : v0+rows, H] = dS_vt[rows x kt] * hidden^T[H x kt]^T
      StoreParams s;
      memset(&s, 0, sizeof(s));
      s.g.M = rows;
      s.g.N = H;
      s.g.lda = pl.Tpad;
      s.g.ldb = pl.Tpad;
      if (pl.kmajor) {  // A = dS[t][v] and B = hidden[t][h], both read in place with t as the contraction index
        s.g.nseg = 1;
        s.g.seg[0] = GemmSeg{pl.tv_hi, (const bf16_t*)hidden, kt};
        s.g.lda = 256;
        s.g.a_blk = tv_blk;
        s.g.ldb = H;
        s.g.kb_valid = T;
      } else if (f32) {
        s.g.nseg = 3;
        s.g.seg[0] = GemmSeg{pl.vt_hi, pl.hT_hi, kt};
        s.g.seg[1] = GemmSeg{pl.vt_hi, pl.hT_lo, kt};
        s.g.seg[2] = GemmSeg{pl.vt_lo, pl.hT_hi, kt};
      } else {
        s.g.nseg = 1;
        s.g.seg[0] = GemmSeg{pl.vt_hi, pl.hT_hi, kt};
      }
      s.ldc = H;
      s.alpha = 1.f;
      if (f32)
        s.c_out_f32 = (float*)dW_out + (size_t)v0 * H;
      else
        s.c_out_bf16 = (bf16_t*)dW_out + (size_t)v0 * H;
      {
        PhaseScope ph(kPhaseDw, st);
        rc = pl.kmajor ? run_store_gemm_kmajor(tn, s, true, true, st) : run_store_gemm(tn, s, tn.gemm_variant, st);
      }
      if (rc) return rc;
    }
    if (dbias_out) {
      float* o32 = f32 ? (float*)dbias_out + v0 : nullptr;
      bf16_t* o16 = f32 ? nullptr : (bf16_t*)dbias_out + v0;
      if (pl.kmajor)
        hipLaunchKernelGGL(panel_col_sum_kernel, dim3((rows + 63) / 64), dim3(256), 0, st, pl.tv_hi, pl.tv_lo,
                           (long long)pl.panel, tv_blk, T, rows, o32, o16);
      else
        hipLaunchKernelGGL(panel_row_sum_kernel, dim3((rows + 3) / 4), dim3(256), 0, st, pl.vt_hi, pl.vt_lo,
                           (long long)pl.Tpad, rows, T, o32, o16);
      HIP_TRY(hipGetLastError());
    }
  }
  return 0;
}

int fgrpo_keep_supported(int T, int H, int V, int dtype) { return keep_supported(g_tune, T, H, V, dtype) ? 1 : 0; }

size_t fgrpo_logits_keep_bytes(int T, int V) { return (T > 0 && V > 0) ? keep_bytes(T, V) : 0; }

int fgrpo_logprob_fwd_keep(const void* hidden, const void* weight, const void* bias, const int64_t* labels,
                           float inv_temp, int T, int H, int V, int dtype, float* lp_out, float* ent_out,
                           float* lse_out, void* logits_keep, size_t logits_keep_bytes, void* ws, size_t ws_bytes,
                           void* stream) {
  if (T <= 0 || H <= 0 || V <= 0) return fail(FGRPO_ERR_BAD_ARG, "logprob_fwd_keep: T=%d H=%d V=%d", T, H, V);
  if (!keep_supported(g_tune, T, H, V, dtype))
    return fail(FGRPO_ERR_UNSUPPORTED, "logprob_fwd_keep: needs bf16, H %% 64 == 0 and V/256 x H/256 tiles for half the CUs (T=%d H=%d V=%d)", T, H, V);
  if (!logits_keep || !aligned16(logits_keep) || logits_keep_bytes < keep_bytes(T, V))
    return fail(FGRPO_ERR_WORKSPACE, "logprob_fwd_keep: logits buffer null, misaligned or smaller than %zu bytes", keep_bytes(T, V));
  return logprob_fwd_impl(hidden, weight, bias, labels, inv_temp, T, H, V, dtype, lp_out, ent_out, lse_out, ws, ws_bytes,
                          stream, logits_keep);
}

namespace {
// Vocabulary panels of the kept-logits backward.  One by default: each gradient GEMM is a single launch over the
// whole vocabulary, dH is written once and nothing is accumulated (measured at T=32768, H=1536, V=151936:
// 1 or 2 panels 26.8 ms, 7 panels 27.2, 10 panels 30.7).  The tuning key keep_panels splits them.
void kept_panels(const Tuning& tn, int T, int H, int V, int& panel, int& npanels) {
  (void)T;
  (void)H;
  int np = tn.keep_panels > 0 ? tn.keep_panels : 1;
  const int max_np = (V + 255) / 256;
  np = np < 1 ? 1 : (np > max_np ? max_np : np);
  panel = (int)round_up((V + np - 1) / np, 256);
  npanels = (V + panel - 1) / panel;
}
}  // namespace

namespace {
// dHidden's tiles come in device rounds (one 256 x 256 tile per CU, each walking the whole vocabulary: 3.4 ms at
// V = 151936, H = 1536); a token count just past a whole number of rounds (T = 33000: 129 x 6 tiles = 3.02 rounds)
// would spend a fourth round on a handful of CUs (measured 14.1 ms against 10.3 at T = 32768).  Plan: row tiles
// [0, main_tiles) as whole tiles in whole rounds; the others' contraction in ksplit pieces of kchunk columns, a
// work-group each (at most kDhPartRounds per CU, which bounds the fp32 tiles they write); then a fixed-order sum of
// the pieces.  The plan is taken when its rounds are at least 5 % fewer (T = 33000: 11.2 ms, 24000: 8.3 against
// 10.4, 12000: 4.1 against 6.9; a last round that is half full gains little, the device is power-limited and
// gives the CUs that do run more clock).
struct DhSplitPlan {
  int main_tiles;   // == tiles_m: no split
  int ksplit, kchunk;
};
constexpr int kDhPartRounds = 8;      // fp32 tiles the split contraction may write: this many per CU (the workspace is sized from the plan)
DhSplitPlan plan_tail_split(int T, int H, int kv, double* rounds_out = nullptr) {
  const int tiles_m = (T + 255) / 256, tiles_n = (H + 255) / 256, slots = num_cus(), per_xcd = slots / 8;
  DhSplitPlan d{tiles_m, 1, 0};
  if (rounds_out) *rounds_out = (double)(((long long)tiles_m * tiles_n + slots - 1) / slots);
  if (H % 4 != 0 || tiles_n > per_xcd) return d;
  // time in device rounds of whole tiles.  Whole-tile launches deal row tiles round-robin to the 8 XCDs (or hand
  // each a contiguous range): an XCD runs its share x tiles_n work-groups on slots / 8 CUs.
  auto whole_rounds = [&](int row_tiles) { return ((row_tiles + 7) / 8 * tiles_n + per_xcd - 1) / per_xcd; };
  const int blocks = (kv + 255) / 256;                         // 256-column blocks of the contraction
  double best = (double)whole_rounds(tiles_m);
  const int full = tiles_m * tiles_n / slots;
  // candidates: the last partial round alone in pieces (after `full` or `full - 1` whole rounds), or every tile in
  // pieces - then the launch's work is a whole number of pieces whatever the tile count (T = 16384, H = 3584: 896
  // tiles = 3.5 rounds, four as whole tiles; as 1792 half contractions seven rounds of half the length)
  int mains[3] = {8 * (full * per_xcd / tiles_n), full > 0 ? 8 * ((full - 1) * per_xcd / tiles_n) : 0, 0};
  for (int c = 0; c < 3; ++c) {
    const int main_tiles = mains[c];
    if (c > 0 && main_tiles == mains[c - 1]) continue;
    const int tail = (tiles_m - main_tiles) * tiles_n;
    if (tail <= 0) continue;
    for (int ks = 2; ks <= 16 && tail * ks <= kDhPartRounds * slots; ++ks) {
      const int per = (blocks + ks - 1) / ks;
      if (per < 8) break;                                      // pieces under 32 K steps are not worth their tile store
      const int pieces = (blocks + per - 1) / per;
      const double cost = whole_rounds(main_tiles) + (double)((tail * pieces + slots - 1) / slots) * per / blocks + 0.03;
      if (cost < best * 0.95) {
        best = cost;
        d.main_tiles = main_tiles;
        d.ksplit = pieces;
        d.kchunk = per * 256;
      }
    }
  }
  if (rounds_out) *rounds_out = best;
  return d;
}
// Row length of the scaled, transposed copy of hidden: the padded token count plus 192 elements.  Rows 2 * Tpad bytes
// apart (a multiple of 512, at T = 32768 exactly 64 KiB) all start in the same memory channel, and a tile of the dW
// product reads 256 of them side by side.  Measured on that product at T = 32768, H = 1536: no padding 11.03 ms,
// 64 bytes 11.86 (rows then straddle 128-byte lines), 128 bytes 10.69, 256 / 384 / 640 / 2176 bytes 10.55-10.59.
long long kept_hs_ld(int T) { return round_up(T, 256) + 192; }

// Workspace of the kept-numerators backward, laid out from the tuning state the call itself will use: the fp32 dH
// accumulator exists only when the products are split into vocabulary panels, the fp32 tiles of the split
// contraction only when the plan takes it.
struct KeptBwdPlan {
  int panel, npanels;     // vocabulary panels of the two products
  DhSplitPlan split;      // of dHidden's last row tiles (one panel only)
  float* row_scale;       // [T]
  int* k_runs;            // live runs of the token axis for the dW product
  int* m_tile_live;       // live 256-row tiles for the dH product
  bf16_t* hidden_scaled;  // [H x (Tpad + 192)]: diag(a) hidden, transposed (the token contiguous), zero from T to Tpad
  float* dh_acc;          // [T x H] fp32, panels > 1 only
  float* dh_part;         // fp32 tiles of the split contraction of dHidden's last row tiles
  float* bias32;          // [V] fp32 copy of the bias for the recomputing fall-back
  size_t bytes;
};
void plan_kept_bwd(const Tuning& tn, KeptBwdPlan& pl, void* ws, int T, int H, int V, bool has_bias, bool want_dh,
                   bool want_dw) {
  kept_panels(tn, T, H, V, pl.panel, pl.npanels);
  const int tiles_m = (T + 255) / 256;
  pl.split = (want_dh && pl.npanels == 1 && tn.tail_split != 0) ? plan_tail_split(T, H, (int)round_up(V, 256))
                                                                : DhSplitPlan{tiles_m, 1, 0};
  Carver cv(ws);
  pl.row_scale = cv.take<float>((size_t)T);
  pl.k_runs = cv.take<int>((size_t)(2 + 2 * kRunCap));
  pl.m_tile_live = cv.take<int>((size_t)tiles_m);
  pl.hidden_scaled = want_dw ? cv.take<bf16_t>((size_t)H * kept_hs_ld(T)) : nullptr;
  pl.dh_acc = (want_dh && pl.npanels > 1) ? cv.take<float>((size_t)T * H) : nullptr;
  pl.dh_part = pl.split.ksplit > 1 ? cv.take<float>((size_t)pl.split.ksplit * (T - pl.split.main_tiles * 256) * H) : nullptr;
  pl.bias32 = has_bias ? cv.take<float>((size_t)V) : nullptr;
  pl.bytes = cv.total();
}

// Where the products of one call go when the caller walks the tokens in chunks: dW (and dbias) are sums over all
// tokens, carried in fp32 from chunk to chunk.
struct KeptBwdSums {
  const float* dw_in = nullptr;     // [V x H] fp32 sum of the earlier chunks, or null
  float* dw_out_f32 = nullptr;      // where the sum goes on (null: this is the last chunk, dW_out takes it in `dtype`)
  const float* db_in = nullptr;     // the same for dbias [V]
  float* db_out_f32 = nullptr;
};

int kept_bwd_impl(const Tuning& tn, const void* hidden, const void* weight, const void* bias, const int64_t* labels,
                  const float* lse, const float* g, const float* gout_dev, float inv_temp, int T, int H, int V,
                  void* logits_keep, void* dH_out, void* dW_out, void* dbias_out, const KeptBwdSums& sums, void* ws,
                  size_t ws_bytes, hipStream_t st, const KeepAux* aux_in = nullptr) {
  const bool want_dh = dH_out != nullptr, want_dw = dW_out != nullptr || sums.dw_out_f32 != nullptr;
  const bool want_db = dbias_out != nullptr || sums.db_out_f32 != nullptr;
  KeptBwdPlan pl;
  plan_kept_bwd(tn, pl, ws, T, H, V, bias != nullptr, want_dh, want_dw);
  if (!ws || !aligned16(ws) || ws_bytes < pl.bytes)
    return fail(FGRPO_ERR_WORKSPACE, "lmhead_bwd_kept: workspace null, misaligned or smaller than %zu bytes", pl.bytes);
  const int Tpad = (int)round_up(T, 256);
  const long long blk = (long long)Tpad * 256;
  bf16_t* ek = (bf16_t*)logits_keep;
  const int panel = pl.panel, npanels = pl.npanels;
  const KeepAux aux = aux_in ? *aux_in : keep_aux_of(logits_keep, T, V);
  int* flag = aux.flag;
  // rows without a gradient (zero advantage, ignored label) are skipped by 256-row tile (dH) and 64-row K step (dW)
  const bool skip_dead = tn.keep_skip_dead != 0 && (T + 63) / 64 <= kLiveMaxChunks;

  {
    PhaseScope ph(kPhaseDlogits, st);
    KeepPrepParams k{ek, blk, aux.ref2, aux.xy, (const long long*)labels, lse, g, gout_dev, inv_temp,
                     (const bf16_t*)hidden, T, H, V, pl.row_scale, flag};
    hipLaunchKernelGGL(keep_backward_prep_kernel, dim3((T + 3) / 4), dim3(256), 0, st, k);
    HIP_TRY(hipGetLastError());
    {
      // Out-of-range batches (the forward raised the buffer's flag): the decision is taken on the device.  This launch
      // returns at once unless the flag is set; when it is, it overwrites the whole buffer with dLogits recomputed
      // from the operands (the kernel of the recomputing backward, one panel over the whole vocabulary, same
      // layout), and the prep kernel above has set the row factors to 1: the products below then are that backward.
      DsParams d;
      memset(&d, 0, sizeof(d));
      int rc = stage_logit_operands(d.g, hidden, weight, T, H, V, FGRPO_BF16, false, H, nullptr, nullptr, nullptr, nullptr, st);
      if (rc) return rc;
      if (bias) {
        hipLaunchKernelGGL(to_f32_kernel, dim3((V + 255) / 256), dim3(256), 0, st, bias, 0, pl.bias32, V);
        HIP_TRY(hipGetLastError());
      }
      d.bias = bias ? pl.bias32 : nullptr;
      d.labels = (const long long*)labels;
      d.lse = lse;
      d.gtok = g;
      d.gout = gout_dev;
      d.inv_temp = inv_temp;
      d.v0 = 0;
      d.tiles_t = Tpad / 256;
      d.tiles_v = (V + 255) / 256;
      d.nsplit = choose_nsplit(d.tiles_t, d.tiles_v, num_cus(), tn.ds_nsplit > 0 ? tn.ds_nsplit : tn.fwd_nsplit, 8);
      d.group_t = tn.ds_group_t > 0 ? tn.ds_group_t : d.nsplit == 8 ? 2 : tn.fwd_group_t > 0 ? tn.fwd_group_t : 1;
      d.tv_hi = ek;
      d.ld_tv = round_up(V, 256);
      d.tv_blk = blk;
      d.gate = flag;
      rc = launch_ds_variant(8, false, d, st);
      if (rc) return rc;
    }
    if (want_dw)
      hipLaunchKernelGGL(keep_scaled_transpose_kernel, dim3(Tpad / 64, H / 64), dim3(256), 0, st, (const bf16_t*)hidden,
                         (const float*)pl.row_scale, T, H, Tpad, kept_hs_ld(T), pl.hidden_scaled);
    if (skip_dead) {
      KeepLiveParams lv{pl.row_scale, T, (T + 63) / 64, Tpad / 64, pl.k_runs, pl.m_tile_live};
      hipLaunchKernelGGL(keep_live_runs_kernel, dim3(1), dim3(1024), 0, st, lv);
    }
  }
  HIP_TRY(hipGetLastError());

  int rc = 0;
  for (int pi = 0; pi < npanels; ++pi) {
    const int v0 = pi * panel;
    const int rows = (V - v0) < panel ? (V - v0) : panel;      // vocabulary rows of W / dW in this panel
    const int kv = (int)round_up(rows, 256);                   // columns of the panel (zero past V)
    bf16_t* ek_p = ek + (long long)(v0 / 256) * blk;
    if (want_dh) {   // dH[T x H] (+)= diag(a) E'[T x kv] W[v0 : v0+rows, H]: A column-blocked K-contiguous, B = W read in place
      StoreParams s;
      memset(&s, 0, sizeof(s));
      s.g.M = T;
      s.g.N = H;
      s.g.lda = 256;
      s.g.a_blk = blk;
      s.g.ldb = H;
      s.g.nseg = 1;
      s.g.seg[0] = GemmSeg{ek_p, (const bf16_t*)weight + (size_t)v0 * H, kv};
      s.g.kb_valid = rows;
      s.ldc = H;
      s.alpha = 1.f;
      s.row_scale = pl.row_scale;
      s.m_tile_live = skip_dead ? pl.m_tile_live : nullptr;
      const bool first = (pi == 0), last = (pi == npanels - 1);
      s.c_in = first ? nullptr : pl.dh_acc;
      if (last)
        s.c_out_bf16 = (bf16_t*)dH_out;
      else
        s.c_out_f32 = pl.dh_acc;
      {
        // raster: the work-groups that share a tile of the [T x V] buffer (all tiles across H) run side by side,
        // so each XCD streams its rows of the buffer once (measured against groups of 4: dH 11.3 vs 11.5 ms,
        // dW 11.7 vs 12.1 at T=32768, H=1536, V=151936)
        PhaseScope ph(kPhaseDh, st);
        const DhSplitPlan sp = pl.split;
        if (sp.ksplit <= 1) {
          rc = run_store_gemm_kmajor(tn, s, false, true, st, skip_dead ? -1 : 1);
        } else {
          // whole rounds of whole tiles, then the last row tiles with their contraction in pieces, then the sum
          const int r0 = sp.main_tiles * 256, tr = T - r0;
          if (r0 > 0) {
            StoreParams m = s;
            m.g.M = r0;
            rc = run_store_gemm_kmajor(tn, m, false, true, st, skip_dead ? -1 : 1);
            if (rc) return rc;
          }
          StoreParams t = s;
          t.g.M = tr;
          t.g.seg[0].A = ek_p + (long long)r0 * 256;               // row r0 of every 256-column block
          t.c_out_bf16 = nullptr;
          t.c_out_f32 = pl.dh_part;
          t.row_scale = nullptr;                                    // applied once, to the sum
          t.m_tile_live = skip_dead ? pl.m_tile_live + sp.main_tiles : nullptr;
          t.ksplit = sp.ksplit;
          t.kchunk = sp.kchunk;
          t.part_slice = (long long)tr * H;
          t.tiles_m = (tr + 255) / 256;
          t.tiles_n = (H + 255) / 256;
          t.nblocks = t.tiles_m * t.tiles_n * sp.ksplit;
          t.wide_stores = can_store_wide(tn, t);
          rc = launch_store_splitk(t, st);
          if (rc) return rc;
          const long long quads = (long long)tr * (H / 4);
          hipLaunchKernelGGL(splitk_reduce_kernel, dim3((unsigned)((quads + 255) / 256)), dim3(256), 0, st,
                             (const float*)pl.dh_part, sp.ksplit, t.part_slice, tr, H, (long long)H,
                             (const float*)pl.row_scale + r0, (bf16_t*)dH_out + (size_t)r0 * H);
          HIP_TRY(hipGetLastError());
        }
      }
      if (rc) return rc;
    }
    if (want_dw) {  // dW[v0 : v0+rows, H] = E'^T[rows x Tpad] (diag(a) hidden)^T[H x Tpad]^T: A read where the forward left it
                    // (the token is its row), B a token-contiguous copy, so that only A needs transposing LDS reads
      StoreParams s;
      memset(&s, 0, sizeof(s));
      s.g.M = rows;
      s.g.N = H;
      s.g.lda = 256;
      s.g.a_blk = blk;
      s.g.ldb = kept_hs_ld(T);
      s.g.nseg = 1;
      s.g.seg[0] = GemmSeg{ek_p, pl.hidden_scaled, Tpad};
      s.g.ka_valid = T;
      s.g.k_runs = skip_dead ? pl.k_runs : nullptr;
      s.ldc = H;
      s.alpha = 1.f;
      s.c_in = sums.dw_in ? sums.dw_in + (size_t)v0 * H : nullptr;
      if (sums.dw_out_f32)
        s.c_out_f32 = sums.dw_out_f32 + (size_t)v0 * H;
      else
        s.c_out_bf16 = (bf16_t*)dW_out + (size_t)v0 * H;
      {
        PhaseScope ph(kPhaseDw, st);
        rc = run_store_gemm_kmajor(tn, s, true, false, st, 1);
      }
      if (rc) return rc;
    }
  }
  if (want_db) {
    PhaseScope ph(kPhaseOther, st);
    hipLaunchKernelGGL(keep_col_sum_kernel, dim3((V + 63) / 64), dim3(256), 0, st, ek, blk, pl.row_scale, T, V,
                       sums.db_in, sums.db_out_f32, sums.db_out_f32 ? nullptr : (bf16_t*)dbias_out);
    HIP_TRY(hipGetLastError());
  }
  return 0;
}
}  // namespace

size_t fgrpo_lmhead_bwd_kept_workspace(int T, int H, int V, int dtype) {
  if (T <= 0 || H <= 0 || V <= 0 || dtype != FGRPO_BF16) return 0;
  KeptBwdPlan pl;
  plan_kept_bwd(g_tune, pl, nullptr, T, H, V, true, true, true);
  return pl.bytes;
}

int fgrpo_keep_overflowed(const void* logits_keep, int T, int V, void* stream) {
  if (!logits_keep || T <= 0 || V <= 0) return fail(FGRPO_ERR_BAD_ARG, "keep_overflowed: bad argument");
  int flag = 0;
  HIP_TRY(hipMemcpyAsync(&flag, keep_flag_of(const_cast<void*>(logits_keep), T, V), sizeof(int), hipMemcpyDeviceToHost,
                         (hipStream_t)stream));
  HIP_TRY(hipStreamSynchronize((hipStream_t)stream));
  return flag != 0 ? 1 : 0;
}

int fgrpo_lmhead_bwd_kept(const void* hidden, const void* weight, const void* bias, const int64_t* labels,
                          const float* lse, const float* g, const float* gout_dev, float inv_temp, int T, int H, int V,
                          int dtype, void* logits_keep, size_t logits_keep_bytes, void* dH_out, void* dW_out,
                          void* dbias_out, void* ws, size_t ws_bytes, void* stream) {
  if (!hidden || !weight || !labels || !lse || !g) return fail(FGRPO_ERR_BAD_ARG, "lmhead_bwd_kept: null argument");
  if (T <= 0 || H <= 0 || V <= 0) return fail(FGRPO_ERR_BAD_ARG, "lmhead_bwd_kept: T=%d H=%d V=%d", T, H, V);
  if (!(inv_temp > 0.f)) return fail(FGRPO_ERR_BAD_ARG, "lmhead_bwd_kept: inv_temperature must be positive");
  const Tuning tn = g_tune;
  if (!keep_supported(tn, T, H, V, dtype))
    return fail(FGRPO_ERR_UNSUPPORTED, "lmhead_bwd_kept: needs bf16, H %% 64 == 0 and V/256 x H/256 tiles for half the CUs (T=%d H=%d V=%d)", T, H, V);
  if (!logits_keep || !aligned16(logits_keep) || logits_keep_bytes < keep_bytes(T, V))
    return fail(FGRPO_ERR_WORKSPACE, "lmhead_bwd_kept: kept buffer null, misaligned or smaller than %zu bytes", keep_bytes(T, V));
  if (dbias_out && !bias) return fail(FGRPO_ERR_BAD_ARG, "lmhead_bwd_kept: dbias requested without a bias");
  if (!aligned16(hidden) || !aligned16(weight)) return fail(FGRPO_ERR_ALIGN, "lmhead_bwd_kept: hidden/weight must be 16-byte aligned");
  if (!dH_out && !dW_out && !dbias_out) return 0;
  return kept_bwd_impl(tn, hidden, weight, bias, labels, lse, g, gout_dev, inv_temp, T, H, V, logits_keep, dH_out, dW_out,
                       dbias_out, KeptBwdSums{}, ws, ws_bytes, (hipStream_t)stream);
}

int fgrpo_phase_timing_begin(void) {
  std::lock_guard<std::mutex> lock(g_phase_mu);
  PhaseTimer& t = g_phase;
  if (!t.created) {
    for (int i = 0; i < 2 * FGRPO_MAX_TIMED_PHASES; ++i) HIP_TRY(hipEventCreate(&t.ev[i]));
    t.created = true;
  }
  t.n = t.dropped = 0;
  t.on = true;
  return 0;
}

int fgrpo_phase_timing_end(float* ms_by_phase, int* brackets_by_phase) {
  std::lock_guard<std::mutex> lock(g_phase_mu);
  PhaseTimer& t = g_phase;
  if (!t.on) return fail(FGRPO_ERR_BAD_ARG, "phase_timing_end without phase_timing_begin");
  t.on = false;
  if (!ms_by_phase || !brackets_by_phase) return fail(FGRPO_ERR_BAD_ARG, "phase_timing_end: null argument");
  for (int k = 0; k < FGRPO_NUM_PHASES; ++k) ms_by_phase[k] = 0.f, brackets_by_phase[k] = 0;
  if (t.n > 0) HIP_TRY(hipEventSynchronize(t.ev[2 * (t.n - 1) + 1]));
  for (int i = 0; i < t.n; ++i) {
    float ms = 0.f;
    HIP_TRY(hipEventElapsedTime(&ms, t.ev[2 * i], t.ev[2 * i + 1]));
    const int k = (t.kind[i] >= 0 && t.kind[i] < FGRPO_NUM_PHASES) ? t.kind[i] : kPhaseOther;
    ms_by_phase[k] += ms;
    ++brackets_by_phase[k];
  }
  return t.dropped;
}

size_t fgrpo_loss_fwd_workspace(int T, int nseq) {
  if (T <= 0) return 0;
  Carver cv(nullptr);
  cv.take<double>(2 * (size_t)((T + kLossThreads - 1) / kLossThreads));
  cv.take<float>((size_t)T);
  cv.take<int>((size_t)(nseq > 0 ? nseq : 1));
  return cv.total();
}

int fgrpo_loss_fwd(const float* lp, const float* old_lp, const float* ref_lp, const float* adv, const int64_t* labels,
                   const int32_t* cu, int nseq, int T, float clip_low, float clip_high, float clip_c, float kl_beta,
                   int agg_mode, double denom_override, float* loss_out, float* g_out, float* log_ratio, float* clip1,
                   float* unclipped, float* clipped, float* scal_out, void* ws, size_t ws_bytes, void* stream) {
  hipStream_t st = (hipStream_t)stream;
  if (!lp || !adv || !labels || !loss_out || !g_out) return fail(FGRPO_ERR_BAD_ARG, "loss_fwd: null argument");
  if (T <= 0) return fail(FGRPO_ERR_BAD_ARG, "loss_fwd: T=%d", T);
  if (agg_mode != FGRPO_AGG_TOKEN_MEAN && agg_mode != FGRPO_AGG_SAMPLE_MEAN)
    return fail(FGRPO_ERR_BAD_ARG, "loss_fwd: agg_mode=%d", agg_mode);
  if (agg_mode == FGRPO_AGG_SAMPLE_MEAN && (!cu || nseq <= 0))
    return fail(FGRPO_ERR_BAD_ARG, "loss_fwd: sample_mean needs cu_seqlens");
  if (!ws || !aligned16(ws) || ws_bytes < fgrpo_loss_fwd_workspace(T, nseq))
    return fail(FGRPO_ERR_WORKSPACE, "loss_fwd: workspace too small");
  const int nblocks = (T + kLossThreads - 1) / kLossThreads;
  Carver cv(ws);
  LossParams p;
  memset(&p, 0, sizeof(p));
  p.partial = cv.take<double>(2 * (size_t)nblocks);
  float* tokw = cv.take<float>((size_t)T);
  int* segc = cv.take<int>((size_t)(nseq > 0 ? nseq : 1));
  p.lp = lp;
  p.old_lp = old_lp;
  p.ref_lp = ref_lp;
  p.adv = adv;
  p.labels = (const long long*)labels;
  p.T = T;
  p.clip_low = clip_low;
  p.clip_high = clip_high;
  p.clip_c = clip_c;
  p.kl_beta = kl_beta;
  p.agg_mode = agg_mode;
  p.denom_override = denom_override;
  p.g = g_out;
  p.log_ratio = log_ratio;
  p.clip1 = clip1;
  p.unclipped = unclipped;
  p.clipped = clipped;
  p.loss = loss_out;
  p.scal = scal_out;
  if (agg_mode == FGRPO_AGG_SAMPLE_MEAN) {
    // tokens outside every segment keep weight 0
    hipLaunchKernelGGL(fill_f32_kernel, dim3((T + 255) / 256), dim3(256), 0, st, tokw, 0.f, T);
    HIP_TRY(hipGetLastError());
    hipLaunchKernelGGL(segment_valid_weight_kernel, dim3((nseq + 3) / 4), dim3(256), 0, st, p.labels, cu, nseq, T, segc,
                       tokw);
    HIP_TRY(hipGetLastError());
    p.tokw = tokw;
    p.seg_cnt = segc;
    p.nseq = nseq;
  }
  hipLaunchKernelGGL(grpo_loss_tokens_kernel, dim3(nblocks), dim3(kLossThreads), 0, st, p);
  HIP_TRY(hipGetLastError());
  hipLaunchKernelGGL(grpo_loss_finalize_kernel, dim3(std::min(nblocks, kFinalizeBlocks)), dim3(kLossThreads), 0, st, p, nblocks);
  HIP_TRY(hipGetLastError());
  return 0;
}

int fgrpo_loss_prepare(const int64_t* labels, const int32_t* cu, int nseq, int T, int agg_mode, double denom_override,
                       float* tokw_out, int32_t* seg_cnt_out, double* pre_out, void* stream) {
  hipStream_t st = (hipStream_t)stream;
  if (!labels || !pre_out || T <= 0) return fail(FGRPO_ERR_BAD_ARG, "loss_prepare: bad argument");
  if (agg_mode != FGRPO_AGG_TOKEN_MEAN && agg_mode != FGRPO_AGG_SAMPLE_MEAN)
    return fail(FGRPO_ERR_BAD_ARG, "loss_prepare: agg_mode=%d", agg_mode);
  const bool by_sample = agg_mode == FGRPO_AGG_SAMPLE_MEAN;
  if (by_sample && (!cu || nseq <= 0 || !tokw_out || !seg_cnt_out))
    return fail(FGRPO_ERR_BAD_ARG, "loss_prepare: sample_mean needs cu_seqlens, tokw_out and seg_cnt_out");
  if (by_sample) {
    // tokens outside every segment keep weight 0
    hipLaunchKernelGGL(fill_f32_kernel, dim3((T + 255) / 256), dim3(256), 0, st, tokw_out, 0.f, T);
    HIP_TRY(hipGetLastError());
    hipLaunchKernelGGL(segment_valid_weight_kernel, dim3((nseq + 3) / 4), dim3(256), 0, st, (const long long*)labels, cu,
                       nseq, T, seg_cnt_out, tokw_out);
    HIP_TRY(hipGetLastError());
  }
  hipLaunchKernelGGL(grpo_loss_prepare_kernel, dim3(1), dim3(1024), 0, st, (const long long*)labels, T,
                     by_sample ? (const int*)seg_cnt_out : nullptr, by_sample ? nseq : 0, agg_mode, denom_override, pre_out);
  HIP_TRY(hipGetLastError());
  return 0;
}

extern "C++" {
namespace {
// Token chunks of the chunked step.  The caller's bound is rounded down to whole 256-token tiles; under it three ways
// of cutting T tokens are weighed: the tokens dealt evenly over the chunks the bound needs; whole chunks of the bound
// and one shorter chunk for the rest; or whole chunks, with the last of them and the rest dealt evenly over two.
// What decides is how the chunks' tile counts fall on the device: T = 33000 is 129 token tiles; five chunks of 26 give
// the forward 26 x 9 = 234 work-groups per launch (a tenth of the CUs idle, measured 38.1 ms/step); four chunks of 32
// run at the full-device shape but leave one tile that pays a whole pass over the dW sums (36.5 ms); three of 32 and
// two of 17 and 16 avoid both.  The estimate counts K steps of 64 per CU: a forward tile H / 64 + its epilogue, a dHidden round V / 64 (in pieces
// where plan_tail_split says so), a dW tile tokens / 64 + the read-modify-write of its fp32 sums.
double chunk_cost_estimate(int cnt, int H, int V) {
  const int slots = num_cus();
  const int tiles_t = (cnt + 255) / 256, tiles_v = (V + 255) / 256, tiles_h = (H + 255) / 256;
  const int prefer = (16384LL * H * 2 > (192LL << 20)) ? 8 : 4;
  const int ns = choose_nsplit(tiles_t, tiles_v, slots, 0, prefer);
  const double fwd = (double)split_cost(tiles_t, tiles_v, slots, ns) * (H / 64.0 + 5.0);
  double dh_rounds = 0.0;
  (void)plan_tail_split(cnt, H, (int)round_up(V, 256), &dh_rounds);
  const double dh = dh_rounds * (round_up(V, 256) / 64.0 + 8.0);
  const double dw = (double)(((long long)tiles_v * tiles_h + slots - 1) / slots) * (round_up(cnt, 256) / 64.0 + 12.0);
  return fwd + dh + dw + 40.0;     // + the small launches of a chunk
}
// The chunks of a call, in token order (every size but the last a multiple of 256, none above the bound).
std::vector<int> chunk_sizes(const Tuning& tn, int T, int H, int V, int chunk_tokens) {
  long long c = chunk_tokens > 0 ? chunk_tokens : 8192;
  c = c / 256 * 256;
  if (c < 256) c = 256;
  if (c >= T) return std::vector<int>(1, T);
  const int n = (int)((T + c - 1) / c);
  const int even = (int)round_up((T + n - 1) / n, 256);
  auto cut = [&](int chunk, int nfull, std::initializer_list<int> tail) {
    std::vector<int> v((size_t)nfull, chunk);
    for (int t : tail)
      if (t > 0) v.push_back(t);
    return v;
  };
  std::vector<std::vector<int>> cand;
  cand.push_back(cut(even, (T - 1) / even, {T - (T - 1) / even * even}));          // the tokens dealt evenly
  const int full = (int)(T / c), rest = T - full * (int)c;
  if (even != c && H > 0 && V > 0) {
    cand.push_back(cut((int)c, full, {rest}));                                       // whole chunks and the rest
    if (rest > 0 && full >= 1) {                                                     // ... or the last whole chunk and the rest, halved
      const int h1 = (int)round_up(((int)c + rest + 1) / 2, 256);
      cand.push_back(cut((int)c, full - 1, {h1, (int)c + rest - h1}));
    }
  }
  size_t best = 0;
  double best_cost = -1.0;
  for (size_t i = 0; i < cand.size(); ++i) {
    bool ok = true;
    double cost = 0.0;
    int prev = -1;
    double prev_cost = 0.0;
    for (int sz : cand[i]) {
      if (sz != prev) {
        ok = ok && (i == 0 || keep_supported(tn, sz, H, V, FGRPO_BF16));   // a chunk the kernels would refuse rules a cut out
        prev_cost = (H > 0 && V > 0) ? chunk_cost_estimate(sz, H, V) : 0.0;
        prev = sz;
      }
      cost += prev_cost;
    }
    if (ok && (best_cost < 0.0 || cost < best_cost)) {
      best_cost = cost;
      best = i;
    }
  }
  return cand[best];
}
int fused_chunk_tokens(const Tuning& tn, int T, int H, int V, int chunk_tokens) {
  int m = 0;
  for (int sz : chunk_sizes(tn, T, H, V, chunk_tokens)) m = sz > m ? sz : m;
  return (int)round_up(m, 256);
}

struct ChunkedPlan {
  std::vector<int> sizes;   // tokens of each chunk, in order
  int chunk, nchunks;       // the largest chunk (whole tiles); number of chunks
  void* keep;
  size_t keep_bytes;
  void* fwd_ws;
  size_t fwd_bytes;
  void* bwd_ws;
  size_t bwd_bytes;
  float* dw_acc;
  float* db_acc;
  double* partial;
  // the kept forward's pre-pass, run once for the tokens of every chunk: references, target logits, one overflow
  // flag per chunk, and the scratch of the pass itself
  float *ref2, *xy, *pre_xt, *pre_bias32;
  int* flags;
  float4* pre_part;
  size_t bytes;
};
void plan_chunked(const Tuning& tn, ChunkedPlan& pl, void* ws, int T, int H, int V, int chunk_tokens, bool has_bias,
                  bool want_dh, bool want_dw, bool want_db) {
  pl.sizes = chunk_sizes(tn, T, H, V, chunk_tokens);
  pl.nchunks = (int)pl.sizes.size();
  pl.chunk = 0;
  for (int sz : pl.sizes) pl.chunk = sz > pl.chunk ? sz : pl.chunk;
  pl.keep_bytes = keep_bytes(pl.chunk, V);
  pl.fwd_bytes = pl.bwd_bytes = 0;
  int prev = -1;
  for (int cnt : pl.sizes) {
    if (cnt == prev) continue;
    prev = cnt;
    Tuning tf = tn;
    tf.fwd_variant = 8;
    FwdPlan fp;
    plan_fwd(tf, fp, nullptr, cnt, H, V, FGRPO_BF16, has_bias);
    if (fp.bytes > pl.fwd_bytes) pl.fwd_bytes = fp.bytes;
    KeptBwdPlan bp;
    plan_kept_bwd(tn, bp, nullptr, cnt, H, V, has_bias, want_dh, want_dw);
    if (bp.bytes > pl.bwd_bytes) pl.bwd_bytes = bp.bytes;
  }
  Carver cv(ws);
  pl.keep = cv.take<char>(pl.keep_bytes);
  pl.fwd_ws = cv.take<char>(pl.fwd_bytes);
  pl.bwd_ws = cv.take<char>(pl.bwd_bytes);
  pl.dw_acc = (want_dw && pl.nchunks > 1) ? cv.take<float>((size_t)V * H) : nullptr;
  pl.db_acc = (want_db && pl.nchunks > 1) ? cv.take<float>((size_t)V) : nullptr;
  pl.partial = cv.take<double>(2 * (size_t)((T + kLossThreads - 1) / kLossThreads));
  pl.ref2 = cv.take<float>((size_t)T);
  pl.xy = cv.take<float>((size_t)T);
  pl.flags = cv.take<int>((size_t)pl.nchunks);
  pl.pre_part = cv.take<float4>(2 * (size_t)T);
  pl.pre_xt = cv.take<float>((size_t)T);
  pl.pre_bias32 = has_bias ? cv.take<float>((size_t)V) : nullptr;
  pl.bytes = cv.total();
}
}  // namespace
}  // extern "C++"

namespace {
// every chunk - the full ones and the shorter last one - must be a problem the kept-numerators pair handles
bool chunked_supported(const Tuning& tn, int T, int H, int V, int dtype, int chunk_tokens) {
  if (T <= 0 || H <= 0 || V <= 0) return false;
  for (int sz : chunk_sizes(tn, T, H, V, chunk_tokens))
    if (!keep_supported(tn, sz, H, V, dtype)) return false;
  return true;
}
}  // namespace

int fgrpo_grpo_step_chunked_supported(int T, int H, int V, int dtype, int chunk_tokens) {
  return chunked_supported(g_tune, T, H, V, dtype, chunk_tokens) ? 1 : 0;
}

int fgrpo_grpo_step_chunk_tokens(int T, int H, int V, int chunk_tokens) {
  if (T <= 0 || H <= 0 || V <= 0) return fail(FGRPO_ERR_BAD_ARG, "grpo_step_chunk_tokens: T=%d H=%d V=%d", T, H, V);
  return fused_chunk_tokens(g_tune, T, H, V, chunk_tokens);
}

size_t fgrpo_grpo_step_chunked_workspace(int T, int H, int V, int dtype, int chunk_tokens) {
  if (T <= 0 || H <= 0 || V <= 0 || dtype != FGRPO_BF16) return 0;
  ChunkedPlan pl;
  plan_chunked(g_tune, pl, nullptr, T, H, V, chunk_tokens, true, true, true, true);
  return pl.bytes;
}

int fgrpo_grpo_step_chunked(const void* hidden, const void* weight, const void* bias, const int64_t* labels,
                            const float* old_lp, const float* ref_lp, const float* adv, const float* tokw,
                            const double* pre, float inv_temp, int T, int H, int V, int dtype, float clip_low,
                            float clip_high, float clip_c, float kl_beta, int chunk_tokens, float* lp_out, float* ent_out,
                            float* lse_out, float* loss_out, float* g_out, float* log_ratio, float* clip1,
                            float* unclipped, float* clipped, float* scal_out, void* dH_out, void* dW_out,
                            void* dbias_out, void* ws, size_t ws_bytes, void* stream) {
  hipStream_t st = (hipStream_t)stream;
  if (!hidden || !weight || !labels || !adv || !pre || !lp_out || !lse_out || !loss_out || !g_out)
    return fail(FGRPO_ERR_BAD_ARG, "grpo_step_chunked: null argument");
  if (T <= 0 || H <= 0 || V <= 0) return fail(FGRPO_ERR_BAD_ARG, "grpo_step_chunked: T=%d H=%d V=%d", T, H, V);
  if (!(inv_temp > 0.f)) return fail(FGRPO_ERR_BAD_ARG, "grpo_step_chunked: inv_temperature must be positive");
  if (dbias_out && !bias) return fail(FGRPO_ERR_BAD_ARG, "grpo_step_chunked: dbias requested without a bias");
  if (!aligned16(hidden) || !aligned16(weight)) return fail(FGRPO_ERR_ALIGN, "grpo_step_chunked: hidden/weight must be 16-byte aligned");
  const Tuning tn = g_tune;   // one reading of the tuning state per call
  ChunkedPlan pl;
  plan_chunked(tn, pl, ws, T, H, V, chunk_tokens, bias != nullptr, dH_out != nullptr, dW_out != nullptr, dbias_out != nullptr);
  if (!chunked_supported(tn, T, H, V, dtype, chunk_tokens))
    return fail(FGRPO_ERR_UNSUPPORTED, "grpo_step_chunked: every chunk needs bf16, H %% 64 == 0, V/256 x H/256 tiles for half the CUs and V/256 x tokens/256 tiles for half the CUs (T=%d H=%d V=%d, chunks of %d)", T, H, V, pl.chunk);
  if (!ws || !aligned16(ws) || ws_bytes < pl.bytes)
    return fail(FGRPO_ERR_WORKSPACE, "grpo_step_chunked: workspace null, misaligned or smaller than %zu bytes", pl.bytes);

  LossParams lp;
  memset(&lp, 0, sizeof(lp));
  lp.clip_low = clip_low;
  lp.clip_high = clip_high;
  lp.clip_c = clip_c;
  lp.kl_beta = kl_beta;
  lp.pre = pre;
  lp.loss = loss_out;
  lp.scal = scal_out;

  {
    // references of the kept numerators for the tokens of every chunk, in one pass before the first chunk
    // (timed with "everything else": the forward brackets then hold one forward launch and its merge each)
    PhaseScope ph(kPhaseOther, st);
    FwdParams bp;
    memset(&bp, 0, sizeof(bp));
    int rc = stage_logit_operands(bp.g, hidden, weight, T, H, V, dtype, false, H, nullptr, nullptr, nullptr, nullptr, st);
    if (rc) return rc;
    if (bias) {
      hipLaunchKernelGGL(to_f32_kernel, dim3((V + 255) / 256), dim3(256), 0, st, bias, 0, pl.pre_bias32, V);
      HIP_TRY(hipGetLastError());
    }
    bp.bias = bias ? pl.pre_bias32 : nullptr;
    bp.labels = (const long long*)labels;
    bp.inv_temp = inv_temp;
    bp.group_t = tn.fwd_group_t > 0 ? tn.fwd_group_t : 1;
    bp.xt = pl.pre_xt;
    rc = keep_prepass(bp, hidden, weight, labels, T, H, V, 2, pl.pre_part, KeepAux{pl.ref2, pl.xy, pl.flags, true},
                      pl.nchunks, st);
    if (rc) return rc;
  }
  const size_t esz = sizeof(bf16_t);
  std::vector<int> first(pl.sizes.size(), 0);          // first token of each chunk
  for (size_t i = 1; i < first.size(); ++i) first[i] = first[i - 1] + pl.sizes[i - 1];
  for (int ci = 0; ci < pl.nchunks; ++ci) {
    const int t0 = first[ci], cnt = pl.sizes[ci];
    const char* h_c = (const char*)hidden + (size_t)t0 * H * esz;
    const KeepAux aux{pl.ref2 + t0, pl.xy + t0, pl.flags + ci, true};
    int rc;
    {
      PhaseScope ph(kPhaseFwd, st);
      rc = logprob_fwd_impl(h_c, weight, bias, labels + t0, inv_temp, cnt, H, V, dtype, lp_out + t0,
                            ent_out ? ent_out + t0 : nullptr, lse_out + t0, pl.fwd_ws, pl.fwd_bytes, stream, pl.keep, &tn,
                            &aux);
    }
    if (rc) return rc;
    {
      // the objective on this chunk's tokens: the normaliser is known (pre), so g is final as it is written
      PhaseScope ph(kPhaseOther, st);
      LossParams q = lp;
      q.lp = lp_out + t0;
      q.old_lp = old_lp ? old_lp + t0 : nullptr;
      q.ref_lp = ref_lp ? ref_lp + t0 : nullptr;
      q.adv = adv + t0;
      q.labels = (const long long*)labels + t0;
      q.tokw = tokw ? tokw + t0 : nullptr;
      q.T = cnt;
      q.g = g_out + t0;
      q.log_ratio = log_ratio ? log_ratio + t0 : nullptr;
      q.clip1 = clip1 ? clip1 + t0 : nullptr;
      q.unclipped = unclipped ? unclipped + t0 : nullptr;
      q.clipped = clipped ? clipped + t0 : nullptr;
      q.partial = pl.partial + 2 * (size_t)(t0 / kLossThreads);     // chunks start on whole blocks of the token kernel
      hipLaunchKernelGGL(grpo_loss_tokens_kernel, dim3((cnt + kLossThreads - 1) / kLossThreads), dim3(kLossThreads), 0, st, q);
      HIP_TRY(hipGetLastError());
    }
    if (dH_out || dW_out || dbias_out) {
      const bool first = ci == 0, last = ci == pl.nchunks - 1;
      KeptBwdSums sums;
      if (dW_out && pl.nchunks > 1) {
        sums.dw_in = first ? nullptr : pl.dw_acc;
        sums.dw_out_f32 = last ? nullptr : pl.dw_acc;
      }
      if (dbias_out && pl.nchunks > 1) {
        sums.db_in = first ? nullptr : pl.db_acc;
        sums.db_out_f32 = last ? nullptr : pl.db_acc;
      }
      rc = kept_bwd_impl(tn, h_c, weight, bias, labels + t0, lse_out + t0, g_out + t0, nullptr, inv_temp, cnt, H, V,
                         pl.keep, dH_out ? (char*)dH_out + (size_t)t0 * H * esz : nullptr, dW_out, dbias_out, sums,
                         pl.bwd_ws, pl.bwd_bytes, st, &aux);
      if (rc) return rc;
    }
  }
  {
    PhaseScope ph(kPhaseOther, st);
    const int nblocks = (T + kLossThreads - 1) / kLossThreads;
    lp.T = T;
    lp.partial = pl.partial;
    hipLaunchKernelGGL(grpo_loss_finalize_kernel, dim3(1), dim3(kLossThreads), 0, st, lp, nblocks);
    HIP_TRY(hipGetLastError());
  }
  return 0;
}

int fgrpo_scale_inplace(void* x, long long n, int dtype, const float* scale_dev, void* stream) {
  if (!x || !scale_dev || n < 0) return fail(FGRPO_ERR_BAD_ARG, "scale_inplace: bad argument");
  if (dtype != FGRPO_BF16 && dtype != FGRPO_F32) return fail(FGRPO_ERR_BAD_ARG, "scale_inplace: dtype=%d", dtype);
  if (!aligned16(x)) return fail(FGRPO_ERR_ALIGN, "scale_inplace: the array must be 16-byte aligned");
  if (n == 0) return 0;
  const long long nv = n / (dtype == FGRPO_F32 ? 4 : 8);
  long long nb = (nv + 255) / 256;
  nb = nb < 1 ? 1 : (nb > 4096 ? 4096 : nb);
  hipLaunchKernelGGL(scale_inplace_kernel, dim3((unsigned)nb), dim3(256), 0, (hipStream_t)stream, x, n,
                     dtype == FGRPO_F32, scale_dev);
  HIP_TRY(hipGetLastError());
  return 0;
}

int fgrpo_metrics(const int64_t* idx, int n, int T, const float* log_ratio, const float* entropy,
                  const float* old_entropy, const float* adv, const float* unclipped, const float* clipped,
                  float clip_low, float clip_high, double* stats_out, double* partial_ws, void* stream) {
  if (!stats_out || n < 0 || T <= 0) return fail(FGRPO_ERR_BAD_ARG, "metrics: bad argument");
  if (n > 0 && (!idx || !log_ratio || !adv || !unclipped || !clipped)) return fail(FGRPO_ERR_BAD_ARG, "metrics: null argument");
  // one work-group per 2048 positions, at most kMetricBlocks; without scratch (or for few positions) a single one
  int nb = partial_ws ? (n + 2047) / 2048 : 1;
  nb = nb < 1 ? 1 : (nb > kMetricBlocks ? kMetricBlocks : nb);
  MetricParams p{(const long long*)idx, n, T, log_ratio, entropy, old_entropy, adv, unclipped, clipped, clip_low, clip_high,
                 nb == 1 ? stats_out : partial_ws};
  hipLaunchKernelGGL(grpo_metrics_kernel, dim3(nb), dim3(1024), 0, (hipStream_t)stream, p);
  HIP_TRY(hipGetLastError());
  if (nb > 1) {
    hipLaunchKernelGGL(grpo_metrics_reduce_kernel, dim3(1), dim3(64 * kNumStats), 0, (hipStream_t)stream, partial_ws, nb,
                       stats_out);
    HIP_TRY(hipGetLastError());
  }
  return 0;
}

int fgrpo_group_advantages(const void* rewards, int rewards_f64, const int32_t* goff, int ngroups, int n_rewards,
                           double eps, float* out_f32, double* out_f64, void* stream) {
  if (!rewards || !goff || ngroups <= 0 || n_rewards < 0 || (!out_f32 && !out_f64))
    return fail(FGRPO_ERR_BAD_ARG, "group_advantages: bad argument");
  hipLaunchKernelGGL(group_advantage_kernel, dim3((ngroups + 3) / 4), dim3(256), 0, (hipStream_t)stream, rewards,
                     rewards_f64, goff, ngroups, n_rewards, eps, out_f32, out_f64);
  HIP_TRY(hipGetLastError());
  return 0;
}

int fgrpo_segment_broadcast(const void* values, int values_f64, const int32_t* cu, int nseq, int T, float* out,
                            void* stream) {
  if (!values || !cu || !out || nseq <= 0 || T < 0) return fail(FGRPO_ERR_BAD_ARG, "segment_broadcast: bad argument");
  hipLaunchKernelGGL(segment_broadcast_kernel, dim3((nseq + 3) / 4), dim3(256), 0, (hipStream_t)stream, values,
                     values_f64, cu, nseq, T, out);
  HIP_TRY(hipGetLastError());
  return 0;
}

int fgrpo_segment_reduce(const float* x, const int64_t* labels, const int32_t* cu, int nseq, int T, float* sum_out,
                         float* mean_out, int32_t* count_out, void* stream) {
  if (!x || !cu || nseq <= 0 || T < 0) return fail(FGRPO_ERR_BAD_ARG, "segment_reduce: bad argument");
  hipLaunchKernelGGL(segment_reduce_kernel, dim3((nseq + 3) / 4), dim3(256), 0, (hipStream_t)stream, x,
                     (const long long*)labels, cu, nseq, T, sum_out, mean_out, count_out);
  HIP_TRY(hipGetLastError());
  return 0;
}

int fgrpo_output_indices(const int32_t* tok_off, const int32_t* in_len, const int32_t* out_off, int nsamples,
                         int n_out, int64_t* out, void* stream) {
  if (!tok_off || !in_len || !out_off || !out || nsamples <= 0 || n_out < 0)
    return fail(FGRPO_ERR_BAD_ARG, "output_indices: bad argument");
  hipLaunchKernelGGL(output_indices_kernel, dim3((nsamples + 3) / 4), dim3(256), 0, (hipStream_t)stream, tok_off, in_len,
                     out_off, nsamples, n_out, (long long*)out);
  HIP_TRY(hipGetLastError());
  return 0;
}

int fgrpo_build_labels(const int64_t* ids, const int32_t* tok_off, const int32_t* in_len, const int32_t* out_len,
                       int nsamples, int T, int64_t* labels_out, void* stream) {
  if (!ids || !tok_off || !in_len || !out_len || !labels_out || nsamples <= 0 || T <= 0)
    return fail(FGRPO_ERR_BAD_ARG, "build_labels: bad argument");
  hipStream_t st = (hipStream_t)stream;
  // tokens outside every sample are masked
  hipLaunchKernelGGL(fill_i64_kernel, dim3((T + 255) / 256), dim3(256), 0, st, (long long*)labels_out, -100LL, T);
  HIP_TRY(hipGetLastError());
  hipLaunchKernelGGL(build_labels_kernel, dim3((nsamples + 3) / 4), dim3(256), 0, st, (const long long*)ids, tok_off,
                     in_len, out_len, nsamples, T, (long long*)labels_out);
  HIP_TRY(hipGetLastError());
  return 0;
}

int fgrpo_segment_starts(const int64_t* position_ids, int T, int32_t* cu_out, int max_out, int32_t* count_out,
                         void* stream) {
  if (!position_ids || !cu_out || !count_out || T <= 0 || max_out <= 0) return fail(FGRPO_ERR_BAD_ARG, "segment_starts: bad argument");
  hipLaunchKernelGGL(segment_starts_kernel, dim3(1), dim3(1024), 0, (hipStream_t)stream, (const long long*)position_ids,
                     T, cu_out, max_out, count_out);
  HIP_TRY(hipGetLastError());
  return 0;
}

int fgrpo_logits_logprob_entropy(const void* logits, int dtype, long long ld, int N, int V, const int64_t* labels,
                                 long long ignore_index, int use_ignore, float* lp, float* ent, float* lse,
                                 void* stream) {
  if (!logits || N <= 0 || V <= 0 || ld < V) return fail(FGRPO_ERR_BAD_ARG, "logits_logprob_entropy: bad argument");
  if (lp && !labels) return fail(FGRPO_ERR_BAD_ARG, "logits_logprob_entropy: lp requested without labels");
  if (dtype != FGRPO_BF16 && dtype != FGRPO_F32) return fail(FGRPO_ERR_BAD_ARG, "logits_logprob_entropy: dtype=%d", dtype);
  RowParams p{logits, dtype == FGRPO_F32, ld, N, V, (const long long*)labels, ignore_index, use_ignore, lp, ent, lse};
  hipLaunchKernelGGL(logits_row_stats_kernel, dim3(N), dim3(256), 0, (hipStream_t)stream, p);
  HIP_TRY(hipGetLastError());
  return 0;
}

int fgrpo_logits_logprob_bwd(const void* logits, int dtype, long long ld, int N, int V, const int64_t* labels,
                             long long ignore_index, int use_ignore, const float* g, const float* lse, void* dlogits,
                             long long ld_out, void* stream) {
  if (!logits || !labels || !g || !lse || !dlogits || N <= 0 || V <= 0 || ld < V || ld_out < V)
    return fail(FGRPO_ERR_BAD_ARG, "logits_logprob_bwd: bad argument");
  if (dtype != FGRPO_BF16 && dtype != FGRPO_F32) return fail(FGRPO_ERR_BAD_ARG, "logits_logprob_bwd: dtype=%d", dtype);
  RowBwdParams p{{logits, dtype == FGRPO_F32, ld, N, V, (const long long*)labels, ignore_index, use_ignore, nullptr, nullptr, nullptr},
                 g, lse, dlogits, ld_out};
  hipLaunchKernelGGL(logits_row_bwd_kernel, dim3(N), dim3(256), 0, (hipStream_t)stream, p);
  HIP_TRY(hipGetLastError());
  return 0;
}

int fgrpo_gemm_nt(const void* A, const void* B, int M, int N, int K, long long lda, long long ldb, const float* c_in,
                  float* c_out_f32, void* c_out_bf16, long long ldc, float alpha, int variant, void* stream) {
  if (!A || !B || (!c_out_f32 == !c_out_bf16)) return fail(FGRPO_ERR_BAD_ARG, "gemm_nt: need A, B and exactly one output");
  if (ldc < N) return fail(FGRPO_ERR_BAD_ARG, "gemm_nt: ldc < N");
  StoreParams s;
  memset(&s, 0, sizeof(s));
  s.g.M = M;
  s.g.N = N;
  s.g.lda = lda;
  s.g.ldb = ldb;
  s.g.nseg = 1;
  s.g.seg[0] = GemmSeg{(const bf16_t*)A, (const bf16_t*)B, K};
  s.c_in = c_in;
  s.c_out_f32 = c_out_f32;
  s.c_out_bf16 = (bf16_t*)c_out_bf16;
  s.ldc = ldc;
  s.alpha = alpha;
  if (variant < 0 || variant >= kNumCfg) return fail(FGRPO_ERR_BAD_ARG, "gemm_nt: variant=%d", variant);
  // the hook runs exactly the requested variant
  Tuning tn = g_tune;
  tn.small_variant = -1;
  return run_store_gemm(tn, s, variant, (hipStream_t)stream);
}

int fgrpo_gemm_kmajor(const void* A, const void* B, int M, int N, int K, long long lda, long long ldb, int a_kmajor,
                      int b_kmajor, long long a_blk, int k_valid, const float* c_in, float* c_out_f32,
                      void* c_out_bf16, long long ldc, float alpha, void* stream) {
  if (!A || !B || (!c_out_f32 == !c_out_bf16)) return fail(FGRPO_ERR_BAD_ARG, "gemm_kmajor: need A, B and exactly one output");
  if (ldc < N) return fail(FGRPO_ERR_BAD_ARG, "gemm_kmajor: ldc < N");
  if (!a_kmajor && !b_kmajor && !a_blk) return fail(FGRPO_ERR_BAD_ARG, "gemm_kmajor: plain layouts go through gemm_nt");
  if (k_valid < 0 || k_valid > K) return fail(FGRPO_ERR_BAD_ARG, "gemm_kmajor: k_valid=%d", k_valid);
  StoreParams s;
  memset(&s, 0, sizeof(s));
  s.g.M = M;
  s.g.N = N;
  s.g.lda = lda;
  s.g.ldb = ldb;
  s.g.nseg = 1;
  s.g.seg[0] = GemmSeg{(const bf16_t*)A, (const bf16_t*)B, K};
  s.g.a_blk = a_blk;
  s.g.ka_valid = (a_kmajor && !b_kmajor) ? k_valid : 0;
  s.g.kb_valid = b_kmajor ? k_valid : 0;
  s.c_in = c_in;
  s.c_out_f32 = c_out_f32;
  s.c_out_bf16 = (bf16_t*)c_out_bf16;
  s.ldc = ldc;
  s.alpha = alpha;
  if (!a_kmajor && !b_kmajor) {  // K-contiguous operands, A column-blocked
    Tuning tn = g_tune;
    tn.small_variant = -1;
    return run_store_gemm(tn, s, 8, (hipStream_t)stream);
  }
  return run_store_gemm_kmajor(g_tune, s, a_kmajor != 0, b_kmajor != 0, (hipStream_t)stream);
}

}  // extern "C"
