// Host-side pieces shared by the translation units of libfgrpo.so: error reporting, tile configurations, tuning
// state, the tile-kernel launch helper and the launch functions each unit defines for the others.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/fgrpo.h"
#include "lmhead_kernels.h"

namespace fgrpo {

// Records the message for fgrpo_last_error() (per thread) and returns `code`.
int fail(int code, const char* fmt, ...) __attribute__((format(printf, 2, 3)));

#define HIP_TRY(expr)                                                                  \
  do {                                                                                 \
    hipError_t e_ = (expr);                                                            \
    if (e_ != hipSuccess) return ::fgrpo::fail(FGRPO_ERR_HIP, "%s: %s", #expr, hipGetErrorString(e_)); \
  } while (0)

inline long long round_up(long long x, long long m) { return (x + m - 1) / m * m; }
inline bool aligned16(const void* p) { return (((uintptr_t)p) & 15) == 0; }

// ---- tile configurations ---------------------------------------------------------
// id 0: 256x256x64, 4 wavefronts of 128x128, one work-group per CU
// id 1: 256x128x64, 4 wavefronts of 128x64
// id 2: 256x128x32, 4 wavefronts of 128x64, two work-groups per CU
// id 3: 256x256x32, 8 wavefronts of 128x64 (two per SIMD)
// id 4: 128x128x64, 4 wavefronts of 64x64, two work-groups per CU (small problems)
typedef TileCfg<256, 256, 64, 2, 2, 1> Cfg0;
typedef TileCfg<256, 128, 64, 2, 2, 1> Cfg1;
typedef TileCfg<256, 128, 32, 2, 2, 2> Cfg2;
typedef TileCfg<256, 256, 32, 2, 4, 2> Cfg3;
typedef TileCfg<128, 128, 64, 2, 2, 2> Cfg4;
// id 5: 256x256x32, 4 wavefronts, direct-to-LDS loads, 5 LDS stages, look-ahead fragment prefetch
// id 6: 256x256x64, 4 wavefronts, direct-to-LDS loads, 2 LDS stages
// id 7: 256x128x32, 4 wavefronts of 128x64, direct-to-LDS, 4 stages, two work-groups per CU
typedef TileCfg<256, 256, 32, 2, 2, 1, 5, true> Cfg5;
typedef TileCfg<256, 256, 64, 2, 2, 1, 2, true> Cfg6;
typedef TileCfg<256, 128, 32, 2, 2, 2, 3, true> Cfg7;
// id 8/9: as 6/5 with 8 wavefronts of 128x64 (two per SIMD)
typedef TileCfg<256, 256, 64, 2, 4, 2, 2, true> Cfg8;
typedef TileCfg<256, 256, 32, 2, 4, 2, 5, true> Cfg9;
constexpr int kNumCfg = 10;

struct CfgInfo {
  int bm, bn, bk, nt, lds, wgs_per_cu;
};
template <class C>
constexpr CfgInfo info_of(int wgs) {
  return CfgInfo{C::BM, C::BN, C::BK, C::NT, C::LDS_BYTES, wgs};
}
inline constexpr CfgInfo kCfg[kNumCfg] = {info_of<Cfg0>(1), info_of<Cfg1>(1), info_of<Cfg2>(2), info_of<Cfg3>(1),
                                          info_of<Cfg4>(2), info_of<Cfg5>(1), info_of<Cfg6>(1), info_of<Cfg7>(2),
                                          info_of<Cfg8>(1), info_of<Cfg9>(1)};

#define DISPATCH_VARIANT(variant, fn, ...)                \
  switch (variant) {                                      \
    case 0: rc = fn<Cfg0>(__VA_ARGS__); break;            \
    case 1: rc = fn<Cfg1>(__VA_ARGS__); break;            \
    case 2: rc = fn<Cfg2>(__VA_ARGS__); break;            \
    case 3: rc = fn<Cfg3>(__VA_ARGS__); break;            \
    case 5: rc = fn<Cfg5>(__VA_ARGS__); break;            \
    case 6: rc = fn<Cfg6>(__VA_ARGS__); break;            \
    case 7: rc = fn<Cfg7>(__VA_ARGS__); break;            \
    case 8: rc = fn<Cfg8>(__VA_ARGS__); break;            \
    case 9: rc = fn<Cfg9>(__VA_ARGS__); break;            \
    default: rc = fn<Cfg4>(__VA_ARGS__); break;           \
  }

// ---- tuning (fgrpo_set_tuning) -----------------------------------------------------
// Plain ints written by fgrpo_set_tuning and read when a call is planned.  An entry point that plans and launches
// copies the struct once at its top (Tuning snapshot = g_tune) so that a concurrent set_tuning cannot change the
// plan between the workspace check and the launch.
struct Tuning {
  int fwd_variant = 8;
  int ds_variant = 8;
  int gemm_variant = 8;
  int fwd_nsplit = 0;   // 0 = heuristic
  int fwd_group_t = 8;
  int ds_nsplit = 0;    // dLogits kernel: vocabulary splits of a panel; 0 = as the forward
  int ds_group_t = 0;   // dLogits kernel: token tiles per raster group; 0 = as the forward
  int dh_group_m = 0;   // dHidden GEMM raster group; 0 = gemm_group_m
  int dw_group_m = 0;   // dW GEMM raster group; 0 = gemm_group_m
  int gemm_group_m = 4;
  int panel_cols = 0;      // vocabulary panel width of the backward when the caller gives no bound; 0 = a quarter of [T x V], 2^25 .. 2^30 elements
  int small_variant = 4;   // used when a problem has fewer than small_tiles tiles of the big variant
  int bwd_kmajor = 2;      // 0: transposed copies; 1: the dW GEMM reads dLogits and hidden in place; 2: the dH GEMM reads W in place too
  int attn_heads = 0;      // query heads per work-group of the attention forward / dQ kernels (1, 2, 4); 0 = heuristic
  int attn_qside = 0;      // forward / dQ kernels: 1 = tiles staged through registers, compiler-scheduled LDS reads (3: dQ only); 0, 2 = the hand-scheduled forms
  int attn_dkv = 0;        // dK/dV kernel: 1 = one wavefront per 32 keys, 2 = a pair of wavefronts per 32 keys; 0 = default
  int wide_stores = 1;     // GEMM epilogues write 16-byte pieces through an LDS patch where alignment allows
  int keep_skip_dead = 1;  // kept-path backward skips stretches of tokens that carry no gradient
  int tail_split = 1;        // kept-path dHidden: last partial device round as a split contraction; forward: token regions
  int keep_panels = 0;     // kept-logits backward: vocabulary panels of the gradient GEMMs; 0 = one
};
extern Tuning g_tune;

int num_cus();

// Kernels with more than 64 KiB of dynamic LDS need the limit raised once per device and kernel: the flag array
// belongs to this instantiation, i.e. to the kernel named by the template argument.
template <auto Kern>
int raise_lds(int bytes) {
  static bool done[64] = {false};
  int dev = 0;
  HIP_TRY(hipGetDevice(&dev));
  if (dev >= 0 && dev < 64 && done[dev]) return 0;
  HIP_TRY(hipFuncSetAttribute(reinterpret_cast<const void*>(Kern), hipFuncAttributeMaxDynamicSharedMemorySize, bytes));
  if (dev >= 0 && dev < 64) done[dev] = true;
  return 0;
}

template <auto Kern, class C, class P>
int launch_tile_kernel(const P& p, int nblocks, hipStream_t st) {
  if (nblocks <= 0) return 0;
  int rc = raise_lds<Kern>(C::LDS_BYTES);
  if (rc) return rc;
  hipLaunchKernelGGL(Kern, dim3(nblocks), dim3(C::NT), C::LDS_BYTES, st, p);
  HIP_TRY(hipGetLastError());
  return 0;
}

// ---- launch functions defined in launch_lmhead.hip / launch_gemm.hip -------------------
// `variant` is a tile configuration id (already chosen by the caller).  The LM-head kernels exist for the ids
// lmhead_variant_built() accepts; the others are refused with FGRPO_ERR_UNSUPPORTED.
bool lmhead_variant_built(int variant);
int launch_fwd_variant(int variant, const FwdParams& p, hipStream_t st);
// the forward that also keeps the bf16 logits (tile id 8 only)
int launch_fwd_keep(const FwdParams& p, hipStream_t st);
// split: fp32 inputs, dS written as bf16 hi + lo halves (small tile only)
int launch_ds_variant(int variant, bool split, const DsParams& p, hipStream_t st);
int launch_store_variant(int variant, const StoreParams& p, hipStream_t st);
// 256x256x64 tile with one or both operands contraction-major
int launch_store_kmajor(bool akm, bool bkm, const StoreParams& p, hipStream_t st);
int launch_store_splitk(const StoreParams& p, hipStream_t st);

}  // namespace fgrpo
