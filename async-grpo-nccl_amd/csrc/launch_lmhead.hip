// Instantiations and launches of the two LM-head tile kernels (vocabulary statistics of the forward, dLogits
// panels of the recomputing backward).  Built for the tile configurations whose kernels stay inside the register
// file (ids 2, 3, 4, 7, 8, 9): with the 128x128 wavefront tiles of ids 0, 1, 5 and 6 the epilogues spill over a
// hundred registers to scratch, which is slow everywhere and unsafe next to the inline-assembly fragment reads of
// the two-buffer direct-to-LDS loop; those ids are refused.
#include "host_common.h"

namespace fgrpo {
namespace {
template <class C>
int launch_fwd(const FwdParams& p, hipStream_t st) {
  return launch_tile_kernel<lmhead_fwd_kernel<C>, C>(p, p.tiles_t * p.nsplit, st);
}
template <class C>
int launch_ds(const DsParams& p, hipStream_t st) {
  return launch_tile_kernel<lmhead_ds_kernel<C, false>, C>(p, p.tiles_t * p.nsplit, st);
}
}  // namespace

#define DISPATCH_LMHEAD(variant, fn, ...)                                                          \
  switch (variant) {                                                                               \
    case 2: return fn<Cfg2>(__VA_ARGS__);                                                          \
    case 3: return fn<Cfg3>(__VA_ARGS__);                                                          \
    case 4: return fn<Cfg4>(__VA_ARGS__);                                                          \
    case 7: return fn<Cfg7>(__VA_ARGS__);                                                          \
    case 8: return fn<Cfg8>(__VA_ARGS__);                                                          \
    case 9: return fn<Cfg9>(__VA_ARGS__);                                                          \
    default: return fail(FGRPO_ERR_UNSUPPORTED, "tile configuration %d is not built for the LM-head kernels (2, 3, 4, 7, 8, 9 are)", variant); \
  }

bool lmhead_variant_built(int variant) {
  return variant == 2 || variant == 3 || variant == 4 || variant == 7 || variant == 8 || variant == 9;
}

int launch_fwd_variant(int variant, const FwdParams& p, hipStream_t st) {
  DISPATCH_LMHEAD(variant, launch_fwd, p, st);
}

int launch_fwd_keep(const FwdParams& p, hipStream_t st) {
  return launch_tile_kernel<lmhead_fwd_kernel<Cfg8, true>, Cfg8>(p, p.tiles_t * p.nsplit, st);
}

int launch_ds_variant(int variant, bool split, const DsParams& p, hipStream_t st) {
  // fp32 inputs: dS is written as bf16 hi + lo halves; only the small tile carries that epilogue
  if (split) return launch_tile_kernel<lmhead_ds_kernel<Cfg4, true>, Cfg4>(p, p.tiles_t * p.nsplit, st);
  DISPATCH_LMHEAD(variant, launch_ds, p, st);
}

}  // namespace fgrpo
