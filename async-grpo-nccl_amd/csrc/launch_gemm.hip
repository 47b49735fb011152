// Instantiations and launches of the plain GEMM with store epilogue: every tile configuration with K-contiguous
// operands, and the 256x256x64 tile with contraction-major operands (the gradient GEMMs that read dLogits,
// hidden and W where they lie).
#include "host_common.h"

namespace fgrpo {
namespace {
template <class C>
int launch_store(const StoreParams& p, hipStream_t st) {
  return launch_tile_kernel<gemm_store_kernel<C, false, false>, C>(p, p.nblocks, st);
}
}  // namespace

int launch_store_variant(int variant, const StoreParams& p, hipStream_t st) {
  int rc = 0;
  DISPATCH_VARIANT(variant, launch_store, p, st);
  return rc;
}

int launch_store_splitk(const StoreParams& p, hipStream_t st) {
  return launch_tile_kernel<gemm_store_kernel<Cfg8, false, true, true>, Cfg8>(p, p.nblocks, st);
}

int launch_store_kmajor(bool akm, bool bkm, const StoreParams& p, hipStream_t st) {
  const int nb = p.nblocks;
  if (akm && bkm) return launch_tile_kernel<gemm_store_kernel<Cfg8, true, true>, Cfg8>(p, nb, st);
  if (akm) return launch_tile_kernel<gemm_store_kernel<Cfg8, true, false>, Cfg8>(p, nb, st);
  if (bkm) return launch_tile_kernel<gemm_store_kernel<Cfg8, false, true>, Cfg8>(p, nb, st);
  return fail(FGRPO_ERR_BAD_ARG, "gemm(k-major): no k-major operand");
}

}  // namespace fgrpo
