// Packed variable-length attention: C entry points, argument checks and launches (kernels in attn_kernels.h).
#include <string.h>

#include "host_common.h"
#include "attn_kernels.h"

using namespace fgrpo;

namespace {
// Query heads per work-group of the query-side kernels (tile = 128 / heads tokens).  Short segments gain from short
// tiles (less masked work on the diagonal and at segment boundaries) as long as the heads of a group fill the
// work-group; long ones do not care, and a lone head per K/V head has nothing to share.
int attn_heads_per_group(int G, int T, int n_seq) {
  if (g_tune.attn_heads == 1 || g_tune.attn_heads == 2 || g_tune.attn_heads == 4) return g_tune.attn_heads;
  if (G <= 1 || (long long)T >= 8192LL * n_seq) return 1;      // measured: -10..-22 % up to 2048-token segments, +1 % at 8192
  if (G % 4 == 0) return 4;
  if (G % 2 == 0) return 2;
  return G >= 3 ? 4 : 1;
}

template <template <int, int> class Launcher>
int launch_query_side(int D, int hb, AttnParams& p, int T, int Hq, int Hkv, int32_t* bounds_ws, hipStream_t st) {
  const int rb = 128 / hb, G = Hq / Hkv;
  p.order_q = bounds_ws + attn_order_offset(T, hb == 1 ? 1 : hb == 2 ? 2 : 3);
  const long long units = (long long)((T + rb - 1) / rb) * Hkv;            // (tile, K/V head)
  const dim3 grid((unsigned)(((units + 7) / 8 * 8) * ((G + hb - 1) / hb)));
  if (D == 128) {
    if (hb == 1) Launcher<128, 1>::run(grid, st, p);
    else if (hb == 2) Launcher<128, 2>::run(grid, st, p);
    else Launcher<128, 4>::run(grid, st, p);
  } else {
    if (hb == 1) Launcher<64, 1>::run(grid, st, p);
    else if (hb == 2) Launcher<64, 2>::run(grid, st, p);
    else Launcher<64, 4>::run(grid, st, p);
  }
  HIP_TRY(hipGetLastError());
  return 0;
}
template <int HD, int HB>
struct FwdLauncher {
  static void run(dim3 grid, hipStream_t st, const AttnParams& p) {
    if (g_tune.attn_qside == 1) hipLaunchKernelGGL((varlen_attn_fwd_kernel<HD, HB>), grid, dim3(256), 0, st, p);
    else hipLaunchKernelGGL((varlen_attn_fwd2_kernel<HD, HB>), grid, dim3(256), 0, st, p);
  }
};
template <int HD, int HB>
struct DqLauncher {
  static void run(dim3 grid, hipStream_t st, const AttnParams& p) {
    if (g_tune.attn_qside == 1 || g_tune.attn_qside == 3) hipLaunchKernelGGL((varlen_attn_dq_kernel<HD, HB>), grid, dim3(256), 0, st, p);
    else hipLaunchKernelGGL((varlen_attn_dq2_kernel<HD, HB>), grid, dim3(256), 0, st, p);
  }
};
}  // namespace

extern "C" {

// ---- packed variable-length attention ------------------------------------------------------------------
namespace {
int check_attn(const char* who, const void* q, const void* k, const void* v, long long q_st, long long q_sh,
               long long k_st, long long k_sh, long long v_st, long long v_sh, const int32_t* cu, int n_seq, int T,
               int Hq, int Hkv, int D, float scale, const int32_t* bounds_ws) {
  if (!q || !k || !v || !cu || !bounds_ws) return fail(FGRPO_ERR_BAD_ARG, "%s: null argument", who);
  if (T <= 0 || n_seq <= 0 || Hq <= 0 || Hkv <= 0 || Hq % Hkv != 0)
    return fail(FGRPO_ERR_BAD_ARG, "%s: T=%d n_seq=%d Hq=%d Hkv=%d", who, T, n_seq, Hq, Hkv);
  if (D != 128 && D != 64) return fail(FGRPO_ERR_BAD_ARG, "%s: head dimension %d not supported (128 or 64)", who, D);
  if (!(scale > 0.f)) return fail(FGRPO_ERR_BAD_ARG, "%s: softmax scale must be positive", who);
  if (!aligned16(q) || !aligned16(k) || !aligned16(v)) return fail(FGRPO_ERR_ALIGN, "%s: q/k/v must be 16-byte aligned", who);
  const long long st[6] = {q_st, q_sh, k_st, k_sh, v_st, v_sh};
  for (int i = 0; i < 6; ++i)
    if (st[i] <= 0 || st[i] % 8 != 0) return fail(FGRPO_ERR_ALIGN, "%s: strides must be positive multiples of 8 elements", who);
  return 0;
}

void fill_attn(AttnParams& p, const void* q, const void* k, const void* v, long long q_st, long long q_sh,
               long long k_st, long long k_sh, long long v_st, long long v_sh, int T, int Hq, int Hkv, float scale,
               int causal, int32_t* bounds_ws) {
  memset(&p, 0, sizeof(p));
  p.q = (const bf16_t*)q;
  p.k = (const bf16_t*)k;
  p.v = (const bf16_t*)v;
  p.q_st = q_st, p.q_sh = q_sh, p.k_st = k_st, p.k_sh = k_sh, p.v_st = v_st, p.v_sh = v_sh;
  p.seg_start = bounds_ws;
  p.seg_end = bounds_ws + T;
  p.order_k = bounds_ws + attn_order_offset(T, 0);
  p.order_q = bounds_ws + attn_order_offset(T, 1);      // the query-side launches pick the list of their tile size
  p.T = T, p.Hq = Hq, p.Hkv = Hkv;
  p.scale = scale;
  p.causal = causal != 0;
}
}  // namespace

int fgrpo_varlen_attn_bounds(const int32_t* cu, int n_seq, int T, int causal, int32_t* bounds_ws, void* stream) {
  hipStream_t st = (hipStream_t)stream;
  if (!cu || !bounds_ws || T <= 0 || n_seq <= 0) return fail(FGRPO_ERR_BAD_ARG, "varlen_attn_bounds: bad argument");
  hipLaunchKernelGGL(segment_bounds_kernel, dim3((T + 255) / 256), dim3(256), 0, st, cu, n_seq, T, bounds_ws, bounds_ws + T);
  HIP_TRY(hipGetLastError());
  hipLaunchKernelGGL(attn_tile_order_kernel, dim3(4, kAttnOrderSlices), dim3(1024), 0, st, bounds_ws, bounds_ws + T, T, causal != 0, bounds_ws);
  HIP_TRY(hipGetLastError());
  return 0;
}

int fgrpo_varlen_attn_fwd(const void* q, const void* k, const void* v, long long q_st, long long q_sh, long long k_st,
                          long long k_sh, long long v_st, long long v_sh, const int32_t* cu, int n_seq, int T, int Hq,
                          int Hkv, int D, float scale, int causal, void* out, float* lse, int32_t* bounds_ws,
                          int bounds_valid, void* stream) {
  hipStream_t st = (hipStream_t)stream;
  int rc = check_attn("varlen_attn_fwd", q, k, v, q_st, q_sh, k_st, k_sh, v_st, v_sh, cu, n_seq, T, Hq, Hkv, D, scale, bounds_ws);
  if (rc) return rc;
  if (!out || !lse) return fail(FGRPO_ERR_BAD_ARG, "varlen_attn_fwd: null output");
  if (!aligned16(out)) return fail(FGRPO_ERR_ALIGN, "varlen_attn_fwd: out must be 16-byte aligned");
  AttnParams p;
  fill_attn(p, q, k, v, q_st, q_sh, k_st, k_sh, v_st, v_sh, T, Hq, Hkv, scale, causal, bounds_ws);
  p.out = (bf16_t*)out;
  p.lse = lse;
  if (!bounds_valid) {   // else bounds_ws still holds what an earlier call with the same segments wrote
    rc = fgrpo_varlen_attn_bounds(cu, n_seq, T, causal, bounds_ws, stream);
    if (rc) return rc;
  }
  return launch_query_side<FwdLauncher>(D, attn_heads_per_group(Hq / Hkv, T, n_seq), p, T, Hq, Hkv, bounds_ws, st);
}

int fgrpo_varlen_attn_bwd(const void* dout, const void* q, const void* k, const void* v, const void* out, const float* lse,
                          long long q_st, long long q_sh, long long k_st, long long k_sh, long long v_st, long long v_sh,
                          const int32_t* cu, int n_seq, int T, int Hq, int Hkv, int D, float scale, int causal, void* dq,
                          void* dk, void* dv, float* delta_ws, int32_t* bounds_ws, int bounds_valid, void* stream) {
  hipStream_t st = (hipStream_t)stream;
  int rc = check_attn("varlen_attn_bwd", q, k, v, q_st, q_sh, k_st, k_sh, v_st, v_sh, cu, n_seq, T, Hq, Hkv, D, scale, bounds_ws);
  if (rc) return rc;
  if (!dout || !out || !lse || !dq || !dk || !dv || !delta_ws) return fail(FGRPO_ERR_BAD_ARG, "varlen_attn_bwd: null argument");
  if (!aligned16(dout) || !aligned16(out) || !aligned16(dq) || !aligned16(dk) || !aligned16(dv))
    return fail(FGRPO_ERR_ALIGN, "varlen_attn_bwd: dout/out/dq/dk/dv must be 16-byte aligned");
  AttnParams p;
  fill_attn(p, q, k, v, q_st, q_sh, k_st, k_sh, v_st, v_sh, T, Hq, Hkv, scale, causal, bounds_ws);
  p.lse = const_cast<float*>(lse);
  p.dout = (const bf16_t*)dout;
  p.delta = delta_ws;
  p.out_fwd = (const bf16_t*)out;
  p.dq = (bf16_t*)dq;
  p.dk = (bf16_t*)dk;
  p.dv = (bf16_t*)dv;
  if (!bounds_valid) {   // else bounds_ws still holds what an earlier call with the same segments wrote
    rc = fgrpo_varlen_attn_bounds(cu, n_seq, T, causal, bounds_ws, stream);
    if (rc) return rc;
  }
  rc = launch_query_side<DqLauncher>(D, attn_heads_per_group(Hq / Hkv, T, n_seq), p, T, Hq, Hkv, bounds_ws, st);
  if (rc) return rc;
  const dim3 grid_k(Hkv, (T + kAttnBQ - 1) / kAttnBQ);
  if (g_tune.attn_dkv == 1) {
    if (D == 128) hipLaunchKernelGGL(varlen_attn_dkv_kernel<128>, grid_k, dim3(256), 0, st, p);
    else hipLaunchKernelGGL(varlen_attn_dkv_kernel<64>, grid_k, dim3(256), 0, st, p);
  } else if (D == 128) {
    rc = raise_lds<varlen_attn_dkv2_kernel<128>>(kAttnDkv2Lds<128>);
    if (rc) return rc;
    hipLaunchKernelGGL(varlen_attn_dkv2_kernel<128>, grid_k, dim3(512), kAttnDkv2Lds<128>, st, p);
  } else {
    rc = raise_lds<varlen_attn_dkv2_kernel<64>>(kAttnDkv2Lds<64>);
    if (rc) return rc;
    hipLaunchKernelGGL(varlen_attn_dkv2_kernel<64>, grid_k, dim3(512), kAttnDkv2Lds<64>, st, p);
  }
  HIP_TRY(hipGetLastError());
  return 0;
}

}  // extern "C"
