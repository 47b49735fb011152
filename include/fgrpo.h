/* fgrpo: C ABI of the MI355X (gfx950) fused logprob + GRPO hot path.
 *
 * Plain pointers and sizes only; every pointer named *_dev / every array is
 * DEVICE memory unless the comment says host.  Every call is asynchronous on
 * `stream` (a hipStream_t passed as void*), allocates nothing and keeps no
 * state between calls except tuning knobs.  Return value: 0 on success, a
 * negative FGRPO_ERR_* otherwise; fgrpo_last_error() gives the message of the
 * calling thread's last failure.
 *
 * Each entry point names the reference interface it replaces
 * (paths relative to the reference repository engineerA314/async-grpo-nccl).
 */
#ifndef FGRPO_H
#define FGRPO_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define FGRPO_OK 0
#define FGRPO_ERR_BAD_ARG (-1)     /* null pointer, non-positive size, bad enum */
#define FGRPO_ERR_UNSUPPORTED (-2) /* shape/dtype outside what the kernels handle */
#define FGRPO_ERR_WORKSPACE (-3)   /* workspace missing, misaligned or too small */
#define FGRPO_ERR_HIP (-4)         /* a HIP runtime call failed */
#define FGRPO_ERR_ALIGN (-5)       /* operand base not 16-byte aligned */

#define FGRPO_BF16 0
#define FGRPO_F32 1

#define FGRPO_AGG_TOKEN_MEAN 0
#define FGRPO_AGG_SAMPLE_MEAN 1

#define FGRPO_NUM_STATS 16

int fgrpo_version(void);
const char* fgrpo_last_error(void);

/* Tuning knobs (kernel variant ids, vocabulary splits, raster groups).  Unknown
 * keys return FGRPO_ERR_BAD_ARG.  Not part of the reference interface. */
int fgrpo_set_tuning(const char* key, int value);
int fgrpo_get_tuning(const char* key);

/* ---- LM-head projection -> log-softmax -> target gather (+ entropy) --------
 * Replaces the body of fused_log_probs_and_entropy_fn (grpo_loss.py:211-250)
 * and the chunk loop of grpo_loss_and_entropy_ce_fn (grpo_loss.py:286-313):
 *   x_t = (W h_t + b) * inv_temperature
 *   lp_t  = [y_t != -100] * (x_t[y_t] - logsumexp x_t)
 *   ent_t = [y_t != -100] * (logsumexp x_t - sum softmax(x_t) x_t)
 * hidden [T x H], weight [V x H] row-major in `dtype`; bias [V] in `dtype` or
 * NULL; labels_shifted [T] int64 (already shifted by one, -100 = ignored).
 * lp_out/ent_out/lse_out: fp32 [T]; ent_out and lse_out may be NULL.
 * The [T x V] logits never exist in memory. */
size_t fgrpo_logprob_fwd_workspace(int T, int H, int V, int dtype);
int fgrpo_logprob_fwd(const void* hidden, const void* weight, const void* bias,
                      const int64_t* labels_shifted, float inv_temperature,
                      int T, int H, int V, int dtype,
                      float* lp_out, float* ent_out, float* lse_out,
                      void* workspace, size_t workspace_bytes, void* stream);

/* Same computation and results as fgrpo_logprob_fwd, for callers that cannot allocate (code under HIP graph
 * capture, tight serving loops, harnesses that forbid hipMalloc): it takes no workspace and calls no allocating
 * routine.  Its scratch (per-split soft-max partials and target logits, what fgrpo_logprob_fwd_workspace sizes)
 * lives in a buffer of FGRPO_STATIC_SCRATCH_BYTES built into the library's device image, one copy per GPU, held
 * until the process ends.  A call that would need more returns FGRPO_ERR_WORKSPACE (bf16 inputs with H a multiple
 * of 64 need 16 * splits + 4 bytes per token: 2.2 MB at T = 32768, no bias; fp32 inputs and other H also stage
 * operand copies there and fit only at small sizes).  All calls on one GPU share the buffer: calls that overlap on
 * one GPU (different streams or threads) race; calls ordered on one stream do not.  Nothing in the buffer has to
 * start at zero.  No counterpart in the reference. */
#define FGRPO_STATIC_SCRATCH_BYTES (8u << 20)
int fgrpo_logprob_fwd_static(const void* hidden, const void* weight, const void* bias,
                             const int64_t* labels_shifted, float inv_temperature,
                             int T, int H, int V, int dtype,
                             float* lp_out, float* ent_out, float* lse_out, void* stream);

/* ---- backward of the above (what autograd derives from grpo_loss.py:290-296
 * through torch.matmul / gather / logsumexp):
 *   dX_t = g_t * gout * inv_temperature * (onehot(y_t) - softmax(x_t))
 *   dH = dX W ; dW = dX^T H ; dbias = sum_t dX_t
 * Logits are recomputed per tile; only one vocabulary panel of dX (bf16) lives
 * in the workspace at a time.  g [T] fp32 = d loss / d lp; gout_dev = device
 * scalar with the upstream gradient of the loss (NULL = 1); lse [T] from the
 * forward.  dH_out [T x H], dW_out [V x H], dbias_out [V] in `dtype`; each may
 * be NULL.  panel_elems_hint: upper bound on T*panel_width; <=0 = the library's
 * own bound, a quarter of T*V clamped to 2^25 .. 2^30 elements.  Within the
 * bound the panel count is fitted to whole rounds of the dW GEMM's tiles. */
size_t fgrpo_lmhead_bwd_workspace(int T, int H, int V, int dtype, long long panel_elems_hint);
/* Vocabulary columns of one dLogits panel that fgrpo_lmhead_bwd will use for these arguments (a multiple of 256;
 * the backward makes ceil(V / columns) passes).  A query for callers that size or report memory; no counterpart
 * in the reference, whose chunks are token rows (grpo_loss.py:280-316). */
int fgrpo_lmhead_bwd_panel_cols(int T, int H, int V, int dtype, long long panel_elems_hint);
int fgrpo_lmhead_bwd(const void* hidden, const void* weight, const void* bias,
                     const int64_t* labels_shifted, const float* lse, const float* g,
                     const float* gout_dev, float inv_temperature,
                     int T, int H, int V, int dtype,
                     void* dH_out, void* dW_out, void* dbias_out,
                     long long panel_elems_hint,
                     void* workspace, size_t workspace_bytes, void* stream);

/* ---- the same forward / backward pair WITHOUT recomputation: the soft-max numerators are kept ---------------
 * The reference keeps every chunk's logits alive for autograd (grpo_loss.py:286-313: 9.96 GB of bf16 at T = 32768,
 * V = 151936) and its backward reads them back; fgrpo_lmhead_bwd instead recomputes them (a fourth [T x V x H]
 * product).  Where memory allows - 288 GB of HBM per MI355X - this pair keeps a [T x V] bf16 matrix as the
 * reference does, in the form the backward needs: fgrpo_logprob_fwd_keep is fgrpo_logprob_fwd that also writes
 *   E[t, v] = exp(x_tv / temperature - ref_t),   ref_t = x_t[y_t] / temperature + 40,
 * the exponential its statistics compute anyway, re-based on a per-token reference fixed before the sweep (a dot
 * product per token).  The probability is E[t, v] * exp(ref_t - lse_t), so dLogits = diag(a) E' with one factor
 * a_t per token and E' = E but for the target's element of each row, which fgrpo_lmhead_bwd_kept patches in place:
 * no pass over [T x V] is needed and the two gradient products read the buffer as it lies (dH = diag(a) E' W with
 * the factor in the epilogue, dW = E'^T (diag(a) hidden)): 6 instead of 8 T*H*V products per step.  The buffer
 * survives the backward (a second backward may reuse it).  lp / entropy / lse are computed as in
 * fgrpo_logprob_fwd and are bit-identical to its results.
 * Range: E[t][v] = exp(x_tv / temperature - ref_t) in bf16 with ref_t = max(target logit, largest logit among the
 * first 512 vocabulary rows) / temperature + 40: finite as long as no logit of a scored token lies more than 123
 * (in units of log probability) above that maximum; the forward raises a flag in the buffer otherwise,
 * and fgrpo_lmhead_bwd_kept, which reads it on the device, then recomputes dLogits into the buffer before its two products (fgrpo_keep_overflowed() reports the flag to the host).  Rows of ignored tokens are stored as exact zeros.
 * logits_keep: fgrpo_logits_keep_bytes(T, V) bytes, 16-byte aligned: [ceil(V/256)][round_up(T,256)][256] bf16,
 * then the references and the flag.  workspace of the backward: fgrpo_lmhead_bwd_kept_workspace bytes (the token
 * factors, the scaled transposed copy of hidden, and an fp32 dH accumulator used only when the tuning key keep_panels splits
 * the products into vocabulary panels).
 * Supported (fgrpo_keep_supported() != 0): bf16, H a multiple of 64, V/256 x H/256 tiles for at least half the
 * CUs (any token count); anything
 * else returns FGRPO_ERR_UNSUPPORTED - use the recomputing pair.  dH_out / dW_out / dbias_out as in
 * fgrpo_lmhead_bwd. */
int fgrpo_keep_supported(int T, int H, int V, int dtype);
size_t fgrpo_logits_keep_bytes(int T, int V);
int fgrpo_logprob_fwd_keep(const void* hidden, const void* weight, const void* bias,
                           const int64_t* labels_shifted, float inv_temperature,
                           int T, int H, int V, int dtype,
                           float* lp_out, float* ent_out, float* lse_out,
                           void* logits_keep, size_t logits_keep_bytes,
                           void* workspace, size_t workspace_bytes, void* stream);
/* 1 when the kept values may have overflowed, 0 when they are good, negative on error.  Synchronises `stream`.
 * A query for tests and reports: fgrpo_lmhead_bwd_kept and fgrpo_grpo_step_chunked read the flag on the device
 * themselves (when it is set, a launch that otherwise returns at once overwrites the buffer with dLogits recomputed
 * from the operands, and the same two products then give the recomputing backward's gradients), so no caller has to
 * wait for the forward before queueing the backward. */
int fgrpo_keep_overflowed(const void* logits_keep, int T, int V, void* stream);
size_t fgrpo_lmhead_bwd_kept_workspace(int T, int H, int V, int dtype);
int fgrpo_lmhead_bwd_kept(const void* hidden, const void* weight, const void* bias,
                          const int64_t* labels_shifted, const float* lse, const float* g,
                          const float* gout_dev, float inv_temperature,
                          int T, int H, int V, int dtype,
                          void* logits_keep, size_t logits_keep_bytes,
                          void* dH_out, void* dW_out, void* dbias_out,
                          void* workspace, size_t workspace_bytes, void* stream);

/* ---- diagnostics: GPU time per phase of the backward ------------------------------------------------------
 * Between fgrpo_phase_timing_begin() and fgrpo_phase_timing_end() every fgrpo_lmhead_bwd / fgrpo_lmhead_bwd_kept
 * call of the process (whatever thread makes it: autograd runs backwards on its own) brackets its launches with
 * HIP events on the call's stream (the library creates FGRPO_MAX_TIMED_PHASES event pairs on first use; later
 * brackets are counted as dropped).  Meant for one stream at a time.  _end waits
 * for the last event and returns, per phase, the summed milliseconds and the number of brackets:
 * phase 0 = dLogits (recomputing kernel, or the in-place pass over kept logits), 1 = dHidden product,
 * 2 = dW product, 3 = everything else (operand staging, bias sums, the objective kernels of
 * fgrpo_grpo_step_chunked), 4 = the forward launches of fgrpo_grpo_step_chunked.  Returns the number of dropped brackets
 * (0 = all timed) or a negative error.  Timing is off unless begun; no counterpart in the reference. */
#define FGRPO_NUM_PHASES 5
#define FGRPO_MAX_TIMED_PHASES 1024
int fgrpo_phase_timing_begin(void);
int fgrpo_phase_timing_end(float* ms_by_phase, int* brackets_by_phase);

/* ---- per-token GRPO objective -------------------------------------------------
 * Replaces the tail of grpo_loss_and_entropy_ce_fn (grpo_loss.py:318-348):
 * ratio, dual clip, masked mean.  old_lp NULL => ratio 1 (grpo_loss.py:318-319).
 * Extensions not in the reference: ref_lp/kl_beta (k3 KL penalty per token) and
 * agg_mode SAMPLE_MEAN over cu_seqlens [nseq+1] int32 (mean over samples of the
 * per-sample token mean); denom_override > 0 replaces the normaliser.
 * Outputs (fp32): loss_out scalar; g_out [T] = d loss / d lp; log_ratio, clip1,
 * unclipped, clipped [T] (each may be NULL); scal_out [4] (may be NULL) =
 * {1/normaliser, valid tokens, non-empty samples, unnormalised sum}. */
size_t fgrpo_loss_fwd_workspace(int T, int nseq);
int fgrpo_loss_fwd(const float* lp, const float* old_lp, const float* ref_lp, const float* adv,
                   const int64_t* labels_shifted, const int32_t* cu_seqlens, int nseq, int T,
                   float clip_low, float clip_high, float clip_ratio_c, float kl_beta,
                   int agg_mode, double denom_override,
                   float* loss_out, float* g_out, float* log_ratio, float* clip1,
                   float* unclipped, float* clipped, float* scal_out,
                   void* workspace, size_t workspace_bytes, void* stream);

/* ---- the whole training step of one packed micro-batch, token chunk by token chunk --------------------------
 * Replaces the chunk loop of grpo_loss_and_entropy_ce_fn (grpo_loss.py:280-316), the objective behind it
 * (grpo_loss.py:318-348) AND what autograd later derives from them, in one call that never holds more than one
 * token chunk of [. x V]: for each chunk of `chunk` tokens
 *   forward with kept numerators (fgrpo_logprob_fwd_keep) into ONE chunk-sized buffer  ->  the objective on the
 *   chunk's tokens  ->  that chunk's rows of dH (written once)  ->  its contribution to dW (and dbias), carried
 *   in fp32 from chunk to chunk in a fixed order, converted by the last chunk's product.
 * This is possible because every normaliser of the objective (valid tokens, tokens per sample, samples) depends on
 * the labels and cu_seqlens only: fgrpo_loss_prepare forms them first - tokw_out [T] = 1 / (valid tokens of the
 * token's sample) and seg_cnt_out [nseq] for FGRPO_AGG_SAMPLE_MEAN (both may be NULL for TOKEN_MEAN), pre_out [4]
 * doubles = {normaliser, valid tokens, non-empty samples, 1 / normaliser rounded to fp32} - and
 * g_t = d loss / d lp_t is final as soon as lp_t is.  The gradients are those of the loss itself (upstream gradient
 * 1); a caller whose autograd later delivers another upstream scalar multiplies them with fgrpo_scale_inplace
 * (x[i] *= *scale_dev for n elements of `dtype`; a scale of exactly 1 returns without touching the array).
 * Executed matrix work: 6 T H V (the reference's own three products), against 8 T H V for the recomputing pair;
 * transient: fgrpo_logits_keep_bytes(chunk, V) + the fp32 dW sum (V x H x 4 bytes, only with more than one chunk).
 * chunk_tokens <= 0: 8192.  No chunk exceeds the bound (rounded down to whole 256-token tiles); under it the tokens
 * are dealt evenly over ceil(T / bound) chunks, or cut into whole chunks of the bound and a shorter last one, or into
 * whole chunks with the last of them and the rest dealt over two - whichever fills the device best (an estimate from
 * the tile counts; it depends on the arguments only).  fgrpo_grpo_step_chunk_tokens(T, H, V, chunk_tokens) returns
 * the largest chunk of the call (whole tiles): what the kept-numerator buffer is sized for.  Results do not depend on the
 * chunk size beyond fp32 summation order (of a token's vocabulary partial sums, whose split follows the token count
 * of a launch, and of dW across chunks): two calls with the same chunk size are bit-identical.
 * old_lp / ref_lp / tokw may be NULL (ratio 1 / no KL term / token mean); kl_beta as in fgrpo_loss_fwd.  Outputs as
 * in fgrpo_logprob_fwd and fgrpo_loss_fwd (lse_out and g_out are required: the gradients are formed from them);
 * dH_out [T x H], dW_out [V x H], dbias_out [V] in `dtype`, each may be NULL.  Supported
 * (fgrpo_grpo_step_chunked_supported() != 0) where fgrpo_keep_supported holds for the chunk and for the shorter last
 * chunk; otherwise FGRPO_ERR_UNSUPPORTED (use the recomputing pair).
 * Out-of-range chunks (see fgrpo_logprob_fwd_keep) are recomputed on the device, chunk by chunk, without a host
 * synchronisation: the call can be captured in a HIP graph. */
int fgrpo_loss_prepare(const int64_t* labels_shifted, const int32_t* cu_seqlens, int nseq, int T,
                       int agg_mode, double denom_override,
                       float* tokw_out, int32_t* seg_cnt_out, double* pre_out, void* stream);
int fgrpo_grpo_step_chunk_tokens(int T, int H, int V, int chunk_tokens);
int fgrpo_grpo_step_chunked_supported(int T, int H, int V, int dtype, int chunk_tokens);
size_t fgrpo_grpo_step_chunked_workspace(int T, int H, int V, int dtype, int chunk_tokens);
int fgrpo_grpo_step_chunked(const void* hidden, const void* weight, const void* bias,
                            const int64_t* labels_shifted, const float* old_lp, const float* ref_lp,
                            const float* adv, const float* tokw, const double* pre,
                            float inv_temperature, int T, int H, int V, int dtype,
                            float clip_low, float clip_high, float clip_ratio_c, float kl_beta,
                            int chunk_tokens,
                            float* lp_out, float* ent_out, float* lse_out, float* loss_out, float* g_out,
                            float* log_ratio, float* clip1, float* unclipped, float* clipped, float* scal_out,
                            void* dH_out, void* dW_out, void* dbias_out,
                            void* workspace, size_t workspace_bytes, void* stream);
int fgrpo_scale_inplace(void* x, long long n, int dtype, const float* scale_dev, void* stream);

/* ---- diagnostics on the output-token positions ---------------------------------
 * Replaces the ~20 .item() reductions of compute_dual_clip_grpo_loss
 * (grpo_loss.py:408-498) with one launch.  idx [n] int64 positions into the
 * [T] arrays.  stats_out: FGRPO_NUM_STATS doubles =
 * {n, sum|lr|, sum lr, sum lr^2, sum(r-1-lr), #(r>1+hi), #(r<1-lo), sum ent,
 *  sum old_ent, sum adv, sum adv^2, #(adv>0), #(adv==0), #(clipped>unclipped),
 *  0, #out-of-range idx}.  partial_ws: FGRPO_NUM_STATS * FGRPO_METRIC_BLOCKS doubles of
 * scratch for the two-stage sum (fixed order: results are bit-reproducible), or NULL
 * for a single work-group. */
#define FGRPO_METRIC_BLOCKS 128
int fgrpo_metrics(const int64_t* idx, int n, int T, const float* log_ratio, const float* entropy,
                  const float* old_entropy, const float* adv, const float* unclipped,
                  const float* clipped, float clip_low, float clip_high,
                  double* stats_out, double* partial_ws, void* stream);

/* ---- group-normalised advantages ------------------------------------------------
 * Replaces vllm_worker.py:788-796 (and normalize_rewards, :77-92):
 * (r - mean) / (population std + eps) per group; group_offsets [ngroups+1] int32.
 * rewards [n_rewards] fp32 or fp64 (rewards_f64 != 0); out_f32 / out_f64 may be NULL.
 * Offsets are read on the device and clamped into [0, n_rewards]. */
int fgrpo_group_advantages(const void* rewards, int rewards_f64, const int32_t* group_offsets,
                           int ngroups, int n_rewards, double eps, float* out_f32, double* out_f64,
                           void* stream);

/* ---- segmented helpers over cu_seqlens [nseq+1] int32 ---------------------------
 * fgrpo_segment_broadcast replaces broadcast_values (sample_processing_utils.py:69-105):
 * out[t] = values[s(t)].  fgrpo_segment_reduce gives per-sample sums / means /
 * counts of a per-token array, masked by labels != -100 when labels is given.
 * T = length of the per-token arrays; cu_seqlens entries are clamped into [0, T]. */
int fgrpo_segment_broadcast(const void* values, int values_f64, const int32_t* cu_seqlens, int nseq,
                            int T, float* out, void* stream);
int fgrpo_segment_reduce(const float* x, const int64_t* labels, const int32_t* cu_seqlens, int nseq,
                         int T, float* sum_out, float* mean_out, int32_t* count_out, void* stream);

/* ---- batch shaping --------------------------------------------------------------
 * fgrpo_output_indices replaces get_output_logits_indices_numba
 * (sample_processing_utils.py:29-67): sample i, packed at token offset
 * tok_off[i] with prompt length in_len[i], contributes the positions
 * tok_off[i]+in_len[i]-1+j, j in [0, out_off[i+1]-out_off[i]), written at
 * out[out_off[i]+j].  tok_off, in_len [nsamples], out_off [nsamples+1] int32;
 * out has n_out entries (out_off is clamped into [0, n_out]).
 * fgrpo_segment_starts replaces the cu_seqlens derivation of
 * gpu_process_worker.py:239-252: cu_out = ordered indices t with
 * position_ids[t]==0, then T; *count_out = entries produced (boundaries + 1),
 * at most max_out of them are stored. */
int fgrpo_output_indices(const int32_t* tok_off, const int32_t* in_len, const int32_t* out_off,
                         int nsamples, int n_out, int64_t* out, void* stream);
int fgrpo_segment_starts(const int64_t* position_ids, int T, int32_t* cu_out, int max_out,
                         int32_t* count_out, void* stream);
/* fgrpo_build_labels replaces the per-sample label loop of the rollout worker
 * (vllm_worker.py:768-774) for a packed batch that is already on the device:
 * inside sample i (tokens tok_off[i] .. tok_off[i+1] of ids [T]) the generated
 * span [in_len[i], in_len[i]+out_len[i]) keeps its token id, every other
 * position is -100.  tok_off [nsamples+1], in_len, out_len [nsamples] int32. */
int fgrpo_build_labels(const int64_t* ids, const int32_t* tok_off, const int32_t* in_len,
                       const int32_t* out_len, int nsamples, int T, int64_t* labels_out, void* stream);

/* ---- row soft-max on materialised logits ----------------------------------------
 * Replaces logprobs_from_logits (grpo_loss.py:146-173) and entropy_from_logits
 * (grpo_loss.py:203-208) for callers that already hold logits [N x V] (ld =
 * row stride in elements).  labels may be NULL when lp is NULL.  use_ignore = 0
 * disables the ignore_index test.  The backward writes
 * dlogits = g (onehot - softmax) in the logits' dtype, rows ld_out elements apart
 * (ld_out >= V; the rows of logits and dlogits need not share a stride). */
int fgrpo_logits_logprob_entropy(const void* logits, int dtype, long long ld, int N, int V,
                                 const int64_t* labels, long long ignore_index, int use_ignore,
                                 float* lp, float* ent, float* lse, void* stream);
int fgrpo_logits_logprob_bwd(const void* logits, int dtype, long long ld, int N, int V,
                             const int64_t* labels, long long ignore_index, int use_ignore,
                             const float* g, const float* lse, void* dlogits, long long ld_out, void* stream);

/* ---- test hook: the GEMM core on its own -----------------------------------------
 * C[m,n] = alpha * sum_k A[m,k] B[n,k] (+ c_in); A [M x K], B [N x K] bf16,
 * K a multiple of 64.  No counterpart in the reference. */
int fgrpo_gemm_nt(const void* A, const void* B, int M, int N, int K, long long lda, long long ldb,
                  const float* c_in, float* c_out_f32, void* c_out_bf16, long long ldc, float alpha,
                  int variant, void* stream);

/* Same contraction with the operand layouts the gradient GEMMs of fgrpo_lmhead_bwd
 * use to read dLogits, W and hidden in place.  a_kmajor != 0: A is stored [K x M]
 * (contraction index = row), else [M x K]; likewise B.  a_blk != 0: A is kept as
 * 256-column blocks, stored element (r, c) at A + (c/256)*a_blk + r*256 + c%256
 * (lda must be 256; r, c are the row and the contiguous index as stored).
 * k_valid > 0: rows k >= k_valid of the K-major operand (of B when both are
 * K-major) are not read; the other operand must exist and hold zeros there.
 * K a multiple of 64.  No counterpart in the reference. */
int fgrpo_gemm_kmajor(const void* A, const void* B, int M, int N, int K, long long lda, long long ldb,
                      int a_kmajor, int b_kmajor, long long a_blk, int k_valid, const float* c_in,
                      float* c_out_f32, void* c_out_bf16, long long ldc, float alpha, void* stream);

/* ---- packed variable-length attention ----------------------------------------------
 * Replaces the flash-attn call of the reference's packed path,
 * flash_attn_varlen_func(q, k, v, cu_seqlens_q=cu, cu_seqlens_k=cu, ..., softmax_scale, causal)
 * (gpu_process_worker.py:265-276), with the K/V head repeat of its grouped-query wrapper
 * (gpu_process_worker.py:154-161) done by head index: query head j reads K/V head j / (Hq/Hkv).
 * q [T, Hq, D], k / v [T, Hkv, D] bf16, D == 128 or 64, innermost dimension contiguous, token and head
 * strides in elements (multiples of 8), bases 16-byte aligned.  cu_seqlens [n_seq+1] int32 as built
 * at gpu_process_worker.py:239-252 (the same vector for queries and keys).  bounds_ws: 2*T + 2*ceil(T/128) + ceil(T/64) + ceil(T/32) int32
 * of scratch.  out [T, Hq, D] bf16 contiguous; lse [Hq, T] fp32 (natural log of the softmax
 * denominator), needed by the backward.  dropout is not supported (the reference passes 0).
 * bounds_valid != 0: bounds_ws was filled by an earlier call with the same cu_seqlens, T and causal flag (another
 * layer of the same batch, or the forward of this backward) and is used as it is; 0: it is (re)built first.
 * fgrpo_varlen_attn_bounds builds it alone (per-token segment bounds as the wrapper derives them from cu_seqlens,
 * gpu_process_worker.py:239-252, and the launch order of the tiles). */
int fgrpo_varlen_attn_bounds(const int32_t* cu_seqlens, int n_seq, int T, int causal, int32_t* bounds_ws,
                             void* stream);
int fgrpo_varlen_attn_fwd(const void* q, const void* k, const void* v, long long q_stride_t, long long q_stride_h,
                          long long k_stride_t, long long k_stride_h, long long v_stride_t, long long v_stride_h,
                          const int32_t* cu_seqlens, int n_seq, int T, int Hq, int Hkv, int D, float softmax_scale,
                          int causal, void* out, float* lse, int32_t* bounds_ws, int bounds_valid, void* stream);

/* Backward of the above (autograd of flash_attn_varlen_func in the reference).  dout, out
 * [T, Hq, D] bf16 contiguous; dq [T, Hq, D], dk / dv [T, Hkv, D] bf16 contiguous;
 * delta_ws: Hq*T fp32 of scratch.  bounds_valid != 0: bounds_ws is the buffer a forward (or backward) call
 * with the same cu_seqlens, T and causal flag filled, and is used as it is. */
int fgrpo_varlen_attn_bwd(const void* dout, const void* q, const void* k, const void* v, const void* out,
                          const float* lse, long long q_stride_t, long long q_stride_h, long long k_stride_t,
                          long long k_stride_h, long long v_stride_t, long long v_stride_h, const int32_t* cu_seqlens,
                          int n_seq, int T, int Hq, int Hkv, int D, float softmax_scale, int causal, void* dq, void* dk,
                          void* dv, float* delta_ws, int32_t* bounds_ws, int bounds_valid, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* FGRPO_H */
