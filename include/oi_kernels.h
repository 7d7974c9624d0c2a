/*
 * C-ABI of the MI355X (gfx950) policy-loss kernels.
 *
 * The reference (allenai/open-instruct) has no native interface for this path: its boundary is
 * plain Python functions on torch tensors.  Each entry point below names the reference function
 * whose arithmetic it carries; the Python package binds them with ctypes and exposes the
 * reference's own names and signatures on top.
 *
 * Conventions
 *  - Every pointer is DEVICE memory owned by the caller.  The library never allocates, frees or
 *    keeps a pointer after the call returns.  Scratch memory is passed in as `workspace` and sized
 *    by the matching oi_*_workspace_bytes().  Workspaces and fp32 accumulators (wsum) must be
 *    ordinary device allocations (hipMalloc, a torch tensor): the kernels add to them with the
 *    L2's floating-point atomics, which fine-grained or host-mapped memory does not support.
 *  - Work is enqueued on `stream` (a hipStream_t passed as void*; NULL = the null stream) and the
 *    call returns without waiting for it.
 *  - Return value: 0 on success, a negative OI_E* code for a rejected argument (nothing was
 *    launched), a positive value = the hipError_t of a failed launch.
 *  - Calls are re-entrant.  The only state the library keeps between calls is looked up once per
 *    device under a lock and never changes afterwards: the CU count, and the device address of the
 *    static scratch array of oi_grpo_fused_fwd_static (the one entry point that shares memory
 *    between calls; see there).
 *  - Row-major everywhere; strides are in ELEMENTS, not bytes.
 *  - Token ids / labels are int64, sequence boundaries int32, masks one byte per token (0 / 1).
 */
#ifndef OI_KERNELS_H
#define OI_KERNELS_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define OI_OK 0
#define OI_EINVAL (-1)     /* a size or scalar argument is out of range            */
#define OI_ENULL (-2)      /* a required pointer is NULL                            */
#define OI_EALIGN (-3)     /* pointer/stride alignment the kernel needs is not met  */
#define OI_EDTYPE (-4)     /* unknown or unsupported dtype tag                      */
#define OI_EWORKSPACE (-5) /* workspace_bytes is smaller than the op needs          */
#define OI_ETOOLARGE (-6)  /* larger than the static scratch of a *_static entry    */

#define OI_DTYPE_F32 0
#define OI_DTYPE_BF16 1
#define OI_DTYPE_F16 2

#define OI_LOSS_DAPO 0
#define OI_LOSS_CISPO 1

/* Library ABI version (major * 1000 + minor). */
int oi_version(void);
/* Human-readable text for a negative OI_E* code (static storage). */
const char* oi_error_string(int code);

/* ------------------------------------------------------------------------------------------
 * Row-wise log-softmax gather + entropy over materialised logits.
 *
 * Carries open_instruct/model_utils.py:587-600 (log_softmax_and_gather),
 * open_instruct/model_utils.py:326-333 (entropy_from_logits) and, with the label clamp done by
 * the caller, open_instruct/padding_free_collator.py:10-16 (calculate_per_token_logps).  The
 * division by temperature of open_instruct/grpo_utils.py:560 is folded in as `inv_temperature`.
 *
 * Rows are addressed as row = o * n_inner + i  ->  logits + o * stride_outer + i * stride_inner,
 * which covers the reference's non-contiguous `logits[:, :-1]` view (n_outer = B, n_inner = T-1,
 * stride_outer = T*V, stride_inner = V).  The vocabulary dim has stride 1.
 *
 *   logprob[row] = z[index[row]] * inv_T - logsumexp(z * inv_T)
 *   entropy[row] = logsumexp(z * inv_T) - sum_j softmax(z * inv_T)_j * z_j * inv_T   (optional)
 *   lse[row]     = logsumexp(z * inv_T)                                              (optional)
 *
 * All three outputs are fp32, contiguous, n_outer * n_inner long.  index values outside [0, V)
 * are clamped into range (never a fault).  One pass over the logits.
 * ------------------------------------------------------------------------------------------ */
int oi_lsg_entropy_fwd(const void* logits, int dtype, int64_t n_outer, int64_t n_inner, int64_t stride_outer,
                       int64_t stride_inner, int64_t vocab, const int64_t* index, float inv_temperature,
                       float* logprob, float* entropy, float* lse, void* stream);

/*
 * Backward of the gather-logprob above (autograd supplies it in the reference; formula
 * d z_j = g * inv_T * (1[j == index] - softmax_j)).  Reads logits + lse, writes dlogits in the
 * logits' dtype with its own outer/inner strides.  Rows whose grad_logprob is exactly 0 are
 * written as zeros without reading their logits.  `dlogits` may alias `logits` (in-place) when
 * the strides are equal.
 */
int oi_lsg_bwd(const void* logits, int dtype, int64_t n_outer, int64_t n_inner, int64_t stride_outer,
               int64_t stride_inner, int64_t vocab, const int64_t* index, const float* lse,
               const float* grad_logprob, float inv_temperature, void* dlogits, int64_t out_stride_outer,
               int64_t out_stride_inner, void* stream);

/*
 * GRPO on materialised logits in one launch: forward (logprob / entropy / lse as
 * oi_lsg_entropy_fwd) and the gradient of the GRPO loss with respect to the logits.  A row stays
 * on its CU (LDS and registers) between the statistics pass and the gradient pass; only what a row
 * has beyond 16384 16-byte pieces is read a second time, from the caches.  HBM sees one read and
 * one write of the [rows, vocab] tensor instead of two reads and a write.  Fuses the sequence open_instruct/grpo_utils.py:541-574 (forward_for_logprobs) ->
 * open_instruct/grpo_utils.py:504-538 (compute_grpo_loss) -> open_instruct/grpo_fast.py:702-724
 * (masked mean, backward) for callers that hold the logits.
 *
 *   ratio = exp(logprob - old) (1 when old_logprobs is NULL), loss_token = pg + beta * kl as in
 *   oi_grpo_terms_fwd, g = token_coef[row] * d loss_token / d logprob,
 *   dlogits[row, j] = g * inv_T * (1[j == index] - softmax_j).
 * token_coef (fp32 per row) carries the loss denominators, which depend on the mask alone:
 * scale / denominator on response tokens, 0 elsewhere (such rows get a zero gradient row).
 * Requirement: 16-byte aligned rows (pointers and strides of logits and dlogits) of at least 16
 * bytes; OI_EALIGN otherwise (use the two-pass entry points).  dlogits must not alias logits (OI_EINVAL).  The scalar loss and
 * its statistics come from oi_grpo_fused_fwd on `logprob`.
 */
int oi_lsg_grpo_fwd_bwd(const void* logits, int dtype, int64_t n_outer, int64_t n_inner, int64_t stride_outer,
                        int64_t stride_inner, int64_t vocab, const int64_t* index, float inv_temperature,
                        const float* old_logprobs, const float* ref_logprobs, const float* advantages,
                        const float* rho_weights, const float* token_coef, int loss_fn, float ratio_lo,
                        float ratio_hi, int kl_estimator, float beta, float* logprob, float* entropy, float* lse,
                        void* dlogits, int64_t out_stride_outer, int64_t out_stride_inner, void* stream);

/*
 * data[i] *= *scale over a contiguous tensor of n elements (dtype tag as above), where `scale` is
 * a DEVICE scalar; when it is exactly 1 the kernel leaves the data untouched.  No reference
 * counterpart: it applies the upstream gradient of the loss to the gradient that
 * oi_lsg_grpo_fwd_bwd stored, the step autograd performs at open_instruct/grpo_fast.py:724
 * (`loss.backward()`), without a host read of the scalar.
 */
int oi_scale_by_device_scalar(void* data, int dtype, int64_t n, const float* scale, void* stream);

/* ------------------------------------------------------------------------------------------
 * Per-token GRPO loss terms.  Carries open_instruct/grpo_utils.py:504-538 (compute_grpo_loss)
 * with open_instruct/model_utils.py:793-818 (estimate_kl) for the selected estimator.
 * All tensors fp32, contiguous, n elements.  ref_logprobs may be NULL (kl = 0).
 * ratio_lo / ratio_hi are the clamp bounds themselves, i.e. 1 - clip_lower and 1 + clip_higher
 * evaluated by the caller in double and rounded once to fp32, as torch does for a Python scalar.
 * ------------------------------------------------------------------------------------------ */
int oi_grpo_terms_fwd(const float* new_logprobs, const float* ratio, const float* advantages,
                      const float* ref_logprobs, const float* rho_weights, int64_t n, int loss_fn, float ratio_lo,
                      float ratio_hi, int kl_estimator, float* pg_loss, float* clipfrac, float* kl, void* stream);

/* Backward of oi_grpo_terms_fwd towards new_logprobs and ratio (either output may be NULL).
 * grad_pg / grad_kl are the upstream gradients of pg_loss / kl (either may be NULL = zeros). */
int oi_grpo_terms_bwd(const float* new_logprobs, const float* ratio, const float* advantages,
                      const float* ref_logprobs, const float* rho_weights, const float* grad_pg,
                      const float* grad_kl, int64_t n, int loss_fn, float ratio_lo, float ratio_hi,
                      int kl_estimator, float* d_new_logprobs, float* d_ratio, void* stream);

/*
 * Fused scalar GRPO loss over a [rows, cols] micro-batch.  Carries the loss assembly of
 * open_instruct/grpo_fast.py:702-724 / open_instruct/olmo_core_train_modules.py:547-568:
 *   ratio = exp(new - old); (pg, clipfrac, kl) as above;
 *   loss  = masked_mean(pg + beta * kl, mask, axis, denominator) * scale
 * together with the no-grad statistics of open_instruct/grpo_utils.py:699-729 in the same pass.
 *
 * axis_mode 0: masked_mean(axis=None) - one denominator (`denominator` if > 0, else mask.sum()).
 * axis_mode 1: masked_mean(axis=1)    - per-row means, then the mean over rows.
 * old_logprobs / ref_logprobs / rho_weights / entropy may be NULL (old NULL => ratio == 1 with
 * gradient, as when old = new.detach(); ref NULL => kl = 0; rho NULL => 1).
 *
 * out_stats (fp32[OI_GRPO_NUM_STATS]): [0] loss, [1] masked mean pg, [2..5] masked mean of KL
 * estimators 0..3, [6] masked mean clipfrac, [7] masked mean ratio, [8] masked mean entropy,
 * [9] mask.sum(), [10..12] masked means of the rho drop indicators (any / below the lower bound /
 * above the upper bound), [13] masked mean of rho_weights, [14] masked mean of the rho clamp
 * indicator (the five metric tensors of open_instruct/grpo_utils.py:446-452; 0 for a NULL
 * pointer, [13] is 1 without rho_weights), [15] = [2 + kl_estimator] * beta, the "loss/kl_avg" of
 * open_instruct/grpo_utils.py:718.  row_denoms (fp32[rows]) receives the reciprocal denominator
 * applied to each row's tokens, which oi_grpo_fused_bwd consumes.  rows * ceil(cols / 1024) must
 * stay below 2^31 (one block per row and 1024 columns).
 */
#define OI_GRPO_NUM_STATS 16
size_t oi_grpo_fused_workspace_bytes(int64_t rows, int64_t cols);
int oi_grpo_fused_fwd(const float* new_logprobs, const float* old_logprobs, const float* ref_logprobs,
                      const float* advantages, const uint8_t* mask, const float* rho_weights, const float* entropy,
                      const float* rho_drop_any, const float* rho_drop_low, const float* rho_drop_high,
                      const float* rho_clipped, int64_t rows, int64_t cols, int loss_fn, float ratio_lo,
                      float ratio_hi, int kl_estimator, float beta, int axis_mode, float denominator, float scale,
                      float* out_stats, float* row_denoms, void* workspace, size_t workspace_bytes, void* stream);
/*
 * oi_grpo_fused_fwd for callers that cannot allocate device memory (code under HIP graph capture,
 * tight serving loops, harnesses that forbid hipMalloc).  It has no counterpart in the reference.
 * Same arguments, results and kernels as oi_grpo_fused_fwd, without the workspace: the partial
 * sums live in a file-scope device array of the library (OI_GRPO_STATIC_MAX_BLOCKS * 15 floats =
 * 480 KB, held on every GPU the library runs on until the process ends).  The call allocates and
 * frees nothing.  Limit: rows * ceil(cols / 1024) <= OI_GRPO_STATIC_MAX_BLOCKS, OI_ETOOLARGE
 * beyond it (nothing is launched).  The first call on a device looks up the array's address on
 * that device (hipGetSymbolAddress); make it before a stream capture starts.  All calls on one GPU
 * share the array: calls that overlap in time on one GPU (two streams, two threads) race; calls
 * in stream order do not, and nothing has to be cleared between them.
 */
#define OI_GRPO_STATIC_MAX_BLOCKS 8192
int oi_grpo_fused_fwd_static(const float* new_logprobs, const float* old_logprobs, const float* ref_logprobs,
                             const float* advantages, const uint8_t* mask, const float* rho_weights,
                             const float* entropy, const float* rho_drop_any, const float* rho_drop_low,
                             const float* rho_drop_high, const float* rho_clipped, int64_t rows, int64_t cols,
                             int loss_fn, float ratio_lo, float ratio_hi, int kl_estimator, float beta, int axis_mode,
                             float denominator, float scale, float* out_stats, float* row_denoms, void* stream);

/*
 * The same statistics for a caller that already holds the per-token terms.  Carries
 * open_instruct/grpo_utils.py:699-729 (populate_sample_loss_stats) in two launches: masked means
 * of pg_loss, clipfrac, ratio, of the four KL estimators of clamp(new - ref, +-40) (zeros when
 * ref_logprobs is NULL), of entropy and of the rho metric tensors.  Statistic q (numbering of
 * oi_grpo_fused_fwd; [0] is the caller's own loss and is never written) goes to
 * out_stats[q * out_stride] when bit q of write_mask is set, so one column of a
 * [OI_GRPO_NUM_STATS, num_samples] table can be filled in place.  Workspace as for
 * oi_grpo_fused_fwd.
 */
int oi_grpo_stats_from_terms(const float* pg_loss, const float* clipfrac, const float* ratio,
                             const float* new_logprobs, const float* ref_logprobs, const uint8_t* mask,
                             const float* entropy, const float* rho_weight, const float* rho_drop_any,
                             const float* rho_drop_low, const float* rho_drop_high, const float* rho_clipped,
                             int64_t rows, int64_t cols, int kl_estimator, float beta, float* out_stats,
                             int64_t out_stride, uint32_t write_mask, void* workspace, size_t workspace_bytes,
                             void* stream);
/* d loss / d new_logprobs (fp32 [rows, cols]); grad_loss is a DEVICE scalar (upstream gradient; NULL = 1). */
int oi_grpo_fused_bwd(const float* new_logprobs, const float* old_logprobs, const float* ref_logprobs,
                      const float* advantages, const uint8_t* mask, const float* rho_weights, int64_t rows,
                      int64_t cols, int loss_fn, float ratio_lo, float ratio_hi, int kl_estimator, float beta,
                      float scale, const float* row_denoms, const float* grad_loss, float* d_new_logprobs,
                      void* stream);

/* ------------------------------------------------------------------------------------------
 * Small per-token helpers of the GRPO step (fp32, contiguous).
 * oi_estimate_kl_*: open_instruct/model_utils.py:793-818 - out is [4, n]: d, d^2/2,
 *   expm1(-d)+d, ratio*d.  The backward takes grad_out [4, n]; d_diff / d_ratio may be NULL.
 * oi_mask_logprobs_*: open_instruct/grpo_utils.py:340-344 - positions off the mask and NaNs
 *   become `fill` (INVALID_LOGPROB = 1.0 in the reference, open_instruct/utils.py:83).
 * oi_rho_correction: open_instruct/grpo_utils.py:372-463 - per token rho = exp(clamp(old - vllm,
 *   +-10)) on the mask (1 elsewhere), optional per-row geometric mean / TV-divergence drop rule,
 *   drop outside (mask_lower, mask_upper), clamp to [clamp_lower, clamp_upper] (a bound of 0
 *   disables it); six fp32 [rows, cols] outputs: rho, weights, dropped, dropped-low,
 *   dropped-high, clamped-flag.
 * ------------------------------------------------------------------------------------------ */
int oi_estimate_kl_fwd(const float* ref_logprobs_diff, const float* ratio, int64_t n, float* out, void* stream);
int oi_estimate_kl_bwd(const float* ref_logprobs_diff, const float* ratio, const float* grad_out, int64_t n,
                       float* d_diff, float* d_ratio, void* stream);
int oi_mask_logprobs_fwd(const float* logprobs, const uint8_t* mask, int64_t n, float fill, float* out,
                         void* stream);
int oi_mask_logprobs_bwd(const float* logprobs, const uint8_t* mask, const float* grad_out, int64_t n,
                         float* d_logprobs, void* stream);
int oi_rho_correction(const float* old_logprobs, const float* vllm_logprobs, const uint8_t* mask,
                      const float* advantages, int64_t rows, int64_t cols, int sequence_level, int tv_divergence,
                      float mask_lower, float mask_upper, float clamp_lower, float clamp_upper, float* rho,
                      float* weights, float* drop_any, float* drop_low, float* drop_high, float* clipped,
                      void* stream);

/* Group-normalised advantages.  Carries open_instruct/data_loader.py:1472-1484: population std,
 * mode 0 "standard" (s - mean) / (std + 1e-8), mode 1 "centered" s - mean.  Computed in fp64 like
 * the reference's numpy, stored as fp32.  scores: fp64 [n_groups * group_size]. */
int oi_group_advantages(const double* scores, int64_t n_groups, int64_t group_size, int mode, float* advantages,
                        void* stream);

/* ------------------------------------------------------------------------------------------
 * Masked mean.  Carries open_instruct/rl_utils.py:426-448 for fp32 values [extra, rows, cols]
 * and a byte or fp32 mask [rows, cols] (mask_is_float selects).  axis_mode as above;
 * out: fp32 [extra].  row_denoms (fp32 [rows], may be NULL) as above.  extra <= 65535 and
 * extra * rows * ceil(cols / 1024) < 2^31.
 * ------------------------------------------------------------------------------------------ */
size_t oi_masked_mean_workspace_bytes(int64_t extra, int64_t rows, int64_t cols);
int oi_masked_mean_fwd(const float* values, const void* mask, int mask_is_float, int64_t extra, int64_t rows,
                       int64_t cols, int axis_mode, float denominator, float* out, float* row_denoms,
                       void* workspace, size_t workspace_bytes, void* stream);
/* d values[e, r, c] = grad_out[e] * mask[r, c] * row_denoms[r]. */
int oi_masked_mean_bwd(const float* grad_out, const void* mask, int mask_is_float, const float* row_denoms,
                       int64_t extra, int64_t rows, int64_t cols, float* d_values, void* stream);

/* ------------------------------------------------------------------------------------------
 * Per-sequence log-probability sums.
 * Packed rows (cu_seq_lens != NULL): carries open_instruct/padding_free_collator.py:202-229 -
 * per_token_logps / labels are one packed row of `total` positions, cu_seq_lens int32 [n_seqs+1];
 * position t < total-1 is kept when labels[t+1] != -100 and belongs to the segment given by the
 * boundaries shifted left by one (leading 0 kept, tail clamped into the last segment).
 * Padded rows (cu_seq_lens == NULL): carries open_instruct/dpo_utils.py:689-712 - n_seqs rows of
 * `total` positions each.  average != 0 divides by max(count, 1).
 * out: fp32 [n_seqs]; counts: fp32 [n_seqs] (kept positions, may be NULL).  Deterministic.
 * ------------------------------------------------------------------------------------------ */
int oi_seq_logp_fwd(const float* per_token_logps, const int64_t* labels, const int32_t* cu_seq_lens, int64_t n_seqs,
                    int64_t total, int average, float* out, float* counts, void* stream);
/* d per_token_logps (same shape as the input; the dropped last position(s) get 0).  `counts` is
 * the forward's output and is required when average != 0. */
int oi_seq_logp_bwd(const float* grad_out, const int64_t* labels, const int32_t* cu_seq_lens, const float* counts,
                    int64_t n_seqs, int64_t total, int average, float* d_per_token_logps, void* stream);

/* ------------------------------------------------------------------------------------------
 * Debug statistics of locally recomputed logprobs against the sampler's logprobs.  Carries
 * open_instruct/grpo_utils.py:345-369 (compute_vllm_local_debug_metrics) in one launch.
 * A position is valid where mask != 0 and other_logprobs is not NaN.  out_stats (fp32[4]):
 *   [0] mean |local - other|, [1] max |local - other|, [2] unbiased std of |local - other|
 *   (0 when fewer than 2 valid positions), [3] mean exp(other) * (other - local); all 0 when no
 *   position is valid.  Sums are accumulated in fp64.
 * ------------------------------------------------------------------------------------------ */
#define OI_LOGPROB_DIFF_NUM_STATS 4
int oi_logprob_diff_stats(const float* local_logprobs, const float* other_logprobs, const uint8_t* mask, int64_t n,
                          float* out_stats, void* stream);

/* ------------------------------------------------------------------------------------------
 * Sigmoid preference loss per pair.  Carries open_instruct/dpo_utils.py:523-563 (dpo_loss) and,
 * with ref pointers NULL and `margin` = gamma/beta, open_instruct/dpo_utils.py:617-642
 * (simpo_loss):   x = (pc - pr) - (rc - rr) - margin
 *                 loss = -(1 - ls) * logsigmoid(beta x) - ls * logsigmoid(-beta x)
 * `weights` (may be NULL) multiplies the loss per pair (open_instruct/dpo_utils.py:566-613, wpo).
 * rewards: beta * (p - ref) (ref treated as 0 when NULL); either may be NULL.
 * ------------------------------------------------------------------------------------------ */
int oi_dpo_sigmoid_fwd(const float* policy_chosen, const float* policy_rejected, const float* ref_chosen,
                       const float* ref_rejected, const float* weights, int64_t n_pairs, float beta,
                       float label_smoothing, float margin, float* losses, float* chosen_rewards,
                       float* rejected_rewards, void* stream);
int oi_dpo_sigmoid_bwd(const float* policy_chosen, const float* policy_rejected, const float* ref_chosen,
                       const float* ref_rejected, const float* weights, const float* grad_losses, int64_t n_pairs,
                       float beta, float label_smoothing, float margin, float* d_policy_chosen,
                       float* d_policy_rejected, void* stream);

/* ------------------------------------------------------------------------------------------
 * Packing of query/response pairs into training rows.  Carries the per-token part of
 * open_instruct/rl_utils.py:227-375 (pack_sequences: concatenation with padding tokens dropped
 * from the responses, document-id response mask, intra-pack attention ids, per-document position
 * ids (open_instruct/rl_utils.py:215-224), `dones`, sampler logprobs with NaN on query tokens)
 * and the advantage broadcast of open_instruct/data_loader.py:1509-1514 in one launch.
 *
 * Inputs are the ragged lists in CSR form: q_tokens / r_tokens (int64, all queries / responses
 * back to back), q_offsets / r_offsets (int64 [n_seqs + 1]), r_tool_mask (one byte per response
 * token, may be NULL unless mask_tool_use), r_logprobs (fp32 per response token).  The greedy
 * assignment of sequences to rows is O(n_seqs) scalar work and stays with the caller, who passes
 *   dst_offsets[i] = position of sequence i's first token in the flat outputs (rows back to back),
 *   mask_base[i]   = index of the first sequence in sequence i's row (attention id = i + 1 - base).
 * Outputs (flat, one entry per kept token): query_responses, attention_masks, position_ids,
 * response_masks (0 on query tokens, i + 1 on response tokens, or only where r_tool_mask != 0 when
 * mask_tool_use), dones (i + 1 on the last token of sequence i, else 0), vllm_logprobs and, when
 * `advantages` (fp32 [n_seqs]) is given, out_advantages = advantages[i] where response_masks != 0.
 * ------------------------------------------------------------------------------------------ */
int oi_pack_sequences(const int64_t* q_tokens, const int64_t* q_offsets, const int64_t* r_tokens,
                      const int64_t* r_offsets, const uint8_t* r_tool_mask, const float* r_logprobs,
                      const float* advantages, const int64_t* dst_offsets, const int32_t* mask_base, int64_t n_seqs,
                      int64_t pad_token_id, int mask_tool_use, int64_t* query_responses, int64_t* attention_masks,
                      int64_t* position_ids, int64_t* response_masks, int64_t* dones, float* vllm_logprobs,
                      float* out_advantages, void* stream);

/* ------------------------------------------------------------------------------------------
 * Fused lm_head projection + per-token logprob / entropy, logits never materialised.
 *
 * Replaces the pair "lm_head GEMM -> calculate_per_token_logps" of
 * open_instruct/olmo_core_train_modules.py:71-76 (DPOLMHead.forward) and
 * open_instruct/grpo_utils.py:558-572 (forward_for_logprobs); no single reference function
 * computes it.  hidden: bf16 [n_tokens, hidden_dim]; weight: bf16 [vocab, hidden_dim] (both
 * row-major, 16-byte aligned, hidden_dim a multiple of 64; n_tokens, vocab and hidden_dim at most
 * 2^22 per call); labels int64 [n_tokens], negative
 * labels are scored as token 0 (clamp(min=0) at open_instruct/padding_free_collator.py:15).
 *
 *   z = hidden @ weight^T (bf16 MFMA, fp32 accumulate), logprob/entropy/lse as for oi_lsg_*.
 *
 * row_mask (one byte per token, may be NULL = every row): rows whose byte is 0 are not multiplied
 * and their outputs are 0 (prompt and padding positions, whose results the reference masks out
 * afterwards: open_instruct/grpo_utils.py:340-344, open_instruct/dpo_utils.py:689-712).  The
 * selection is made on the device: a row index is built from the mask and the selected rows are
 * gathered into the workspace, every kernel reads the selected count from device memory, the host
 * never waits.  The workspace is sized for all n_tokens rows either way.
 * ------------------------------------------------------------------------------------------ */
size_t oi_lmhead_fwd_workspace_bytes(int64_t n_tokens, int64_t hidden_dim, int64_t vocab, int with_row_mask);
int oi_lmhead_logp_fwd(const void* hidden, const void* weight, const int64_t* labels, const uint8_t* row_mask,
                       int64_t n_tokens, int64_t hidden_dim, int64_t vocab, float inv_temperature, float* logprob,
                       float* entropy, float* lse, void* workspace, size_t workspace_bytes, void* stream);

/*
 * Backward: recomputes the logits tile by tile,
 *   dZ[n, v] = grad_logprob[n] * inv_T * (1[v == label_n] - exp(z[n,v] * inv_T - lse[n])),
 *   d_hidden = dZ @ weight   (bf16 [n_tokens, hidden_dim]),
 *   d_weight = dZ^T @ hidden (bf16 [vocab, hidden_dim]; NULL skips it).
 * Vocabulary is processed in chunks of 32768 columns; only one chunk of dZ (bf16, token-major)
 * lives in the workspace at a time, next to the fp32 accumulator of d_hidden.  Both products
 * read weight, hidden and dZ where they lie (no transposed copies), so the workspace is the same
 * with and without d_weight.  row_mask as in the forward (rows left out get a zero d_hidden row
 * and add nothing to d_weight); skip_zero_grad_rows != 0 also leaves out rows whose grad_logprob is
 * exactly 0, which changes no result.
 * d_hidden and d_weight must be 4-byte aligned.  logprob is the forward's output for the same rows:
 * the label's entry of dZ is taken from it as -grad * inv_T * expm1(logprob), which stays exact
 * where the label's probability is close to 1.
 */
size_t oi_lmhead_bwd_workspace_bytes(int64_t n_tokens, int64_t hidden_dim, int64_t vocab, int want_d_weight,
                                     int with_row_selection);
int oi_lmhead_logp_bwd(const void* hidden, const void* weight, const int64_t* labels, const float* lse,
                       const float* grad_logprob, const uint8_t* row_mask, int skip_zero_grad_rows, int64_t n_tokens,
                       int64_t hidden_dim, int64_t vocab, float inv_temperature, const float* logprob, void* d_hidden,
                       void* d_weight, void* workspace, size_t workspace_bytes, void* stream);

/*
 * Kept exponentials (what the two entry-point families below share).  The forward evaluates
 * 2^(x[n,v] - max) for its statistics anyway (x = z * inv_T * log2 e); where a backward pass follows
 * that can use them, it also stores them, as bf16, relative to a per-token reference exponent:
 *   e'[n, v] = 2^(x[n,v] - xref[n]),   xref[n] = x[n, label_n]  (a dot product taken beforehand),
 * so that dZ[n, v] = s_n * (e'[n, v] - 1[v = label_n] * 2^(lse2_n - xref[n])) with the per-token
 * factor s_n = -g_n * inv_T * 2^(xref[n] - lse2_n) moved out of the products and the label's entry
 * rebuilt from the fp32 logprob.  Relative to the label's own logit the stored numbers and the
 * factor stay inside the bf16 / fp32 range whatever the magnitude of the logits and the
 * temperature, as long as the token's largest logit is less than 64 binary orders (44 nats) above
 * its label's.  A token beyond that (a label of probability below about e^-44), or whose logits hold
 * a NaN, is flagged on the device and served by the recomputing backward instead, inside the same
 * call and without a host read: results are those of the reference's exact log_softmax
 * (open_instruct/padding_free_collator.py:10-16, open_instruct/model_utils.py:587-600) either way.
 */

/*
 * Forward + backward for callers that need d_hidden only (a frozen lm_head: the DPO / reward passes of
 * open_instruct/dpo_utils.py:959-1019 through DPOLMHead when the head's weight takes no gradient, or
 * any d_weight == NULL use of oi_lmhead_logp_bwd).  With e' and xref as above,
 *   d_hidden[n] = s_n * sum_{v != label_n} e'[n,v] * weight[v]  -  g_n * inv_T * expm1(logprob_n) * weight[label_n],
 * and the sum does not depend on the upstream gradient g: oi_lmhead_logp_fwd_wsum computes it together
 * with logprob / entropy / lse while the logits exist (one chunk of 65536 vocabulary columns at a
 * time: the chunk's exponentials as bf16 in the workspace, then wsum (+)= E_chunk @ weight_chunk in
 * fp32), and oi_lmhead_dh_from_wsum turns it into d_hidden in one pass over [n_tokens, hidden_dim].
 * Matrix work of forward + backward: 4 N H V instead of 6 N H V, nothing is recomputed, nothing of size
 * [tokens, vocab] exists.
 * wsum: fp32 [n_tokens, hidden_dim], 16-byte aligned; xref: fp32 [n_tokens]; unsafe: one byte per
 * token (set for flagged tokens): all three are outputs of the forward call that the caller holds
 * until the backward call.  Row j of wsum / xref belongs to the j-th selected row (rows in ascending
 * order; every row without a row_mask), unsafe is indexed like the caller's rows.  The backward call
 * takes the same hidden / labels / row_mask and the forward's lse and logprob; rows left out get a zero
 * d_hidden row, flagged rows are recomputed (the workspace holds the recomputing backward's buffers,
 * which are only touched for such rows).  d_hidden: bf16 [n_tokens, hidden_dim], 8-byte aligned.
 */
size_t oi_lmhead_fwd_wsum_workspace_bytes(int64_t n_tokens, int64_t hidden_dim, int64_t vocab, int with_row_mask);
int oi_lmhead_logp_fwd_wsum(const void* hidden, const void* weight, const int64_t* labels, const uint8_t* row_mask,
                            int64_t n_tokens, int64_t hidden_dim, int64_t vocab, float inv_temperature, float* logprob,
                            float* entropy, float* lse, float* wsum, float* xref, uint8_t* unsafe, void* workspace,
                            size_t workspace_bytes, void* stream);
size_t oi_lmhead_dh_workspace_bytes(int64_t n_tokens, int64_t hidden_dim, int64_t vocab);
int oi_lmhead_dh_from_wsum(const void* hidden, const void* weight, const int64_t* labels, const float* lse,
                           const float* logprob, const float* grad_logprob, const uint8_t* row_mask, const float* wsum,
                           const float* xref, const uint8_t* unsafe, int64_t n_tokens, int64_t hidden_dim,
                           int64_t vocab, float inv_temperature, void* d_hidden, void* workspace,
                           size_t workspace_bytes, void* stream);

/*
 * The whole GRPO step on hidden states in one call: fused lm_head forward (logprob, entropy),
 * scalar loss with its statistics, and the backward to d_hidden / d_weight, for an upstream
 * gradient of 1 on the loss.  It replaces, for a model that hands out its final hidden states, the
 * sequence open_instruct/grpo_utils.py:558-572 (lm_head, log_softmax_and_gather, entropy) ->
 * open_instruct/grpo_utils.py:504-538 (compute_grpo_loss) -> open_instruct/grpo_fast.py:702-724
 * (masked_mean, loss.backward()); no single reference function computes it.
 *
 * hidden: bf16 [rows * cols, hidden_dim]; labels int64, mask (one byte per token) and the fp32 side
 * tensors are [rows, cols]; `mask` is the response mask: it selects the rows that are multiplied
 * and the tokens that enter the loss.  old_logprobs NULL: ratio 1 with gradient; ref_logprobs NULL:
 * no KL term; rho_weights NULL: 1.  Loss arguments and out_stats as for oi_grpo_fused_fwd (the rho
 * indicator statistics [10..12, 14] are 0 here).  logprob / entropy (may be NULL) are fp32
 * [rows, cols], 0 off the mask.  d_weight NULL skips that product.  A token's upstream gradient
 * depends only on its own logprob once the denominators are known, and those come from the mask, so
 * the backward is enqueued straight behind the forward: nothing returns to the host in between.
 *
 * slab_tokens == 0: one forward over all selected rows, then the recomputing backward of
 * oi_lmhead_logp_bwd (8 N H V of matrix work).
 * slab_tokens > 0 (rounded up to a multiple of 256): the step runs in slabs of at most that many
 * selected tokens and recomputes nothing.  The selected rows are split on the device into the fewest
 * equal slabs; a slab's forward leaves its kept exponentials (every vocabulary column, bf16, see
 * above) in a slab-sized buffer inside the workspace, the slab's tokens get their upstream gradient
 * at once, and both products read the buffer before the next slab overwrites it: d_hidden rows are
 * final, d_weight accumulates in fp32 over the slabs (deterministic: slab after slab) and is rounded
 * to bf16 once.  6 N H V of matrix work instead of 8 N H V; the workspace holds [slab, vocab] bf16 and,
 * with d_weight and more than one slab, an fp32 [vocab, hidden_dim], never anything of size
 * [tokens, vocab].  Flagged tokens (see above) are recomputed after the last slab.
 * oi_lmhead_grpo_workspace_bytes takes the same slab_tokens and whether d_weight is wanted.
 */
size_t oi_lmhead_grpo_workspace_bytes(int64_t rows, int64_t cols, int64_t hidden_dim, int64_t vocab,
                                      int want_d_weight, int64_t slab_tokens);
int oi_lmhead_grpo_fwd_bwd(const void* hidden, const void* weight, const int64_t* labels, const uint8_t* mask,
                           const float* old_logprobs, const float* ref_logprobs, const float* advantages,
                           const float* rho_weights, int64_t rows, int64_t cols, int64_t hidden_dim, int64_t vocab,
                           float inv_temperature, int loss_fn, float ratio_lo, float ratio_hi, int kl_estimator,
                           float beta, int axis_mode, float denominator, float scale, float* logprob, float* entropy,
                           float* out_stats, void* d_hidden, void* d_weight, int64_t slab_tokens, void* workspace,
                           size_t workspace_bytes, void* stream);

/*
 * The whole DPO step on hidden states in one call, with nothing recomputed and with a d_weight: the
 * fused lm_head forward (per-token logps), the per-sequence sums, the sigmoid preference loss per pair
 * and the backward to d_hidden / d_weight.  It replaces, for a model that hands its final hidden
 * states to the head, the sequence open_instruct/olmo_core_train_modules.py:71-76 (DPOLMHead: w_out,
 * calculate_per_token_logps) -> open_instruct/padding_free_collator.py:202-229 or
 * open_instruct/dpo_utils.py:689-712 (per-sequence logps) -> open_instruct/dpo_utils.py:523-563 /
 * :617-642 (dpo_loss / simpo_loss) -> losses.mean().backward()
 * (open_instruct/olmo_core_train_modules.py:190-207); no single reference function computes it.
 *
 * hidden: bf16 [n, hidden_dim]; labels: the batch's own (unshifted) int64 labels; position t is scored
 * against labels[t + 1] when that is not -100.  cu_seq_lens NULL: n_seqs padded rows of `total`
 * positions (n = n_seqs * total); otherwise one packed row of `total` positions with boundaries
 * cu_seq_lens int32 [n_seqs + 1] (n = total), segments as for oi_seq_logp_fwd.  The first n_seqs / 2
 * sequences are the chosen answers, the others the rejected ones, pair i = (i, n_seqs / 2 + i)
 * (open_instruct/dpo_utils.py:876-877).  ref_chosen / ref_rejected (fp32 [n_seqs / 2], both or
 * neither), beta, label_smoothing, margin as for oi_dpo_sigmoid_fwd; average_log_prob != 0 divides
 * every sequence sum by its count (dpo_norm, simpo).  grad_scale is d (caller's scalar) / d losses[i],
 * e.g. 1 / (n_seqs / 2) for losses.mean().
 * Outputs: per_token_logps fp32 [n] (0 where nothing is scored), seq_logps fp32 [n_seqs], losses and
 * (optional) rewards fp32 [n_seqs / 2], d_hidden bf16 [n, hidden_dim] (zero rows where nothing is
 * scored), d_weight bf16 [vocab, hidden_dim] (NULL skips it).
 *
 * The step runs like the slab-wise oi_lmhead_grpo_fwd_bwd, with the slabs (at most slab_tokens
 * scored rows, > 0) filled with whole pairs: a token's upstream gradient depends on the sums of both
 * sequences of its pair, so a pair's rows are gathered next to each other (the row index is built on
 * the device in pair order) and a slab ends where the next pair would not fit.  A pair with more
 * scored rows than a slab holds is cut across slabs and its tokens take the recomputing backward
 * after the last slab, like flagged tokens; pass a slab_tokens of at least the largest pair to avoid
 * that.  6 N H V of matrix work; the workspace holds [slab, vocab] bf16 and, with d_weight, an fp32
 * [vocab, hidden_dim].
 */
size_t oi_lmhead_dpo_workspace_bytes(int64_t n_seqs, int64_t total, int packed, int64_t hidden_dim, int64_t vocab,
                                     int want_d_weight, int64_t slab_tokens);
int oi_lmhead_dpo_fwd_bwd(const void* hidden, const void* weight, const int64_t* labels, const int32_t* cu_seq_lens,
                          int64_t n_seqs, int64_t total, int64_t hidden_dim, int64_t vocab, float inv_temperature,
                          const float* ref_chosen, const float* ref_rejected, float beta, float label_smoothing,
                          float margin, int average_log_prob, float grad_scale, float* per_token_logps,
                          float* seq_logps, float* losses, float* chosen_rewards, float* rejected_rewards,
                          void* d_hidden, void* d_weight, int64_t slab_tokens, void* workspace, size_t workspace_bytes,
                          void* stream);

/*
 * Timing probe of the slab-wise entry points (no reference counterpart; it exists for the
 * measurement harness, which has to time one kernel inside a call that launches several).  Between
 * oi_lmhead_probe_arm(kernel) and oi_lmhead_probe_read the slab-wise calls of this process record a
 * pair of HIP events, on the stream of the call, around every launch of the chosen tile kernel:
 * 0 = the forward that keeps its exponentials, 1 = the d_hidden product, 2 = the d_weight product
 * (at most 1024 launches; later ones are not recorded).  oi_lmhead_probe_read waits for the recorded
 * events, writes the duration of each recorded launch in milliseconds to ms[0 .. min(n, capacity)),
 * the number of recorded launches to *n_launches, and disarms the probe.  Launches whose slab is
 * empty are recorded too (they take a few microseconds).  Not thread-safe; do not arm it around a
 * call that is captured into a graph.
 */
int oi_lmhead_probe_arm(int kernel);
int oi_lmhead_probe_read(float* ms, int capacity, int* n_launches);

/*
 * The bf16 MFMA main loop of the lm_head kernels as a plain product (no reference counterpart;
 * it exists so that the tile engine can be tested and timed on its own):
 *   out[m, n] (+)= sum_k A[m, k] * B[n, k]      A: bf16 [M, K] (row stride lda), B: bf16 [N, K] (ldb)
 * K must be a multiple of 64, A and B 16-byte aligned, lda/ldb multiples of 8 and at most 2^22 (or
 * 0 = every row aliases row 0).  Exactly one of out_f32 / out_bf16 is written (row stride ldo; out_bf16
 * 4-byte aligned when ldo is even, its rows are then stored as pairs); accumulate != 0 adds to the
 * existing fp32 output.
 */
int oi_gemm_bf16_tn(const void* A, int64_t lda, int64_t M, const void* B, int64_t ldb, int64_t N, int64_t K,
                    float* out_f32, void* out_bf16, int64_t ldo, int accumulate, void* stream);

/*
 * The same product with either operand in k-major order (no reference counterpart; test and timing
 * hook of the operand layouts that the backward of the fused lm_head uses to read weight, hidden
 * and dZ where they lie):
 *   out[m, n] (+)= sum_k a(m, k) * b(n, k),   a(m, k) = a_k_major ? A[k * lda + m] : A[m * lda + k],
 *                                             b(n, k) = b_k_major ? B[k * ldb + n] : B[n * ldb + k].
 * K must be a multiple of 64; lda/ldb positive multiples of 8, at most 2^22 and at least the
 * operand's contiguous extent; M (N) a multiple of 8 when A (B) is k-major.
 */
int oi_gemm_bf16_layouts(const void* A, int64_t lda, int a_k_major, const void* B, int64_t ldb, int b_k_major,
                         int64_t M, int64_t N, int64_t K, float* out_f32, void* out_bf16, int64_t ldo,
                         int accumulate, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* OI_KERNELS_H */
