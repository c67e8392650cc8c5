/* verl_amd.h -- C ABI of libverl_amd.so: MI355X (gfx950) kernels for verl's per-token
 * policy-math path.
 *
 * Conventions
 *   - every pointer is a DEVICE pointer unless its name ends in _host;
 *   - every function is asynchronous on `stream` (a hipStream_t passed as void*), allocates
 *     nothing and keeps no state between calls: scratch comes from the caller through
 *     (workspace, workspace_bytes); the matching *_workspace_bytes() gives the size needed;
 *   - the reductions (masked moments, agg_loss, policy / value / KL loss, the advantage
 *     estimators) finish inside one launch through arrival counters in the FIRST
 *     VAMD_TICKET_BYTES of their workspace: those bytes must be zero on entry, or as an earlier
 *     call of this library left them, and are zero again when the call has completed -- except two
 *     32-bit words that no kernel depends on: byte 132, an epoch that vamd_grpo_advantage advances, and
 *     byte 136 (VAMD_TICKET_GAVE_UP_OFFSET), a count of the workgroups that gave up a bounded wait on this
 *     buffer and carried on by other means, which a host may read now and then --
 *     so a caller may zero a buffer once and reuse it for calls that are ordered on one stream;
 *   - return value: 0 on success, a negative VAMD_E* code otherwise; vamd_last_error() returns a
 *     thread-local description of the last failure on the calling thread;
 *   - "mask" arguments come with a VAMD_MASK_* code naming their element type; the value used is
 *     (float)mask[i], and mask[i] != 0 decides membership, exactly as
 *     masked_sum does in the reference (verl/utils/torch_functional.py:283-284).
 *
 * Each entry point cites the reference interface it stands behind (paths relative to the
 * reference tree).
 */
#ifndef VERL_AMD_H_
#define VERL_AMD_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define VAMD_OK 0
#define VAMD_EINVAL (-1)    /* bad shape / null pointer / unsupported option */
#define VAMD_EWORKSPACE (-2) /* workspace missing or too small */
#define VAMD_EHIP (-3)      /* a HIP runtime call failed; see vamd_last_error() */

#define VAMD_TICKET_BYTES 16640 /* 65 arrival counters, 256 bytes apart */
#define VAMD_TICKET_GAVE_UP_OFFSET 136 /* u32: workgroups that ever gave up a bounded wait on this buffer */

#define VAMD_MASK_F32 0
#define VAMD_MASK_I64 1
#define VAMD_MASK_U8 2 /* torch.bool and torch.uint8 */
#define VAMD_MASK_I32 3

/* loss_agg_mode of agg_loss (verl/trainer/ppo/core_algos.py:1025-1080) */
#define VAMD_AGG_TOKEN_MEAN 0
#define VAMD_AGG_SEQ_MEAN_TOKEN_SUM 1
#define VAMD_AGG_SEQ_MEAN_TOKEN_MEAN 2
#define VAMD_AGG_SEQ_MEAN_TOKEN_SUM_NORM 3

/* estimator of kl_penalty_forward (verl/trainer/ppo/core_algos.py:1868-1902) */
#define VAMD_KL_K1 0  /* "kl", "k1": logprob - ref */
#define VAMD_KL_ABS 1 /* "abs" */
#define VAMD_KL_K2 2  /* "mse", "k2": 0.5 (logprob - ref)^2 */
#define VAMD_KL_K3 3  /* "low_var_kl", "k3": exp(k) - k - 1, k = clamp(ref - logprob, -20, 20), clamped to [-10, 10] */

/* outcome-reward advantage estimators that reduce a response to one score and normalise it inside its
 * prompt group (verl/trainer/ppo/core_algos.py:266-330, :421-579, :657-753) */
#define VAMD_ADV_GRPO 0            /* (s - mean) / (std + eps), or s - mean */
#define VAMD_ADV_RLOO 1            /* s n/(n-1) - mean n/(n-1); a single-member group keeps s */
#define VAMD_ADV_RLOO_VECTORIZED 2 /* the same; a single-member group gets 0 */
#define VAMD_ADV_MEAN_BASELINE 3   /* s - mean: REINFORCE++ baseline before its whitening */
#define VAMD_ADV_OPO 4             /* s - sum(len s) / sum(len), len = response length */
#define VAMD_ADV_GPG 5             /* alpha (s - mean) / f_norm, alpha = batch / max(#{s != 0}, 1) */
#define VAMD_ADV_GRPO_PASSK 6      /* best response of a group: (max - second max) [/ (std + eps)]; others 0;
                                      every group needs at least two responses (checked by the caller) */

/* policy-loss variants of the registry (core_algos.py:1159-1447, :1721-1779) */
#define VAMD_PL_VANILLA 0 /* clipped PPO with the dual-clip floor */
#define VAMD_PL_GPG 1     /* -log_prob A */
#define VAMD_PL_CISPO 2   /* -sg(clip(ratio)) A log_prob */
#define VAMD_PL_SAPO 3    /* -4/tau sigmoid(tau (ratio - 1)) A, tau by the sign of A */
#define VAMD_PL_GSPO 4    /* clipped objective on the sequence-level importance ratio */
#define VAMD_PL_REINFORCE 5 /* -log_prob A; the KL metric is taken against old_log_prob = the rollout policy */
#define VAMD_PL_GEO_MEAN 6  /* GMPO: -A_seq exp(mean_t of the sign-aware clipped log-ratio); mean over all rows */

/* token-level return recurrences (core_algos.py:582-654) */
#define VAMD_RETURNS_REMAX 0        /* returns = reverse cumsum of r m; adv = returns - baseline_i m */
#define VAMD_RETURNS_REINFORCE_PP 1 /* R_t = r_t + gamma c, c <- R_t m_t; adv = masked_whiten(R, m) m */

/* Bumped whenever an entry point changes its signature or a workspace its layout; a binding compares it with
 * the header it was written against. */
#define VAMD_ABI_VERSION 5
int vamd_abi_version(void);
const char* vamd_last_error(void);

/* Process-wide switch for the kernels whose workgroups wait for each other inside one launch (vamd_gae with
 * whiten = 1, vamd_grpo_advantage, GSPO / GMPO in vamd_policy_loss_variant_forward): 0 keeps every entry point to
 * launches that never wait, 1 allows the waiting forms, a negative value hands the decision back to the environment
 * variable VAMD_WAITING_KERNELS (unset or anything but "0" = allowed).  Meant for a host that has seen one bounded
 * wait run out (vamd_gae reports it in moments_out[4]) on a GPU it shares with other long-running kernels: a
 * time-out costs about a second of polling, and the conditions behind it rarely go away between two calls.
 * No counterpart in the reference, whose estimators are sequences of torch launches. */
void vamd_set_waiting_kernels(int allowed);
int vamd_waiting_kernels_enabled(void);

/* ------------------------------------------------------------------------------------------
 * Fused vocab-projection log-prob / entropy head.
 * Replaces kernels.efficient_entropy_forward / efficient_entropy_backward behind
 * LinearCrossEntropy (verl/utils/kernel/linear_cross_entropy.py:40-116,
 * verl/utils/kernel/kernels.py:563-753 and :1512-1723).
 *
 *   hidden [n_tokens, hidden_size] bf16 row-major, weight [vocab, hidden_size] bf16 row-major,
 *   labels [n_tokens] int64 in [0, vocab).  hidden_size % 128 == 0 (kernels.py:593); any vocab
 *   (the vocabulary tail is masked as the reference does); a logits cache needs vocab % 8 == 0.
 *   z = hidden . weight^T * rcp_temperature ; logprobs = z[label] - lse(z) ;
 *   entropy = lse(z) - sum softmax(z) z.
 *   lse[n] and mean_z[n] (= sum softmax(z) z) are saved for the backward pass in place of the
 *   reference's (maximum, accumulate, entropy_b) triple.
 *   logits_cache: NULL, or [n_tokens, vocab] fp32 (16-byte aligned) that receives z.  Handing the
 *   same buffer to vamd_lce_backward replaces its logits-recompute GEMM by a streaming pass: a
 *   trade of 4 * n_tokens * vocab bytes of HBM (10 GB at 16384 x 152064) for a quarter of the
 *   step's matrix work.  Results do not depend on the choice beyond fp32 rounding of z.
 *   sum_pi_squared: NULL, or [n_tokens] fp32 that receives sum_j softmax(z)_j^2
 *   (calculate_sum_pi_squared_from_logits, verl/utils/torch_functional.py:680-694), carried as a
 *   fifth running sum of the same online softmax; the reference cannot combine this statistic with
 *   its fused kernels (verl/workers/actor/dp_actor.py:107-111).
 */
size_t vamd_lce_forward_workspace_bytes(int64_t n_tokens, int64_t hidden_size, int64_t vocab);
int vamd_lce_forward(const void* hidden, const void* weight, const int64_t* labels, int64_t n_tokens,
                     int64_t hidden_size, int64_t vocab, float rcp_temperature, float* logprobs, float* entropy,
                     float* lse, float* mean_z, float* logits_cache, float* sum_pi_squared, void* workspace,
                     size_t workspace_bytes, void* stream);

/* The forward pass for callers that cannot allocate device memory or hand over a workspace: code under
 * HIP graph capture, tight serving loops, harnesses that forbid hipMalloc.  It has no counterpart in the
 * reference.  Same arguments, arithmetic and results as vamd_lce_forward without a logits cache; the
 * softmax partials of the (token tile, vocabulary split) workgroups go to a buffer built into the library
 * (VAMD_LCE_STATIC_MAX_TOKENS * 20 + 512 bytes of device memory, held by every GPU the library is
 * used on until the process ends).  n_tokens above VAMD_LCE_STATIC_MAX_TOKENS is refused with VAMD_EINVAL.
 * The call allocates nothing and records no memset.  All calls on one GPU share the one buffer: calls on
 * different streams of the same GPU that may overlap race on it; calls ordered on one stream do not.
 * The first call on a device looks up the buffer's address and raises the kernels' LDS limit, so make it
 * before a capture begins. */
#define VAMD_LCE_STATIC_MAX_TOKENS 65536
int vamd_lce_forward_static(const void* hidden, const void* weight, const int64_t* labels, int64_t n_tokens,
                            int64_t hidden_size, int64_t vocab, float rcp_temperature, float* logprobs,
                            float* entropy, float* lse, float* mean_z, float* sum_pi_squared, void* stream);

/* Backward: d_logits = [g_lp (onehot - p) - g_ent p (z - mean_z)] * rcp_temperature is formed one
 * vocabulary chunk at a time as a bf16 [n_pad, vocab_chunk] panel in the workspace -- from logits
 * recomputed tile by tile on the matrix cores (logits_cache == NULL: no [n_tokens, vocab] tensor ever
 * exists, as in the reference, kernels.py:1374-1509) or from the cache the forward call filled (a
 * streaming pass instead of the recompute GEMM) -- and consumed by d_hidden = d_logits . weight and
 * d_weight = d_logits^T . hidden, both accumulated in fp32 and rounded to bf16 once.
 *   d_logprobs [n] fp32 or NULL (treated as zeros);
 *   d_entropy  [n] fp32 or NULL, in which case the constant d_entropy_scalar is used for every
 *   token (an entropy-bonus coefficient folded into the backward pass);
 *   d_hidden [n, hidden_size] bf16 out; d_weight [vocab, hidden_size] bf16 out.
 *   d_weight_mode says where this call's weight gradient goes (token-chunked callers sum several calls):
 *     VAMD_DW_STORE            d_weight = bf16(g)                                (d_weight_acc32 unused)
 *     VAMD_DW_ADD_BF16         d_weight = bf16(d_weight + g): one bf16 rounding of the running sum per call,
 *                              what `weight.grad += d_weight` does in the reference's bf16 training
 *     VAMD_DW_F32_STORE        d_weight_acc32 = g                                (d_weight may be NULL)
 *     VAMD_DW_F32_ADD          d_weight_acc32 += g                               (d_weight may be NULL)
 *     VAMD_DW_F32_ADD_FINISH   d_weight_acc32 += g; d_weight = bf16(d_weight_acc32): the sum over all token
 *                              chunks is rounded once
 *     VAMD_DW_NONE             no weight gradient: the d_weight GEMM is not run (a frozen lm_head)
 *   d_weight_acc32: [vocab, hidden_size] fp32, 16-byte aligned, for the three F32 modes.
 *   d_hidden may be NULL when the hidden states need no gradient: the d_hidden GEMM is then not run.  Like the
 *   reference's torch backend, which allocates and accumulates only the gradients whose inputs require them
 *   (verl/utils/experimental/torch_functional.py:150-156, :184-187); one of the two must be asked for.
 * vocab_chunk = 0 lets the library choose how many vocabulary columns of d_logits are staged
 * at a time (the workspace holds one [n_pad, vocab_chunk] bf16 panel plus an fp32 d_hidden
 * accumulator); pass the same value to the workspace query.
 */
#define VAMD_DW_STORE 0
#define VAMD_DW_ADD_BF16 1
#define VAMD_DW_F32_STORE 2
#define VAMD_DW_F32_ADD 3
#define VAMD_DW_F32_ADD_FINISH 4
#define VAMD_DW_NONE 5
size_t vamd_lce_backward_workspace_bytes(int64_t n_tokens, int64_t hidden_size, int64_t vocab, int64_t vocab_chunk);
int vamd_lce_backward(const void* hidden, const void* weight, const int64_t* labels, int64_t n_tokens,
                      int64_t hidden_size, int64_t vocab, float rcp_temperature, const float* lse,
                      const float* mean_z, const float* d_logprobs, const float* d_entropy, float d_entropy_scalar,
                      const float* logits_cache, void* d_hidden, void* d_weight, int d_weight_mode,
                      float* d_weight_acc32, int64_t vocab_chunk, void* workspace, size_t workspace_bytes,
                      void* stream);

/* ------------------------------------------------------------------------------------------
 * Per-token log-prob / entropy from materialised logits: the unfused definitions the actor uses when the
 * fused head is off.  logprobs_from_logits / _v2 / _naive (verl/utils/torch_functional.py:72-100, :148-200),
 * entropy_from_logits / entropy_from_logits_with_chunking (:224-263).
 *   logits [n_rows, vocab] with row pitch ld (elements), element type VAMD_DT_*; arithmetic in fp32;
 *   labels [n_rows] int64 (may be NULL when logprobs is NULL).  A label outside [0, vocab) -- an ignore index such
 *   as -100, a padding id -- reads no logit: its logprobs entry is 0 and it receives no one-hot term in the
 *   backward pass (the reference's gather would fault on it; 0 is what flash-attn's cross_entropy_loss returns
 *   for its ignore index).
 *   logprobs = z[label] - lse(z); entropy = lse(z) - sum softmax(z) z; lse and mean_z (= sum softmax(z) z) are
 *   what the backward pass needs.  Every output is fp32 [n_rows] and may be NULL if not wanted.
 * One pass over the logits (online softmax), no workspace. */
#define VAMD_DT_F32 0
#define VAMD_DT_BF16 1
#define VAMD_DT_F16 2
int vamd_row_softmax_stats(const void* logits, int dtype, int64_t n_rows, int64_t vocab, int64_t ld,
                           const int64_t* labels, float* logprobs, float* entropy, float* lse, float* mean_z,
                           void* stream);
/* d_logits = d_logprobs (onehot(label) - p) - d_entropy p (z - mean_z), p = exp(z - lse): what autograd hands back
 * through log_softmax + gather (logprobs_from_logits_naive) and through logsumexp - sum softmax * z
 * (entropy_from_logits).  d_logprobs / d_entropy: fp32 [n_rows], either may be NULL (no contribution);
 * d_logits has the element type of logits and row pitch ld_out, and may be the logits buffer itself (in place, the
 * reference's inplace_backward). */
int vamd_row_softmax_backward(const void* logits, int dtype, int64_t n_rows, int64_t vocab, int64_t ld,
                              const int64_t* labels, const float* lse, const float* mean_z, const float* d_logprobs,
                              const float* d_entropy, void* d_logits, int64_t ld_out, void* stream);
/* clip_by_value (verl/utils/torch_functional.py:203-221): out = max(min(x, hi), lo) over n fp32 elements, and its
 * gradients with torch's rule for binary min / max (the selected operand takes the gradient, equal operands half
 * each); d_x / d_lo / d_hi may be NULL.  A NaN in x, lo or hi gives a NaN output, as torch.min / torch.max of two
 * tensors do, and (every comparison with it being false) the whole upstream gradient to both operands of that
 * min / max, which is what torch's backward formulas produce. */
int vamd_clip_by_value(const float* x, const float* lo, const float* hi, int64_t n, float* out, void* stream);
int vamd_clip_by_value_backward(const float* x, const float* lo, const float* hi, const float* grad_out, int64_t n,
                                float* d_x, float* d_lo, float* d_hi, void* stream);

/* ------------------------------------------------------------------------------------------
 * Masked reductions: verl/utils/torch_functional.py:266-339.
 * vamd_masked_moments writes out[0..3] (double): sum(m), sum(where(m,v,0)*m),
 * sum(where(m,v,0)^2*m), count(m != 0)  -- the sufficient statistics of masked_sum / masked_mean /
 * masked_var.  rows x cols elements; with per_row != 0 it writes 4 doubles per row instead
 * (masked_sum / masked_mean with axis=-1).
 */
size_t vamd_masked_moments_workspace_bytes(int64_t rows, int64_t cols);
int vamd_masked_moments(const float* values, const void* mask, int mask_dtype, int64_t rows, int64_t cols,
                        int per_row, double* out, void* workspace, size_t workspace_bytes, void* stream);
/* The same reduction with the results the callers are after derived in the same launch (each output may be NULL):
 * moments as above; sum = masked_sum; mean = masked_mean = sum / (sum(mask) + 1e-8); denom = sum(mask) + 1e-8
 * (fp32, [rows] with per_row != 0, else [1]); whiten_stats [4] = (mean, rsqrt(unbiased var + 1e-8), shift) of
 * masked_whiten over the whole input (per_row must be 0), ready for vamd_affine_by_stats.  Same workspace as
 * vamd_masked_moments. */
int vamd_masked_reduce(const float* values, const void* mask, int mask_dtype, int64_t rows, int64_t cols,
                       int per_row, double* moments, float* sum, float* mean, float* denom, float* whiten_stats,
                       int shift_mean, void* workspace, size_t workspace_bytes, void* stream);

/* out[i] = (values[i] - stats[0]) * stats[1] + stats[2], stats being three DEVICE floats
 * (mean, rsqrt(var + 1e-8), re-added mean or 0): the elementwise half of masked_whiten
 * (torch_functional.py:335-339).  vamd_whiten_stats fills stats from vamd_masked_moments'
 * output following masked_var's unbiased rule; flags_host receives nothing -- the M in {0,1}
 * error of masked_var (:311-316) is raised by the host wrapper from the moments. */
int vamd_whiten_stats(const double* moments, int shift_mean, float* stats, void* stream);
/* out[i] = ((values[i] - mean) * rstd + shift) * mask[i]: whitening followed by the mask product of the
 * REINFORCE++ estimators (core_algos.py:472, :615-616). */
int vamd_affine_by_stats_masked(const float* values, const float* stats, const void* mask, int mask_dtype, int64_t n,
                                float* out, void* stream);
int vamd_affine_by_stats(const float* values, const float* stats, int64_t n, float* out, void* stream);

/* ------------------------------------------------------------------------------------------
 * GAE: compute_gae_advantage_return (verl/trainer/ppo/core_algos.py:214-262).
 * rewards, values [B, L] fp32, mask [B, L]; advantages (whitened) and returns [B, L] fp32 out.
 * The recurrence is evaluated as a chunked associative scan (a most-recent-valid-value scan for the
 * bootstrap value, then a one-variable affine scan for the advantage); masked steps carry the state.
 * whiten == 0 leaves the raw advantages (the value before :261).  With whiten == 1 the whole estimator is one
 * launch whose workgroups meet once (the grid is capped at what the device holds at a time): the masked
 * moments are folded, and every workgroup whitens what it produced.  whiten == 2 does the same in two launches
 * whose workgroups never wait for each other; VAMD_WAITING_KERNELS=0 in the environment makes 1 behave as 2 (and
 * keeps vamd_grpo_advantage / vamd_group_outcome_advantage to their several-launch paths), for a GPU that other
 * long-running kernels share.
 * moments_out (5 doubles, may be NULL) receives the masked moments of the raw advantages (sum m, sum g m,
 * sum g^2 m, count) so the host can raise masked_var's M in {0,1} error; moments_out[4] is 0, or 1 if the
 * workgroups' bounded wait for each other ran out (the advantages are then left raw; VAMD_GATE_SPIN_LIMIT in the
 * environment overrides the bound).
 */
size_t vamd_gae_workspace_bytes(int64_t batch, int64_t length);
int vamd_gae(const float* rewards, const float* values, const void* mask, int mask_dtype, int64_t batch,
             int64_t length, float gamma, float lam, int whiten, float* advantages, float* returns,
             double* moments_out, void* workspace, size_t workspace_bytes, void* stream);

/* ------------------------------------------------------------------------------------------
 * GRPO: compute_grpo_outcome_advantage (core_algos.py:266-330) and its vectorised twin
 * (:333-357) with group_mean_std (verl/utils/groupwise.py:163-223).
 * group_ids [B] int64, contiguous ids in [0, n_groups) (the host factorises arbitrary labels as
 * groupwise.as_torch_index does).  std_mode 0: unbiased torch.std (loop form); 1:
 * sqrt(clamp(var, min=eps)) (vectorised form).  scores_out [B] (may be NULL) receives the
 * normalised scalar per response.
 * Up to 8192 responses the estimator is one launch: every workgroup leaves its rows' scores in memory, waits
 * (a bounded number of polls) for the scores of its groups' other members, and derives the group statistics
 * itself; a workgroup whose wait runs out sums the members' rows itself, to the same bits, so the result does
 * not depend on the launch's workgroups all running at once.  Larger batches, and VAMD_WAITING_KERNELS=0, take
 * a row-sum launch, a statistics launch and a broadcast launch.
 */
size_t vamd_grpo_workspace_bytes(int64_t batch, int64_t length, int64_t n_groups);
int vamd_grpo_advantage(const float* rewards, const void* mask, int mask_dtype, const int64_t* group_ids,
                        int64_t batch, int64_t length, int64_t n_groups, float epsilon, int norm_by_std,
                        int std_mode, float* advantages, float* scores_out, void* workspace,
                        size_t workspace_bytes, void* stream);

/* The group-normalised outcome estimators above behind one entry point; vamd_grpo_advantage is the
 * VAMD_ADV_GRPO case.  std_mode and norm_by_std only matter for GRPO, f_norm only for GPG.  Estimators
 * other than GRPO support at most 2048 groups.  The REINFORCE++-baseline estimator is
 * VAMD_ADV_MEAN_BASELINE followed by masked whitening (vamd_masked_moments, vamd_whiten_stats,
 * vamd_affine_by_stats_masked). */
size_t vamd_group_outcome_advantage_workspace_bytes(int64_t batch, int64_t length, int64_t n_groups);
int vamd_group_outcome_advantage(const float* rewards, const void* mask, int mask_dtype, const int64_t* group_ids,
                                 int64_t batch, int64_t length, int64_t n_groups, int estimator, float epsilon,
                                 int norm_by_std, int std_mode, float f_norm, float* advantages, float* scores_out,
                                 void* workspace, size_t workspace_bytes, void* stream);

/* ReMax and REINFORCE++ (core_algos.py:621-654, :582-618): returns[batch, length] by a reverse scan over
 * each response, then the advantages (ReMax: returns - row_baseline[i] * mask; REINFORCE++: whitened
 * returns * mask, row_baseline unused and may be NULL).  moments_out (optional, 3 doubles): sum(m),
 * sum(R m), sum(R^2 m) of the returns, from which a caller checks that at least two tokens are valid. */
size_t vamd_returns_advantage_workspace_bytes(int64_t batch, int64_t length);
int vamd_returns_advantage(const float* rewards, const void* mask, int mask_dtype, const float* row_baseline,
                           int64_t batch, int64_t length, float gamma, int mode, float* advantages, float* returns,
                           double* moments_out, void* workspace, size_t workspace_bytes, void* stream);

/* Optimal token baseline (compute_optimal_token_baseline_advantage, core_algos.py:756-873):
 * returns = reverse cumulative sum of rewards * mask; W = forward cumulative sum of
 * (1 - 2 exp(old_log_probs) + sum_pi_squared) [* is_weights^2] * mask; per prompt group and column
 * baseline = sum(returns W mask) / (sum(W mask) + epsilon), 0 for a group of one;
 * advantages = (returns - baseline) * mask.  The groups arrive as a row permutation: rows_by_group
 * lists the rows of group 0 first (each group's rows in ascending order), group_offsets
 * [n_groups + 1] delimits the groups.  tail_start (optional, [batch]): the baseline of row i counts as 0
 * from column tail_start[i] on (the reference's handle_zero_tail, :858-868).  is_weights may be NULL.
 * packed != 0 selects the multi-turn variant (compute_multi_turn_optimal_token_baseline_advantage,
 * :876-1004): the k-th valid token of every trajectory shares baseline column k, tail_start counts in
 * those packed columns, and rows_by_group must leave out the rows that have no valid token (their
 * advantages are 0; n_groups may then be 0).  returns is always laid out like rewards. */
size_t vamd_otb_advantage_workspace_bytes(int64_t batch, int64_t length, int packed);
int vamd_otb_advantage(const float* rewards, const void* mask, int mask_dtype, const float* old_log_probs,
                       const float* sum_pi_squared, const float* is_weights, const int64_t* rows_by_group,
                       const int64_t* group_offsets, const int64_t* tail_start, int64_t batch, int64_t length,
                       int64_t n_groups, int packed, float epsilon, float* advantages, float* returns,
                       void* workspace, size_t workspace_bytes, void* stream);

/* group_mean_std (verl/utils/groupwise.py:163-223): mean/std/count per group, singleton -> (0,1). */
int vamd_group_mean_std(const float* scores, const int64_t* group_ids, int64_t n, int64_t n_groups, float eps,
                        float* mean, float* std, float* count, void* stream);

/* ------------------------------------------------------------------------------------------
 * Remove-padding output -> response window (verl/workers/actor/dp_actor.py:316-344: pad_input to
 * [batch, seqlen], then the columns [-response_length - 1, -1)).  a / b / c: per-token values [nnz] in the
 * order of indices (b, c optional); indices: the tokens' flat positions row * seqlen + col, ascending;
 * out_*: [batch, response_length], every element written (0 where no token lies).  The gather is the
 * backward direction: d_a[i] = d_out_a[row][j] for tokens inside the window, 0 for the others.
 */
int vamd_response_window_scatter(const float* a, const float* b, const float* c, const int64_t* indices,
                                 int64_t nnz, int64_t batch, int64_t seqlen, int64_t response_length, float* out_a,
                                 float* out_b, float* out_c, void* stream);
int vamd_response_window_gather(const float* d_out_a, const float* d_out_b, const int64_t* indices, int64_t nnz,
                                int64_t batch, int64_t seqlen, int64_t response_length, float* d_a, float* d_b,
                                void* stream);

/* ------------------------------------------------------------------------------------------
 * compute_data_metrics (verl/trainer/ppo/metric_utils.py:81-225): every statistic of the step's batch
 * in one launch.  The five [batch, response_length] fp32 tensors and response_mask are read once;
 * attention_mask is [batch, prompt_length + response_length] (any VAMD_MASK_* element type) and gives
 * the prompt and response lengths (:67-70).  values may be NULL (use_critic=False: the VAL_* slots
 * and VF_EXPLAINED_VAR are then meaningless).  out: VAMD_DM_COUNT device doubles, indexed by the
 * constants below.  Sequence scores/rewards are taken over non-aborted rows (response length != 0);
 * means over an empty set come out as NaN, which the caller turns into the reference's exceptions.
 */
enum {
  VAMD_DM_SCORE_MEAN = 0, VAMD_DM_SCORE_MAX, VAMD_DM_SCORE_MIN,
  VAMD_DM_REWARD_MEAN, VAMD_DM_REWARD_MAX, VAMD_DM_REWARD_MIN,
  VAMD_DM_ADV_MEAN, VAMD_DM_ADV_MAX, VAMD_DM_ADV_MIN,
  VAMD_DM_RET_MEAN, VAMD_DM_RET_MAX, VAMD_DM_RET_MIN,
  VAMD_DM_VAL_MEAN, VAMD_DM_VAL_MAX, VAMD_DM_VAL_MIN,
  VAMD_DM_VF_EXPLAINED_VAR,
  VAMD_DM_RESP_LEN_MEAN, VAMD_DM_RESP_LEN_MAX, VAMD_DM_RESP_LEN_MIN, VAMD_DM_RESP_LEN_CLIP,
  VAMD_DM_RESP_LEN_NA_MEAN, VAMD_DM_RESP_LEN_NA_MAX, VAMD_DM_RESP_LEN_NA_MIN, VAMD_DM_RESP_LEN_NA_CLIP,
  VAMD_DM_ABORTED_RATIO,
  VAMD_DM_PROMPT_LEN_MEAN, VAMD_DM_PROMPT_LEN_MAX, VAMD_DM_PROMPT_LEN_MIN, VAMD_DM_PROMPT_LEN_CLIP,
  VAMD_DM_VALID_TOKENS, /* number of response_mask != 0 elements */
  VAMD_DM_NON_ABORTED,  /* number of rows with a non-zero response length */
  VAMD_DM_COUNT
};
size_t vamd_data_metrics_workspace_bytes(int64_t batch, int64_t response_length);
int vamd_data_metrics(const float* token_level_scores, const float* token_level_rewards, const float* advantages,
                      const float* returns, const float* values, const void* response_mask, int mask_dtype,
                      const void* attention_mask, int attention_dtype, int64_t batch, int64_t prompt_length,
                      int64_t response_length, double* out, void* workspace, size_t workspace_bytes, void* stream);

/* ------------------------------------------------------------------------------------------
 * Rollout-correction importance weights and off-policy diagnostics
 * (verl/trainer/ppo/rollout_corr_helper.py: compute_rollout_correction_weights :481-598,
 * compute_is_metrics :601-712, compute_offpolicy_metrics :835-937) in one pass over old_log_prob,
 * rollout_log_prob and the (binary) response mask.
 *   level VAMD_IS_NONE: metrics only.  rollout_log_prob may then be NULL, which leaves only
 *     TRAINING_PPL, TRAINING_LOG_PPL and VALID_TOKENS defined.
 *   level VAMD_IS_TOKEN: weights = min(exp(clamp(old - rollout, -20, 20)), threshold) * mask.
 *   level VAMD_IS_SEQUENCE: one weight per row from the row's summed log ratio, broadcast over the mask.
 * batch_normalize != 0 divides the weights by their batch mean (per token, or per non-empty sequence)
 * when that mean exceeds 1e-8; IS_BATCH_NORM_FACTOR reports the divisor (1 when not applied).
 * The IS_* metrics describe the weights before truncation, as in the reference.
 * metrics: VAMD_RC_COUNT device doubles indexed by the constants below.
 */
#define VAMD_IS_NONE 0
#define VAMD_IS_TOKEN 1
#define VAMD_IS_SEQUENCE 2
enum {
  VAMD_RC_TRAINING_PPL = 0, VAMD_RC_TRAINING_LOG_PPL, VAMD_RC_KL, VAMD_RC_K3_KL, VAMD_RC_ROLLOUT_PPL,
  VAMD_RC_ROLLOUT_LOG_PPL, VAMD_RC_LOG_PPL_DIFF, VAMD_RC_LOG_PPL_ABS_DIFF, VAMD_RC_LOG_PPL_DIFF_MAX,
  VAMD_RC_LOG_PPL_DIFF_MIN, VAMD_RC_PPL_RATIO, VAMD_RC_CHI2_TOKEN, VAMD_RC_CHI2_SEQ,
  VAMD_RC_IS_MEAN, VAMD_RC_IS_MAX, VAMD_RC_IS_MIN, VAMD_RC_IS_FRACTION_HIGH, VAMD_RC_IS_FRACTION_LOW,
  VAMD_RC_IS_STD, VAMD_RC_IS_ESS, VAMD_RC_IS_SEQ_MEAN, VAMD_RC_IS_SEQ_STD, VAMD_RC_IS_SEQ_MAX,
  VAMD_RC_IS_SEQ_MIN, VAMD_RC_IS_SEQ_MAX_DEVIATION, VAMD_RC_IS_SEQ_FRACTION_HIGH, VAMD_RC_IS_SEQ_FRACTION_LOW,
  VAMD_RC_IS_BATCH_NORM_FACTOR,
  VAMD_RC_VALID_TOKENS, /* number of mask != 0 elements */
  VAMD_RC_COUNT
};
size_t vamd_rollout_correction_workspace_bytes(int64_t batch, int64_t length);
int vamd_rollout_correction(const float* old_log_prob, const float* rollout_log_prob, const void* mask,
                            int mask_dtype, int64_t batch, int64_t length, int level, float threshold,
                            int batch_normalize, float* weights, double* metrics, void* workspace,
                            size_t workspace_bytes, void* stream);

/* Per-row sums for compute_variance_proxy_metrics (verl/trainer/ppo/metric_utils.py:306-412).  records: doubles
 * [5][chunks][batch] with chunks = vamd_rollout_rs_chunks(length): number of valid tokens, sum of advantages,
 * sum of w = 1 - 2 exp(old_log_prob) + sum_pi_squared (times is_weight^2 when is_weights is given), sum of the
 * importance weights, sum of w / max(is_weight^2, 1e-10), each over the valid tokens.  is_weights may be NULL
 * (slots 3 and 4 are then 0). */
int vamd_variance_proxy_rows(const float* advantages, const float* old_log_probs, const float* sum_pi_squared,
                             const float* is_weights, const void* mask, int mask_dtype, int64_t batch,
                             int64_t length, double* records, void* stream);

/* Rejection sampling of the rollout correction (compute_rollout_rejection_mask,
 * rollout_corr_helper.py:163-357) as two streaming passes around a host step.  Records are doubles laid out
 * [slot][chunk][row] with chunk count vamd_rollout_rs_chunks(length).
 *   vamd_rollout_rs_row_stats: 6 slots per (row, chunk): number of valid tokens, sum of k1 = -r, of
 *     k2 = r^2 / 2 and of k3 = exp(r) - 1 - r over them (r = old - rollout clamped to +-20), max k2, max k3
 *     (-inf without a valid token).  The host folds the chunks, evaluates the sequence-level options and builds
 *     row_keep [batch] (uint8).
 *   vamd_rollout_rs_apply: new_mask = mask where row_keep and every token-level option keep the token, else 0,
 *     in the mask's element type.  Token option j: estimators[j] in {0: k1, 1: k2, 2: k3}; k1 keeps
 *     lower[j] <= k1 <= upper[j] (the logs of the ratio bounds), the others keep k <= upper[j].  The three
 *     tables are host arrays of n_token_options (<= 3) entries.  Records: slot 0 = valid tokens the new mask
 *     drops; then 8 slots per token option: sum, max, -min, count above upper, count below lower (k1 only), sum
 *     and sum of squares of the value clamped to [lower or 0, upper], count rejected by this option. */
int64_t vamd_rollout_rs_chunks(int64_t length);
int vamd_rollout_rs_row_stats(const float* old_log_prob, const float* rollout_log_prob, const void* mask,
                              int mask_dtype, int64_t batch, int64_t length, double* records, void* stream);
int vamd_rollout_rs_apply(const float* old_log_prob, const float* rollout_log_prob, const void* mask, int mask_dtype,
                          int64_t batch, int64_t length, const uint8_t* row_keep, int n_token_options,
                          const int* estimators, const float* lower, const float* upper, void* new_mask,
                          double* records, void* stream);

/* ------------------------------------------------------------------------------------------
 * agg_loss (core_algos.py:1025-1080), forward and backward.
 * out_loss: 1 device float.  coef_out [rows] floats: d loss / d loss_mat[i][t] = coef_out[i] *
 * (float)mask[i][t]; the backward entry point multiplies by the upstream scalar *d_loss.
 * batch_num_tokens / global_batch_size / loss_scale_factor < 0 mean "None" in the reference.
 */
size_t vamd_agg_loss_workspace_bytes(int64_t rows, int64_t cols);
int vamd_agg_loss_forward(const float* loss_mat, const void* mask, int mask_dtype, int64_t rows, int64_t cols,
                          int mode, double dp_size, double batch_num_tokens, double global_batch_size,
                          double loss_scale_factor, float* out_loss, float* coef_out, void* workspace,
                          size_t workspace_bytes, void* stream);
int vamd_agg_loss_backward(const float* d_loss, const float* coef, const void* mask, int mask_dtype, int64_t rows,
                           int64_t cols, float* d_loss_mat, void* stream);

/* ------------------------------------------------------------------------------------------
 * compute_policy_loss_vanilla (core_algos.py:1159-1250): clipped + dual-clip PPO objective.
 * Forward (one pass over old_log_prob, log_prob, advantages, mask [rows, cols]) writes
 *   out[0] = pg_loss, out[1] = pg_clipfrac, out[2] = ppo_kl, out[3] = pg_clipfrac_lower
 * and, when grad_unscaled != NULL, g[i][t] = d(per-token loss)/d log_prob * (float)mask (the
 * row coefficient of agg_loss is applied in the backward entry point, which writes
 * d_log_prob = g * coef[row] * *d_loss).  is_weights may be NULL.
 */
size_t vamd_policy_loss_workspace_bytes(int64_t rows, int64_t cols);
int vamd_policy_loss_forward(const float* old_log_prob, const float* log_prob, const float* advantages,
                             const void* mask, int mask_dtype, const float* is_weights, int64_t rows, int64_t cols,
                             float clip_low, float clip_high, float clip_c, int mode, double dp_size,
                             double batch_num_tokens, double global_batch_size, double loss_scale_factor,
                             float* out, float* grad_unscaled, float* coef_out, void* workspace,
                             size_t workspace_bytes, void* stream);
/* The same pass for the other registered policy losses.  out[0..3] as above with the counters a variant
 * does not define left at 0 (GPG: all three; SAPO: both clip fractions; CISPO / GSPO:
 * pg_clipfrac_lower); ppo_kl of GSPO averages the unclamped log-ratio, as the reference does.  tau_pos /
 * tau_neg are SAPO's; clip_c is only read by VAMD_PL_VANILLA.  GSPO needs the per-row mean of
 * log_prob - old_log_prob first (its sequence-level ratio).  REINFORCE (core_algos.py:1984-2061) reports
 * only ppo_kl.  GEO_MEAN (:1635-1718) clips the log-ratio to [-clip_low, clip_high], needs per-row
 * geometric means first (is_weights enter there, as exp(mean log(w + 1e-10))), ignores mode and the four
 * agg_loss scalars (the loss is the mean over all rows) and reports all three metrics.  The per-row
 * quantities of GSPO and GEO_MEAN come from a pre-pass launch, or -- while the whole launch fits the
 * device at once and VAMD_WAITING_KERNELS is not 0 -- from the loss launch itself, whose workgroups then
 * wait for the other chunks of their row a bounded number of polls (VAMD_GATE_SPIN_LIMIT) and compute
 * what did not arrive themselves. */
size_t vamd_policy_loss_variant_workspace_bytes(int64_t rows, int64_t cols);
int vamd_policy_loss_variant_forward(int variant, const float* old_log_prob, const float* log_prob,
                                     const float* advantages, const void* mask, int mask_dtype,
                                     const float* is_weights, int64_t rows, int64_t cols, float clip_low,
                                     float clip_high, float clip_c, float tau_pos, float tau_neg, int mode,
                                     double dp_size, double batch_num_tokens, double global_batch_size,
                                     double loss_scale_factor, float* out, float* grad_unscaled, float* coef_out,
                                     void* workspace, size_t workspace_bytes, void* stream);
/* The two covariance-based policy losses.  kind 0 = KL-Cov (core_algos.py:1555-1632): -A ratio everywhere plus
 * ppo_kl_coef |log ratio| on the max(1, int(n select_ratio)) valid tokens with the largest covariance
 * (A - mean A)(log_prob - mean log_prob); out[2] is masked_mean(|log ratio|).  kind 1 = Clip-Cov (:1450-1552): the
 * clipped surrogate (clip_low / clip_high) with min(max(int(select_ratio sum(mask)), 1), #candidates) tokens, drawn
 * uniformly at random (seed) from the valid, unclipped tokens whose covariance lies strictly inside
 * (cov_lb, cov_ub), contributing neither loss nor gradient; out[1] is their share of the valid tokens, out[2]
 * masked_mean(-log ratio).  out[0] = loss, out[3] = 0.  selected_out (optional, rows * cols bytes) receives 1 for
 * the selected tokens.  grad_unscaled / coef_out and the agg_loss scalars as for vamd_policy_loss_forward.  The
 * workspace is plain scratch (no arrival counters); tokens whose selection key equals the threshold exactly share
 * the remaining places in arrival order. */
size_t vamd_policy_loss_cov_workspace_bytes(int64_t rows, int64_t cols);
int vamd_policy_loss_cov_forward(int kind, const float* old_log_prob, const float* log_prob, const float* advantages,
                                 const void* mask, int mask_dtype, const float* is_weights, int64_t rows,
                                 int64_t cols, float clip_low, float clip_high, float cov_lb, float cov_ub,
                                 double select_ratio, float ppo_kl_coef, uint64_t seed, int mode, double dp_size,
                                 double batch_num_tokens, double global_batch_size, double loss_scale_factor,
                                 float* out, float* grad_unscaled, float* coef_out, uint8_t* selected_out,
                                 void* workspace, size_t workspace_bytes, void* stream);
int vamd_scale_rows(const float* g, const float* coef, const float* d_loss, float extra_scale, int64_t rows,
                    int64_t cols, float* out, void* stream);

/* compute_value_loss (core_algos.py:1799-1838): out[0] = vf_loss, out[1] = vf_clipfrac;
 * grad_unscaled as above (d per-token loss / d vpreds * mask, before the 0.5 and agg_loss row
 * coefficient, which vamd_scale_rows applies). */
size_t vamd_value_loss_workspace_bytes(int64_t rows, int64_t cols);
int vamd_value_loss_forward(const float* vpreds, const float* returns, const float* values, const void* mask,
                            int mask_dtype, int64_t rows, int64_t cols, float cliprange_value, int mode,
                            float* out, float* grad_unscaled, float* coef_out, void* workspace,
                            size_t workspace_bytes, void* stream);

/* kl_penalty / kl_penalty_forward (core_algos.py:1841-1902), elementwise over n values:
 * kld[i] (optional) and grad[i] = d kld / d logprob (optional; d kld / d ref_logprob is its
 * negative).  straight_through != 0 keeps the estimator's value and replaces its gradient by
 * that of k2, (logprob - ref): the reference's "+" variants (core_algos.py:1854-1864). */
int vamd_kl_penalty(const float* logprob, const float* ref_logprob, int64_t n, int kind, int straight_through,
                    float* kld, float* grad, void* stream);

/* apply_kl_penalty (verl/trainer/ppo/ray_trainer.py:70-109) without its controller update:
 * kld = kl_penalty(logprob, ref_logprob) * mask; token_level_rewards = scores - beta * kld;
 * current_kl[0] (1 device float) = mean over rows of masked_mean(kld, mask, axis=-1).  With
 * kind = VAMD_KL_K1 and an all-ones mask the rewards are compute_rewards (core_algos.py:1009-1022). */
size_t vamd_apply_kl_penalty_workspace_bytes(int64_t rows, int64_t cols);
int vamd_apply_kl_penalty(const float* scores, const float* logprob, const float* ref_logprob, const void* mask,
                          int mask_dtype, int64_t rows, int64_t cols, int kind, float beta,
                          float* token_level_rewards, float* current_kl, void* workspace, size_t workspace_bytes,
                          void* stream);

/* agg_loss(kl_penalty(logprob, ref_logprob), mask, mode) in one pass: the kl_loss of the actor
 * update (verl/workers/actor/dp_actor.py:640-646).  out[0] = kl_loss; grad_unscaled (optional) =
 * d kld / d logprob * mask, to be scaled by coef_out[row] and the upstream gradient with
 * vamd_scale_rows.  The last four scalars are agg_loss's (negative = None). */
size_t vamd_kl_loss_workspace_bytes(int64_t rows, int64_t cols);
int vamd_kl_loss_forward(const float* logprob, const float* ref_logprob, const void* mask, int mask_dtype,
                         int64_t rows, int64_t cols, int kind, int straight_through, int mode, double dp_size,
                         double batch_num_tokens, double global_batch_size, double loss_scale_factor, float* out,
                         float* grad_unscaled, float* coef_out, void* workspace, size_t workspace_bytes,
                         void* stream);

/* ==========================================================================================
 * MEASUREMENT AIDS.  Nothing below is part of the drop-in: none of these entry points has a counterpart in the
 * reference and no caller of the policy math needs them.  They exist so that bench.py and the profiler passes
 * can time kernels on their launch stream, turn counter units into bytes and read the board's matrix-pipe
 * ceiling with the library's own code.
 * ========================================================================================== */
/* Measurement aid (no counterpart in the reference): a plain 16-byte-per-lane copy of `bytes`
 * (a multiple of 16, both pointers 16-byte aligned) from src to dst.  Profilers read its memory
 * counters next to those of the other kernels to turn counter units into bytes. */
int vamd_copy_bytes(const void* src, void* dst, int64_t bytes, void* stream);
/* out[i] = a[i] + b[i] + c[i] + d[i] over n floats (n % 4 == 0, 16-byte aligned pointers): a second yardstick,
 * the memory traffic of a fused loss kernel with its gradient and nothing else.  No counterpart in the reference. */
int vamd_sum4(const float* a, const float* b, const float* c, const float* d, float* out, int64_t n, void* stream);
/* Benchmark aid (no counterpart in the reference): a loop of independent bf16 matrix instructions on register
 * operands, no memory traffic, `workgroups` workgroups of 8 wavefronts, `iters` rounds of 8 (32x32x16) or 32
 * (16x16x32) instructions per wavefront.  seed: workgroups * 512 * 32 device words the operand fragments are taken
 * from (zeros: nothing toggles; random bf16: the data the board's power management sees in a real GEMM);
 * out: workgroups * 512 floats.  vamd_mfma_yardstick_flops gives the flops of one launch. */
#define VAMD_MFMA_32X32X16 0
#define VAMD_MFMA_16X16X32 1
int64_t vamd_mfma_yardstick_flops(int shape, int workgroups, int iters);
int vamd_mfma_yardstick(int shape, const void* seed, float* out, int workgroups, int iters, void* stream);

/* Benchmark aid (no counterpart in the reference): with timing enabled, every head kernel
 * launch of the process is bracketed by HIP events on its stream.  vamd_lce_timing_collect
 * waits for them and adds up milliseconds and launch counts per kernel, indexed
 * 0 forward, 1 merge, 2 d_logits panel from recomputed logits (the recompute GEMM), 3 gradient GEMMs
 * (d_hidden + d_weight), 4 d_logits panel from cached logits (arrays of VAMD_LCE_TIMING_KERNELS). */
#define VAMD_LCE_TIMING_KERNELS 5
int vamd_lce_timing_enable(int on);
int vamd_lce_timing_collect(double* ms_by_kernel_host, int64_t* launches_by_kernel_host);

#ifdef __cplusplus
}
#endif
#endif /* VERL_AMD_H_ */
