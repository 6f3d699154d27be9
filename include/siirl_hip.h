/*
 * siirl_hip.h -- C ABI of libsiirl_hip.so: the per-token RL loss path of siiRL on MI355X (gfx950).
 *
 * Conventions
 *   - Every pointer is a device pointer on the current HIP device unless its comment says "host".
 *   - Every entry point enqueues its kernels on `stream` (a hipStream_t passed as void*; NULL is the
 *     default stream) and returns without synchronising.  Nothing here allocates device memory:
 *     outputs and workspaces are the caller's.
 *   - Return value: SIIRL_OK, or a negative siirl_status.  siirl_hip_last_error() gives the message
 *     of the last failure on the calling thread.
 *   - Two-dimensional operands are row-major with unit inner stride.
 *
 * The reference (sii-research/siiRL) has no FFI on this path: its boundary is a set of Python
 * callables.  Each entry point names the reference function (file:line under the reference root)
 * whose device arithmetic it replaces; the Python modules of siirl_amd mirror the Python signatures on top.
 */
#ifndef SIIRL_HIP_H
#define SIIRL_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef void* siirl_stream_t; /* hipStream_t */

typedef enum siirl_status {
  SIIRL_OK = 0,
  SIIRL_ERR_INVALID_ARGUMENT = -1, /* null pointer, negative size, bad enum, misaligned operand */
  SIIRL_ERR_UNSUPPORTED = -2,      /* valid request this build does not implement */
  SIIRL_ERR_HIP = -3,              /* a HIP runtime call failed; message holds hipGetErrorString */
  SIIRL_ERR_WORKSPACE = -4         /* workspace smaller than the *_workspace_bytes() figure */
} siirl_status;

typedef enum siirl_dtype {
  SIIRL_F32 = 0,
  SIIRL_BF16 = 1,
  SIIRL_F16 = 2,
  SIIRL_F64 = 3,
  SIIRL_I64 = 4,
  SIIRL_I32 = 5,
  SIIRL_U8 = 6 /* also torch.bool */
} siirl_dtype;

/* loss_agg_mode of agg_loss, siirl/dag_worker/core_algos.py:536-569 */
typedef enum siirl_agg_mode {
  SIIRL_AGG_TOKEN_MEAN = 0,             /* "token-mean" */
  SIIRL_AGG_SEQ_MEAN_TOKEN_SUM = 1,     /* "seq-mean-token-sum" */
  SIIRL_AGG_SEQ_MEAN_TOKEN_MEAN = 2,    /* "seq-mean-token-mean" */
  SIIRL_AGG_SEQ_MEAN_TOKEN_SUM_NORM = 3 /* "seq-mean-token-sum-norm" */
} siirl_agg_mode;

/* registered policy losses, siirl/dag_worker/core_algos.py:572,710,795,865,898,998,1074 */
typedef enum siirl_loss_mode {
  SIIRL_LOSS_VANILLA = 0,  /* "vanilla" */
  SIIRL_LOSS_GSPO = 1,     /* "gspo" */
  SIIRL_LOSS_CPGD = 2,     /* "cpgd" */
  SIIRL_LOSS_GPG = 3,      /* "gpg" */
  SIIRL_LOSS_GEO_MEAN = 4, /* "geo_mean" (GMPO) */
  SIIRL_LOSS_KL_COV = 5,   /* "kl_cov"   (siirl_actor_loss_cov_fwd / _bwd only) */
  SIIRL_LOSS_CLIP_COV = 6  /* "clip_cov" (siirl_actor_loss_cov_fwd / _bwd only) */
} siirl_loss_mode;

/* kl_penalty estimators, siirl/dag_worker/core_algos.py:1241-1276 */
typedef enum siirl_kl_mode {
  SIIRL_KL_K1 = 0,  /* "kl", "k1" */
  SIIRL_KL_ABS = 1, /* "abs" */
  SIIRL_KL_K2 = 2,  /* "mse", "k2" */
  SIIRL_KL_K3 = 3   /* "low_var_kl", "k3" */
} siirl_kl_mode;

/* ------------------------------------------------------------------------------------------ misc */

/* ABI version of this header (major * 1000 + minor); siirl_hip_abi_version() returns the one the library was built
 * from.  A host compiled against another version must not call the library. */
#define SIIRL_HIP_ABI_VERSION 1010
int siirl_hip_abi_version(void);

/* Message of the last failing call on this thread ("" if none).  Host pointer, valid until the
 * thread's next failing call. */
const char* siirl_hip_last_error(void);

/* ---------------------------------------------------------- log-prob and entropy from logits */

/* A label with this value marks a row nothing is wanted of (a prompt token of a packed batch, see
 * siirl_mark_rows_outside_response): siirl_logprob_entropy_fwd writes 0 to all of the row's outputs without reading
 * its logits, siirl_logprob_entropy_bwd counts both upstream gradients of the row as zero: with
 * SIIRL_BWD_SKIP_ZERO_ROWS the row's gradient is written as zeros unread; without that flag it is zero as well unless
 * the row holds +inf or NaN logits (contiguous rows are then still read, with their probabilities forced to 0).  The
 * single-launch step entry points (siirl_logprob_entropy_fwd_bwd, siirl_actor_step_fused) do the same in one go:
 * log-prob and entropy 0 and a gradient of zeros, the row unread.  The lm_head entry points know no special labels
 * (any label outside [0, V) gives NaN there). */
#define SIIRL_LABEL_SKIP_ROW (-101)

/*
 * Forward: one streaming pass over logits[T, V] (row r starts at logits + r * row_stride elements).
 * With z = x * inv_temperature, per row:
 *     lse[r]     = logsumexp(z)
 *     ex[r]      = sum softmax(z) * z
 *     logprob[r] = z[labels[r]] - lse[r]          (0 when labels[r] == -100, the ignore_index of flash-attn's
 *                                                  cross_entropy_loss; NaN for any other label outside [0, V))
 *     entropy[r] = lse[r] - ex[r]
 * A row whose label is SIIRL_LABEL_SKIP_ROW is not read: its four outputs are 0.
 * Outputs are fp32.  labels and logprob may both be NULL (entropy only); entropy may be NULL;
 * lse is required; ex is required when entropy is requested and may be NULL otherwise.
 * logits_dtype: SIIRL_F32, SIIRL_BF16 or SIIRL_F16.  Accumulation is fp32.
 *
 * Replaces: logprobs_from_logits    siirl/utils/model_utils/torch_functional.py:56-116
 *           entropy_from_logits     siirl/utils/model_utils/torch_functional.py:128-143
 *           logits.div_(temperature) siirl/engine/actor/dp_actor.py:176 (pass inv_temperature = 1 if
 *           the caller already divided).
 */
int siirl_logprob_entropy_fwd(const void* logits, int logits_dtype, int64_t T, int64_t V, int64_t row_stride,
                              const int64_t* labels, float inv_temperature, float* logprob, float* entropy,
                              float* lse, float* ex, siirl_stream_t stream);

#define SIIRL_BWD_SKIP_ZERO_ROWS 1u /* rows whose upstream gradients are all zero are written as zeros unread */

/*
 * Backward: one pass that re-reads logits and writes
 *     dlogits[r, v] = inv_T * ( g_logprob[r] * (1[v == labels[r]] - p) - g_entropy[r] * p * (z - ex[r]) ),
 *     p = exp(z - lse[r]),  z = x * inv_T,
 * in the dtype of the logits (round to nearest even).  g_logprob or g_entropy may be NULL (that
 * branch contributes nothing); labels is required when g_logprob is given and may be given without it; ex is
 * required iff g_entropy is.
 * A row whose label is -100 (ignored) takes no gradient from g_logprob; a row whose label is SIIRL_LABEL_SKIP_ROW
 * takes none at all (see there).
 * dlogits may be the logits buffer itself (in-place backward, same stride), otherwise the two must
 * not overlap.  lse / ex are the forward's outputs for the same inv_temperature.
 *
 * Replaces: autograd backward of the two functions above, i.e. the closed form of
 *           siirl/utils/experimental/torch_functional.py:49-62 and siirl/utils/kernel/kernels.py:828-835;
 *           in-place mode mirrors inplace_backward of torch_functional.py:56,85-90.
 */
int siirl_logprob_entropy_bwd(const void* logits, int logits_dtype, int64_t T, int64_t V, int64_t row_stride,
                              const int64_t* labels, float inv_temperature, const float* lse, const float* ex,
                              const float* g_logprob, const float* g_entropy, void* dlogits,
                              int64_t dlogits_row_stride, uint32_t flags, siirl_stream_t stream);

/*
 * Forward and backward in one launch for upstream gradients that are known per row: logprob / entropy as the
 * forward writes them, dlogits as the backward does, from one pass over HBM plus a partial second read (half of a
 * 152064-entry bf16 row stays in LDS between the passes).  g_logprob or g_entropy may be NULL; logprob / entropy
 * outputs may be NULL.  No in-place mode.
 * Replaces: logprobs_from_logits + entropy_from_logits siirl/utils/model_utils/torch_functional.py:56-116,128-143
 *           and their autograd backward (closed form siirl/utils/experimental/torch_functional.py:49-62).
 */
int siirl_logprob_entropy_fwd_bwd(const void* logits, int logits_dtype, int64_t T, int64_t V, int64_t row_stride,
                                  const int64_t* labels, float inv_temperature, const float* g_logprob,
                                  const float* g_entropy, float* logprob, float* entropy, void* dlogits,
                                  int64_t dlogits_row_stride, siirl_stream_t stream);

/*
 * The actor's micro-batch step from logits to dlogits in one launch, for the token-separable policy losses
 * (vanilla, cpgd, gpg): per row, logprob and entropy, then the gradient of
 *   loss = (pg_loss - entropy_coeff * agg(entropy) + kl_coef * agg(kl_penalty(logprob, ref)) + drift term) * scale
 * with respect to that row's logprob and entropy, evaluated in-kernel from the per-token operands (arrays of T
 * floats: old_log_prob -- NULL means on-policy, old = logprob --, advantages, ref_log_prob or NULL, is_weights or
 * NULL) and the aggregation weights w_policy / w_aux (siirl_agg_weights), then dlogits.  Rows with zero weights
 * get zero gradients without a second read.  The scalar loss and the logged metrics are obtained afterwards from
 * the returned logprob / entropy with siirl_actor_loss_fwd (a [B, L]-sized pass).
 * Replaces: siirl/engine/actor/dp_actor.py:170-231,403-501 between the logits and their gradient, i.e.
 *           logprobs_from_logits + entropy_from_logits + the policy loss + backward() through them.
 */
int siirl_actor_step_fused(const void* logits, int logits_dtype, int64_t T, int64_t V, int64_t row_stride,
                           const int64_t* labels, float inv_temperature, const float* old_log_prob,
                           const float* advantages, const float* ref_log_prob, const float* is_weights,
                           const float* w_policy, const float* w_aux, int loss_mode, float clip_low, float clip_high,
                           float clip_c, float log_ratio_clamp, float entropy_coeff, int kl_mode,
                           int kl_straight_through, float kl_coef, float policy_drift_coeff, float loss_scale,
                           float* logprob, float* entropy, void* dlogits, int64_t dlogits_row_stride,
                           siirl_stream_t stream);

/* ------------------------------------------------------------ [B, L] loss arithmetic of the actor */

/* Bytes of scratch the *_fwd entry points below need for a [B, L] problem. */
size_t siirl_loss_workspace_bytes(int64_t B, int64_t L);

/* Layout of the 16-float result block `out16` written by siirl_agg_loss_fwd / siirl_actor_loss_fwd. */
#define SIIRL_OUT_LOSS 0         /* (policy_loss) * loss_scale, the scalar that is back-propagated      */
#define SIIRL_OUT_PG_LOSS 1      /* pg_loss (for siirl_agg_loss_fwd: the aggregated value)              */
#define SIIRL_OUT_PG_CLIPFRAC 2  /* masked_mean(l2 > l1)                                                */
#define SIIRL_OUT_PPO_KL 3       /* masked_mean(-(log_prob - old_log_prob))                             */
#define SIIRL_OUT_PG_CLIPFRAC_LOWER 4
#define SIIRL_OUT_ENTROPY_LOSS 5 /* agg_loss(entropy)            (0 when entropy is NULL)               */
#define SIIRL_OUT_KL_LOSS 6      /* agg_loss(kl_penalty(lp,ref)) (0 when ref_log_prob is NULL)          */
#define SIIRL_OUT_RATIO_MEAN 7   /* mean / min / max over ALL B*L tokens of exp(log_prob - old_log_prob) */
#define SIIRL_OUT_RATIO_MIN 8
#define SIIRL_OUT_RATIO_MAX 9
#define SIIRL_OUT_MASK_TOTAL 10  /* sum of the mask                                                     */
#define SIIRL_OUT_POLICY_LOSS 11 /* pg_loss - entropy_coeff * entropy_loss + kl_coef * kl_loss + drift term */
#define SIIRL_OUT_DRIFT_LOSS 12  /* agg_loss(policy drift)       (0 when policy_drift_coeff is 0)       */

/*
 * agg_loss(loss_mat, loss_mask, loss_agg_mode): scalar aggregation of a [B, L] fp32 matrix.
 * mask_dtype: U8 (bool), I32, I64, F32, BF16 or F16.  out16[SIIRL_OUT_PG_LOSS] receives the value,
 * row_msum[B] the per-row mask sums (saved for the backward).  token-mean is
 * sum(where(mask, v, 0) * mask) / (sum(mask) + 1e-8); seq-mean-token-mean has no epsilon, so a row with
 * an empty mask yields NaN, as in the reference.
 * Replaces: agg_loss siirl/dag_worker/core_algos.py:536-569; masked_sum / masked_mean
 *           siirl/utils/model_utils/torch_functional.py:146-168 (token-mean numerator and value).
 */
int siirl_agg_loss_fwd(const float* loss_mat, const void* mask, int mask_dtype, int64_t B, int64_t L,
                       int agg_mode, float* out16, float* row_msum, void* workspace, size_t workspace_bytes,
                       siirl_stream_t stream);

/*
 * weights[b, t] = d agg_loss / d loss_mat[b, t] for the given mask and mode (a function of the mask alone):
 * token-mean m / (sum m + 1e-8), seq-mean-token-sum m / B, seq-mean-token-mean m / (row sum) / B,
 * seq-mean-token-sum-norm m / L.  out16 / row_msum / workspace as for siirl_agg_loss_fwd.
 * Replaces: the backward of agg_loss siirl/dag_worker/core_algos.py:536-569 for a unit upstream gradient.
 */
int siirl_agg_weights(const void* mask, int mask_dtype, int64_t B, int64_t L, int agg_mode, float* weights,
                      float* out16, float* row_msum, void* workspace, size_t workspace_bytes, siirl_stream_t stream);

/* d(loss_mat) = g_out[0] * d(agg)/d(loss_mat).  g_out is a device scalar. */
int siirl_agg_loss_bwd(const float* g_out, const void* mask, int mask_dtype, const float* out16,
                       const float* row_msum, int64_t B, int64_t L, int agg_mode, float* d_loss_mat,
                       siirl_stream_t stream);

/*
 * The actor's loss for one micro-batch in one pass over [B, L] fp32 operands:
 *   pg_loss, pg_clipfrac, ppo_kl, pg_clipfrac_lower  = policy loss `loss_mode` (vanilla: PPO/GRPO/DAPO clip
 *        with dual clip `clip_c`; gspo: sequence-level ratio, always seq-mean-token-mean; cpgd: the
 *        log-probability clipped at old + log(1 -+ eps), importance weights unused; gpg: -log_prob * A, the
 *        three metrics zero; geo_mean: per sequence -mean(A) * exp(mean of the clipped log-ratios), plain mean
 *        over sequences whatever agg_mode says),
 *   entropy_loss = agg_loss(entropy)                       when entropy != NULL,
 *   kl_loss      = agg_loss(kl_penalty(log_prob, ref))     when ref_log_prob != NULL,
 *   drift_loss   = agg_loss(clamp(exp(log_prob - old) - 1, max = 2) * log_prob), the weight not
 *                  differentiated,                         when policy_drift_coeff != 0,
 *   loss = (pg_loss - entropy_coeff * entropy_loss + kl_coef * kl_loss + policy_drift_coeff * drift_loss)
 *          * loss_scale,
 * plus the ratio statistics the actor logs.  is_weights (rollout importance weights) may be NULL.
 * row_msum[B] and row_s[B] (gspo: the per-sequence mean log-ratio; geo_mean: the per-sequence loss; may be
 * NULL for the other modes) are saved for the backward.  Called with entropy = ref_log_prob = NULL and loss_scale = 1 this is exactly
 * compute_policy_loss_vanilla / compute_policy_loss_gspo.  log_ratio_clamp bounds |log_prob - old_log_prob|
 * before the exponential in the vanilla loss: 20 as in core_algos.py:758, +infinity for the legacy
 * compute_policy_loss (core_algos.py:631-707) which does not clamp.
 * Replaces: siirl/dag_worker/core_algos.py:710-792 (vanilla), :795-862 (gspo), :572-629 (cpgd), :865-895
 *           (gpg), :1074-1153 (geo_mean), :1215-1276 (kl_penalty), and the composition in
 *           siirl/engine/actor/dp_actor.py:455-513 (drift term :488-494).
 */
int siirl_actor_loss_fwd(const float* old_log_prob, const float* log_prob, const float* advantages,
                         const void* mask, int mask_dtype, const float* is_weights, const float* entropy,
                         const float* ref_log_prob, int64_t B, int64_t L, int loss_mode, float clip_low,
                         float clip_high, float clip_c, float log_ratio_clamp, int agg_mode, float entropy_coeff,
                         int kl_mode, int kl_straight_through, float kl_coef, float policy_drift_coeff,
                         float loss_scale, float* out16, float* row_msum, float* row_s, void* workspace,
                         size_t workspace_bytes, siirl_stream_t stream);

/*
 * siirl_actor_loss_fwd for callers that cannot allocate or bring a workspace (code under HIP graph capture,
 * tight serving loops, harnesses that forbid hipMalloc): same operands, same kernels, same results bit for bit,
 * with the scratch taken from a buffer that is part of the library's device image (one copy per GPU, held until the
 * process ends): SIIRL_ACTOR_LOSS_STATIC_SLOTS slices of SIIRL_ACTOR_LOSS_STATIC_SCRATCH_BYTES each.  The call
 * allocates nothing and frees nothing.  `slot` in [0, SIIRL_ACTOR_LOSS_STATIC_SLOTS) names the slice this call uses
 * (anything else is refused with SIIRL_ERR_INVALID_ARGUMENT): calls that may overlap in time on one GPU -- different
 * streams or threads -- must be given different slots and then do not touch each other's scratch; calls that share
 * a slot and overlap race; calls on one stream may share a slot.  A [B, L] problem whose
 * siirl_loss_workspace_bytes(B, L) exceeds a slice (64 bytes per 2048-token segment of a row: about 65 000
 * segments) is refused with SIIRL_ERR_WORKSPACE.  The first call on each GPU looks the buffer's address up
 * (hipGetSymbolAddress) and must happen outside stream capture.
 * This entry point has no counterpart in the reference.
 */
#define SIIRL_ACTOR_LOSS_STATIC_SCRATCH_BYTES (4u << 20)
#define SIIRL_ACTOR_LOSS_STATIC_SLOTS 4
int siirl_actor_loss_fwd_static(const float* old_log_prob, const float* log_prob, const float* advantages,
                                const void* mask, int mask_dtype, const float* is_weights, const float* entropy,
                                const float* ref_log_prob, int64_t B, int64_t L, int loss_mode, float clip_low,
                                float clip_high, float clip_c, float log_ratio_clamp, int agg_mode,
                                float entropy_coeff, int kl_mode, int kl_straight_through, float kl_coef,
                                float policy_drift_coeff, float loss_scale, float* out16, float* row_msum,
                                float* row_s, int slot, siirl_stream_t stream);

/*
 * Backward of siirl_actor_loss_fwd for an upstream gradient g_loss[0] (device scalar) on out16[SIIRL_OUT_LOSS]:
 * d_log_prob[B, L] and, when entropy was given, d_entropy[B, L].  Ties follow autograd: maximum / minimum
 * split the gradient 1/2 : 1/2, clamp passes it on the closed interval.
 */
int siirl_actor_loss_bwd(const float* g_loss, const float* old_log_prob, const float* log_prob,
                         const float* advantages, const void* mask, int mask_dtype, const float* is_weights,
                         const float* entropy, const float* ref_log_prob, int64_t B, int64_t L, int loss_mode,
                         float clip_low, float clip_high, float clip_c, float log_ratio_clamp, int agg_mode,
                         float entropy_coeff, int kl_mode, int kl_straight_through, float kl_coef,
                         float policy_drift_coeff, float loss_scale, const float* out16, const float* row_msum,
                         const float* row_s, float* d_log_prob, float* d_entropy, siirl_stream_t stream);

/*
 * The two covariance losses (Clip-Cov, KL-Cov) pick a few tokens of the batch by the covariance of advantage and
 * log-probability and treat them differently.  This entry point writes the scores that the pick is made from,
 *   cov[b, t] = (A - mean A) * (log_prob - mean log_prob),
 * SIIRL_LOSS_KL_COV: plain means over the tokens with mask > 0, cov = -inf where mask <= 0 (the caller takes the
 * max(1, int(n * kl_cov_ratio)) largest); SIIRL_LOSS_CLIP_COV: masked means sum(v * m) / (sum(m) + 1e-8), cov = -inf
 * where mask <= 0 (no candidate there) and where the PPO clip already bites (-A * clamp(ratio, 1 - clip_low, 1 + clip_high) > -A * ratio,
 * ratio = exp(log_prob - old_log_prob)); the caller draws its tokens among clip_cov_lb < cov < clip_cov_ub.
 * stats[6] (device) receives {count of mask > 0, sum of the mask, mean A, mean log_prob, and the float32 rounding
 * residues of the first two: count = stats[0] + stats[4] and mask sum = stats[1] + stats[5] exactly}.  old_log_prob may be NULL
 * for SIIRL_LOSS_KL_COV.  workspace: siirl_cov_workspace_bytes(), 8-byte aligned.
 * Replaces: siirl/dag_worker/core_algos.py:952-971 (clip_cov) and :1047-1055 (kl_cov).
 */
size_t siirl_cov_workspace_bytes(void);
int siirl_cov_scores(const float* old_log_prob, const float* log_prob, const float* advantages, const void* mask,
                     int mask_dtype, int64_t B, int64_t L, int loss_mode, float clip_low, float clip_high, float* cov,
                     float* stats, void* workspace, size_t workspace_bytes, siirl_stream_t stream);

/*
 * marks[i] = value for the k largest of scores[0..n) and 0 for the rest: the selection step of KL-Cov (the
 * max(1, int(n_valid * kl_cov_ratio)) tokens of largest covariance get the coefficient of their KL term), in place of
 * torch.topk followed by an indexed assignment.  Radix select over three streaming passes; entries equal to the k-th
 * largest are taken lowest index first until k are marked; NaN ranks above every number (as for torch.topk), -0 and
 * +0 are one value.  Deterministic (no atomics on memory).  n < 2^32, 0 <= k <= n; scores and marks must not
 * overlap.  workspace: siirl_topk_mark_workspace_bytes(), 16-byte aligned.
 * Replaces: siirl/dag_worker/core_algos.py:1055-1063 (torch.topk(cov, k).indices and the assignment through them).
 */
size_t siirl_topk_mark_workspace_bytes(void);
int siirl_topk_mark(const float* scores, int64_t n, int64_t k, float value, float* marks, void* workspace,
                    size_t workspace_bytes, siirl_stream_t stream);

/*
 * Flat indices, ascending, of the entries with lower_open < scores[i] < upper_open: Clip-Cov's candidate list (the
 * tokens whose covariance lies inside (clip_cov_lb, clip_cov_ub); masked and already-clipped tokens carry -inf and
 * stay out), in place of three comparisons, two logical ands and torch.nonzero.  Two steps, because the caller sizes
 * the list: siirl_range_select_count leaves the number of such entries in *count (a device uint32) and the per-chunk
 * counts in the workspace; after reading the count the caller passes the same scores and workspace, untouched, to
 * siirl_range_select_write together with a list of `capacity` >= count entries (nothing is written beyond capacity).
 * n < 2^32.  workspace: siirl_range_select_workspace_bytes(), 4-byte aligned.
 * Replaces: siirl/dag_worker/core_algos.py:974-975.
 */
size_t siirl_range_select_workspace_bytes(void);
int siirl_range_select_count(const float* scores, int64_t n, float lower_open, float upper_open, uint32_t* count,
                             void* workspace, size_t workspace_bytes, siirl_stream_t stream);
int siirl_range_select_write(const float* scores, int64_t n, float lower_open, float upper_open, const void* workspace,
                             int64_t* indices, int64_t capacity, siirl_stream_t stream);

/*
 * siirl_actor_loss_fwd for the two covariance losses: the same composition (entropy, KL and drift terms, ratio
 * statistics, loss_scale) around a policy term that takes one more [B, L] fp32 operand, token_aux:
 *   SIIRL_LOSS_KL_COV:   tok = -A * ratio + token_aux * |log_prob - old_log_prob|  (token_aux = ppo_kl_coef on the
 *        selected tokens, 0 elsewhere); out16[SIIRL_OUT_PPO_KL] is masked_mean(|log_prob - old_log_prob|), the two
 *        clip fractions are 0;
 *   SIIRL_LOSS_CLIP_COV: tok = max(-A * ratio, -A * clamp(ratio, 1 - clip_low, 1 + clip_high)) where token_aux == 0
 *        and 0 where token_aux != 0 (the dropped tokens); out16[SIIRL_OUT_PG_CLIPFRAC] is the masked share of dropped
 *        tokens, out16[SIIRL_OUT_PPO_KL] masked_mean(-(log_prob - old_log_prob)).
 * Neither clamps the log-ratio, neither has a dual clip; both multiply by is_weights when given and aggregate with
 * agg_mode.  Workspace as for siirl_actor_loss_fwd.
 * Replaces: compute_policy_loss_clip_cov siirl/dag_worker/core_algos.py:898-995 (after the draw, :983-995) and
 *           compute_policy_loss_kl_cov :998-1071 (after the selection, :1061-1071).
 */
int siirl_actor_loss_cov_fwd(const float* old_log_prob, const float* log_prob, const float* advantages,
                             const void* mask, int mask_dtype, const float* is_weights, const float* entropy,
                             const float* ref_log_prob, const float* token_aux, int64_t B, int64_t L, int loss_mode,
                             float clip_low, float clip_high, int agg_mode, float entropy_coeff, int kl_mode,
                             int kl_straight_through, float kl_coef, float policy_drift_coeff, float loss_scale,
                             float* out16, float* row_msum, void* workspace, size_t workspace_bytes,
                             siirl_stream_t stream);

/* Backward of siirl_actor_loss_cov_fwd, as siirl_actor_loss_bwd; |x| passes sign(x), 0 at 0. */
int siirl_actor_loss_cov_bwd(const float* g_loss, const float* old_log_prob, const float* log_prob,
                             const float* advantages, const void* mask, int mask_dtype, const float* is_weights,
                             const float* entropy, const float* ref_log_prob, const float* token_aux, int64_t B,
                             int64_t L, int loss_mode, float clip_low, float clip_high, int agg_mode,
                             float entropy_coeff, int kl_mode, int kl_straight_through, float kl_coef,
                             float policy_drift_coeff, float loss_scale, const float* out16, const float* row_msum,
                             float* d_log_prob, float* d_entropy, siirl_stream_t stream);

/*
 * Clipped value loss of the critic over [B, L] fp32 operands:
 *   vclip = max(min(vpreds, values + c), values - c),  tok = max((vpreds - returns)^2, (vclip - returns)^2),
 *   out16[SIIRL_OUT_LOSS] = vf_loss = 0.5 * agg_loss(tok),  out16[SIIRL_OUT_PG_CLIPFRAC] = vf_clipfrac =
 *   masked_mean((vclip - returns)^2 > (vpreds - returns)^2);  out16[SIIRL_OUT_PG_LOSS] holds agg_loss(tok).
 * The backward writes d vf_loss / d vpreds times g_loss[0], with autograd's tie rules for max / min.
 * Replaces: compute_value_loss siirl/dag_worker/core_algos.py:1173-1212 (clip_by_value
 *           siirl/utils/model_utils/torch_functional.py:119-125).
 */
int siirl_value_loss_fwd(const float* vpreds, const float* returns, const float* values, const void* mask,
                         int mask_dtype, int64_t B, int64_t L, float cliprange_value, int agg_mode, float* out16,
                         float* row_msum, void* workspace, size_t workspace_bytes, siirl_stream_t stream);
int siirl_value_loss_bwd(const float* g_loss, const float* vpreds, const float* returns, const float* values,
                         const void* mask, int mask_dtype, int64_t B, int64_t L, float cliprange_value, int agg_mode,
                         const float* out16, const float* row_msum, float* d_vpreds, siirl_stream_t stream);

/*
 * kl_penalty, elementwise over n fp32 values.  straight_through != 0 gives the k2 gradient
 * (log_prob - ref) whatever the estimator.  d_logprob or d_ref_logprob may be NULL.
 * Replaces: kl_penalty / kl_penalty_forward siirl/dag_worker/core_algos.py:1215-1276.
 */
int siirl_kl_penalty_fwd(const float* logprob, const float* ref_logprob, int64_t n, int kl_mode, float* out,
                         siirl_stream_t stream);
int siirl_kl_penalty_bwd(const float* g, const float* logprob, const float* ref_logprob, int64_t n, int kl_mode,
                         int straight_through, float* d_logprob, float* d_ref_logprob, siirl_stream_t stream);

/*
 * masked_sum / masked_mean over a [B, L] fp32 matrix: row_sum[b] = sum_t where(mask, v, 0) * mask,
 * row_mean[b] = row_sum[b] / (sum_t mask + 1e-8), total2 = {sum over all, sum / (sum(mask) + 1e-8)},
 * row_msum[b] = sum_t mask, mask_total[0] = sum(mask) (the denominators, kept for the backward).
 * Any output may be NULL.  Workspace as for the loss entry points.  A reduction over other axes is this one after
 * the caller has moved the reduced axes last.
 * Replaces: masked_sum / masked_mean siirl/utils/model_utils/torch_functional.py:146-168.
 */
int siirl_masked_reduce(const float* values, const void* mask, int mask_dtype, int64_t B, int64_t L, float* row_sum,
                        float* row_mean, float* total2, float* row_msum, float* mask_total, void* workspace,
                        size_t workspace_bytes, siirl_stream_t stream);

/*
 * Backward of the above: d_values[b, t] = g[per_row ? b : 0] * mask[b, t], divided by (mask_sums[per_row ? b : 0]
 * + 1e-8) when mask_sums is given (the mean; NULL for the sum).  g holds B entries (per_row) or one.
 */
int siirl_masked_reduce_bwd(const float* g, const void* mask, int mask_dtype, int64_t B, int64_t L, int per_row,
                            const float* mask_sums, float* d_values, siirl_stream_t stream);

/*
 * KL penalty folded into the reward: kld = kl_penalty(old_log_prob, ref_log_prob) * mask,
 * token_level_rewards = token_level_scores - beta * kld, row_kl[b] = masked_mean(kld, mask) of row b,
 * current_kl[0] = mean_b row_kl[b] (device scalar; the controller update stays on the host).
 * Replaces: apply_kl_penalty siirl/dag_worker/core_algos.py:1358-1397 (device arithmetic).
 */
int siirl_kl_in_reward(const float* token_level_scores, const float* old_log_prob, const float* ref_log_prob,
                       const void* mask, int mask_dtype, int64_t B, int64_t L, int kl_mode, float beta,
                       float* token_level_rewards, float* row_kl, float* current_kl, siirl_stream_t stream);

/* ------------------------------------------------------------------- remove-padding bookkeeping */

/*
 * unpad_input's index computation for a 0/1 attention mask [B, S]: seqlens[b] = attended positions of row b,
 * cu_seqlens[B + 1] = [0, cumsum(seqlens)] (int32, so B * S < 2^31), indices[0 .. nnz) = flat positions b * S + s
 * of the attended tokens in ascending order (capacity B * S), info2 = {nnz, max seqlen}.
 * Replaces: unpad_input of flash-attn's bert_padding (flash-attn 2.7.3 / 2.8.2) as called at
 *           siirl/engine/actor/dp_actor.py:112.
 */
int siirl_unpad_indices(const void* attention_mask, int mask_dtype, int64_t B, int64_t S, int32_t* seqlens,
                        int32_t* cu_seqlens, int64_t* indices, int64_t* info2, siirl_stream_t stream);

/*
 * index_first_axis: dst[j, :] = src[indices[j], :] for n rows of row_bytes (a multiple of 4) each; and pad_input:
 * dst[total_rows, :] = 0, then dst[indices[j], :] = src[j, :].  Each is the other's backward.  src of the gather
 * has src_rows rows; an index outside [0, src_rows) (gather: the row reads as zeros) or [0, total_rows) (scatter:
 * the row is dropped) never touches memory.
 * Replaces: index_first_axis / pad_input of flash-attn's bert_padding, siirl/engine/actor/dp_actor.py:117-119,215-226.
 */
int siirl_gather_rows(const void* src, const int64_t* indices, int64_t n, int64_t row_bytes, int64_t src_rows,
                      void* dst, siirl_stream_t stream);
int siirl_scatter_rows(const void* src, const int64_t* indices, int64_t n, int64_t row_bytes, int64_t total_rows,
                       void* dst, siirl_stream_t stream);

/*
 * ids_rmpad[j] = input_ids[indices[j]] and labels_rolled[j] = input_ids[indices[(j + 1) % nnz]]: the packed ids and
 * the next-token labels in one pass (either output may be NULL).  input_ids has n_ids entries; an index outside
 * [0, n_ids) yields -1 instead of a read.
 * Replaces: unpad_input on input_ids + torch.roll(input_ids_rmpad, shifts=-1), siirl/engine/actor/dp_actor.py:112-127.
 */
int siirl_unpad_ids_labels(const int64_t* input_ids, int64_t n_ids, const int64_t* indices, int64_t nnz,
                           int64_t* ids_rmpad, int64_t* labels_rolled, siirl_stream_t stream);

/*
 * labels[j] = SIIRL_LABEL_SKIP_ROW for every packed token j whose position in its sequence,
 * indices[j] mod S, lies outside [S - L - 1, S - 2]: the rows of the packed logits whose log-prob and entropy the
 * response window does not keep.  The log-prob entry points then neither read those rows nor send a gradient into
 * them.  Other labels are left as they are.
 * Replaces: the work the reference spends on rows it then drops with the slice
 *           full_log_probs.squeeze(-1)[:, -response_length - 1 : -1]  siirl/engine/actor/dp_actor.py:214-231.
 */
int siirl_mark_rows_outside_response(const int64_t* indices, int64_t nnz, int64_t S, int64_t L, int64_t* labels,
                                     siirl_stream_t stream);

/*
 * pad_input followed by the response window: out[b, t] = full[b, S - L - 1 + t], t in [0, L), where full is the
 * zero-padded [B, S] scatter of values[nnz] at `indices` -- without materialising full.  The gather is its backward.
 * Indices outside [0, B * S) are ignored (scatter) or read as zero (gather).
 * Replaces: pad_input(...).squeeze(-1)[:, -response_length - 1 : -1], siirl/engine/actor/dp_actor.py:214-231.
 */
int siirl_response_scatter(const float* values, const int64_t* indices, int64_t nnz, int64_t B, int64_t S, int64_t L,
                           float* out, siirl_stream_t stream);
int siirl_response_gather(const float* grad, const int64_t* indices, int64_t nnz, int64_t B, int64_t S, int64_t L,
                          float* d_values, siirl_stream_t stream);

/*
 * Response mask from the generated ids [B, L] (int64 or int32): mask[b, t] = 1 while no end-of-sequence token
 * occurs strictly before position t of row b (the first such token is still attended), 0 from the next position on.
 * eos_tokens is a HOST array of n_eos <= SIIRL_MAX_EOS_TOKENS ids (n_eos = 0: all ones); mask takes any mask dtype.
 * Replaces: get_response_mask / get_eos_mask, siirl/utils/model_utils/torch_functional.py:209-254
 *           ((cumsum(eos) - eos) == 0 along the row).
 */
#define SIIRL_MAX_EOS_TOKENS 16
int siirl_eos_response_mask(const void* response_id, int id_dtype, int64_t B, int64_t L, const int64_t* eos_tokens,
                            int n_eos, void* mask, int mask_dtype, siirl_stream_t stream);

/* ------------------------------------------------------------------- outcome reward placement */

/*
 * reward_tensor[B, L] (fp32) = 0 except reward_tensor[b, valid_b - 1] = scores[b] + overlong_b, where valid_b is the
 * sum of attention_mask[b, prompt_width : prompt_width + L] and, when overlong_enable != 0,
 * overlong_b = min(-(valid_b - (max_resp_len - buffer_len)) / buffer_len * penalty_factor, 0), else 0, in
 * float32 arithmetic (the reference computes it on a 0-d tensor).  valid_b == 0 writes the last column (Python's index -1).
 * overlong_reward[B] and valid_response_length[B] are optional outputs.
 * Replaces: the reward tensor construction of DAPORewardManager.__call__ siirl/engine/reward_manager/dapo.py:57-126.
 */
int siirl_place_outcome_reward(const double* scores, const void* attention_mask, int mask_dtype, int64_t B,
                               int64_t prompt_width, int64_t L, int overlong_enable, double max_resp_len,
                               double overlong_buffer_len, double overlong_penalty_factor, float* reward_tensor,
                               double* overlong_reward, int64_t* valid_response_length, siirl_stream_t stream);

/* ------------------------------------------------------------------- logged batch statistics */

/* Order of the 32-float block written by siirl_data_metrics (unused tail entries are 0). */
enum {
  SIIRL_METRIC_SCORE_MEAN = 0, SIIRL_METRIC_SCORE_MAX, SIIRL_METRIC_SCORE_MIN,
  SIIRL_METRIC_REWARD_MEAN, SIIRL_METRIC_REWARD_MAX, SIIRL_METRIC_REWARD_MIN,
  SIIRL_METRIC_ADV_MEAN, SIIRL_METRIC_ADV_MAX, SIIRL_METRIC_ADV_MIN,
  SIIRL_METRIC_RETURNS_MEAN, SIIRL_METRIC_RETURNS_MAX, SIIRL_METRIC_RETURNS_MIN,
  SIIRL_METRIC_VALUES_MEAN, SIIRL_METRIC_VALUES_MAX, SIIRL_METRIC_VALUES_MIN, SIIRL_METRIC_VF_EXPLAINED_VAR,
  SIIRL_METRIC_RESP_LEN_MEAN, SIIRL_METRIC_RESP_LEN_MAX, SIIRL_METRIC_RESP_LEN_MIN, SIIRL_METRIC_RESP_CLIP_RATIO,
  SIIRL_METRIC_CORRECT_LEN_MAX, SIIRL_METRIC_CORRECT_LEN_MIN, SIIRL_METRIC_CORRECT_LEN_MEAN,
  SIIRL_METRIC_WRONG_LEN_MAX, SIIRL_METRIC_WRONG_LEN_MIN, SIIRL_METRIC_WRONG_LEN_MEAN,
  SIIRL_METRIC_PROMPT_LEN_MEAN, SIIRL_METRIC_PROMPT_LEN_MAX, SIIRL_METRIC_PROMPT_LEN_MIN,
  SIIRL_METRIC_PROMPT_CLIP_RATIO, SIIRL_METRIC_VALID_TOKENS, SIIRL_METRIC_COUNT = 32
};

size_t siirl_data_metrics_workspace_bytes(int64_t B, int64_t L);

/*
 * The statistics the trainer logs per step from [B, L] fp32 tensors: mean / max / min of the per-sequence score
 * and reward sums; mean / max / min over the tokens selected by response_mask.bool() of advantages, returns and
 * (when values != NULL) values, plus 1 - var(returns - values) / (var(returns) + 1e-5) with unbiased variances;
 * response length (mask count per row) mean / max / min, the fraction equal to L, the same split by
 * reward sum > 0.5 ("correct") or not (0 when the class is empty); prompt length statistics from the first
 * prompt_width columns of attention_mask [B, prompt_width + L] and the fraction equal to prompt_width.
 * Replaces: compute_data_metric / _compute_response_info siirl/utils/metrics/metric_utils.py:36-183.
 */
int siirl_data_metrics(const float* token_level_scores, const float* token_level_rewards, const float* advantages,
                       const float* returns, const float* values, const void* response_mask,
                       int response_mask_dtype, const void* attention_mask, int attention_mask_dtype, int64_t B,
                       int64_t L, int64_t prompt_width, float* out32, void* workspace, size_t workspace_bytes,
                       siirl_stream_t stream);

/* ------------------------------------------------------------------- GAE and masked whitening */

/* Bytes of scratch siirl_masked_whiten needs (a constant; 8-byte aligned buffer). */
size_t siirl_whiten_workspace_bytes(void);

/*
 * masked_whiten over n fp32 values: mean = masked_mean(values, mask), var = masked_mean((values - mean)^2, mask)
 * * n_mask / (n_mask - 1), out = (values - mean) * rsqrt(var + 1e-8) (+ mean when shift_mean == 0), applied to
 * every element.  out may be the values buffer.  stats3 receives {mean, var, n_mask}; the reference raises
 * ValueError for n_mask 0 or 1 -- here the caller reads stats3[2] (the outputs are then not meaningful).
 * Replaces: masked_mean / masked_var / masked_whiten siirl/utils/model_utils/torch_functional.py:154-206.
 */
int siirl_masked_whiten(const float* values, const void* mask, int mask_dtype, int64_t n, int shift_mean, float* out,
                        float* stats3, void* workspace, size_t workspace_bytes, siirl_stream_t stream);

/* Order of evaluation of the GAE scan. */
typedef enum siirl_gae_order {
  SIIRL_GAE_EXACT_ORDER = 0, /* one sequential pass per row, the reference's float32 operation order */
  SIIRL_GAE_CHUNKED = 1      /* rows cut into up to 16 chunks scanned in parallel and stitched by their affine maps */
} siirl_gae_order;

/* Bytes of scratch siirl_gae_advantage_return needs (8-byte aligned buffer). */
size_t siirl_gae_workspace_bytes(int64_t B, int64_t L);

/*
 * Generalised advantage estimation over [B, L] fp32 operands, scanning each row from its last token:
 *   delta = r_t + gamma * V_next - V_t,  A_t = delta + gamma * lam * A_next; a token with mask 0 keeps V_next and
 *   A_next of the token after it (both start at 0).  returns = A + values (before whitening);
 *   advantages = masked_whiten(A, mask).  With SIIRL_GAE_EXACT_ORDER the scan is evaluated in the reference's
 *   float32 operation order and `returns` is bit-identical to the reference's; SIIRL_GAE_CHUNKED shortens the
 *   dependent chain 16-fold for long rows (same arithmetic inside a chunk; the state entering a chunk goes through
 *   the chunks' composed maps, which changes its rounding: results agree to float32 accuracy, not bit for bit).
 *   stats3 as for siirl_masked_whiten.
 * Replaces: compute_gae_advantage_return siirl/dag_worker/core_algos.py:229-276.
 */
int siirl_gae_advantage_return(const float* token_level_rewards, const float* values, const void* mask,
                               int mask_dtype, int64_t B, int64_t L, double gamma, double lam, float* advantages,
                               float* returns, float* stats3, void* workspace, size_t workspace_bytes, int order,
                               siirl_stream_t stream);

/* ------------------------------------------------------------------- per-prompt group statistics */

/*
 * GRPO outcome advantage: s_i = sum_t rewards[i, t]; per group of equal uid the mean and the unbiased
 * (N-1) standard deviation (a group of one: mean 0, std 1); a_i = (s_i - mean) / (std + epsilon), or
 * s_i - mean when norm_adv_by_std == 0; advantages[i, t] = a_i * mask[i, t].  uid values are arbitrary.
 * scratch_2B: 2*B floats of scratch; on return scratch_2B[0..B) holds the scores s_i and [B..2B) the a_i.
 * Replaces: compute_grpo_outcome_advantage siirl/dag_worker/core_algos.py:279-348.
 */
int siirl_grpo_outcome_advantage(const float* token_level_rewards, const void* mask, int mask_dtype,
                                 const int64_t* uid, int64_t B, int64_t L, float epsilon, int norm_adv_by_std,
                                 float* advantages, float* scratch_2B, siirl_stream_t stream);

/*
 * DAPO dynamic sampling: keep[i] = 1 iff the uid-group of trajectory i has a single member or
 * np.std(metric of the group) > 0, with numpy's arithmetic (population std, pairwise summation, in the
 * dtype of the metric: SIIRL_F32 or SIIRL_F64) reproduced bit for bit.  group_size (int32[B], may be
 * NULL) receives each trajectory's group size.  The kept indices are the positions of the ones, ascending.
 * Replaces: the group test of dynamic_sampling siirl/user_interface/filter_interface/dapo.py:66-93.
 */
int siirl_group_keep_mask(const void* metric, int metric_dtype, const int64_t* uid, int64_t B, uint8_t* keep,
                          int32_t* group_size, siirl_stream_t stream);

/* ------------------------------------------------------------------- multi-agent GAE (MARFT) */

#define SIIRL_MARFT_MAX_AGENTS 16

/* What the reference's assignment into a tensor of the mask's dtype keeps of each float32 result. */
typedef enum siirl_marft_store {
  SIIRL_MARFT_STORE_FLOAT = 0,     /* the value itself */
  SIIRL_MARFT_STORE_TRUNCATED = 1, /* its integer part (the reference's outputs take the integer mask's dtype) */
  SIIRL_MARFT_STORE_NONZERO = 2    /* 1 where it is not zero (bool masks) */
} siirl_marft_store;

/*
 * GAE over the trajectories of multi-agent requests, before whitening.  The batch of B rows holds each request as
 * chain_len[c] consecutive rows from chain_start[c] (its steps, last step first); agent g (0 .. n_agents - 1, the
 * last one being the batch's own response) has fp32 rewards / values [B, widths[g]] and an integer mask
 * [B, widths[g]] whose row sum is the number of generated tokens, which sit at the front of the row.  One
 * accumulator runs over a request: rows in order, agents from last to first, tokens from the last generated one to
 * the first;  delta = gamma * V[t+1] - V[t] inside an agent's tokens and rew + gamma * V_next - V at its last token,
 * where V_next is the first value of the next agent in the row, or for the last agent the first agent's first value
 * in the row before (nothing in a request's first row);  gae = delta + gamma_lam * gae;  advantages[g][row, t] = gae,
 * returns[g][row, t] = gae + V[t]; every other element of the outputs is zero.  float32 operation order of the
 * reference: bit-identical results.  gamma_lam is the product as the caller's arithmetic yields it (the
 * reference multiplies two Python floats in double and rounds the product once).
 * token_level_rewards / values / masks / advantages / returns / widths: HOST arrays of n_agents device pointers
 * (row lengths); chain_start / chain_len: device int64[n_chains]; status: device int32, 0 on success, 1 when a mask
 * row summed to more than its length (clamped; the reference raises IndexError), 2 when a request's rows leave the
 * batch (that request is skipped).
 * Replaces: compute_marft_gae_advantage_return siirl/dag_worker/core_algos.py:351-450 (the whitening of :451 is
 *           siirl_masked_whiten per agent).
 */
int siirl_marft_gae(const float* const* token_level_rewards, const float* const* values, const void* const* masks,
                    int mask_dtype, const int64_t* widths, int n_agents, int64_t B, const int64_t* chain_start,
                    const int64_t* chain_len, int64_t n_chains, float gamma, float gamma_lam, int store_mode,
                    float* const* advantages, float* const* returns, int32_t* status, siirl_stream_t stream);

/* ------------------------------------------------- lm_head projection fused with log-prob / entropy */

/* Bytes of scratch for the two entry points below, for 16-bit operands (SIIRL_BF16, SIIRL_F16) and, `_dtype`, for
 * the operand dtype given (SIIRL_F32 operands are staged as three bf16 terms per element: 6 more bytes per element of
 * hidden and of weight). */
size_t siirl_fused_linear_fwd_workspace_bytes(int64_t T, int64_t H, int64_t V);
size_t siirl_fused_linear_bwd_workspace_bytes(int64_t T, int64_t H, int64_t V, int want_d_hidden, int want_d_weight);
size_t siirl_fused_linear_fwd_workspace_bytes_dtype(int dtype, int64_t T, int64_t H, int64_t V);
size_t siirl_fused_linear_bwd_workspace_bytes_dtype(int dtype, int64_t T, int64_t H, int64_t V, int want_d_hidden,
                                                    int want_d_weight);
/* Bytes of the optional saved_logits buffer of the two entry points below: 4 bytes per logit, whole 256 x 256 tiles. */
size_t siirl_fused_linear_saved_logits_bytes(int64_t T, int64_t V);

/*
 * Forward: z = (hidden[T, H] . weight[V, H]^T) * inv_temperature is formed tile by tile on the matrix cores
 * (fp32 accumulation) and reduced in the epilogue; no [T, V] tensor is needed.
 * dtype of hidden and weight: SIIRL_BF16 or SIIRL_F16 (exact products of the operands on the bf16 / fp16 matrix
 * instructions), or SIIRL_F32: each operand is first staged in the workspace as three bf16 terms per element
 * (x = hi + lo, a.b ~ hi.hi + hi.lo + lo.hi, relative error 2^-16 per product) and the same bf16 kernels run over
 * K = 3 H -- the reference's matmul in the input dtype (experimental/torch_functional.py:21) to better than TF32.
 * Outputs as siirl_logprob_entropy_fwd: logprob[T] (with labels), entropy[T], lse[T], ex[T], all fp32.
 * saved_logits (may be NULL): siirl_fused_linear_saved_logits_bytes(T, V) bytes, 16-byte aligned, into which the
 * fp32 accumulator tiles are parked in the kernel's own lane order for the backward; an opaque buffer, trading
 * memory for the backward's recomputation.
 * H a multiple of 64; hidden and weight row-major, contiguous, 16-byte aligned; workspace 256-byte aligned.
 * Replaces: FusedLinearForPPO.forward  siirl/utils/experimental/torch_functional.py:20-32,70-133
 *           linear_cross_entropy fwd   siirl/utils/kernel/linear_cross_entropy.py:40-88 ->
 *                                      siirl/utils/kernel/kernels.py:507-696 (reduction "none", no TP group)
 */
int siirl_fused_linear_logprob_entropy_fwd(const void* hidden, const void* weight, int dtype, const int64_t* labels,
                                           int64_t T, int64_t H, int64_t V, float inv_temperature, float* logprob,
                                           float* entropy, float* lse, float* ex, float* saved_logits, void* workspace,
                                           size_t workspace_bytes, siirl_stream_t stream);

/*
 * Backward: for upstream gradients g_logprob[T] / g_entropy[T] (either may be NULL) writes
 * d_hidden[T, H] and / or d_weight[V, H] in the operands' dtype (either may be NULL).  The vocabulary is walked in
 * slabs of 8192 columns: the slab's logits are recomputed -- or, when saved_logits holds what the forward call with
 * the same hidden, weight and inv_temperature parked there, read back --, dlogits = inv_T * (g_lp (onehot - p)
 * - g_H p (z - ex)) is written to scratch as bf16 (token-major, one layout for both consumers), then
 * d_hidden += dlogits . W_slab (fp32 accumulation across slabs, rounded once) and d_weight_slab = dlogits^T . hidden.
 * Both routes give the same bits.  For SIIRL_F16 and SIIRL_F32 operands the logits are recomputed as in the forward;
 * the two gradient GEMMs multiply the bf16 dlogits (bf16 for its range: a softmax gradient underflows fp16) with
 * hidden and W rounded to bf16, so the gradients carry one more 2^-9 rounding than with bf16 operands; the reference
 * rounds dlogits to the operands' dtype at the same place (experimental/torch_functional.py:62).
 * Replaces: FusedLinearForPPO.backward siirl/utils/experimental/torch_functional.py:35-67,135-188
 *           linear_cross_entropy bwd   siirl/utils/kernel/kernels.py:1378-1586 (the split-N d_logits strategy
 *                                      :1263-1375,1523-1581)
 */
int siirl_fused_linear_logprob_entropy_bwd(const void* hidden, const void* weight, int dtype, const int64_t* labels,
                                           int64_t T, int64_t H, int64_t V, float inv_temperature, const float* lse,
                                           const float* ex, const float* saved_logits, const float* g_logprob,
                                           const float* g_entropy, void* d_hidden, void* d_weight, void* workspace,
                                           size_t workspace_bytes, siirl_stream_t stream);

/*
 * The same backward restricted to the n_rows token rows listed in rows[] (distinct indices into [0, T), any
 * order): the rows whose upstream gradients are not both zero.  The actor takes the log-probs of every packed token
 * but only the response slice reaches the loss, so the rows of prompt tokens arrive with zero gradients; they
 * contribute nothing to either result and are left out of all three GEMMs here.  Rows not listed get zeros in
 * d_hidden; d_weight sums over the listed rows only.  The results are those of
 * siirl_fused_linear_logprob_entropy_bwd on the gathered operands, bit for bit (against the full call d_weight
 * differs by the rounding order of its sum over tokens).  n_rows == 0 writes zeros.  The logits are always
 * recomputed on this route.  workspace: siirl_fused_linear_bwd_rows_workspace_bytes(n_rows, ...) bytes, 256-byte
 * aligned.
 * Replaces: FusedLinearForPPO.backward siirl/utils/experimental/torch_functional.py:35-67,135-188 as reached from
 *           siirl/engine/actor/dp_actor.py:170-172 (log-probs of all packed tokens) and :228-231 (only the
 *           response slice [:, -response_length - 1 : -1] is used).
 */
size_t siirl_fused_linear_bwd_rows_workspace_bytes(int64_t n_rows, int64_t H, int64_t V, int want_d_hidden,
                                                   int want_d_weight);
size_t siirl_fused_linear_bwd_rows_workspace_bytes_dtype(int dtype, int64_t n_rows, int64_t H, int64_t V,
                                                         int want_d_hidden, int want_d_weight);
int siirl_fused_linear_logprob_entropy_bwd_rows(const void* hidden, const void* weight, int dtype, const int64_t* labels,
                                                int64_t T, int64_t H, int64_t V, float inv_temperature, const float* lse,
                                                const float* ex, const float* g_logprob, const float* g_entropy,
                                                const int64_t* rows, int64_t n_rows, void* d_hidden, void* d_weight,
                                                void* workspace, size_t workspace_bytes, siirl_stream_t stream);

#ifdef __cplusplus
}
#endif
#endif /* SIIRL_HIP_H */
