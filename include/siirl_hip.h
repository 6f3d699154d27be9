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

/* registered policy losses, siirl/dag_worker/core_algos.py:710,795 */
typedef enum siirl_loss_mode { SIIRL_LOSS_VANILLA = 0, SIIRL_LOSS_GSPO = 1 } siirl_loss_mode;

/* kl_penalty estimators, siirl/dag_worker/core_algos.py:1241-1276 */
typedef enum siirl_kl_mode {
  SIIRL_KL_K1 = 0,  /* "kl", "k1" */
  SIIRL_KL_ABS = 1, /* "abs" */
  SIIRL_KL_K2 = 2,  /* "mse", "k2" */
  SIIRL_KL_K3 = 3   /* "low_var_kl", "k3" */
} siirl_kl_mode;

/* ------------------------------------------------------------------------------------------ misc */

/* ABI version of this header (major * 1000 + minor). */
int siirl_hip_abi_version(void);

/* Message of the last failing call on this thread ("" if none).  Host pointer, valid until the
 * thread's next failing call. */
const char* siirl_hip_last_error(void);

/* ---------------------------------------------------------- log-prob and entropy from logits */

/*
 * Forward: one streaming pass over logits[T, V] (row r starts at logits + r * row_stride elements).
 * With z = x * inv_temperature, per row:
 *     lse[r]     = logsumexp(z)
 *     ex[r]      = sum softmax(z) * z
 *     logprob[r] = z[labels[r]] - lse[r]          (NaN when labels[r] is outside [0, V))
 *     entropy[r] = lse[r] - ex[r]
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
 * branch contributes nothing); labels is required iff g_logprob is given; ex iff g_entropy is.
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

#ifdef __cplusplus
}
#endif
#endif /* SIIRL_HIP_H */
