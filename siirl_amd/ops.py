"""Loads the ``torch.library`` layer of the package and gives its plain operators fake kernels.

The operators themselves are C++ (``csrc/torch_ops.cpp`` -> ``lib/libsiirl_torch.so``,
``TORCH_LIBRARY(siirl_hip, m)``): each checks its operands, allocates its outputs with ATen and hands raw
device pointers plus torch's current stream to the C ABI of ``libsiirl_hip.so``.  Two kinds exist:

* plain operators, one per entry point of the path (``logprob_entropy_fwd`` ... ``fused_linear_logprob_entropy_bwd``),
  registered for the GPU only; the fake kernels below give their output shapes to FakeTensor tracing;
* differentiable operators (``logprob_entropy``, ``actor_loss``, ``agg_loss``, ``masked_reduce``, ``value_loss``,
  ``kl_penalty``, ``fused_linear_logprob_entropy``) whose autograd nodes live in C++: what the Python mirrors of the
  reference's functions call in eager mode.

There is deliberately no CPU kernel."""

from __future__ import annotations

import torch

from . import _lib

_NS = "siirl_hip"
TORCH_LIB_PATH = _lib.LIB_PATH.parent / "libsiirl_torch.so"


def _load() -> None:
    if hasattr(torch.ops.siirl_hip, "logprob_entropy_fwd"):
        return
    _lib.lib()  # libsiirl_hip.so first: ABI check, and the loader then finds it already mapped
    if not TORCH_LIB_PATH.exists():
        raise _lib.SiirlHipError(f"{TORCH_LIB_PATH} is missing: build it with `python -m siirl_amd.build`.  "
                                 "siirl_amd has no CPU or eager fallback.")
    torch.ops.load_library(str(TORCH_LIB_PATH))


_load()
_fake = torch.library.register_fake


def row_blocks(x: torch.Tensor):
    """Splits a ``(..., V)`` tensor with unit inner stride into blocks of uniformly strided rows:
    yields ``(element_offset, n_rows, row_stride)``.  A contiguous tensor, or a row-sliced 2-D view,
    is a single block; a ``[B, S, V]`` slice along ``S`` gives ``B`` blocks."""
    V = x.shape[-1]
    if x.stride(-1) != 1 and V > 1:
        raise ValueError("siirl_amd: the vocab axis of logits must have stride 1")
    lead_shape, lead_stride = list(x.shape[:-1]), list(x.stride()[:-1])
    # drop size-1 axes, then peel trailing leading-axes that collapse into one uniformly strided axis
    dims = [(n, s) for n, s in zip(lead_shape, lead_stride) if n != 1]
    if not dims:
        yield 0, 1 if x.numel() else 0, max(V, 1)
        return
    n_in, s_in = dims[-1]
    k = len(dims) - 1
    while k > 0 and dims[k - 1][1] == n_in * s_in:
        n_in *= dims[k - 1][0]
        k -= 1
    outer = dims[:k]
    if s_in < V:
        raise ValueError("siirl_amd: overlapping logits rows are not supported")

    def rec(level, off):
        if level == len(outer):
            yield off, n_in, s_in
            return
        n, s = outer[level]
        for i in range(n):
            yield from rec(level + 1, off + i * s)

    yield from rec(0, 0)


@_fake(f"{_NS}::logprob_entropy_fwd")
def _(logits, labels, inv_temperature, want_entropy):
    lead = logits.shape[:-1]
    mk = lambda shape: logits.new_empty(shape, dtype=torch.float32)  # noqa: E731
    return (mk(lead if labels is not None else (0,)), mk(lead if want_entropy else (0,)), mk(lead),
            mk(lead if want_entropy else (0,)))


@_fake(f"{_NS}::logprob_entropy_bwd")
def _(logits, labels, inv_temperature, lse, ex, g_logprob, g_entropy, skip_zero_rows):
    return logits.new_empty(logits.shape)


@_fake(f"{_NS}::logprob_entropy_bwd_")
def _(logits, labels, inv_temperature, lse, ex, g_logprob, g_entropy, skip_zero_rows):
    return None


@_fake(f"{_NS}::grpo_advantage")
def _(token_level_rewards, mask, uid, epsilon, norm_by_std):
    return token_level_rewards.new_empty(token_level_rewards.shape, dtype=torch.float32)


@_fake(f"{_NS}::group_keep_mask")
def _(metric, uid):
    return uid.new_empty(uid.shape, dtype=torch.uint8), uid.new_empty(uid.shape, dtype=torch.int32)


@_fake(f"{_NS}::agg_loss_fwd")
def _(loss_mat, mask, agg_mode):
    return loss_mat.new_empty(16, dtype=torch.float32), loss_mat.new_empty(loss_mat.shape[0], dtype=torch.float32)


@_fake(f"{_NS}::agg_loss_bwd")
def _(g, mask, out16, row_msum, agg_mode):
    return out16.new_empty(mask.shape, dtype=torch.float32)


@_fake(f"{_NS}::masked_reduce_fwd")
def _(values, mask, per_row, want_mean):
    B = values.shape[0]
    return values.new_empty(B if per_row else 2, dtype=torch.float32), values.new_empty(B if per_row else 1,
                                                                                       dtype=torch.float32)


@_fake(f"{_NS}::masked_reduce_bwd")
def _(g, mask, per_row, mask_sums):
    return g.new_empty(mask.shape, dtype=torch.float32)


@_fake(f"{_NS}::policy_loss_fwd")
def _(old_log_prob, log_prob, advantages, mask, is_weights, entropy, ref_log_prob, loss_mode, clip_low, clip_high,
      clip_c, log_ratio_clamp, agg_mode, entropy_coeff, kl_mode, kl_straight_through, kl_coef, policy_drift_coeff,
      loss_scale, token_aux=None):
    B = log_prob.shape[0]
    mk = lambda n: log_prob.new_empty(n, dtype=torch.float32)  # noqa: E731
    return mk(16), mk(B), mk(B)


@_fake(f"{_NS}::policy_loss_bwd")
def _(g_loss, old_log_prob, log_prob, advantages, mask, is_weights, entropy, ref_log_prob, loss_mode, clip_low,
      clip_high, clip_c, log_ratio_clamp, agg_mode, entropy_coeff, kl_mode, kl_straight_through, kl_coef,
      policy_drift_coeff, loss_scale, out16, row_msum, row_s, token_aux=None):
    return (log_prob.new_empty(log_prob.shape, dtype=torch.float32),
            log_prob.new_empty(log_prob.shape if entropy is not None else (0,), dtype=torch.float32))


@_fake(f"{_NS}::cov_scores")
def _(old_log_prob, log_prob, advantages, mask, loss_mode, clip_low, clip_high):
    return log_prob.new_empty(log_prob.shape, dtype=torch.float32), log_prob.new_empty(6, dtype=torch.float32)


@_fake(f"{_NS}::topk_mark")
def _(scores, k, value):
    return scores.new_empty(scores.shape, dtype=torch.float32)


@_fake(f"{_NS}::range_indices")
def _(scores, lower, upper):
    # the length of the list depends on the data: an unbacked size, as for torch.nonzero
    return scores.new_empty(torch.library.get_ctx().new_dynamic_size(), dtype=torch.int64)


@_fake(f"{_NS}::kl_penalty_fwd")
def _(log_prob, ref_log_prob, kl_mode):
    return log_prob.new_empty(log_prob.shape, dtype=torch.float32)


@_fake(f"{_NS}::kl_penalty_bwd")
def _(g, log_prob, ref_log_prob, kl_mode, straight_through, need_log_prob, need_ref):
    mk = lambda need: log_prob.new_empty(log_prob.shape if need else (0,), dtype=torch.float32)  # noqa: E731
    return mk(need_log_prob), mk(need_ref)


@_fake(f"{_NS}::fused_linear_logprob_entropy_fwd")
def _(hidden, weight, labels, inv_temperature, save_logits=False):
    mk = lambda: hidden.new_empty(hidden.shape[0], dtype=torch.float32)  # noqa: E731
    T, V = hidden.shape[0], weight.shape[0]
    n = ((V + 255) // 256) * ((T + 255) // 256) * 65536 if save_logits else 0
    return mk(), mk(), mk(), mk(), hidden.new_empty(n, dtype=torch.float32)


@_fake(f"{_NS}::fused_linear_logprob_entropy_bwd")
def _(hidden, weight, labels, inv_temperature, lse, ex, g_logprob, g_entropy, need_hidden, need_weight, saved=None,
      skip_zero_rows=False):
    return (hidden.new_empty(hidden.shape if need_hidden else (0,)),
            weight.new_empty(weight.shape if need_weight else (0,)))
