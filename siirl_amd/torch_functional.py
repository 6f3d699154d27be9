"""Log-prob / entropy from logits and masked reductions, with the reference's Python signatures.

Mirror of ``siirl/utils/model_utils/torch_functional.py:41-168`` of the reference: same names, same
argument meaning.  The arithmetic runs in ``libsiirl_hip.so``; tensors must live on the GPU.

Differences a caller can observe, all deliberate:

* results for 16-bit logits are fp32 (what the reference returns on its flash-attn dispatch,
  ``torch_functional.py:73-79,85-90``); accumulation is always fp32;
* ``logprobs_from_logits(..., inplace_backward=False)`` also computes the entropy in the same pass over
  the row and parks it, so that the ``entropy_from_logits(logits)`` call that the actor issues next on
  the same tensor (``siirl/engine/actor/dp_actor.py:179-195``) costs no second pass and both gradients
  are written by one backward kernel.  ``set_pairing(False)`` turns this off.
"""

from __future__ import annotations

import weakref
from typing import Optional

import torch

from . import ops  # noqa: F401  (registers torch.ops.siirl_hip.*)

_fwd = torch.ops.siirl_hip.logprob_entropy_fwd
_bwd = torch.ops.siirl_hip.logprob_entropy_bwd
_bwd_ = torch.ops.siirl_hip.logprob_entropy_bwd_

_SKIP_ZERO_ROWS = True


def set_skip_zero_rows(flag: bool) -> None:
    """Backward writes zeros, without reading the row, where both upstream gradients are zero
    (padding rows).  On by default; identical results for finite logits."""
    global _SKIP_ZERO_ROWS
    _SKIP_ZERO_ROWS = bool(flag)


class _LogprobEntropy(torch.autograd.Function):
    """(logits, labels) -> (logprob, entropy) with one forward pass and one backward pass over the rows."""

    @staticmethod
    def forward(ctx, logits, labels, inv_temperature, want_entropy, inplace_backward):
        lp, ent, lse, ex = _fwd(logits, labels, inv_temperature, want_entropy)
        ctx.save_for_backward(logits, labels if labels is not None else lse.new_empty(0), lse, ex)
        ctx.has_labels = labels is not None
        ctx.want_entropy = want_entropy
        ctx.inv_temperature = inv_temperature
        ctx.inplace = inplace_backward
        ctx.set_materialize_grads(False)
        if labels is None:
            ctx.mark_non_differentiable(lp)
        if not want_entropy:
            ctx.mark_non_differentiable(ent)
        return lp, ent

    @staticmethod
    def backward(ctx, g_lp, g_ent):
        logits, labels, lse, ex = ctx.saved_tensors
        if not ctx.has_labels:
            labels, g_lp = None, None
        if not ctx.want_entropy:
            g_ent = None
        if g_lp is None and g_ent is None:
            return None, None, None, None, None
        args = (logits, labels if g_lp is not None else None, ctx.inv_temperature, lse,
                ex if g_ent is not None else None, g_lp, g_ent, _SKIP_ZERO_ROWS)
        if ctx.inplace:
            _bwd_(*args)
            return logits, None, None, None, None
        return _bwd(*args), None, None, None, None


def _check_logits(logits):
    if not isinstance(logits, torch.Tensor) or logits.dim() < 1:
        raise TypeError("logits must be a tensor of shape (..., vocab_size)")
    if logits.dtype not in (torch.float32, torch.bfloat16, torch.float16):
        raise TypeError(f"logits dtype {logits.dtype} is not supported (float32, bfloat16, float16)")
    if logits.shape[-1] > 1 and logits.stride(-1) != 1:
        logits = logits.contiguous()
    return logits


def logprobs_and_entropy_from_logits(logits: torch.Tensor, labels: torch.Tensor, temperature: float = 1.0,
                                     inplace_backward: bool = False):
    """Both per-token outputs of the actor's post-logits step in one pass: ``(logprob, entropy)`` of
    ``logits / temperature``.  The division is folded into the kernels, ``logits`` is left untouched
    (the reference divides in place first, ``siirl/engine/actor/dp_actor.py:176``)."""
    logits = _check_logits(logits)
    return _LogprobEntropy.apply(logits, labels, 1.0 / float(temperature), True, inplace_backward)


# ------------------------------------------------------------------------------ pairing slot

_PAIRING = True
_slot = None  # (weakref to logits, _version, grad_enabled, entropy)


def set_pairing(flag: bool) -> None:
    global _PAIRING, _slot
    _PAIRING, _slot = bool(flag), None


def _park(logits, entropy):
    global _slot
    _slot = (weakref.ref(logits), logits._version, torch.is_grad_enabled(), entropy)


def _claim(logits):
    global _slot
    if _slot is None:
        return None
    ref, version, grad_mode, entropy = _slot
    if ref() is logits and logits._version == version and torch.is_grad_enabled() == grad_mode:
        _slot = None
        return entropy
    if ref() is None:
        _slot = None
    return None


# ------------------------------------------------------------------------------ reference API


def gather_from_labels(data: torch.Tensor, label: torch.Tensor) -> torch.Tensor:
    """reference ``torch_functional.py:41-53`` (plain indexing; not a hot op)."""
    return torch.gather(data, -1, label.unsqueeze(-1)).squeeze(-1)


def logprobs_from_logits(logits: torch.Tensor, labels: torch.Tensor, inplace_backward: bool = True):
    """Log-probability of ``labels`` under ``softmax(logits)``, shape ``logits.shape[:-1]``
    (reference ``torch_functional.py:56-82``).  With ``inplace_backward=True`` the backward pass
    overwrites ``logits`` with its gradient, as the reference's flash-attn path does (``:85-90``)."""
    logits = _check_logits(logits)
    if _PAIRING and not inplace_backward:
        lp, ent = _LogprobEntropy.apply(logits, labels, 1.0, True, False)
        _park(logits, ent)
        return lp
    lp, _ = _LogprobEntropy.apply(logits, labels, 1.0, False, bool(inplace_backward))
    return lp


def logprobs_from_logits_v2(logits: torch.Tensor, labels: torch.Tensor):
    """reference ``torch_functional.py:99-116``; same kernel, never in place."""
    return logprobs_from_logits(logits, labels, inplace_backward=False)


logprobs_from_logits_naive = logprobs_from_logits_v2  # reference :93-96


def entropy_from_logits(logits: torch.Tensor):
    """Entropy of ``softmax(logits)`` per row (reference ``torch_functional.py:128-132``)."""
    logits = _check_logits(logits)
    parked = _claim(logits) if _PAIRING else None
    if parked is not None:
        return parked
    _, ent = _LogprobEntropy.apply(logits, None, 1.0, True, False)
    return ent


def entropy_from_logits_with_chunking(logits: torch.Tensor, chunk_size: int = 2048):
    """reference ``torch_functional.py:135-143``.  The chunking there bounds the fp32 temporaries; the
    kernel has none, so the whole tensor goes in one launch.  2-D input, fp32 output, as there."""
    if logits.dim() != 2:
        raise ValueError("entropy_from_logits_with_chunking expects a 2-D tensor")
    return entropy_from_logits(logits)


# ------------------------------------------------------------------------------ masked reductions


def _masked_reduce(values: torch.Tensor, mask: torch.Tensor, axis, want_mean: bool):
    from . import _lib
    from . import core_algos as CA

    if not values.is_cuda:
        raise RuntimeError("siirl_amd: masked reductions run on the GPU only (no CPU fallback)")
    nd = values.dim()
    if isinstance(axis, (tuple, list)):
        axis = axis[0] if len(axis) == 1 else (None if sorted(a % nd for a in axis) == list(range(nd)) else axis)
    per_row = axis is not None
    if per_row and (not isinstance(axis, int) or axis % nd != nd - 1):
        raise NotImplementedError("siirl_amd: masked_sum / masked_mean reduce over all elements or over the last axis")
    if values.requires_grad and torch.is_grad_enabled():
        if want_mean and not per_row:  # identical arithmetic to agg_loss(..., 'token-mean'), which has a backward
            return CA.agg_loss(values, mask.expand_as(values), "token-mean")
        raise NotImplementedError("siirl_amd: only masked_mean over all elements is differentiable here")
    dev = values.device
    mask = mask.expand_as(values)
    v = CA._as_2d(CA._f32(values, dev)) if nd >= 1 else CA._f32(values, dev).reshape(1, 1)
    m, mcode = CA._mask_arg(CA._as_2d(mask) if nd >= 1 else mask.reshape(1, 1), dev)
    B, L = v.shape
    ws, nws = CA._workspace(B, L, dev)
    row = torch.empty(B, dtype=torch.float32, device=dev) if per_row else None
    tot = None if per_row else torch.empty(2, dtype=torch.float32, device=dev)
    with torch.cuda.device(dev):
        rc = _lib.lib().siirl_masked_reduce(_lib.ptr(v), _lib.ptr(m), mcode, B, L,
                                            _lib.ptr(row) if (per_row and not want_mean) else None,
                                            _lib.ptr(row) if (per_row and want_mean) else None, _lib.ptr(tot),
                                            _lib.ptr(ws), nws, _lib.current_stream(dev))
    _lib.check(rc, "siirl_masked_reduce")
    if per_row:
        return row.reshape(values.shape[:-1])
    return tot[1] if want_mean else tot[0]


def masked_sum(values: torch.Tensor, mask: torch.Tensor, axis=None):
    """``sum(where(mask, values, 0) * mask)`` over everything or over the last axis (reference
    ``torch_functional.py:146-151``); fp32 result."""
    return _masked_reduce(values, mask, axis, want_mean=False)


def masked_mean(values: torch.Tensor, mask: torch.Tensor, axis=None):
    """``masked_sum / (mask.sum + 1e-8)`` (reference ``torch_functional.py:154-168``)."""
    return _masked_reduce(values, mask, axis, want_mean=True)


def clip_by_value(x: torch.Tensor, tensor_min: torch.Tensor, tensor_max: torch.Tensor):
    """``max(min(x, tensor_max), tensor_min)`` with tensor bounds (reference ``torch_functional.py:119-125``);
    plain torch, it is not on the hot path by itself (the value loss fuses it)."""
    return torch.max(torch.min(x, tensor_max), tensor_min)


def _check_whiten_count(n: float):
    """The two ``ValueError``s of the reference's ``masked_var`` (``torch_functional.py:178-184``)."""
    if n == 0:
        raise ValueError("At least one element in the mask has to be 1.")
    if n == 1:
        raise ValueError("The sum of the mask is one, which can cause a division by zero.")


def _whiten(values: torch.Tensor, mask: torch.Tensor, shift_mean: bool):
    from . import _lib
    from . import core_algos as CA

    if not values.is_cuda:
        raise RuntimeError("siirl_amd: masked_var / masked_whiten run on the GPU only (no CPU fallback)")
    dev = values.device
    v = CA._f32(values, dev)
    m, mcode = CA._mask_arg(mask.expand_as(values), dev)
    out = torch.empty_like(v)
    stats = torch.empty(3, dtype=torch.float32, device=dev)
    nws = _lib.lib().siirl_whiten_workspace_bytes()
    ws = torch.empty(nws, dtype=torch.uint8, device=dev)
    with torch.cuda.device(dev):
        rc = _lib.lib().siirl_masked_whiten(_lib.ptr(v), _lib.ptr(m), mcode, v.numel(), int(bool(shift_mean)),
                                            _lib.ptr(out), _lib.ptr(stats), _lib.ptr(ws), nws,
                                            _lib.current_stream(dev))
    _lib.check(rc, "siirl_masked_whiten")
    return out, stats


def masked_var(values: torch.Tensor, mask: torch.Tensor, unbiased: bool = True):
    """Variance over the masked elements (reference ``torch_functional.py:171-187``), 0-d fp32."""
    _, stats = _whiten(values, mask, True)
    n = float(stats[2])
    if unbiased:
        _check_whiten_count(n)
        return stats[1]
    return stats[1] * ((n - 1.0) / n) if n > 1 else stats[1]


def masked_whiten(values: torch.Tensor, mask: torch.Tensor, shift_mean: bool = True):
    """``(values - mean) * rsqrt(var + 1e-8)`` with masked mean and unbiased masked variance, applied to every
    element (reference ``torch_functional.py:190-206``); no gradient (the reference uses it under ``no_grad``)."""
    out, stats = _whiten(values, mask, shift_mean)
    _check_whiten_count(float(stats[2]))
    return out.reshape(values.shape)


# ------------------------------------------------------------------------------ response masks and rmpad glue


def get_response_mask(response_id: torch.Tensor, eos_token=2, dtype=torch.int64):
    """1 up to and including the first end-of-sequence token of each row, 0 after it; ``eos_token`` is an int or a
    list of ints (reference ``torch_functional.py:209-229``: ``(cumsum(isin) - isin) == 0``)."""
    if not response_id.is_cuda:
        raise RuntimeError(f"siirl_amd: `response_id` is on {response_id.device}; these ops run on the GPU only")
    if response_id.dim() != 2:
        raise ValueError(f"response_id must be [batch, response_length], got {tuple(response_id.shape)}")
    if response_id.dtype not in (torch.int64, torch.int32):
        raise TypeError(f"response_id dtype {response_id.dtype} is not supported (int64, int32)")
    import ctypes

    from . import _lib

    toks = [int(t) for t in (eos_token if isinstance(eos_token, (list, tuple)) else [eos_token])]
    if len(toks) > _lib.MAX_EOS_TOKENS:
        raise ValueError(f"at most {_lib.MAX_EOS_TOKENS} end-of-sequence tokens are supported, got {len(toks)}")
    ids = response_id.contiguous()
    B, L = ids.shape
    out_dtype = torch.uint8 if dtype == torch.bool else dtype
    out = torch.empty(B, L, dtype=out_dtype, device=ids.device)
    arr = (ctypes.c_int64 * max(len(toks), 1))(*toks)
    with torch.cuda.device(ids.device):
        rc = _lib.lib().siirl_eos_response_mask(_lib.ptr(ids), _lib.dtype_code(ids.dtype), B, L, arr, len(toks),
                                                _lib.ptr(out), _lib.dtype_code(out_dtype),
                                                _lib.current_stream(ids.device))
    _lib.check(rc, "siirl_eos_response_mask")
    return out.view(torch.bool) if dtype == torch.bool else out


def get_eos_mask(response_id: torch.Tensor, eos_token: int = 2, dtype=torch.int64):
    """The single-token form (reference ``torch_functional.py:232-254``); same mask."""
    return get_response_mask(response_id, int(eos_token), dtype)


def get_unpad_data(attention_mask: torch.Tensor):
    """``(indices, cu_seqlens, max_seqlen_in_batch)`` of the attended positions (reference
    ``torch_functional.py:638-647``)."""
    from . import padding

    indices, cu, max_seqlen, _ = padding._unpad_indices(attention_mask)
    return indices, cu, max_seqlen


def log_probs_from_logits_response(input_ids, logits, response_length):
    """Log-probs of the response tokens from padded logits ``[batch, seqlen, vocab]`` (reference
    ``torch_functional.py:431-444``).  The ``[:, -response_length - 1 : -1]`` window is read in place through its
    row stride; no copy of the logits is made."""
    response_logits = logits[:, -response_length - 1:-1]
    response = input_ids[:, -response_length:]
    return logprobs_from_logits(logits=response_logits, labels=response)


def log_probs_from_logits_all_rmpad(input_ids_rmpad, logits_rmpad, indices, batch_size, seqlen, response_length):
    """Response log-probs ``[batch, response_length]`` from packed ids ``[1, nnz]`` and packed logits
    ``[nnz, vocab]`` (reference ``torch_functional.py:474-500``): labels are the ids rolled by one, the packed
    log-probs are scattered straight into the response window."""
    from . import padding

    ids = input_ids_rmpad.reshape(-1)
    rolled = torch.roll(ids, shifts=-1, dims=0)
    full_log_probs_rmpad = logprobs_from_logits(logits=logits_rmpad, labels=rolled)
    return padding.pad_and_slice_response(full_log_probs_rmpad, indices, batch_size, seqlen, response_length)


def log_probs_from_logits_response_rmpad(input_ids, attention_mask, logits_rmpad, response_length):
    """Same result from padded ids ``[batch, seqlen]`` + attention mask and packed logits (reference
    ``torch_functional.py:447-471``)."""
    from . import padding

    batch_size, seqlen = input_ids.shape
    _, rolled, indices, _, _ = padding.unpad_ids_and_labels(input_ids, attention_mask)
    full_log_probs_rmpad = logprobs_from_logits(logits=logits_rmpad, labels=rolled)
    return padding.pad_and_slice_response(full_log_probs_rmpad, indices, batch_size, seqlen, response_length)


def remove_pad_token(input_ids: torch.Tensor, attention_mask: torch.Tensor):
    """Per-row python lists of the last ``mask.sum()`` ids (reference ``torch_functional.py:416-428``); host-side
    list building, one device-to-host copy for the whole batch."""
    ids = input_ids.cpu()
    counts = attention_mask.sum(dim=-1).cpu().tolist()
    return [row[len(row) - int(n):].numpy().tolist() for row, n in zip(ids, counts)]
