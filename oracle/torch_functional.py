"""Oracle (test infrastructure): log-prob / entropy from logits and the masked reductions.

Restates ``siirl/utils/model_utils/torch_functional.py:41-206`` of the reference on the CPU.

Precision policy.  The reference's fp32 branch (``torch_functional.py:103-107``) is
``gather(x) - logsumexp(x)``; for 16-bit logits the deployed path is flash-attn's fp32
cross-entropy (``:73-79,85-90``) and the chunked entropy upcasts with ``.float()``
(``:139-142``).  The oracle therefore upcasts 16-bit logits and applies the fp32 (or, on
request, fp64) formula.  ``literal_bf16=True`` reproduces the reference's no-flash-attn
16-bit branch (``:108-115``, ``:128-132``), whose results are rounded to the input dtype;
it is a side note, not the parity target.
"""

from __future__ import annotations

import torch
import torch.nn.functional as F


def _work_dtype(x: torch.Tensor, dtype):
    if dtype is not None:
        return dtype
    return torch.float64 if x.dtype == torch.float64 else torch.float32


def gather_from_labels(data: torch.Tensor, label: torch.Tensor) -> torch.Tensor:
    """``data[..., label]`` along the last axis (reference ``torch_functional.py:41-53``)."""
    return data.gather(-1, label.unsqueeze(-1)).squeeze(-1)


def logprobs_from_logits(logits, labels, inplace_backward=True, *, dtype=None, literal_bf16=False):
    """Per-row ``x[y] - logsumexp(x)`` (reference ``torch_functional.py:56-82,99-116``).

    ``inplace_backward`` is accepted for signature parity and has no effect on values.
    """
    if literal_bf16 and logits.dtype in (torch.bfloat16, torch.float16):
        # reference :108-115 -- row-wise log_softmax in the input dtype, then gather
        flat = logits.reshape(-1, logits.shape[-1])
        lab = labels.reshape(-1)
        rows = [F.log_softmax(r, dim=-1)[y] for r, y in zip(flat, lab)]
        return torch.stack(rows).reshape(labels.shape)
    x = logits.to(_work_dtype(logits, dtype))
    picked = gather_from_labels(x, labels)
    return picked - torch.logsumexp(x, dim=-1)


def logprobs_from_logits_flash_attn(logits, labels, *, dtype=None):
    """The reference's flash-attn dispatch (``torch_functional.py:73-90``): ``-cross_entropy_loss(logits, labels)[0]``.
    flash-attn (2.7.3 / 2.8.2, not in the reference tree) computes the per-row cross entropy in fp32 with its default
    ``ignore_index=-100``: an ignored row has loss 0 and receives no gradient.  Stated here with torch's own
    ``F.cross_entropy``, which has the same default and the same convention.  Parity with flash-attn's Triton kernel
    itself is unpinned (third party); this function is pinned by the library routine it calls."""
    x = logits.to(_work_dtype(logits, dtype))
    flat = -F.cross_entropy(x.reshape(-1, x.shape[-1]), labels.reshape(-1), reduction="none")
    return flat.reshape(labels.shape)


def entropy_from_logits(logits, *, dtype=None, literal_bf16=False):
    """``H = logsumexp(x) - sum(softmax(x) * x)`` (reference ``torch_functional.py:128-132``)."""
    if literal_bf16:
        p = torch.softmax(logits, dim=-1)
        return torch.logsumexp(logits, dim=-1) - (p * logits).sum(-1)
    x = logits.to(_work_dtype(logits, dtype))
    p = torch.softmax(x, dim=-1)
    return torch.logsumexp(x, dim=-1) - (p * x).sum(-1)


def entropy_from_logits_with_chunking(logits, chunk_size: int = 2048):
    """Row-chunked fp32 entropy of a 2-D tensor (reference ``torch_functional.py:135-143``)."""
    out = torch.zeros(logits.shape[0], dtype=torch.float32)
    for lo in range(0, logits.shape[0], chunk_size):
        out[lo : lo + chunk_size] = entropy_from_logits(logits[lo : lo + chunk_size].float())
    return out


def logprob_entropy_forward(logits, labels, temperature: float = 1.0, *, dtype=None):
    """Both outputs of the actor's post-logits step with the in-place ``logits / T`` of
    ``siirl/engine/actor/dp_actor.py:176`` folded in.  Returns ``(logprob, entropy, lse, ex)``
    where ``lse = logsumexp(z)`` and ``ex = E_p[z]`` for ``z = x / T``."""
    z = logits.to(_work_dtype(logits, dtype)) / temperature
    lse = torch.logsumexp(z, dim=-1)
    p = torch.exp(z - lse.unsqueeze(-1))
    ex = (p * z).sum(-1)
    return gather_from_labels(z, labels) - lse, lse - ex, lse, ex


def logprob_entropy_backward(logits, labels, g_logprob, g_entropy, temperature: float = 1.0, *, dtype=None):
    """Closed-form gradient of ``sum(g_lp * logprob) + sum(g_H * entropy)`` w.r.t. the logits.

    ``dx = (1/T) * [ g_lp * (onehot(y) - p) - g_H * p * (z - E_p[z]) ]`` with ``z = x/T``,
    ``p = softmax(z)``: the explicit form of ``siirl/utils/experimental/torch_functional.py:49-62``
    (``log p + H == z - E_p[z]``) and of ``siirl/utils/kernel/kernels.py:828-835``.
    Either upstream gradient may be ``None``.  Returned in the working dtype (not rounded)."""
    wd = _work_dtype(logits, dtype)
    z = logits.to(wd) / temperature
    lse = torch.logsumexp(z, dim=-1, keepdim=True)
    p = torch.exp(z - lse)
    dz = torch.zeros_like(z)
    if g_logprob is not None:
        g = g_logprob.to(wd).unsqueeze(-1)
        onehot = torch.zeros_like(z).scatter_(-1, labels.unsqueeze(-1), 1.0)
        dz += g * (onehot - p)
    if g_entropy is not None:
        gh = g_entropy.to(wd).unsqueeze(-1)
        ex = (p * z).sum(-1, keepdim=True)
        dz -= gh * p * (z - ex)
    return dz / temperature


def logprob_entropy_backward_autograd(logits, labels, g_logprob, g_entropy, temperature: float = 1.0, *, dtype=None):
    """Same gradient obtained the way the reference obtains it: autograd through the forward."""
    wd = _work_dtype(logits, dtype)
    x = logits.to(wd).detach().clone().requires_grad_(True)
    z = x / temperature
    total = x.new_zeros(())
    if g_logprob is not None:
        total = total + (g_logprob.to(wd) * logprobs_from_logits(z, labels, dtype=wd)).sum()
    if g_entropy is not None:
        total = total + (g_entropy.to(wd) * entropy_from_logits(z, dtype=wd)).sum()
    (grad,) = torch.autograd.grad(total, x)
    return grad


def masked_sum(values, mask, axis=None):
    """``sum(where(mask, v, 0) * mask)`` (reference ``torch_functional.py:146-151``): values outside
    the mask, NaN included, do not contribute."""
    kept = torch.where(mask.bool(), values, 0.0)  # (integer values become float32 here, as in the reference)
    return (kept * mask).sum(axis)


def masked_mean(values, mask, axis=None):
    """``masked_sum / (sum(mask) + 1e-8)`` (reference ``torch_functional.py:154-168``)."""
    return masked_sum(values, mask, axis) / (mask.sum(axis) + 1e-8)


def clip_by_value(x, tensor_min, tensor_max):
    """``max(min(x, tensor_max), tensor_min)`` with tensor bounds (reference ``torch_functional.py:119-125``)."""
    return torch.max(torch.min(x, tensor_max), tensor_min)


def masked_var(values, mask, unbiased=True):
    """Variance over the masked elements (reference ``torch_functional.py:171-187``): the masked mean
    of the squared deviations from the masked mean, times ``n / (n - 1)`` when unbiased.  An empty
    mask or a mask of one element raise ``ValueError`` as the reference does."""
    mean = masked_mean(values, mask)
    variance = masked_mean((values - mean) ** 2, mask)
    if unbiased:
        n = mask.sum()
        if n == 0:
            raise ValueError("At least one element in the mask has to be 1.")
        if n == 1:
            raise ValueError("The sum of the mask is one, which can cause a division by zero.")
        variance = variance * (n / (n - 1))
    return variance


def masked_whiten(values, mask, shift_mean=True):
    """``(values - mean) * rsqrt(var + 1e-8)`` with masked statistics, applied to every element
    (reference ``torch_functional.py:190-206``)."""
    mean, var = masked_mean(values, mask), masked_var(values, mask)
    out = (values - mean) * torch.rsqrt(var + 1e-8)
    if not shift_mean:
        out = out + mean
    return out


# ---------------------------------------------------------------- response-window glue (reference :431-500)


def log_probs_from_logits_response(input_ids, logits, response_length, *, dtype=None):
    """reference ``torch_functional.py:431-444``: logits of positions ``-L-1 .. -2`` score ids ``-L .. -1``."""
    return logprobs_from_logits(logits[:, -response_length - 1:-1], input_ids[:, -response_length:], dtype=dtype)


def log_probs_from_logits_all_rmpad(input_ids_rmpad, logits_rmpad, indices, batch_size, seqlen, response_length, *,
                                    dtype=None):
    """reference ``torch_functional.py:474-500``; ``pad_input`` is flash-attn's zero-filled scatter."""
    ids = input_ids_rmpad.reshape(-1)
    lp = logprobs_from_logits(logits_rmpad, torch.roll(ids, shifts=-1, dims=0), dtype=dtype)
    full = torch.zeros(batch_size * seqlen, dtype=lp.dtype).index_put((indices,), lp).reshape(batch_size, seqlen)
    return full[:, -response_length - 1:-1]


def log_probs_from_logits_response_rmpad(input_ids, attention_mask, logits_rmpad, response_length, *, dtype=None):
    """reference ``torch_functional.py:447-471``."""
    batch_size, seqlen = input_ids.shape
    indices = torch.nonzero(attention_mask.flatten(), as_tuple=False).flatten()
    ids_rmpad = input_ids.flatten()[indices]
    return log_probs_from_logits_all_rmpad(ids_rmpad[None], logits_rmpad, indices, batch_size, seqlen,
                                           response_length, dtype=dtype)
