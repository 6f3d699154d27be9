"""Oracle (test infrastructure): lm_head projection fused with log-prob and entropy.

Restates ``siirl/utils/experimental/torch_functional.py:20-67`` (per-chunk forward and backward
of ``FusedLinearForPPO``); ``siirl/utils/kernel/kernels.py:254-266,343-350,828-835`` computes
the same quantities with an online softmax.  The oracle keeps fp32 (or fp64) outputs; the
reference casts them back to the input dtype (``:32``) and accumulates ``dW`` in the weight's
dtype (``:151,175``) -- ``literal_cast=True`` reproduces that."""

from __future__ import annotations

import torch

from .torch_functional import logprob_entropy_backward, logprob_entropy_forward


def fused_linear_for_ppo_fwd(hidden, weight, input_ids, temperature=1.0, *, dtype=torch.float32,
                             chunk_size=512, literal_cast=False):
    """``logits = (h @ W.T) / T`` chunk by chunk, then log-prob of ``input_ids`` and entropy.
    With ``literal_cast`` the matmul runs in the input dtype and is then upcast (reference
    ``:21-23``); otherwise inputs are upcast first (exact product of the 16-bit values)."""
    h2 = hidden.reshape(-1, hidden.shape[-1])
    ids = input_ids.reshape(-1)
    lps, ents = [], []
    for lo in range(0, h2.shape[0], chunk_size):
        hc = h2[lo : lo + chunk_size]
        if literal_cast:
            logits = ((hc @ weight.t()) / temperature).to(torch.float32)
            lp, ent, _, _ = logprob_entropy_forward(logits, ids[lo : lo + chunk_size])
            lp, ent = lp.to(hidden.dtype), ent.to(hidden.dtype)
        else:
            logits = hc.to(dtype) @ weight.to(dtype).t()
            lp, ent, _, _ = logprob_entropy_forward(logits, ids[lo : lo + chunk_size], temperature, dtype=dtype)
        lps.append(lp)
        ents.append(ent)
    return torch.cat(lps).reshape(input_ids.shape), torch.cat(ents).reshape(input_ids.shape)


def fused_linear_for_ppo_bwd(g_logprob, g_entropy, hidden, weight, input_ids, temperature=1.0, *,
                             dtype=torch.float32, chunk_size=512):
    """``(d hidden, d weight)`` by recomputing each chunk's logits (reference ``:35-67``):
    ``dlogits`` as in ``logprob_entropy_backward`` (the ``1/T`` included), then
    ``dh = dlogits @ W`` and ``dW += dlogits.T @ h``.  Kept in ``dtype`` throughout."""
    h2 = hidden.reshape(-1, hidden.shape[-1]).to(dtype)
    w = weight.to(dtype)
    ids = input_ids.reshape(-1)
    gl = None if g_logprob is None else g_logprob.reshape(-1)
    gh = None if g_entropy is None else g_entropy.reshape(-1)
    dh = torch.zeros_like(h2)
    dw = torch.zeros_like(w)
    for lo in range(0, h2.shape[0], chunk_size):
        sl = slice(lo, lo + chunk_size)
        logits = h2[sl] @ w.t()
        dlogits = logprob_entropy_backward(logits, ids[sl], None if gl is None else gl[sl],
                                           None if gh is None else gh[sl], temperature, dtype=dtype)
        dh[sl] = dlogits @ w
        dw += dlogits.t() @ h2[sl]
    return dh.reshape(hidden.shape), dw
