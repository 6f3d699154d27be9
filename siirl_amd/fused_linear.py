"""lm_head projection fused with log-prob / entropy, with the reference's two Python interfaces.

* ``FusedLinearForPPO`` -- mirror of ``siirl/utils/experimental/torch_functional.py:191-211`` (module) and
  ``:70-188`` (autograd function): ``forward(hidden_states, vocab_weights, input_ids, temperature=1.0)`` returns
  ``(log_probs, entropy)`` shaped like ``input_ids``.
* ``linear_cross_entropy`` -- mirror of ``siirl/utils/kernel/linear_cross_entropy.py:40-117``:
  ``(hidden, weight, labels, temperature, reduction, dist_process_group) -> (logprobs, entropy)``.

Both run the MFMA kernels of ``csrc/fused_linear.hip`` through the C ABI.  Operands are bf16 on the GPU.  The
forward needs no ``[T, V]`` tensor.  When a backward will follow and the buffer fits the limit set with
``set_saved_logits_limit`` (default 16 GiB, or ``SIIRL_AMD_SAVED_LOGITS_LIMIT`` bytes from the environment; 4 bytes
per logit), the forward parks its fp32 logit tiles and the
backward reads them back instead of running the projection a second time: the same bits, a quarter less matrix
work per step.  With the limit at 0 the logits are never stored and the backward recomputes them slab by slab,
which is the reference's memory behaviour.  Outputs are fp32 (the reference's Triton path returns fp32,
``kernels.py:586-593``; its chunked-torch path casts back to the input dtype, ``torch_functional.py:32``, which
``FusedLinearForPPO(cast_outputs=True)`` reproduces).  ``chunk_size`` is accepted and ignored: tiling is the
kernel's business.
"""

from __future__ import annotations

import os
import typing

import torch

from . import ops as _ops_module  # noqa: F401  (registers torch.ops.siirl_hip.*)


# bytes; the environment variable gives a deployment its own default without code changes
_SAVED_LOGITS_LIMIT = int(os.environ.get("SIIRL_AMD_SAVED_LOGITS_LIMIT", 16 << 30))


def set_saved_logits_limit(nbytes: int) -> None:
    """Largest fp32 logit buffer (bytes) the forward may keep for the backward; 0 = always recompute."""
    global _SAVED_LOGITS_LIMIT
    if nbytes < 0:
        raise ValueError(f"the limit must not be negative, got {nbytes}")
    _SAVED_LOGITS_LIMIT = int(nbytes)


def _saved_logits_bytes(T: int, V: int) -> int:
    return ((V + 255) // 256) * ((T + 255) // 256) * (256 * 256 * 4)


class _FusedLinearLogprobEntropy(torch.autograd.Function):
    @staticmethod
    def forward(ctx, hidden, weight, labels, temperature):
        if not hidden.is_cuda or not weight.is_cuda:
            raise RuntimeError("siirl_amd: the fused lm_head path runs on the GPU only (no CPU fallback)")
        if hidden.dtype != torch.bfloat16 or weight.dtype != torch.bfloat16:
            raise TypeError("siirl_amd: the fused lm_head path takes bfloat16 hidden states and weights")
        dev = hidden.device
        h = hidden.detach().contiguous()
        w = weight.detach().contiguous()
        y = labels.detach().to(device=dev, dtype=torch.int64).contiguous()
        T, H = h.shape
        V = w.shape[0]
        if w.shape[1] != H or y.shape != (T,):
            raise ValueError(f"shape mismatch: hidden {tuple(h.shape)}, weight {tuple(w.shape)}, labels {tuple(y.shape)}")
        inv_t = 1.0 / float(temperature)
        save = (ctx.needs_input_grad[0] or ctx.needs_input_grad[1]) and \
            _saved_logits_bytes(T, V) <= _SAVED_LOGITS_LIMIT
        lp, ent, lse, ex, saved = torch.ops.siirl_hip.fused_linear_logprob_entropy_fwd(h, w, y, inv_t, bool(save))
        ctx.save_for_backward(h, w, y, lse, ex, saved)
        ctx.inv_t = inv_t
        ctx.set_materialize_grads(False)
        return lp, ent

    @staticmethod
    def backward(ctx, g_lp, g_ent):
        h, w, y, lse, ex, saved = ctx.saved_tensors
        need_h, need_w = ctx.needs_input_grad[0], ctx.needs_input_grad[1]
        if (g_lp is None and g_ent is None) or not (need_h or need_w):
            return None, None, None, None
        dev = h.device
        f = lambda t: None if t is None else t.detach().to(device=dev, dtype=torch.float32).contiguous()  # noqa: E731
        g_lp, g_ent = f(g_lp), f(g_ent)
        d_h, d_w = torch.ops.siirl_hip.fused_linear_logprob_entropy_bwd(h, w, y, ctx.inv_t, lse, ex, g_lp, g_ent,
                                                                        bool(need_h), bool(need_w), saved)
        return (d_h if need_h else None), (d_w if need_w else None), None, None


def fused_linear_logprob_entropy(hidden: torch.Tensor, weight: torch.Tensor, labels: torch.Tensor,
                                 temperature: float = 1.0):
    """``(logprob, entropy)`` of ``softmax((hidden @ weight.T) / temperature)`` at ``labels``; fp32, shaped like
    ``labels``.  ``hidden`` is ``[..., H]``, ``weight`` ``[V, H]``."""
    lead = hidden.shape[:-1]
    if labels.shape != lead:
        raise ValueError(f"labels shape {tuple(labels.shape)} does not match hidden {tuple(hidden.shape)}")
    lp, ent = _FusedLinearLogprobEntropy.apply(hidden.reshape(-1, hidden.shape[-1]), weight, labels.reshape(-1),
                                               float(temperature))
    return lp.reshape(lead), ent.reshape(lead)


class FusedLinearForPPO(torch.nn.Module):
    """reference ``siirl/utils/experimental/torch_functional.py:191-211``."""

    def __init__(self, chunk_size: int = 512, cast_outputs: bool = False):
        super().__init__()
        self.chunk_size = chunk_size  # kept for signature parity; the kernel tiles by itself
        self.cast_outputs = cast_outputs

    def forward(self, hidden_states: torch.Tensor, vocab_weights: torch.Tensor, input_ids: torch.Tensor,
                temperature: float = 1.0) -> typing.Tuple[torch.Tensor, torch.Tensor]:
        assert hidden_states.ndim in (2, 3), f"Invalid hidden_states shape, received {hidden_states.shape}"
        if hidden_states.ndim == 3:
            assert input_ids.ndim == 2, f"input_ids shape doesn't match, {hidden_states.shape} {input_ids.shape}"
        lp, ent = fused_linear_logprob_entropy(hidden_states, vocab_weights, input_ids.to(torch.int64), temperature)
        if self.cast_outputs:
            lp, ent = lp.to(hidden_states.dtype), ent.to(hidden_states.dtype)
        return lp, ent


def linear_cross_entropy(hidden: torch.Tensor, weight: torch.Tensor, labels: torch.Tensor,
                         temperature: typing.Optional[float] = 1.0, reduction: typing.Optional[str] = "none",
                         dist_process_group=None):
    """reference ``siirl/utils/kernel/linear_cross_entropy.py:40-117``: ``(logprobs, entropy)``, fp32, flattened
    over tokens.  ``reduction`` ("none" | "sum" | "mean") applies to the log-probs as there
    (``kernels.py:353-365``).  A tensor-parallel ``dist_process_group`` is outside this one-GPU build."""
    assert isinstance(temperature, float), f"temperature must be a float, but got {type(temperature)}"
    assert isinstance(reduction, str), f"reduction must be a str, but got {type(reduction)}"
    red = reduction.lower()
    if red not in ("none", "sum", "mean"):
        raise ValueError(f"Invalid reduction: {reduction}")
    if dist_process_group is not None:
        raise NotImplementedError("siirl_amd: vocab-parallel linear_cross_entropy (dist_process_group) is not built")
    h2 = hidden.reshape(-1, hidden.shape[-1])
    lp, ent = _FusedLinearLogprobEntropy.apply(h2, weight, labels.reshape(-1), temperature)
    if red == "sum":
        lp = lp.sum()
    elif red == "mean":
        lp = lp.mean()
    return lp, ent
