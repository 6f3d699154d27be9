"""lm_head projection fused with log-prob / entropy, with the reference's two Python interfaces.

* ``FusedLinearForPPO`` -- mirror of ``siirl/utils/experimental/torch_functional.py:191-211`` (module) and
  ``:70-188`` (autograd function): ``forward(hidden_states, vocab_weights, input_ids, temperature=1.0)`` returns
  ``(log_probs, entropy)`` shaped like ``input_ids``.
* ``linear_cross_entropy`` -- mirror of ``siirl/utils/kernel/linear_cross_entropy.py:40-117``:
  ``(hidden, weight, labels, temperature, reduction, dist_process_group) -> (logprobs, entropy)``.

Both run the MFMA kernels of ``csrc/fused_linear.hip`` through the C ABI.  Operands are bf16, fp16 or fp32 on the GPU (fp16: the half matrix instruction; fp32: three bf16
terms per element, products good to 2^-16; the gradient GEMMs always multiply bf16 dlogits with bf16-rounded
operands and return the operands' dtype).  Neither
pass holds a ``[T, V]`` tensor: the backward recomputes the logits slab by slab, which is the reference's memory
behaviour.  Opt-in trade of memory for time: with ``set_saved_logits_limit(nbytes)`` (or
``SIIRL_AMD_SAVED_LOGITS_LIMIT`` bytes in the environment; default 0 = never), a forward that a backward will follow
parks its fp32 logit tiles (4 bytes per logit) when they fit the limit and the backward reads them back instead of
running the projection a second time: the same bits, a quarter less matrix work per step.  Outputs are fp32 (the reference's Triton path returns fp32,
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
_SAVED_LOGITS_LIMIT = int(os.environ.get("SIIRL_AMD_SAVED_LOGITS_LIMIT", 0))


def set_saved_logits_limit(nbytes: int) -> None:
    """Largest fp32 logit buffer (bytes) the forward may keep for the backward; 0 (the default) = never keep one,
    always recompute."""
    global _SAVED_LOGITS_LIMIT
    if nbytes < 0:
        raise ValueError(f"the limit must not be negative, got {nbytes}")
    _SAVED_LOGITS_LIMIT = int(nbytes)


_SKIP_ZERO_ROWS = False


def set_skip_zero_rows(flag: bool) -> None:
    """``True``: the backward leaves token rows whose upstream gradients are both zero out of its three GEMMs (the
    prompt tokens of a packed batch: the actor keeps only the response slice of the log-probs, reference
    ``siirl/engine/actor/dp_actor.py:170-172,228-231``).  Off by default, because it departs from the reference's
    autograd in two ways: it costs one host synchronisation per backward (the count of such rows; it is therefore
    not applied under stream capture, nor when the logits were parked), and ``d_hidden`` of a skipped row is zero even
    where its hidden state holds NaN or Inf.  ``d_weight`` is summed over the remaining rows, which changes its
    rounding order, not its value."""
    global _SKIP_ZERO_ROWS
    _SKIP_ZERO_ROWS = bool(flag)


def _saved_logits_bytes(T: int, V: int) -> int:
    return ((V + 255) // 256) * ((T + 255) // 256) * (256 * 256 * 4)


def _apply(hidden2d, weight, labels1d, temperature):
    if not hidden2d.is_cuda or not weight.is_cuda:
        raise RuntimeError("siirl_amd: the fused lm_head path runs on the GPU only (no CPU fallback)")
    return torch.ops.siirl_hip.fused_linear_logprob_entropy(hidden2d, weight, labels1d, 1.0 / float(temperature),
                                                            _SAVED_LOGITS_LIMIT, _SKIP_ZERO_ROWS)


def fused_linear_logprob_entropy(hidden: torch.Tensor, weight: torch.Tensor, labels: torch.Tensor,
                                 temperature: float = 1.0):
    """``(logprob, entropy)`` of ``softmax((hidden @ weight.T) / temperature)`` at ``labels``; fp32, shaped like
    ``labels``.  ``hidden`` is ``[..., H]``, ``weight`` ``[V, H]``."""
    lead = hidden.shape[:-1]
    if labels.shape != lead:
        raise ValueError(f"labels shape {tuple(labels.shape)} does not match hidden {tuple(hidden.shape)}")
    lp, ent = _apply(hidden.reshape(-1, hidden.shape[-1]), weight, labels.reshape(-1), temperature)
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
    lp, ent = _apply(h2, weight, labels.reshape(-1), temperature)
    if red == "sum":
        lp = lp.sum()
    elif red == "mean":
        lp = lp.mean()
    return lp, ent
