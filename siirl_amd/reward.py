"""Outcome-reward placement with DAPO's overlong penalty.

Mirror of the tensor-building part of ``DAPORewardManager.__call__`` (reference
``siirl/engine/reward_manager/dapo.py:57-126``): given one scalar score per trajectory (the scoring functions and
the tokenizer are the caller's), build the ``[B, response_length]`` float32 reward tensor with the score -- plus
the overlong penalty when enabled -- at the last valid response token."""

from __future__ import annotations

from collections import defaultdict

import torch

from . import _lib
from .core_algos import _mask_arg, _staging_device

__all__ = ["place_outcome_reward"]


def place_outcome_reward(scores, attention_mask: torch.Tensor, response_length: int, overlong_buffer_cfg=None,
                         max_resp_len=None, return_dict: bool = False):
    """``scores``: ``B`` Python numbers or a tensor; ``attention_mask`` ``[B, prompt + response]``.
    ``overlong_buffer_cfg`` has ``enable``, ``len``, ``penalty_factor`` and ``log`` as in the reference
    (``dapo.py:108-117``).  Returns the reward tensor, or with ``return_dict`` also ``reward_extra_info`` holding
    ``overlong_reward`` / ``overlong`` lists when ``log`` is set."""
    if overlong_buffer_cfg is not None:
        assert max_resp_len is not None, f"max_resp_len must be provided if {overlong_buffer_cfg=}, but got None"
    dev, back = _staging_device(attention_mask)
    B, S = attention_mask.shape
    L = int(response_length)
    if not 1 <= L <= S:
        raise ValueError(f"response_length {L} does not fit attention_mask of width {S}")
    sc = torch.as_tensor(scores, dtype=torch.float64).reshape(-1).to(dev).contiguous()
    if sc.numel() != B:
        raise ValueError(f"{sc.numel()} scores for a batch of {B}")
    am, acode = _mask_arg(attention_mask, dev)
    enable = bool(overlong_buffer_cfg is not None and overlong_buffer_cfg.enable)
    reward = torch.empty(B, L, dtype=torch.float32, device=dev)
    pen = torch.empty(B, dtype=torch.float64, device=dev)
    with torch.cuda.device(dev):
        rc = _lib.lib().siirl_place_outcome_reward(
            _lib.ptr(sc), _lib.ptr(am), acode, B, S - L, L, int(enable),
            float(max_resp_len) if enable else 0.0, float(overlong_buffer_cfg.len) if enable else 1.0,
            float(overlong_buffer_cfg.penalty_factor) if enable else 0.0, _lib.ptr(reward), _lib.ptr(pen), None,
            _lib.current_stream(dev))
    _lib.check(rc, "siirl_place_outcome_reward")
    if back:
        reward = reward.to(attention_mask.device)
    if not return_dict:
        return reward
    extra = defaultdict(list)
    if enable and getattr(overlong_buffer_cfg, "log", False):
        p = pen.tolist()
        extra["overlong_reward"] = p
        extra["overlong"] = [v < 0 for v in p]
    return {"reward_tensor": reward, "reward_extra_info": extra}
