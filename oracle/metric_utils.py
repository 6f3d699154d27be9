"""Oracle (test infrastructure): the per-step data metrics.

Restates ``compute_data_metric`` and ``_compute_response_info`` of the reference
(``siirl/utils/metrics/metric_utils.py:36-183``) on CPU tensors, without the process-memory gauge (``:169``)
and the multi-turn counters (``:172-176``), which are not tensor arithmetic of this path."""

from __future__ import annotations

import torch


def compute_response_info(data: dict):
    """Prompt / response lengths (reference ``metric_utils.py:36-66``)."""
    L = data["responses"].shape[-1]
    prompt_mask = data["attention_mask"][:, :-L]
    response_mask = data["response_mask"] if "response_mask" in data else data["attention_mask"][:, -L:]
    return dict(response_mask=response_mask, prompt_length=prompt_mask.sum(-1).float(),
                response_length=response_mask.sum(-1).float())


def compute_data_metric(data: dict) -> dict:
    """Reference ``metric_utils.py:70-177``: statistics of sequence scores / rewards, of the advantages,
    returns and values under ``response_mask.bool()``, the explained variance of the value function, and
    response / prompt length statistics (overall, and split by reward sum > 0.5)."""
    seq_score = data["token_level_scores"].sum(-1)
    seq_reward = data["token_level_rewards"].sum(-1)
    L = data["responses"].shape[-1]
    max_prompt = data["attention_mask"][:, :-L].size(-1)
    rmask = data["response_mask"].bool()
    info = compute_response_info(data)
    plen, rlen = info["prompt_length"], info["response_length"]
    adv = torch.masked_select(data["advantages"], rmask)
    ret = torch.masked_select(data["returns"], rmask)
    out = {
        "critic/score/mean": seq_score.mean().item(), "critic/score/max": seq_score.max().item(),
        "critic/score/min": seq_score.min().item(),
        "critic/rewards/mean": seq_reward.mean().item(), "critic/rewards/max": seq_reward.max().item(),
        "critic/rewards/min": seq_reward.min().item(),
        "critic/advantages/mean": adv.mean().item(), "critic/advantages/max": adv.max().item(),
        "critic/advantages/min": adv.min().item(),
        "critic/returns/mean": ret.mean().item(), "critic/returns/max": ret.max().item(),
        "critic/returns/min": ret.min().item(),
    }
    if "values" in data:
        val = torch.masked_select(data["values"], rmask)
        out.update({
            "critic/values/mean": val.mean().item(), "critic/values/max": val.max().item(),
            "critic/values/min": val.min().item(),
            "critic/vf_explained_var": (1.0 - torch.var(ret - val) / (torch.var(ret) + 1e-5)).item(),
        })
    correct = seq_reward > 0.5
    groups = {"correct": rlen[correct], "wrong": rlen[~correct]}
    out.update({
        "response/length/mean": rlen.mean().item(), "response/length/max": rlen.max().item(),
        "response/length/min": rlen.min().item(),
        "response/clip_ratio/mean": torch.eq(rlen, L).float().mean().item(),
    })
    for name, g in groups.items():
        for stat in ("max", "min", "mean"):
            out[f"response/{name}_length/{stat}"] = getattr(g, stat)().item() if g.numel() else 0
    out.update({
        "prompt/length/mean": plen.mean().item(), "prompt/length/max": plen.max().item(),
        "prompt/length/min": plen.min().item(),
        "prompt/clip_ratio/mean": torch.eq(plen, max_prompt).float().mean().item(),
    })
    return out
