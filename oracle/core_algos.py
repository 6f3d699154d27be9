"""Oracle (test infrastructure): advantages, policy losses, aggregation and KL penalty.

Restates on the CPU the arithmetic of ``siirl/dag_worker/core_algos.py`` of the reference
(GRPO outcome advantage ``:279-348``, ``agg_loss`` ``:536-569``, the ``vanilla`` loss
``:710-792``, the ``gspo`` loss ``:795-862``, ``kl_penalty`` ``:1215-1276``, KL controllers
``:167-226``, ``apply_kl_penalty`` ``:1358-1397``).  Works in the dtype of its inputs, so the
same code serves as the fp32 statement and, on fp64 inputs, as the high-precision check.
"""

from __future__ import annotations

from collections import OrderedDict
from dataclasses import dataclass
from typing import Optional

import numpy as np
import torch

from .torch_functional import masked_mean

AGG_MODES = ("token-mean", "seq-mean-token-sum", "seq-mean-token-mean", "seq-mean-token-sum-norm")


@dataclass
class LossConfig:
    """The four attributes the loss functions read from the actor config
    (reference ``siirl/params/model_args.py:281-284``; same defaults)."""

    clip_ratio: float = 0.2
    clip_ratio_low: Optional[float] = 0.2
    clip_ratio_high: Optional[float] = 0.2
    clip_ratio_c: float = 3.0


# --------------------------------------------------------------------------- advantages


def compute_grpo_outcome_advantage(token_level_rewards, response_mask, index, epsilon=1e-6,
                                   norm_adv_by_std_in_grpo=True, config=None):
    """Group-normalised outcome advantage (reference ``core_algos.py:279-348``).

    ``s_i = sum_t r_it``; per group of equal ``index``: mean and *unbiased* std (``torch.std``),
    a group of one uses mean 0 / std 1; ``a_i = (s_i - mean) / (std + eps)`` (or ``s_i - mean``);
    broadcast over tokens and multiplied by the mask.  The same tensor is returned twice."""
    scores = token_level_rewards.sum(dim=-1)
    keys = [int(index[i]) for i in range(scores.shape[0])]
    members = OrderedDict()
    for i, k in enumerate(keys):
        members.setdefault(k, []).append(i)
    out = scores.clone()
    for k, rows in members.items():
        if len(rows) == 1:
            mean = torch.zeros((), dtype=scores.dtype)
            std = torch.ones((), dtype=scores.dtype)
        else:
            grp = scores[rows]
            mean, std = grp.mean(), grp.std()  # unbiased (N-1)
        for i in rows:
            out[i] = (scores[i] - mean) / (std + epsilon) if norm_adv_by_std_in_grpo else scores[i] - mean
    adv = out.unsqueeze(-1) * response_mask
    return adv, adv


def grpo_bruteforce(scores, uid, epsilon=1e-6, norm=True):
    """Independent pure-Python statement of the group normalisation for tiny inputs."""
    import math

    s = [float(v) for v in scores]
    u = [int(v) for v in uid]
    out = []
    for i in range(len(s)):
        grp = [s[j] for j in range(len(s)) if u[j] == u[i]]
        if len(grp) == 1:
            mu, sd = 0.0, 1.0
        else:
            mu = sum(grp) / len(grp)
            sd = math.sqrt(sum((g - mu) ** 2 for g in grp) / (len(grp) - 1))
        out.append((s[i] - mu) / (sd + epsilon) if norm else s[i] - mu)
    return out


# --------------------------------------------------------------------------- aggregation


def agg_loss(loss_mat, loss_mask, loss_agg_mode: str):
    """Scalar aggregation of a ``[B, L]`` loss (reference ``core_algos.py:536-569``)."""
    if loss_agg_mode == "token-mean":
        return masked_mean(loss_mat, loss_mask)
    if loss_agg_mode == "seq-mean-token-sum":
        return (loss_mat * loss_mask).sum(-1).mean()
    if loss_agg_mode == "seq-mean-token-mean":
        # no epsilon: a row with an empty mask gives 0/0 = NaN, as in the reference (:557)
        return ((loss_mat * loss_mask).sum(-1) / loss_mask.sum(-1)).mean()
    if loss_agg_mode == "seq-mean-token-sum-norm":
        return (loss_mat * loss_mask).sum(-1).sum() / loss_mask.shape[-1]
    raise ValueError(f"Invalid loss_agg_mode: {loss_agg_mode}")


# --------------------------------------------------------------------------- policy losses


def _clip_bounds(config):
    lo = config.clip_ratio_low if config.clip_ratio_low is not None else config.clip_ratio
    hi = config.clip_ratio_high if config.clip_ratio_high is not None else config.clip_ratio
    return lo, hi


def compute_policy_loss_vanilla(old_log_prob, log_prob, advantages, response_mask,
                                loss_agg_mode="token-mean", config=None, rollout_is_weights=None):
    """PPO / GRPO / DAPO clipped surrogate with dual clip (reference ``core_algos.py:710-792``).
    Returns ``(pg_loss, pg_clipfrac, ppo_kl, pg_clipfrac_lower)``."""
    assert config is not None
    eps_lo, eps_hi = _clip_bounds(config)
    c = config.clip_ratio_c
    assert c > 1.0, f"clip_ratio_c must exceed 1.0, got {c}"

    d = torch.clamp(log_prob - old_log_prob, min=-20.0, max=20.0)
    ratio = torch.exp(d)
    ppo_kl = masked_mean(-d, response_mask)

    l1 = -advantages * ratio
    l2 = -advantages * torch.clamp(ratio, 1 - eps_lo, 1 + eps_hi)
    c1 = torch.maximum(l1, l2)
    pg_clipfrac = masked_mean(torch.gt(l2, l1).to(d.dtype), response_mask)

    l3 = -advantages * c
    c2 = torch.min(l3, c1)
    pg_clipfrac_lower = masked_mean(torch.gt(c1, l3) * (advantages < 0).to(d.dtype), response_mask)

    tok = torch.where(advantages < 0, c2, c1)
    if rollout_is_weights is not None:
        tok = tok * rollout_is_weights
    return agg_loss(tok, response_mask, loss_agg_mode), pg_clipfrac, ppo_kl, pg_clipfrac_lower


def compute_policy_loss_gspo(old_log_prob, log_prob, advantages, response_mask,
                             loss_agg_mode="seq-mean-token-mean", config=None, rollout_is_weights=None):
    """GSPO: sequence-level importance ratio with a token-level gradient (reference
    ``core_algos.py:795-862``).  The aggregation is always ``seq-mean-token-mean`` whatever
    ``loss_agg_mode`` says (``:854``); ``pg_clipfrac_lower`` is a constant zero."""
    assert config is not None
    eps_lo, eps_hi = _clip_bounds(config)

    d = log_prob - old_log_prob
    n = response_mask.sum(-1).clamp(min=1)
    s = (d * response_mask).sum(-1) / n
    log_rho = log_prob - log_prob.detach() + s.detach().unsqueeze(-1)
    rho = torch.exp(torch.clamp(log_rho, max=10.0))

    l1 = -advantages * rho
    l2 = -advantages * torch.clamp(rho, 1 - eps_lo, 1 + eps_hi)
    tok = torch.maximum(l1, l2)
    if rollout_is_weights is not None:
        tok = tok * rollout_is_weights
    pg_loss = agg_loss(tok, response_mask, "seq-mean-token-mean")
    pg_clipfrac = masked_mean(torch.gt(l2, l1).to(d.dtype), response_mask)
    ppo_kl = masked_mean(-d, response_mask)
    return pg_loss, pg_clipfrac, ppo_kl, torch.zeros((), dtype=pg_loss.dtype)


def policy_loss_grad_closed_form(old_log_prob, log_prob, advantages, response_mask, loss_agg_mode,
                                 config, rollout_is_weights=None, mode="vanilla"):
    """d(pg_loss)/d(log_prob) written out by hand, used to cross-check autograd on the functions
    above.  ``w`` is the aggregation weight of each token; the surrogate passes gradient
    ``-A * ratio`` where the unclipped branch is the active one."""
    eps_lo, eps_hi = _clip_bounds(config)
    m = response_mask.to(log_prob.dtype)
    B, L = log_prob.shape
    if mode == "gspo":
        loss_agg_mode = "seq-mean-token-mean"
    if loss_agg_mode == "token-mean":
        w = m / (m.sum() + 1e-8)
    elif loss_agg_mode == "seq-mean-token-sum":
        w = m / B
    elif loss_agg_mode == "seq-mean-token-mean":
        w = m / (B * m.sum(-1, keepdim=True))
    else:
        w = m / L
    if rollout_is_weights is not None:
        w = w * rollout_is_weights
    A = advantages
    if mode == "vanilla":
        raw = log_prob - old_log_prob
        d = raw.clamp(-20.0, 20.0)
        r = torch.exp(d)
        inside = (raw >= -20.0) & (raw <= 20.0)
        # A > 0: max(l1, l2) follows l1 unless r > 1 + eps_hi.   A < 0: l1 is active for
        # r >= 1 - eps_lo, and the dual clip cuts it off once -A*r exceeds -A*c, i.e. r > c.
        pos = (A > 0) & (r <= 1 + eps_hi)
        neg = (A < 0) & (r >= 1 - eps_lo) & (r <= config.clip_ratio_c)
        active = (pos | neg) & inside
        return torch.where(active, w * (-A * r), torch.zeros_like(r))
    n = response_mask.sum(-1).clamp(min=1)
    s = ((log_prob - old_log_prob) * response_mask).sum(-1) / n
    ls = s.unsqueeze(-1).expand(B, L)
    rho = torch.exp(ls.clamp(max=10.0))
    active = (((A > 0) & (rho <= 1 + eps_hi)) | ((A < 0) & (rho >= 1 - eps_lo))) & (ls <= 10.0)
    return torch.where(active, w * (-A * rho), torch.zeros_like(rho))


# --------------------------------------------------------------------------- KL


def kl_penalty_forward(logprob, ref_logprob, kl_penalty: str):
    """Per-token KL estimators (reference ``core_algos.py:1241-1276``)."""
    if kl_penalty in ("kl", "k1"):
        return logprob - ref_logprob
    if kl_penalty == "abs":
        return (logprob - ref_logprob).abs()
    if kl_penalty in ("mse", "k2"):
        return 0.5 * (logprob - ref_logprob).square()
    if kl_penalty in ("low_var_kl", "k3"):
        k = torch.clamp(ref_logprob - logprob, min=-20, max=20)
        return torch.clamp(torch.exp(k) - k - 1, min=-10, max=10)
    raise NotImplementedError(kl_penalty)


def kl_penalty(logprob, ref_logprob, kl_penalty: str):
    """Estimator value, with the k2 gradient when the name ends in ``+`` (reference
    ``core_algos.py:1215-1238``).  Note the reference hands the *suffixed* name to the forward
    (``:1227``), which knows no such name: every ``+`` mode ends in ``NotImplementedError``."""
    value = kl_penalty_forward(logprob, ref_logprob, kl_penalty)
    if not kl_penalty.endswith("+") or kl_penalty in ("mse", "k2"):
        return value
    k2 = 0.5 * (logprob - ref_logprob).square()
    return k2 - k2.detach() + value.detach()


class FixedKLController:
    """reference ``core_algos.py:192-206``"""

    def __init__(self, kl_coef):
        self.value = kl_coef

    def update(self, current_kl, n_steps):
        pass


class AdaptiveKLController:
    """reference ``core_algos.py:167-189``"""

    def __init__(self, init_kl_coef, target_kl, horizon):
        self.value, self.target, self.horizon = init_kl_coef, target_kl, horizon

    def update(self, current_kl, n_steps):
        err = np.clip(current_kl / self.target - 1, -0.2, 0.2)
        self.value *= 1 + err * n_steps / self.horizon


def get_kl_controller(kl_ctrl):
    """reference ``core_algos.py:209-226``"""
    if kl_ctrl.type == "fixed":
        return FixedKLController(kl_ctrl.kl_coef)
    if kl_ctrl.type == "adaptive":
        assert kl_ctrl.horizon > 0
        return AdaptiveKLController(kl_ctrl.kl_coef, kl_ctrl.target_kl, kl_ctrl.horizon)
    raise NotImplementedError


def compute_rewards(token_level_scores, old_log_prob, ref_log_prob, kl_ratio):
    """reference ``core_algos.py:520-533``"""
    return token_level_scores - (old_log_prob - ref_log_prob) * kl_ratio


def apply_kl_penalty(data: dict, kl_ctrl, kl_penalty_type="kl"):
    """KL-in-reward on a dict of tensors (reference ``core_algos.py:1358-1397``)."""
    mask = data["response_mask"]
    kld = kl_penalty(data["old_log_probs"], data["ref_log_prob"], kl_penalty_type) * mask
    beta = kl_ctrl.value
    data["token_level_rewards"] = data["token_level_scores"] - beta * kld
    current_kl = masked_mean(kld, mask, axis=-1).mean(dim=0).item()
    kl_ctrl.update(current_kl=current_kl, n_steps=data["token_level_scores"].shape[0])
    return data, {"actor/reward_kl_penalty": current_kl, "actor/reward_kl_penalty_coeff": beta}
