"""Oracle (test infrastructure): advantages, policy losses, aggregation and KL penalty.

Restates on the CPU the arithmetic of ``siirl/dag_worker/core_algos.py`` of the reference
(GAE ``:229-276``, GRPO outcome advantage ``:279-348``, ``agg_loss`` ``:536-569``, the ``cpgd``
loss ``:572-629``, the ``vanilla`` loss ``:710-792``, the ``gspo`` loss ``:795-862``, ``gpg``
``:865-895``, ``clip_cov`` ``:898-995``, ``kl_cov`` ``:998-1071``, ``geo_mean`` ``:1074-1153``, the CPGD outcome
advantage ``:461-517``, the value loss ``:1173-1212``, ``kl_penalty``
``:1215-1276``, KL controllers ``:167-226``, ``apply_kl_penalty`` ``:1358-1397``) and the CPGD
drift term of ``siirl/engine/actor/dp_actor.py:488-494``.  Works in the dtype of its inputs, so the
same code serves as the fp32 statement and, on fp64 inputs, as the high-precision check.
"""

from __future__ import annotations

from collections import OrderedDict
from dataclasses import dataclass
from typing import Optional

import numpy as np
import torch

from .torch_functional import clip_by_value, masked_mean, masked_whiten

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


def gae_unwhitened(token_level_rewards, values, response_mask, gamma, lam):
    """The reverse scan of the reference's GAE (``core_algos.py:259-273``) before whitening:
    ``delta_t = r_t + gamma * V_next - V_t``, ``A_t = delta_t + gamma * lam * A_next``; a masked
    position keeps ``V_next`` and ``A_next`` of the position after it.  Returns ``(A, A + V)``."""
    nextvalues, lastgaelam = 0, 0
    rev = []
    for t in reversed(range(token_level_rewards.shape[-1])):
        m = response_mask[:, t]
        delta = token_level_rewards[:, t] + gamma * nextvalues - values[:, t]
        cand = delta + gamma * lam * lastgaelam
        nextvalues = values[:, t] * m + (1 - m) * nextvalues
        lastgaelam = cand * m + (1 - m) * lastgaelam
        rev.append(lastgaelam)
    adv = torch.stack(rev[::-1], dim=1)
    return adv, adv + values


def compute_gae_advantage_return(token_level_rewards, values, response_mask, gamma, lam):
    """Generalised advantage estimation, then whitening of the advantages over the mask
    (reference ``core_algos.py:229-276``).  Returns ``(advantages, returns)``; the returns are
    the un-whitened advantages plus the values."""
    adv, returns = gae_unwhitened(token_level_rewards, values, response_mask, gamma, lam)
    return masked_whiten(adv, response_mask), returns


def marft_gae_unwhitened(rewards, values, masks, chains, gamma, lam, out_dtype=None):
    """The token walk of the reference's multi-agent GAE (``core_algos.py:400-448``) on explicit operands:
    ``rewards`` / ``values`` / ``masks`` are lists over the agents (the batch's own response last) of ``[B, L_a]``
    tensors, ``chains`` a list of ``(first_row, n_rows)`` per request (rows = trajectory steps, last step first).
    One accumulator runs through a request: rows in order, agents from last to first, tokens from the last
    generated one (``mask row sum - 1``) down to 0.  Inside an agent ``delta = gamma * V[t + 1] - V[t]``; at its
    last token ``delta = rew + gamma * V_next - V`` with ``V_next`` the next agent's first value in the row, or, for
    the last agent, the first agent's first value in the row before (0 in the request's first row).  The outputs
    take the masks' dtype, as the reference's ``zeros_like(response_mask)`` does (``:386-392``): an integer mask
    truncates every stored advantage and return (``out_dtype`` overrides that, to see the values before the
    truncation).  Arithmetic is that of 0-d tensors and Python floats, as there.
    Returns ``(advantages, returns)``, lists over the agents."""
    adv = [torch.zeros_like(m, dtype=out_dtype) for m in masks]
    ret = [torch.zeros_like(a) for a in adv]
    last = len(masks) - 1
    for first_row, n_rows in chains:
        gae = 0
        for step in range(n_rows):
            row = first_row + step
            for agent in range(last, -1, -1):
                gen = masks[agent][row].sum()
                for t in reversed(range(gen)):
                    v = values[agent][row, t]
                    if t == gen - 1:
                        if agent == last:
                            v_next = 0 if step == 0 else values[0][row - 1, 0]
                        else:
                            v_next = values[agent + 1][row, 0]
                        delta = rewards[agent][row, t] + gamma * v_next - v
                    else:
                        delta = gamma * values[agent][row, t + 1] - v
                    gae = delta + gamma * lam * gae
                    adv[agent][row, t] = gae
                    ret[agent][row, t] = gae + v
    return adv, ret


def compute_marft_gae_advantage_return(data, pre_agent_group_ids, gamma, lam):
    """``siirl/dag_worker/core_algos.py:351-458``.  ``data.batch`` holds ``agent_group_<id>_token_level_rewards`` /
    ``_values`` / ``_response_mask`` for every id of ``pre_agent_group_ids`` and the unprefixed three for the last
    agent; ``data.non_tensor_batch`` holds ``request_id`` (rows of one request are consecutive; the first row of each
    distinct id starts a request) and ``traj_len`` (read at that first row).  As in the reference: the id list is
    indexed by its own values (so it must be 0 .. n - 1) and grows by one id per call (``:395``); every agent's
    advantages are whitened over its mask (``:451``) but the results of all the earlier agents are stored under the
    LAST of the given ids, each overwriting the one before (``:452-454`` use the loop variable left over from
    ``:379``), so only that id's two keys and ``advantages`` / ``returns`` appear in ``data.batch``."""
    prefix = "agent_group_"
    names = [prefix + str(g) + "_" for g in pre_agent_group_ids] + [""]
    rewards = [data.batch[n + "token_level_rewards"] for n in names]
    values = [data.batch[n + "values"] for n in names]
    masks = [data.batch[n + "response_mask"] for n in names]
    last_given = pre_agent_group_ids[-1]
    pre_agent_group_ids.append(last_given + 1)
    seen, chains = set(), []
    for row, rid in enumerate(data.non_tensor_batch["request_id"]):
        if rid not in seen:
            seen.add(rid)
            chains.append((row, int(data.non_tensor_batch["traj_len"][row])))
    with torch.no_grad():
        order = list(pre_agent_group_ids)
        adv, ret = marft_gae_unwhitened([rewards[g] for g in order], [values[g] for g in order],
                                        [masks[g] for g in order], chains, gamma, lam)
        for g in order:
            white = masked_whiten(adv[g], masks[g])
            if g != order[-1]:
                data.batch[prefix + str(last_given) + "_advantages"] = white
                data.batch[prefix + str(last_given) + "_returns"] = ret[g]
            else:
                data.batch["advantages"] = white
                data.batch["returns"] = ret[g]


def pf_ppo_weights(scores, reweight_method: str, weight_pow: float):
    """Resampling weights of PF-PPO from per-sequence scores (reference ``core_algos.py:1296-1327``), with the
    ``+ 1e-8`` floor of ``:1329``."""
    if reweight_method == "pow":
        w = scores.abs() ** weight_pow
    elif reweight_method == "max_min":
        w = ((scores == scores.max()) | (scores == scores.min())).to(torch.float32)
    elif reweight_method == "max_random":
        w = torch.full_like(scores, 0.1)
        w[scores == scores.max()] = 0.4
    else:
        raise ValueError(f"Unsupported reweight_method: {reweight_method}")
    return torch.clamp(w + 1e-8, min=1e-8)


def compute_pf_ppo_reweight_data(data, reweight_method: str = "pow", weight_pow: float = 2.0):
    """``siirl/dag_worker/core_algos.py:1279-1355``: ``batch_size`` rows drawn with replacement (``torch.multinomial``
    on the host generator) with the weights above; tensors, per-row arrays / lists and ``batch_size``-long meta
    lists are indexed with the draw; the input is left alone and a copy returned."""
    import copy

    scores = data.batch["token_level_scores"].sum(dim=-1)
    n = scores.shape[0]
    picks = torch.multinomial(pf_ppo_weights(scores, reweight_method, weight_pow), n, replacement=True)
    out = copy.deepcopy(data)
    out.batch = type(data.batch)({k: t[picks] for k, t in data.batch.items()})
    idx = picks.numpy()
    out.non_tensor_batch = {k: (a[idx] if isinstance(a, np.ndarray) else [a[i] for i in idx])
                            for k, a in data.non_tensor_batch.items()}
    out.meta_info = {k: ([v[i] for i in idx] if isinstance(v, list) and len(v) == n else v)
                     for k, v in data.meta_info.items()}
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


def compute_entropy_loss(logits, response_mask, loss_agg_mode: str = "token-mean"):
    """``siirl/dag_worker/core_algos.py:1156-1170``: aggregated token entropy of ``logits [B, L, V]``."""
    from .torch_functional import entropy_from_logits

    return agg_loss(entropy_from_logits(logits), response_mask, loss_agg_mode)


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


def compute_policy_loss_cpgd(old_log_prob, log_prob, advantages, response_mask,
                             loss_agg_mode="token-mean", config=None, rollout_is_weights=None):
    """CPGD: the log-probability itself is clipped at ``old + log(1 + eps_hi)`` (positive advantage)
    or ``old + log(1 - eps_lo)`` (otherwise) and the loss is ``-clipped * A`` (reference
    ``core_algos.py:572-629``).  ``rollout_is_weights`` is accepted and ignored, as there."""
    import math

    assert config is not None, "Config must be provided for CPGD loss"
    eps_lo, eps_hi = _clip_bounds(config)
    c = config.clip_ratio_c if config.clip_ratio_c is not None else 3.0
    assert c > 1.0, f"clip_ratio_c ({c}) must be > 1.0"
    d = log_prob - old_log_prob
    ratio = torch.exp(d)
    ppo_kl = masked_mean(-d, response_mask)
    clipped = torch.where(advantages > 0,
                          torch.clamp(log_prob, max=math.log(1 + eps_hi) + old_log_prob),
                          torch.clamp(log_prob, min=math.log(1 - eps_lo) + old_log_prob))
    pg_loss = agg_loss(-clipped * advantages, response_mask, loss_agg_mode)
    is_clipped = torch.where(advantages > 0, ratio > 1 + eps_hi, ratio < 1 - eps_lo)
    pg_clipfrac = masked_mean(is_clipped.to(d.dtype), response_mask)
    pg_clipfrac_lower = masked_mean((ratio > c) * (advantages < 0).to(d.dtype), response_mask)
    return pg_loss, pg_clipfrac, ppo_kl, pg_clipfrac_lower


def policy_drift_loss(old_log_prob, log_prob, response_mask, loss_agg_mode):
    """CPGD's drift regulariser as the actor adds it (reference ``dp_actor.py:488-494``):
    ``agg_loss(clamp(exp(lp.detach() - old) - 1, max=2) * lp)``."""
    drift = ((log_prob.detach() - old_log_prob).exp() - 1.0).clamp(max=2.0) * log_prob
    return agg_loss(drift, response_mask, loss_agg_mode)


def compute_policy_loss_gpg(old_log_prob, log_prob, advantages, response_mask,
                            loss_agg_mode="token-mean", config=None, rollout_is_weights=None):
    """GPG: ``-log_prob * A`` (reference ``core_algos.py:865-895``); the three metrics are zeros."""
    tok = -log_prob * advantages
    if rollout_is_weights is not None:
        tok = tok * rollout_is_weights
    z = torch.zeros((), dtype=tok.dtype)
    return agg_loss(tok, response_mask, loss_agg_mode), z, z, z


def compute_policy_loss_geo_mean(old_log_prob, log_prob, advantages, response_mask,
                                 loss_agg_mode="token-mean", config=None, rollout_is_weights=None):
    """GMPO: token log-ratios clipped to ``[-eps_lo, eps_hi]`` on the side the advantage's sign
    makes pessimistic, their masked mean exponentiated (geometric mean of the ratios), times the
    masked-mean advantage of the sequence; plain mean over sequences (reference
    ``core_algos.py:1074-1153``).  ``loss_agg_mode`` is not used."""
    assert config is not None
    eps_lo, eps_hi = _clip_bounds(config)
    d = log_prob - old_log_prob
    ppo_kl = masked_mean(-d, response_mask)
    sgn = torch.sign(advantages)
    dc = torch.clamp(d, -eps_lo, eps_hi)
    x = sgn * torch.min(sgn * d, sgn * dc)
    n = response_mask.sum(dim=-1)
    ratio = torch.exp((x * response_mask).sum(dim=-1) / (n + 1e-8))
    adv = (advantages * response_mask).sum(dim=-1) / (n + 1e-8)
    seq = -adv * ratio
    if rollout_is_weights is not None:
        seq = seq * torch.exp((torch.log(rollout_is_weights + 1e-10) * response_mask).sum(dim=-1) / (n + 1e-8))
    clipped = torch.ne(d, dc)
    pg_clipfrac = masked_mean((clipped * (advantages > 0)).to(d.dtype), response_mask)
    pg_clipfrac_lower = masked_mean((clipped * (advantages < 0)).to(d.dtype), response_mask)
    return torch.mean(seq), pg_clipfrac, ppo_kl, pg_clipfrac_lower


@dataclass
class CovLossConfig:
    """``config.policy_loss`` of the two covariance losses (reference ``siirl/params/model_args.py``, read at
    ``core_algos.py:943-948,1034-1035``); ``None`` selects the default the loss function states."""

    clip_cov_ratio: Optional[float] = None
    clip_cov_lb: Optional[float] = None
    clip_cov_ub: Optional[float] = None
    kl_cov_ratio: Optional[float] = None
    ppo_kl_coef: Optional[float] = None


def clip_cov_candidates(old_log_prob, log_prob, advantages, response_mask, eps_lo, eps_hi, lb, ub):
    """The covariance matrix and the candidate set of Clip-Cov (reference ``core_algos.py:952-975``):
    ``cov = (A - masked_mean(A)) * (lp - masked_mean(lp))``, minus infinity where the mask is zero or where the
    PPO clip already bites (``l2 > l1``); candidates are the tokens with ``lb < cov < ub``, listed in row-major order."""
    ratio = torch.exp(log_prob - old_log_prob)
    l1 = -advantages * ratio
    l2 = -advantages * torch.clamp(ratio, 1 - eps_lo, 1 + eps_hi)
    clip_by_origin = (l2 > l1) & (response_mask > 0)
    cov = (advantages - masked_mean(advantages, response_mask)) * (
        log_prob.detach() - masked_mean(log_prob.detach(), response_mask))
    cov = cov.clone()
    cov[response_mask == 0] = -torch.inf
    cov[clip_by_origin] = -torch.inf
    cand = (cov < ub) & (cov > lb) & (response_mask > 0)
    return cov, torch.nonzero(cand)


def compute_policy_loss_clip_cov(old_log_prob, log_prob, advantages, response_mask, loss_agg_mode="token-mean",
                                 config=None, rollout_is_weights=None, dropped=None):
    """Clip-Cov (reference ``core_algos.py:898-995``): the PPO clip surrogate without dual clip and without the
    +-20 clamp of the log-ratio, with the loss of ``max(int(ratio * sum(mask)), 1)`` randomly chosen candidate tokens
    (``torch.randperm`` on the host, the global generator) set to zero; ``pg_clipfrac`` is the masked share of
    dropped tokens.  ``dropped`` (an ``[n, 2]`` index tensor) overrides the random choice, for tests of the arithmetic
    after the draw.  Returns ``(pg_loss, pg_clipfrac, ppo_kl, 0)``."""
    assert config is not None and config.policy_loss is not None
    pl = config.policy_loss
    ratio_cfg = pl.clip_cov_ratio if pl.clip_cov_ratio is not None else 0.0002
    eps_lo, eps_hi = _clip_bounds(config)
    ub = pl.clip_cov_ub if pl.clip_cov_ub is not None else 5.0
    lb = pl.clip_cov_lb if pl.clip_cov_lb is not None else 1.0
    assert ratio_cfg > 0, "clip_ratio should be larger than 0."

    d = log_prob - old_log_prob
    ratio = torch.exp(d)
    ppo_kl = masked_mean(-d, response_mask)
    l1 = -advantages * ratio
    l2 = -advantages * torch.clamp(ratio, 1 - eps_lo, 1 + eps_hi)
    if dropped is None:
        _, cand = clip_cov_candidates(old_log_prob, log_prob, advantages, response_mask, eps_lo, eps_hi, lb, ub)
        clip_num = max(int(ratio_cfg * response_mask.sum().item()), 1)
        if len(cand) > 0:
            perm = torch.randperm(len(cand))
            dropped = cand[perm[: min(clip_num, len(cand))]]
        else:
            dropped = torch.empty((0, 2), dtype=torch.long)
    corr = torch.ones_like(advantages)
    corr[dropped[:, 0], dropped[:, 1]] = 0
    pg_clipfrac = masked_mean((corr == 0).to(d.dtype), response_mask)
    tok = torch.maximum(l1, l2) * corr
    if rollout_is_weights is not None:
        tok = tok * rollout_is_weights
    return agg_loss(tok, response_mask, loss_agg_mode), pg_clipfrac, ppo_kl, torch.zeros((), dtype=d.dtype)


def kl_cov_selection(log_prob, advantages, response_mask, kl_cov_ratio):
    """Flat indices (into ``[B * L]``) of the tokens KL-Cov penalises (reference ``core_algos.py:1047-1060``): over
    the tokens with a positive mask, ``cov = (A - mean A) * (lp - mean lp)`` with plain means, and the
    ``max(1, int(n * ratio))`` largest values are taken."""
    valid = response_mask > 0
    valid_idx = torch.nonzero(valid.reshape(-1), as_tuple=True)[0]
    a = advantages[valid].detach().reshape(-1)
    lp = log_prob[valid].detach().reshape(-1)
    if min(kl_cov_ratio, len(a)) == 0:
        return valid_idx[:0], None
    cov = (a - a.mean()) * (lp - lp.mean())
    k = max(1, int(len(cov) * kl_cov_ratio))
    return valid_idx[torch.topk(cov, k, largest=True).indices], cov


def compute_policy_loss_kl_cov(old_log_prob, log_prob, advantages, response_mask, loss_agg_mode="token-mean",
                               config=None, rollout_is_weights=None, chosen=None):
    """KL-Cov (reference ``core_algos.py:998-1071``): the unclipped surrogate ``-A * ratio``; the tokens selected by
    ``kl_cov_selection`` additionally pay ``ppo_kl_coef * |lp - old|``.  Returns ``(pg_loss, 0, masked_mean(|lp - old|), 0)``.
    ``chosen`` (flat indices) overrides the selection: for checks of the arithmetic in another precision than the
    one the selection was made in (two tokens of equal covariance sort differently in float32 and float64)."""
    assert config is not None and config.policy_loss is not None
    pl = config.policy_loss
    kl_cov_ratio = pl.kl_cov_ratio if pl.kl_cov_ratio is not None else 0.0002
    coef = pl.ppo_kl_coef if pl.ppo_kl_coef is not None else 1.0
    assert kl_cov_ratio > 0, "kl_cov_ratio should be larger than 0."

    d = log_prob - old_log_prob
    abs_kl = d.abs()
    ratio = torch.exp(d)
    ppo_kl_abs = masked_mean(abs_kl, response_mask)
    plain = -advantages * ratio
    with_kl = -advantages * ratio + coef * abs_kl
    if chosen is None:
        chosen, _ = kl_cov_selection(log_prob, advantages, response_mask, kl_cov_ratio)
    pick = torch.zeros(advantages.numel(), dtype=torch.bool)
    pick[chosen] = True
    tok = torch.where(pick.reshape(advantages.shape), with_kl, plain)
    if rollout_is_weights is not None:
        tok = tok * rollout_is_weights
    zero = torch.zeros((), dtype=d.dtype)
    return agg_loss(tok, response_mask, loss_agg_mode), zero, ppo_kl_abs, zero


def compute_cpgd_outcome_advantage(token_level_rewards, response_mask, index, epsilon=1e-6,
                                   weight_factor_in_cpgd="STD_weight"):
    """CPGD's outcome advantage (reference ``core_algos.py:461-517``): the group statistics of the GRPO estimator (a
    group of one: mean 0, std 1), then ``(s - mean) / (std + eps)`` (``STD_weight``), ``s - mean`` (``naive``) or
    ``(s - mean) * min(B / #groups with std != 0, 3)`` (``clip_filter_like_weight``)."""
    scores = token_level_rewards.sum(dim=-1)
    keys = [index[i].item() if hasattr(index[i], "item") else index[i] for i in range(scores.shape[0])]
    members = OrderedDict()
    for i, k in enumerate(keys):
        members.setdefault(k, []).append(i)
    mean, std = {}, {}
    for k, rows in members.items():
        if len(rows) == 1:
            mean[k], std[k] = torch.zeros((), dtype=scores.dtype), torch.ones((), dtype=scores.dtype)
        else:
            mean[k], std[k] = scores[rows].mean(), scores[rows].std()
    bsz = scores.shape[0]
    out = scores.clone()
    for i, k in enumerate(keys):
        if weight_factor_in_cpgd == "STD_weight":
            out[i] = (scores[i] - mean[k]) / (std[k] + epsilon)
        elif weight_factor_in_cpgd == "clip_filter_like_weight":
            live = sum(int(v != 0) for v in std.values())  # no live group: B / 0 = inf there, clamped to 3
            out[i] = (scores[i] - mean[k]) * (min(bsz / live, 3.0) if live else 3.0)
        elif weight_factor_in_cpgd == "naive":
            out[i] = scores[i] - mean[k]
        else:
            raise NotImplementedError
    out = out.unsqueeze(-1) * response_mask
    return out, out


def compute_value_loss(vpreds, returns, values, response_mask, cliprange_value, loss_agg_mode="token-mean"):
    """Clipped value loss (reference ``core_algos.py:1173-1212``): ``0.5 * agg_loss(max((v - R)^2,
    (clip(v, V_old - c, V_old + c) - R)^2))`` and the fraction of tokens where the clipped term wins."""
    vclip = clip_by_value(vpreds, values - cliprange_value, values + cliprange_value)
    l1 = (vpreds - returns) ** 2
    l2 = (vclip - returns) ** 2
    vf_loss = 0.5 * agg_loss(torch.max(l1, l2), response_mask, loss_agg_mode)
    vf_clipfrac = masked_mean(torch.gt(l2, l1).to(l1.dtype), response_mask)
    return vf_loss, vf_clipfrac


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
