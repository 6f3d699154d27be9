"""Oracle (test infrastructure): the actor's post-logits arithmetic for one micro-batch.

Restates the order of operations of ``siirl/engine/actor/dp_actor.py:170-231`` (logits / T ->
log-prob -> entropy) and ``:403-513`` (policy loss, entropy bonus, KL loss, loss scaling,
backward, metric scalars), with the transformer left out: the micro-batch starts at the
``[B, L, V]`` response logits."""

from __future__ import annotations

from dataclasses import dataclass
from typing import Optional

import torch

from . import core_algos
from .torch_functional import entropy_from_logits, logprobs_from_logits


@dataclass
class ActorConfig:
    """The actor fields that parameterise the path (reference ``siirl/params/model_args.py:281-319``)."""

    clip_ratio: float = 0.2
    clip_ratio_low: Optional[float] = 0.2
    clip_ratio_high: Optional[float] = 0.2
    clip_ratio_c: float = 3.0
    entropy_coeff: float = 0.0
    use_kl_loss: bool = False
    kl_loss_coef: float = 0.001
    kl_loss_type: str = "low_var_kl"
    loss_agg_mode: str = "token-mean"
    loss_mode: str = "vanilla"
    use_cpgd_loss: bool = False
    policy_drift_coeff: float = 0.0
    policy_loss: Optional[core_algos.CovLossConfig] = None  # the covariance losses' parameters


_LOSSES = {"vanilla": core_algos.compute_policy_loss_vanilla, "gspo": core_algos.compute_policy_loss_gspo,
           "cpgd": core_algos.compute_policy_loss_cpgd, "gpg": core_algos.compute_policy_loss_gpg,
           "geo_mean": core_algos.compute_policy_loss_geo_mean, "clip_cov": core_algos.compute_policy_loss_clip_cov,
           "kl_cov": core_algos.compute_policy_loss_kl_cov}


def micro_batch_step(logits, responses, old_log_prob, advantages, response_mask, config: ActorConfig,
                     ref_log_prob=None, temperature=1.0, loss_scale_factor=1.0, on_policy=False,
                     rollout_is_weights=None, dtype=torch.float32):
    """One iteration of the micro-batch loop.  ``logits`` is ``[B, L, V]`` (any float dtype) and is
    not modified.  Returns ``(loss, dlogits, metrics, log_prob, entropy)`` with ``dlogits`` the
    gradient of ``loss`` w.r.t. the *unscaled* logits, in ``dtype``."""
    x = logits.detach().to(dtype).clone().requires_grad_(True)
    z = x / temperature  # dp_actor.py:176 (done in place there)
    log_prob = logprobs_from_logits(z, responses, dtype=dtype)  # :182-186
    want_entropy = config.entropy_coeff != 0  # :423-426
    entropy = entropy_from_logits(z, dtype=dtype) if want_entropy else None  # :189-195

    old = log_prob.detach() if on_policy else old_log_prob  # :436-439
    pg_loss, clipfrac, ppo_kl, clipfrac_lower = _LOSSES[config.loss_mode](
        old_log_prob=old, log_prob=log_prob, advantages=advantages, response_mask=response_mask,
        loss_agg_mode=config.loss_agg_mode, config=config, rollout_is_weights=rollout_is_weights)  # :455-466
    metrics = {}
    policy_loss = pg_loss
    if want_entropy:
        entropy_loss = core_algos.agg_loss(entropy, response_mask, config.loss_agg_mode)  # :469
        policy_loss = pg_loss - entropy_loss * config.entropy_coeff  # :472
        metrics["actor/entropy_loss"] = entropy_loss.item()
    if config.use_kl_loss:
        kld = core_algos.kl_penalty(log_prob, ref_log_prob, config.kl_loss_type)  # :479-481
        kl_loss = core_algos.agg_loss(kld, response_mask, config.loss_agg_mode)  # :482
        policy_loss = policy_loss + kl_loss * config.kl_loss_coef  # :484
        metrics["actor/kl_loss"] = kl_loss.item() * loss_scale_factor
        metrics["actor/kl_coef"] = config.kl_loss_coef
    if config.use_cpgd_loss and config.policy_drift_coeff != 0:  # :488-494
        policy_loss = policy_loss + core_algos.policy_drift_loss(old, log_prob, response_mask, config.loss_agg_mode) \
            * config.policy_drift_coeff
    loss = policy_loss * loss_scale_factor  # :496-500
    (dlogits,) = torch.autograd.grad(loss, x)  # :501
    ratio = (log_prob.detach() - old).exp()
    metrics.update({  # :503-513
        "actor/pg_clip_mean": ratio.mean().item(),
        "actor/pg_clip_min": ratio.min().item(),
        "actor/pg_clip_max": ratio.max().item(),
        "actor/pg_loss": pg_loss.item() * loss_scale_factor,
        "actor/pg_clipfrac": clipfrac.item(),
        "actor/ppo_kl": ppo_kl.item(),
        "actor/pg_clipfrac_lower": float(clipfrac_lower),
    })
    return loss.detach(), dlogits, metrics, log_prob.detach(), None if entropy is None else entropy.detach()
