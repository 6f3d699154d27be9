"""Installs the package's functions over the reference's module globals, for a deployment that does not want to
touch the reference's import lines.

``patch_reference(ref_torch_functional, ref_core_algos)`` takes the two already imported reference modules
(``siirl.utils.model_utils.torch_functional`` and ``siirl.dag_worker.core_algos``) -- or any objects with those
attributes -- and replaces, by name, only the functions whose every caller in the reference hands them device
tensors of the actor's micro-batch:

* ``logprobs_from_logits``, ``entropy_from_logits``, ``entropy_from_logits_with_chunking``
  (``siirl/engine/actor/dp_actor.py:75-84,179-195,254-260``);
* ``agg_loss``, ``kl_penalty``, ``compute_policy_loss`` and the seven registered policy losses
  (``compute_policy_loss_vanilla`` / ``_gspo`` / ``_cpgd`` / ``_gpg`` / ``_clip_cov`` / ``_kl_cov`` / ``_geo_mean``) with
  their registry entries (``dp_actor.py:453-486``).  Three of the reference's own (``clip_cov``, ``kl_cov``,
  ``geo_mean``) refuse the stock actors' config class (``core_algos.py:940,1031,1104``); the replacements read the
  same attributes from any config object and have no such check;
* ``compute_grpo_outcome_advantage``, ``compute_marft_gae_advantage_return`` and ``apply_kl_penalty``, which the
  reference runs on host tensors (``siirl/dag_worker/dagworker.py:542-560,585-630``): the replacements stage host inputs
  to the GPU and return host results.  (The multi-agent GAE is a Python loop over every token in the reference,
  ``core_algos.py:400-448``.)

Deliberately NOT replaced: ``masked_sum`` / ``masked_mean`` / ``masked_var`` / ``masked_whiten``.  The reference's own
``compute_gae_advantage_return`` resolves those globals and calls them on host tensors, where this package's versions
raise (no CPU path); import them from ``siirl_amd.torch_functional`` explicitly where the tensors are on the GPU.
"""

from __future__ import annotations

TORCH_FUNCTIONAL_NAMES = ("logprobs_from_logits", "entropy_from_logits", "entropy_from_logits_with_chunking")
POLICY_LOSSES = {"vanilla": "compute_policy_loss_vanilla", "gspo": "compute_policy_loss_gspo",
                 "cpgd": "compute_policy_loss_cpgd", "gpg": "compute_policy_loss_gpg",
                 "clip_cov": "compute_policy_loss_clip_cov", "kl_cov": "compute_policy_loss_kl_cov",
                 "geo_mean": "compute_policy_loss_geo_mean"}
CORE_ALGOS_NAMES = ("agg_loss", "kl_penalty", "compute_policy_loss", *POLICY_LOSSES.values(),
                    "compute_grpo_outcome_advantage", "compute_marft_gae_advantage_return", "apply_kl_penalty")


def patch_reference(ref_torch_functional, ref_core_algos) -> dict:
    """Returns ``{"module.name": original}`` so that the caller can undo the patch."""
    from . import core_algos as A
    from . import torch_functional as F

    undo = {}
    for name in TORCH_FUNCTIONAL_NAMES:
        undo[f"torch_functional.{name}"] = getattr(ref_torch_functional, name, None)
        setattr(ref_torch_functional, name, getattr(F, name))
    for name in CORE_ALGOS_NAMES:
        undo[f"core_algos.{name}"] = getattr(ref_core_algos, name, None)
        setattr(ref_core_algos, name, getattr(A, name))
    losses = getattr(ref_core_algos, "POLICY_LOSS_REGISTRY", None)
    if losses is not None:
        losses.update({mode: getattr(A, fn) for mode, fn in POLICY_LOSSES.items()})
    estimators = getattr(ref_core_algos, "ADV_ESTIMATOR_REGISTRY", None)
    if estimators is not None:
        estimators["grpo"] = A.compute_grpo_outcome_advantage
    return undo
