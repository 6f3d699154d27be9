"""Installs the package's functions over the reference's module globals, for a deployment that does not want to
touch the reference's import lines.

``patch_reference(ref_torch_functional, ref_core_algos)`` takes the two already imported reference modules
(``siirl.utils.model_utils.torch_functional`` and ``siirl.dag_worker.core_algos``) -- or any objects with those
attributes -- and replaces, by name, only the functions whose every caller in the reference hands them device
tensors of the actor's micro-batch:

* ``logprobs_from_logits``, ``entropy_from_logits``, ``entropy_from_logits_with_chunking``
  (``siirl/engine/actor/dp_actor.py:75-84,179-195,254-260``);
* ``agg_loss``, ``kl_penalty``, ``compute_policy_loss``, ``compute_policy_loss_vanilla``,
  ``compute_policy_loss_gspo`` and the two registry entries (``dp_actor.py:453-486``);
* ``compute_grpo_outcome_advantage`` and ``apply_kl_penalty``, which the reference runs on host tensors
  (``siirl/dag_worker/dagworker.py:542-560``): the replacements stage host inputs to the GPU and return host results.

Deliberately NOT replaced: ``masked_sum`` / ``masked_mean`` / ``masked_var`` / ``masked_whiten``.  The reference's own
``compute_gae_advantage_return``, ``clip_cov`` and ``kl_cov`` resolve those globals and call them on host tensors,
where this package's versions raise (no CPU path); import them from ``siirl_amd.torch_functional`` explicitly where the
tensors are on the GPU.
"""

from __future__ import annotations

TORCH_FUNCTIONAL_NAMES = ("logprobs_from_logits", "entropy_from_logits", "entropy_from_logits_with_chunking")
CORE_ALGOS_NAMES = ("agg_loss", "kl_penalty", "compute_policy_loss", "compute_policy_loss_vanilla",
                    "compute_policy_loss_gspo", "compute_grpo_outcome_advantage", "apply_kl_penalty")


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
        losses.update(vanilla=A.compute_policy_loss_vanilla, gspo=A.compute_policy_loss_gspo)
    estimators = getattr(ref_core_algos, "ADV_ESTIMATOR_REGISTRY", None)
    if estimators is not None:
        estimators["grpo"] = A.compute_grpo_outcome_advantage
    return undo
