"""The start-up patch of ``siirl_amd.integration``, applied to stand-ins for the reference's two modules (CPU only):
the actor-side functions and all seven policy-loss registry entries are replaced, the masked reductions that the
reference also calls on host tensors (compute_gae_advantage_return -> masked_whiten -> masked_mean) are left alone."""
import types

import torch


def _stub_modules():
    F = types.ModuleType("ref_torch_functional")
    A = types.ModuleType("ref_core_algos")

    def masked_mean(values, mask, axis=None):  # the reference's, torch_functional.py:154-168
        return (values * mask).sum(axis=axis) / (mask.sum(axis=axis) + 1e-8)

    def masked_whiten(values, mask):  # resolves the module global, as the reference's does
        return values - F.masked_mean(values, mask)

    for name in ("logprobs_from_logits", "entropy_from_logits", "entropy_from_logits_with_chunking", "masked_sum"):
        setattr(F, name, lambda *a, **k: "reference")
    F.masked_mean, F.masked_whiten = masked_mean, masked_whiten
    modes = ("vanilla", "gspo", "cpgd", "gpg", "clip_cov", "kl_cov", "geo_mean")
    for name in ("agg_loss", "kl_penalty", "compute_policy_loss", "compute_grpo_outcome_advantage", "apply_kl_penalty",
                 "compute_marft_gae_advantage_return", "compute_value_loss", *(f"compute_policy_loss_{m}" for m in modes)):
        setattr(A, name, lambda *a, **k: "reference")
    A.POLICY_LOSS_REGISTRY = {m: getattr(A, f"compute_policy_loss_{m}") for m in modes}
    A.POLICY_LOSS_REGISTRY["users_own"] = A.compute_value_loss
    A.ADV_ESTIMATOR_REGISTRY = {"grpo": A.compute_grpo_outcome_advantage, "gae": object()}
    return F, A


def test_patch_replaces_the_actor_side_and_leaves_host_side_reductions():
    import siirl_amd.core_algos as CA
    import siirl_amd.torch_functional as SF
    from siirl_amd.integration import CORE_ALGOS_NAMES, TORCH_FUNCTIONAL_NAMES, patch_reference

    F, A = _stub_modules()
    gae_before, own_before, masked_sum_before = A.ADV_ESTIMATOR_REGISTRY["gae"], A.POLICY_LOSS_REGISTRY["users_own"], F.masked_sum
    undo = patch_reference(F, A)
    for name in TORCH_FUNCTIONAL_NAMES:
        assert getattr(F, name) is getattr(SF, name)
    for name in CORE_ALGOS_NAMES:
        assert getattr(A, name) is getattr(CA, name)
    for mode in ("vanilla", "gspo", "cpgd", "gpg", "clip_cov", "kl_cov", "geo_mean"):
        assert A.POLICY_LOSS_REGISTRY[mode] is CA.POLICY_LOSS_REGISTRY[mode] is getattr(CA, f"compute_policy_loss_{mode}")
    assert A.POLICY_LOSS_REGISTRY["users_own"] is own_before and A.compute_value_loss is own_before
    assert A.ADV_ESTIMATOR_REGISTRY["grpo"] is CA.compute_grpo_outcome_advantage
    assert A.ADV_ESTIMATOR_REGISTRY["gae"] is gae_before
    assert len(undo) == len(TORCH_FUNCTIONAL_NAMES) + len(CORE_ALGOS_NAMES) + 1 and undo["rebound"] == []
    # the reference's host-side whitening still resolves the reference's own masked_mean and runs on CPU tensors
    assert F.masked_sum is masked_sum_before
    v, m = torch.tensor([[1.0, 2.0, 3.0]]), torch.tensor([[1.0, 1.0, 0.0]])
    assert torch.allclose(F.masked_whiten(v, m), v - 1.5)



def test_patch_reaches_consumers_that_imported_the_names_before_it():
    """``from module import name`` binds by value (the reference's dp_actor.py:32,39, megatron_actor.py:48,
    dagworker.py:45-48): a consumer imported before the patch must be redirected as well, whether it is passed in or
    found in ``sys.modules`` under one of the reference's module names; ``undo_patch`` puts everything back."""
    import sys

    import siirl_amd.core_algos as CA
    import siirl_amd.torch_functional as SF
    from siirl_amd.integration import CONSUMER_MODULES, patch_reference, undo_patch

    F, A = _stub_modules()
    # a stand-in actor module that did `from core_algos import agg_loss, kl_penalty` and
    # `from torch_functional import logprobs_from_logits` before the patch, and also `import torch_functional as F`
    actor = types.ModuleType("standin_dp_actor")
    actor.agg_loss, actor.kl_penalty, actor.compute_policy_loss = A.agg_loss, A.kl_penalty, A.compute_policy_loss
    actor.logprobs_from_logits = F.logprobs_from_logits
    actor.renamed = A.apply_kl_penalty      # `from ... import apply_kl_penalty as renamed`
    actor.F = F
    actor.own_helper = lambda: "own"
    actor.masked_mean = F.masked_mean       # not replaced: must stay
    worker = types.ModuleType(CONSUMER_MODULES[-1])
    worker.apply_kl_penalty = A.apply_kl_penalty
    originals = {"agg_loss": A.agg_loss, "lp": F.logprobs_from_logits, "akl": A.apply_kl_penalty}
    sys.modules[CONSUMER_MODULES[-1]] = worker
    try:
        undo = patch_reference(F, A, consumers=[actor])
        assert actor.agg_loss is CA.agg_loss and actor.kl_penalty is CA.kl_penalty
        assert actor.compute_policy_loss is CA.compute_policy_loss
        assert actor.logprobs_from_logits is SF.logprobs_from_logits
        assert actor.renamed is CA.apply_kl_penalty
        assert actor.F.entropy_from_logits is SF.entropy_from_logits   # attribute-style calls follow the module
        assert actor.own_helper() == "own" and actor.masked_mean is F.masked_mean
        assert worker.apply_kl_penalty is CA.apply_kl_penalty          # found through sys.modules
        names = {(m.__name__, a) for m, a, _ in undo["rebound"]}
        assert ("standin_dp_actor", "agg_loss") in names and (CONSUMER_MODULES[-1], "apply_kl_penalty") in names
        assert len(undo["rebound"]) == 6
        undo_patch(F, A, undo)
        assert actor.agg_loss is originals["agg_loss"] and A.agg_loss is originals["agg_loss"]
        assert actor.logprobs_from_logits is originals["lp"] and F.logprobs_from_logits is originals["lp"]
        assert worker.apply_kl_penalty is originals["akl"] and actor.renamed is originals["akl"]
        assert A.POLICY_LOSS_REGISTRY["vanilla"] is A.compute_policy_loss_vanilla
        assert A.ADV_ESTIMATOR_REGISTRY["grpo"] is A.compute_grpo_outcome_advantage
    finally:
        del sys.modules[CONSUMER_MODULES[-1]]
