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
    assert len(undo) == len(TORCH_FUNCTIONAL_NAMES) + len(CORE_ALGOS_NAMES)
    # the reference's host-side whitening still resolves the reference's own masked_mean and runs on CPU tensors
    assert F.masked_sum is masked_sum_before
    v, m = torch.tensor([[1.0, 2.0, 3.0]]), torch.tensor([[1.0, 1.0, 0.0]])
    assert torch.allclose(F.masked_whiten(v, m), v - 1.5)

