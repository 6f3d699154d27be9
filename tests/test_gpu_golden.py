"""GPU parity against the committed fixtures (tests/golden/oracle_small.npz): the HIP path must reproduce numbers
that were fixed when the fixtures were written, to the tolerances of the task statement."""

import os
from types import SimpleNamespace

import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

G = np.load(os.path.join(os.path.dirname(__file__), "golden", "oracle_small.npz"))


def _bf16(bits):
    return torch.from_numpy(bits.copy()).view(torch.bfloat16)


def test_logprob_entropy_vs_fixtures(dev):
    import siirl_amd.torch_functional as SF

    x, y = _bf16(G["lpe_logits_bf16_bits"]), torch.from_numpy(G["lpe_labels"])
    g_lp, g_h = torch.from_numpy(G["lpe_g_lp"]), torch.from_numpy(G["lpe_g_h"])
    for name, temp in (("t1", 1.0), ("t07", 0.7)):
        xd = x.to(dev).requires_grad_(True)
        lp, ent = SF.logprobs_and_entropy_from_logits(xd, y.to(dev), temperature=temp)
        assert np.abs(lp.detach().cpu().numpy() - G[f"lpe_{name}_logprob"]).max() < 1e-3
        assert np.abs(ent.detach().cpu().numpy() - G[f"lpe_{name}_entropy"]).max() < 1e-3
        (dx,) = torch.autograd.grad([lp, ent], [xd], [g_lp.to(dev), g_h.to(dev)])
        want = torch.from_numpy(G[f"lpe_{name}_dlogits"])
        err = (dx.cpu().double() - want).abs()
        assert (err <= 2.0 ** -7 * want.abs() + 1e-7).all()  # one bf16 ulp


def test_losses_vs_fixtures(dev):
    import siirl_amd.core_algos as CA

    lp, old, ref, adv = (torch.from_numpy(G[f"loss_{k}"]).to(dev) for k in ("lp", "old", "ref", "adv"))
    mask = torch.from_numpy(G["loss_mask"]).to(dev)
    cfg = SimpleNamespace(clip_ratio=0.2, clip_ratio_low=0.2, clip_ratio_high=0.28, clip_ratio_c=3.0)
    for mode in CA.AGG_MODES:
        tag = mode.replace("-", "_")
        x = lp.clone().requires_grad_(True)
        res = CA.compute_policy_loss_vanilla(old, x, adv, mask, mode, cfg)
        assert np.abs(np.array([float(r) for r in res]) - G[f"vanilla_{tag}"]).max() < 1e-3
        res[0].backward()
        assert np.abs(x.grad.cpu().numpy() - G[f"vanilla_{tag}_grad"]).max() < 1e-6
        assert abs(float(CA.agg_loss(lp, mask, mode)) - float(G[f"agg_{tag}"])) < 1e-3
    x = lp.clone().requires_grad_(True)
    gcfg = SimpleNamespace(clip_ratio=0.2, clip_ratio_low=3e-3, clip_ratio_high=4e-3, clip_ratio_c=3.0)
    res = CA.compute_policy_loss_gspo(torch.from_numpy(G["loss_old_gspo"]).to(dev), x, adv, mask, "token-mean", gcfg)
    assert np.abs(np.array([float(r) for r in res]) - G["gspo"]).max() < 1e-3
    res[0].backward()
    assert np.abs(x.grad.cpu().numpy() - G["gspo_grad"]).max() < 1e-6
    for kind in ("kl", "abs", "mse", "low_var_kl"):
        assert np.abs(CA.kl_penalty(lp, ref, kind).cpu().numpy() - G[f"kl_{kind}"]).max() < 1e-3


def test_groups_vs_fixtures(dev):
    import siirl_amd.core_algos as CA
    import siirl_amd.dapo_filter as DF

    rewards, mask, uid = torch.from_numpy(G["grpo_rewards"]), torch.from_numpy(G["grpo_mask"]), G["grpo_uid"]
    for norm, key in ((True, "grpo_adv"), (False, "grpo_adv_nonorm")):
        adv, _ = CA.compute_grpo_outcome_advantage(rewards.to(dev), mask.to(dev), uid, norm_adv_by_std_in_grpo=norm)
        want = G[key]
        assert (np.abs(adv.cpu().numpy() - want) <= 1e-5 * np.abs(want) + 1e-7).all()
    keep = DF.group_keep_mask(G["grpo_rewards"][:, 5], uid, device=dev)
    assert np.array_equal(keep.cpu().numpy(), G["dapo_keep"])
