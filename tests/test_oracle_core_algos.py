"""Pins the oracle's advantage / loss / KL functions (CPU only) against hand-computed cases, brute force and
the known answers the reference's docs hold."""

import math
from types import SimpleNamespace

import numpy as np
import pytest
import torch

from oracle import core_algos as OC

AGGS = ["token-mean", "seq-mean-token-sum", "seq-mean-token-mean", "seq-mean-token-sum-norm"]


def _cfg(lo=0.2, hi=0.2, c=3.0):
    return OC.LossConfig(0.2, lo, hi, c)


# ------------------------------------------------------------------ GRPO


def test_grpo_quickstart_extrema():
    """docs/start/quickstart.rst:137 logs advantages max 1.789 / min -0.730 for rewards in {0, 1}: 1-of-5 and
    2-of-5 successes under the unbiased std.  (The biased std would give 2.0 / -0.816.)"""
    ones = torch.ones(5, 4)
    r = torch.zeros(5, 4)
    r[0, 3] = 1
    a, ret = OC.compute_grpo_outcome_advantage(r, ones, np.zeros(5, dtype=np.int64))
    assert a is ret
    assert abs(a.max().item() - 1.789) < 5e-4 and abs(a.max().item() - 0.8 / (math.sqrt(0.2) + 1e-6)) < 1e-6
    r[1, 3] = 1
    a, _ = OC.compute_grpo_outcome_advantage(r, ones, np.zeros(5, dtype=np.int64))
    assert abs(a.min().item() + 0.730) < 5e-4 and abs(a.min().item() + 0.4 / (math.sqrt(0.3) + 1e-6)) < 1e-6


def test_grpo_bruteforce_and_invariants():
    g = torch.Generator().manual_seed(0)
    B, L = 24, 5
    uid = torch.tensor([3, 3, 3, 3, 10, 10, -5, 7, 7, 7, 7, 7, 7, 7, 7, 2 ** 40, 2 ** 40, 1, 1, 1, 9, 9, 9, 9])
    perm = torch.randperm(B, generator=g)
    uid = uid[perm]
    s = torch.randn(B, generator=g, dtype=torch.float64)
    rewards = torch.zeros(B, L, dtype=torch.float64)
    rewards[:, 2] = s
    mask = (torch.rand(B, L, generator=g) > 0.3).long()
    for norm in (True, False):
        a, _ = OC.compute_grpo_outcome_advantage(rewards, mask, uid.numpy(), norm_adv_by_std_in_grpo=norm)
        want = torch.tensor(OC.grpo_bruteforce(s, uid, norm=norm), dtype=torch.float64)
        assert torch.allclose(a, want[:, None] * mask, atol=1e-12)
    a, _ = OC.compute_grpo_outcome_advantage(rewards, torch.ones(B, L), uid.numpy())
    for u in uid.unique():
        rows = uid == u
        if rows.sum() > 1:
            assert abs(a[rows, 0].sum().item()) < 1e-9  # normalised scores of a group sum to zero
        else:
            assert abs(a[rows, 0].item() - s[rows].item() / (1 + 1e-6)) < 1e-12  # singleton: mean 0, std 1
    # all-equal group is exactly zero; the pair {0, 1} has unbiased std sqrt(1/2)
    r = torch.tensor([[2.0], [2.0], [2.0], [0.0], [1.0]])
    a, _ = OC.compute_grpo_outcome_advantage(r, torch.ones(5, 1), ["a1".replace("a", ""), "1", "1", "2", "2"])
    assert a[:3].abs().max() == 0 and abs(a[4].item() - 0.5 / (math.sqrt(0.5) + 1e-6)) < 1e-6


# ------------------------------------------------------------------ agg_loss


def test_agg_loss_closed_forms():
    v = torch.tensor([[1.0, 2.0, 3.0, 4.0], [10.0, 20.0, 30.0, 40.0]])
    m = torch.tensor([[1, 1, 1, 0], [1, 0, 0, 0]])
    assert abs(float(OC.agg_loss(v, m, "token-mean")) - (1 + 2 + 3 + 10) / 4) < 1e-6
    assert float(OC.agg_loss(v, m, "seq-mean-token-sum")) == (6 + 10) / 2
    assert float(OC.agg_loss(v, m, "seq-mean-token-mean")) == (2 + 10) / 2
    assert float(OC.agg_loss(v, m, "seq-mean-token-sum-norm")) == 16 / 4
    assert abs(float(OC.agg_loss(torch.full((3, 4), 2.5), torch.ones(3, 4), "token-mean")) - 2.5) < 1e-6
    assert math.isnan(float(OC.agg_loss(v, torch.tensor([[1, 1, 1, 0], [0, 0, 0, 0]]), "seq-mean-token-mean")))
    with pytest.raises(ValueError, match="Invalid loss_agg_mode"):
        OC.agg_loss(v, m, "sum")


# ------------------------------------------------------------------ policy losses


def test_vanilla_known_cases():
    cfg = _cfg(0.2, 0.28, 3.0)
    old = torch.zeros(1, 6, dtype=torch.float64)
    mask = torch.ones(1, 6, dtype=torch.int64)
    A = torch.tensor([[1.0, -1.0, 2.0, -2.0, 0.5, -0.5]], dtype=torch.float64)
    pg, cf, kl, cfl = OC.compute_policy_loss_vanilla(old, old.clone(), A, mask, "token-mean", cfg)
    assert abs(float(pg.detach()) + float(A.mean())) < 1e-9 and float(cf) == 0 and float(kl) == 0 and float(cfl) == 0
    lp = torch.log(torch.tensor([[1.5, 0.5, 4.0, 1.1, 1.5, 4.0]], dtype=torch.float64)).requires_grad_(True)
    A2 = torch.tensor([[2.0, -1.0, -1.0, 1.0, -1.0, 1.0]], dtype=torch.float64)
    pg, cf, kl, cfl = OC.compute_policy_loss_vanilla(old, lp, A2, mask, "seq-mean-token-sum", cfg)
    assert abs(float(pg.detach()) - (-2.56 + 0.8 + 3.0 - 1.1 + 1.5 - 1.28)) < 1e-9
    assert abs(float(cf) - 0.5) < 1e-7 and abs(float(cfl) - 1 / 6) < 1e-7
    assert abs(float(kl) + float(lp.detach().mean())) < 1e-7
    pg.backward()
    assert torch.allclose(lp.grad, torch.tensor([[0, 0, 0, -1.1, 1.5, 0]], dtype=torch.float64), atol=1e-9)
    # the +-20 clamp of the log-ratio: value saturates at exp(20), gradient is cut
    lp2 = torch.tensor([[25.0]], dtype=torch.float64, requires_grad=True)
    pg, *_ = OC.compute_policy_loss_vanilla(torch.zeros(1, 1, dtype=torch.float64), lp2, torch.tensor([[-1e-9]], dtype=torch.float64),
                                            torch.ones(1, 1), "token-mean", _cfg(c=1e12))
    assert abs(float(pg.detach()) - 1e-9 * math.exp(20)) < 1e-6
    pg.backward()
    assert float(lp2.grad) == 0.0
    with pytest.raises(AssertionError):
        OC.compute_policy_loss_vanilla(old, old, A, mask, "token-mean", _cfg(c=1.0))


@pytest.mark.parametrize("mode", AGGS)
@pytest.mark.parametrize("mode_fn", ["vanilla", "gspo"])
def test_closed_form_gradient_vs_autograd(mode, mode_fn):
    g = torch.Generator().manual_seed(3)
    B, L = 5, 40
    lp = (torch.randn(B, L, generator=g, dtype=torch.float64) - 1).requires_grad_(True)
    scale = 0.3 if mode_fn == "vanilla" else 0.01
    old = lp.detach() + scale * torch.randn(B, L, generator=g, dtype=torch.float64)
    A = torch.randn(B, 1, generator=g, dtype=torch.float64).expand(B, L)
    mask = (torch.arange(L)[None] < torch.randint(1, L + 1, (B, 1), generator=g)).double()
    isw = torch.rand(B, L, generator=g, dtype=torch.float64) + 0.5
    cfg = _cfg(0.2, 0.28, 3.0) if mode_fn == "vanilla" else _cfg(3e-3, 4e-3)
    fn = OC.compute_policy_loss_vanilla if mode_fn == "vanilla" else OC.compute_policy_loss_gspo
    pg, *_ = fn(old, lp, A, mask, mode, cfg, isw)
    pg.backward()
    cf = OC.policy_loss_grad_closed_form(old, lp.detach(), A, mask, mode, cfg, isw, mode=mode_fn)
    assert torch.allclose(cf, lp.grad, atol=1e-12)


def test_gspo_reduces_to_ppo_for_length_one_and_known_case():
    g = torch.Generator().manual_seed(4)
    lp = torch.randn(9, 1, generator=g, dtype=torch.float64)
    old = lp + 0.2 * torch.randn(9, 1, generator=g, dtype=torch.float64)
    A = torch.randn(9, 1, generator=g, dtype=torch.float64)
    m = torch.ones(9, 1)
    a = OC.compute_policy_loss_gspo(old, lp, A, m, config=_cfg())
    b = OC.compute_policy_loss_vanilla(old, lp, A, m, "seq-mean-token-mean", _cfg(c=1e12))
    assert abs(float(a[0]) - float(b[0])) < 1e-12 and float(a[1]) == float(b[1]) and float(a[3]) == 0
    # sequence ratio = exp(masked mean of the token log-ratios); value is shared by the row's tokens
    lp = torch.tensor([[0.1, 0.3, 9.0]], dtype=torch.float64)
    old = torch.zeros(1, 3, dtype=torch.float64)
    m = torch.tensor([[1.0, 1.0, 0.0]], dtype=torch.float64)
    A = torch.tensor([[2.0, 2.0, 2.0]], dtype=torch.float64)
    pg, cf, kl, _ = OC.compute_policy_loss_gspo(old, lp, A, m, "token-mean", _cfg(0.1, 0.1))
    rho = math.exp(0.2)
    assert abs(float(pg.detach()) - (-2 * 1.1)) < 1e-9 and rho > 1.1 and abs(float(cf) - 1.0) < 1e-7
    assert abs(float(kl) + 0.2) < 1e-7


# ------------------------------------------------------------------ KL


def test_kl_estimators_closed_forms():
    lp = torch.tensor([0.0, -1.0, -2.0, 0.5], dtype=torch.float64)
    ref = torch.tensor([0.0, -1.5, -1.0, 30.0], dtype=torch.float64)
    x = lp - ref
    assert torch.equal(OC.kl_penalty(lp, ref, "kl"), x) and torch.equal(OC.kl_penalty(lp, ref, "k1"), x)
    assert torch.equal(OC.kl_penalty(lp, ref, "abs"), x.abs())
    assert torch.equal(OC.kl_penalty(lp, ref, "mse"), 0.5 * x * x) and torch.equal(OC.kl_penalty(lp, ref, "k2"), 0.5 * x * x)
    k3 = OC.kl_penalty(lp, ref, "low_var_kl")
    assert float(k3[0]) == 0 and (k3 >= 0).all() and float(k3[3]) == 10.0  # clamp at 10
    assert abs(float(k3[1]) - (math.exp(-0.5) + 0.5 - 1)) < 1e-12 and abs(float(k3[2]) - (math.exp(1.0) - 1.0 - 1)) < 1e-12
    assert torch.equal(OC.kl_penalty(lp, ref, "k2"), OC.kl_penalty(ref, lp, "k2"))
    for bad in ("full", "k3+", "whatever"):
        with pytest.raises(NotImplementedError):
            OC.kl_penalty(lp, ref, bad)
    # gradient of k3 is -(e^k - 1) inside both clamps and zero outside
    lpg = lp.clone().requires_grad_(True)
    OC.kl_penalty(lpg, ref, "k3").sum().backward()
    assert abs(float(lpg.grad[1]) + (math.exp(-0.5) - 1)) < 1e-12 and float(lpg.grad[3]) == 0.0


def test_kl_in_reward_and_controller():
    ctrl = OC.AdaptiveKLController(0.1, 0.05, 100)
    ctrl.update(current_kl=0.1, n_steps=50)  # error clipped to +0.2 -> x (1 + 0.2 * 50 / 100)
    assert abs(ctrl.value - 0.11) < 1e-12
    ctrl.update(current_kl=0.0475, n_steps=100)  # error -0.05 -> x 0.95
    assert abs(ctrl.value - 0.11 * 0.95) < 1e-12
    data = {"token_level_scores": torch.tensor([[0.0, 1.0], [0.0, 1.0]]), "old_log_probs": torch.tensor([[-1.0, -1.0], [-2.0, -2.0]]),
            "ref_log_prob": torch.tensor([[-1.5, -1.0], [-1.0, 5.0]]), "response_mask": torch.tensor([[1, 1], [1, 0]])}
    fixed = OC.get_kl_controller(SimpleNamespace(type="fixed", kl_coef=0.5))
    data, metrics = OC.apply_kl_penalty(data, fixed, "kl")
    assert torch.allclose(data["token_level_rewards"], torch.tensor([[-0.25, 1.0], [0.5, 1.0]]))
    assert abs(metrics["actor/reward_kl_penalty"] - ((0.5 + 0) / 2 + (-1.0) / 1) / 2) < 1e-6
    assert metrics["actor/reward_kl_penalty_coeff"] == 0.5 and fixed.value == 0.5
    assert torch.equal(OC.compute_rewards(torch.ones(2), torch.tensor([1.0, 2.0]), torch.tensor([0.0, 4.0]), 0.5), torch.tensor([0.5, 2.0]))
