"""Pins of the oracle's covariance losses (Clip-Cov, KL-Cov) and of the CPGD outcome advantage on the CPU: worked
cases written out with ``math``, brute-force selection, closed-form gradients against autograd, and how the random
draw of Clip-Cov consumes the global generator.  Reference: ``siirl/dag_worker/core_algos.py:461-517,898-1071``."""
import math
from types import SimpleNamespace

import pytest
import torch

from oracle import core_algos as O


def _cfg(**policy_loss):
    return SimpleNamespace(clip_ratio=0.2, clip_ratio_low=0.2, clip_ratio_high=0.28, clip_ratio_c=3.0,
                           policy_loss=O.CovLossConfig(**policy_loss))


# ------------------------------------------------------------------------------------------ KL-Cov


def test_kl_cov_worked_case():
    A = torch.tensor([[1.0, -1.0, 2.0, 0.0]], dtype=torch.float64)
    lp = torch.tensor([[-1.0, -2.0, -0.5, -3.0]], dtype=torch.float64)
    d = [0.1, -0.2, 0.3, 0.0]
    old = lp - torch.tensor([d], dtype=torch.float64)
    m = torch.ones(1, 4, dtype=torch.float64)
    # means 0.5 and -1.625: cov = [0.3125, 0.5625, 1.6875, 0.6875]; one token in four is taken: index 2
    chosen, cov = O.kl_cov_selection(lp, A, m, 0.25)
    assert chosen.tolist() == [2]
    assert cov.tolist() == pytest.approx([0.3125, 0.5625, 1.6875, 0.6875], abs=1e-15)
    coef = 0.7
    loss, z1, kl, z2 = O.compute_policy_loss_kl_cov(old, lp, A, m, "token-mean", _cfg(kl_cov_ratio=0.25, ppo_kl_coef=coef))
    toks = [-1.0 * math.exp(0.1), 1.0 * math.exp(-0.2), -2.0 * math.exp(0.3) + coef * 0.3, 0.0]
    assert float(loss) == pytest.approx(sum(toks) / (4 + 1e-8), rel=1e-14)
    assert float(kl) == pytest.approx((0.1 + 0.2 + 0.3) / (4 + 1e-8), rel=1e-14)
    assert float(z1) == 0.0 and float(z2) == 0.0


def test_kl_cov_cut_moves_only_among_near_ties_when_the_means_are_rounded_differently():
    """The reference centres with float32 ``.mean()`` (``core_algos.py:1055``); the device path sums the means in
    double and rounds once.  The two means can differ in the last bits, so can the covariances, and with them the
    membership exactly at the cut of ``topk`` -- and only there: every token chosen by one and not by the other
    has a covariance within a few float32 spacings of the k-th value."""
    g = torch.Generator().manual_seed(11)
    for n, ratio in ((4096, 0.01), (50000, 0.002), (200000, 0.0002)):
        a = torch.randn(n, generator=g)
        lp = -1.5 + torch.randn(n, generator=g)
        k = max(1, int(n * ratio))
        cov_ref = (a - a.mean()) * (lp - lp.mean())                                   # the reference's arithmetic
        ma, ml = a.double().mean().float(), lp.double().mean().float()                 # double sum, one rounding
        cov_dev = (a - ma) * (lp - ml)
        top_ref = set(torch.topk(cov_ref, k).indices.tolist())
        top_dev = set(torch.topk(cov_dev, k).indices.tolist())
        cut = torch.topk(cov_ref, k).values[-1]
        # a changed mean moves every cov by at most delta = |mean shift| * |other factor| (+ rounding); the cut moves by
        # at most delta as well, so a token that changes sides lies within 2 delta of it
        eps = float(torch.finfo(torch.float32).eps)
        delta = (abs(float(a.mean() - ma)) * float((lp - ml).abs().max())
                 + abs(float(lp.mean() - ml)) * float((a - ma).abs().max()) + 4 * eps * float(cov_ref.abs().max()))
        slack = 2 * delta
        for i in top_ref ^ top_dev:
            assert abs(float(cov_ref[i]) - float(cut)) <= slack, (n, i, float(cov_ref[i]), float(cut), slack)
        assert len(top_ref ^ top_dev) <= max(2, k // 50)


def test_kl_cov_ignores_masked_tokens_and_counts():
    g = torch.Generator().manual_seed(3)
    B, L = 7, 50
    A, lp = torch.randn(B, L, generator=g, dtype=torch.float64), -torch.rand(B, L, generator=g, dtype=torch.float64) * 3
    m = (torch.rand(B, L, generator=g) < 0.6).to(torch.float64)
    A[2, 5], lp[2, 5], m[2, 5] = 1e3, 1e3, 0.0  # the largest product by far, outside the mask
    n = int(m.sum())
    for ratio, k in ((0.0002, 1), (0.05, int(n * 0.05)), (1.0, n)):
        chosen, _ = O.kl_cov_selection(lp, A, m, ratio)
        assert len(chosen) == k and 2 * L + 5 not in chosen.tolist()
        # brute force: sort the valid tokens' products
        valid = [i for i in range(B * L) if m.reshape(-1)[i] > 0]
        ma = sum(float(A.reshape(-1)[i]) for i in valid) / n
        ml = sum(float(lp.reshape(-1)[i]) for i in valid) / n
        prod = sorted(((float(A.reshape(-1)[i]) - ma) * (float(lp.reshape(-1)[i]) - ml), i) for i in valid)
        assert sorted(chosen.tolist()) == sorted(i for _, i in prod[len(prod) - k:])
    empty, cov = O.kl_cov_selection(lp, A, torch.zeros(B, L, dtype=torch.float64), 0.1)
    assert len(empty) == 0 and cov is None


@pytest.mark.parametrize("agg", O.AGG_MODES)
def test_kl_cov_gradient_closed_form(agg):
    g = torch.Generator().manual_seed(11)
    B, L = 5, 24
    A = torch.randn(B, L, generator=g, dtype=torch.float64)
    old = -torch.rand(B, L, generator=g, dtype=torch.float64) * 2
    lp = (old + 0.2 * torch.randn(B, L, generator=g, dtype=torch.float64)).requires_grad_(True)
    m = (torch.rand(B, L, generator=g) < 0.8).to(torch.float64)
    m[:, 0] = 1
    w = torch.rand(B, L, generator=g, dtype=torch.float64) + 0.5
    coef, ratio = 1.3, 0.1
    loss, _, _, _ = O.compute_policy_loss_kl_cov(old, lp, A, m, agg, _cfg(kl_cov_ratio=ratio, ppo_kl_coef=coef), w)
    (grad,) = torch.autograd.grad(loss, lp)
    chosen, _ = O.kl_cov_selection(lp.detach(), A, m, ratio)
    sel = torch.zeros(B * L, dtype=torch.float64)
    sel[chosen] = 1
    sel = sel.reshape(B, L)
    d = (lp - old).detach()
    dtok = (-A * torch.exp(d) + sel * coef * torch.sign(d)) * w
    n_row = m.sum(-1, keepdim=True)
    aggw = {"token-mean": m / (m.sum() + 1e-8), "seq-mean-token-sum": m / B, "seq-mean-token-mean": m / n_row / B,
            "seq-mean-token-sum-norm": m / L}[agg]
    assert torch.allclose(grad, dtok * aggw, rtol=1e-12, atol=1e-15)


# ------------------------------------------------------------------------------------------ Clip-Cov


def _clip_case():
    # ratio = exp(d); eps 0.2 / 0.28.  Token 0: A > 0, ratio 1.5 > 1.28 -> the PPO clip bites (l2 > l1): excluded.
    # Token 3 is masked.  The others are candidates when lb < cov < ub.
    A = torch.tensor([[2.0, 2.0, -1.0, 5.0, 1.0, -3.0]], dtype=torch.float64)
    lp = torch.tensor([[-0.5, -0.2, -2.0, -0.1, -1.0, -2.5]], dtype=torch.float64)
    d = torch.tensor([[math.log(1.5), 0.05, -0.05, 0.0, 0.1, 0.02]], dtype=torch.float64)
    m = torch.tensor([[1.0, 1.0, 1.0, 0.0, 1.0, 1.0]], dtype=torch.float64)
    return lp - d, lp, A, m, d


def test_clip_cov_candidates_worked_case():
    old, lp, A, m, d = _clip_case()
    cov, cand = O.clip_cov_candidates(old, lp, A, m, 0.2, 0.28, 0.5, 5.0)
    ma = (2 + 2 - 1 + 1 - 3) / (5 + 1e-8)
    ml = (-0.5 - 0.2 - 2.0 - 1.0 - 2.5) / (5 + 1e-8)
    want = [(float(A[0, t]) - ma) * (float(lp[0, t]) - ml) for t in range(6)]
    assert math.isinf(float(cov[0, 0])) and float(cov[0, 0]) < 0  # clipped by the PPO bound
    assert math.isinf(float(cov[0, 3])) and float(cov[0, 3]) < 0  # masked
    for t in (1, 2, 4, 5):
        assert float(cov[0, t]) == pytest.approx(want[t], rel=1e-14)
    # want[1] = 1.8 * 1.04 = 1.872, want[2] = -1.2 * -0.76 = 0.912, want[4] = 0.8 * 0.24 = 0.192, want[5] = -3.2 * -1.26 = 4.032
    assert cand.tolist() == [[0, 1], [0, 2], [0, 5]]
    assert O.clip_cov_candidates(old, lp, A, m, 0.2, 0.28, 1.0, 4.0)[1].tolist() == [[0, 1]]


def test_clip_cov_loss_after_the_draw():
    old, lp, A, m, d = _clip_case()
    w = torch.tensor([[1.0, 0.5, 2.0, 1.0, 1.0, 1.5]], dtype=torch.float64)
    dropped = torch.tensor([[0, 2]])
    loss, frac, kl, z = O.compute_policy_loss_clip_cov(old, lp, A, m, "token-mean", _cfg(), w, dropped=dropped)
    r = [math.exp(float(x)) for x in d[0]]
    clip = lambda x: min(max(x, 0.8), 1.28)  # noqa: E731
    tok = [max(-float(A[0, t]) * r[t], -float(A[0, t]) * clip(r[t])) for t in range(6)]
    tok[2] = 0.0
    total = sum(tok[t] * float(w[0, t]) for t in (0, 1, 2, 4, 5))
    assert float(loss) == pytest.approx(total / (5 + 1e-8), rel=1e-14)
    assert float(frac) == pytest.approx(1 / (5 + 1e-8), rel=1e-14)
    assert float(kl) == pytest.approx(-sum(float(d[0, t]) for t in (0, 1, 2, 4, 5)) / (5 + 1e-8), rel=1e-13)
    assert float(z) == 0.0
    # gradient: the dropped token and the token whose ratio sits beyond the bound on the clipped side get none
    lpg = lp.clone().requires_grad_(True)
    loss, *_ = O.compute_policy_loss_clip_cov(old, lpg, A, m, "token-mean", _cfg(), w, dropped=dropped)
    (grad,) = torch.autograd.grad(loss, lpg)
    assert float(grad[0, 2]) == 0.0 and float(grad[0, 0]) == 0.0 and float(grad[0, 3]) == 0.0
    assert float(grad[0, 1]) == pytest.approx(-2.0 * r[1] * 0.5 / (5 + 1e-8), rel=1e-14)


def test_clip_cov_draw_uses_one_host_randperm():
    g = torch.Generator().manual_seed(5)
    B, L = 6, 64
    A = torch.randn(B, L, generator=g, dtype=torch.float64) * 2
    old = -torch.rand(B, L, generator=g, dtype=torch.float64) * 3
    lp = old + 0.05 * torch.randn(B, L, generator=g, dtype=torch.float64)
    m = (torch.rand(B, L, generator=g) < 0.7).to(torch.float64)
    cfg = _cfg(clip_cov_ratio=0.02, clip_cov_lb=0.2, clip_cov_ub=4.0)
    _, cand = O.clip_cov_candidates(old, lp, A, m, 0.2, 0.28, 0.2, 4.0)
    clip_num = max(int(0.02 * float(m.sum())), 1)
    assert len(cand) > clip_num >= 2
    torch.manual_seed(77)
    loss, frac, _, _ = O.compute_policy_loss_clip_cov(old, lp, A, m, "token-mean", cfg)
    after = torch.rand(3)
    torch.manual_seed(77)
    perm = torch.randperm(len(cand))
    assert torch.equal(after, torch.rand(3))  # exactly one randperm(len(candidates)) was drawn, nothing else
    same, frac2, _, _ = O.compute_policy_loss_clip_cov(old, lp, A, m, "token-mean", cfg, dropped=cand[perm[:clip_num]])
    assert float(loss) == float(same) and float(frac) == float(frac2)
    assert float(frac) == pytest.approx(clip_num / (float(m.sum()) + 1e-8), rel=1e-12)
    # fewer candidates than the quota: all of them go, whatever the generator says
    cfg_all = _cfg(clip_cov_ratio=1.0, clip_cov_lb=0.2, clip_cov_ub=4.0)
    a, fa, _, _ = O.compute_policy_loss_clip_cov(old, lp, A, m, "token-mean", cfg_all)
    b, fb, _, _ = O.compute_policy_loss_clip_cov(old, lp, A, m, "token-mean", cfg_all, dropped=cand)
    assert float(a) == float(b) and float(fa) == pytest.approx(len(cand) / (float(m.sum()) + 1e-8), rel=1e-12)


def test_clip_cov_without_candidates_is_the_plain_clip_loss():
    old, lp, A, m, _ = _clip_case()
    cfg = _cfg(clip_cov_lb=100.0, clip_cov_ub=200.0)
    loss, frac, kl, _ = O.compute_policy_loss_clip_cov(old, lp, A, m, "seq-mean-token-sum", cfg)
    legacy = SimpleNamespace(clip_ratio=0.2, clip_ratio_low=0.2, clip_ratio_high=0.28, clip_ratio_c=1e30)
    van, _, vkl, _ = O.compute_policy_loss_vanilla(old, lp, A, m, "seq-mean-token-sum", legacy)
    assert float(frac) == 0.0 and float(loss) == pytest.approx(float(van), rel=1e-14)
    assert float(kl) == pytest.approx(float(vkl), rel=1e-14)


# ------------------------------------------------------------------------------------------ CPGD outcome advantage


def test_cpgd_advantage_modes():
    g = torch.Generator().manual_seed(2)
    B, L = 12, 9
    mask = (torch.rand(B, L, generator=g) < 0.8).to(torch.float64)
    rewards = torch.zeros(B, L, dtype=torch.float64)
    rewards[torch.arange(B), torch.randint(0, L, (B,), generator=g)] = torch.randn(B, generator=g, dtype=torch.float64)
    uid = torch.tensor([0, 0, 0, 1, 1, 2, 3, 3, 3, 3, 4, 4])
    a_std, _ = O.compute_cpgd_outcome_advantage(rewards, mask, uid, weight_factor_in_cpgd="STD_weight")
    a_grpo, _ = O.compute_grpo_outcome_advantage(rewards, mask, uid, norm_adv_by_std_in_grpo=True)
    assert torch.allclose(a_std, a_grpo, rtol=1e-14, atol=0)
    a_naive, _ = O.compute_cpgd_outcome_advantage(rewards, mask, uid, weight_factor_in_cpgd="naive")
    a_plain, _ = O.compute_grpo_outcome_advantage(rewards, mask, uid, norm_adv_by_std_in_grpo=False)
    assert torch.allclose(a_naive, a_plain, rtol=1e-14, atol=0)
    with pytest.raises(NotImplementedError):
        O.compute_cpgd_outcome_advantage(rewards, mask, uid, weight_factor_in_cpgd="other")


def test_cpgd_advantage_clip_filter_worked_case():
    ones = torch.ones(4, 1, dtype=torch.float64)
    # groups {1, 3} (std sqrt 2) and {2, 2} (std 0): one live group of two -> factor min(4 / 1, 3) = 3
    adv, ret = O.compute_cpgd_outcome_advantage(torch.tensor([[1.0], [3.0], [2.0], [2.0]], dtype=torch.float64), ones,
                                                [7, 7, 9, 9], weight_factor_in_cpgd="clip_filter_like_weight")
    assert adv.reshape(-1).tolist() == [-3.0, 3.0, 0.0, 0.0] and ret is adv
    # three live groups (a singleton counts: its std is set to 1) of six rows: factor 2
    adv, _ = O.compute_cpgd_outcome_advantage(
        torch.tensor([[1.0], [3.0], [2.0], [5.0], [0.0], [4.0]], dtype=torch.float64), torch.ones(6, 1, dtype=torch.float64),
        ["a", "a", "b", "c", "c", "c"], weight_factor_in_cpgd="clip_filter_like_weight")
    assert adv.reshape(-1).tolist() == pytest.approx([-2.0, 2.0, 4.0, 4.0, -6.0, 2.0], rel=1e-15)
