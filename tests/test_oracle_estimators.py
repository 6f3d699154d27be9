"""Pins the oracle's GAE / whitening / value loss / CPGD / GPG / GMPO restatements (CPU only).

Each check is a closed form, a brute force or a hand-computed case chosen so that a dropped term, a wrong
sign or a shifted index fails it; none re-types the oracle's own formula."""
import math

import numpy as np
import pytest
import torch

from oracle import core_algos as O
from oracle import torch_functional as OF


def _rand(B, L, seed, dtype=torch.float64):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(B, L, generator=g, dtype=dtype), torch.randn(B, L, generator=g, dtype=dtype))


# ------------------------------------------------------------------------------------------------ GAE


def test_gae_gamma1_lam1_is_reward_to_go_minus_value():
    r, v = _rand(3, 17, 0)
    m = torch.ones(3, 17, dtype=torch.int64)
    adv, ret = O.gae_unwhitened(r, v, m, 1.0, 1.0)
    rtg = torch.flip(torch.cumsum(torch.flip(r, [1]), 1), [1])
    assert torch.allclose(ret, rtg, atol=1e-12)
    assert torch.allclose(adv, rtg - v, atol=1e-12)


def test_gae_lam0_is_td_error():
    r, v = _rand(2, 9, 1)
    m = torch.ones(2, 9, dtype=torch.int64)
    gamma = 0.9
    adv, _ = O.gae_unwhitened(r, v, m, gamma, 0.0)
    vnext = torch.cat([v[:, 1:], torch.zeros(2, 1, dtype=v.dtype)], 1)
    assert torch.allclose(adv, r + gamma * vnext - v, atol=1e-12)


def test_gae_general_matches_double_sum():
    r, v = _rand(2, 11, 2)
    m = torch.ones(2, 11, dtype=torch.int64)
    gamma, lam = 0.97, 0.8
    adv, ret = O.gae_unwhitened(r, v, m, gamma, lam)
    L = 11
    for b in range(2):
        delta = [float(r[b, t]) + gamma * (float(v[b, t + 1]) if t + 1 < L else 0.0) - float(v[b, t]) for t in range(L)]
        for t in range(L):
            a = sum((gamma * lam) ** k * delta[t + k] for k in range(L - t))
            assert abs(float(adv[b, t]) - a) < 1e-10
            assert abs(float(ret[b, t]) - (a + float(v[b, t]))) < 1e-10


def test_gae_trailing_padding_equals_truncation():
    r, v = _rand(2, 12, 3)
    m = torch.ones(2, 12, dtype=torch.int64)
    m[0, 8:] = 0
    m[1, 5:] = 0
    adv, _ = O.gae_unwhitened(r, v, m, 0.95, 0.9)
    for b, n in ((0, 8), (1, 5)):
        a_ref, _ = O.gae_unwhitened(r[b:b + 1, :n], v[b:b + 1, :n], torch.ones(1, n, dtype=torch.int64), 0.95, 0.9)
        assert torch.allclose(adv[b, :n], a_ref[0], atol=1e-12)
        assert torch.all(adv[b, n:] == 0)  # the scan starts from zero and masked positions keep it


def test_gae_interior_masked_tokens_are_skipped():
    # observation tokens inside the response: deleting those columns must not change the other positions, and a
    # masked position carries the advantage of the next unmasked one
    r, v = _rand(1, 10, 4)
    m = torch.tensor([[1, 1, 0, 0, 1, 0, 1, 1, 0, 0]])
    adv, _ = O.gae_unwhitened(r, v, m, 0.9, 0.7)
    keep = m[0].bool()
    a_ref, _ = O.gae_unwhitened(r[:, keep], v[:, keep], torch.ones(1, int(keep.sum()), dtype=torch.int64), 0.9, 0.7)
    assert torch.allclose(adv[0, keep], a_ref[0], atol=1e-12)
    assert adv[0, 2] == adv[0, 4] and adv[0, 3] == adv[0, 4] and adv[0, 5] == adv[0, 6]
    assert adv[0, 8] == 0 and adv[0, 9] == 0


def test_gae_whitens_advantages_only():
    r, v = _rand(4, 16, 5)
    m = (torch.rand(4, 16, generator=torch.Generator().manual_seed(6)) > 0.3).to(torch.int64)
    adv, ret = O.compute_gae_advantage_return(r, v, m, 0.99, 0.95)
    raw, raw_ret = O.gae_unwhitened(r, v, m, 0.99, 0.95)
    assert torch.equal(ret, raw_ret)
    sel = adv[m.bool()].numpy()
    assert abs(sel.mean()) < 1e-7 and abs(sel.var(ddof=1) - 1.0) < 1e-6
    # whitening is an increasing affine map of the raw advantages
    order = torch.argsort(raw.flatten())
    assert torch.all(torch.diff(adv.flatten()[order]) >= 0)


# ------------------------------------------------------------------------------------------ whitening


def test_masked_whiten_matches_numpy_statistics():
    g = torch.Generator().manual_seed(7)
    x = torch.randn(5, 13, generator=g, dtype=torch.float64) * 3 + 2
    m = (torch.rand(5, 13, generator=g) > 0.4).to(torch.int64)
    sel = x[m.bool()].numpy()
    want = (x.numpy() - sel.mean()) / math.sqrt(sel.var(ddof=1) + 1e-8)
    assert np.allclose(OF.masked_whiten(x, m.double()).numpy(), want, atol=1e-7)
    assert np.allclose(OF.masked_whiten(x, m, shift_mean=False).numpy(), want + sel.mean(), atol=1e-6)
    # with an integer mask the Bessel factor n / (n - 1) is a float32 quotient (6e-8 relative)
    assert abs(float(OF.masked_var(x, m)) - sel.var(ddof=1)) < 2e-6
    assert abs(float(OF.masked_var(x, m.double())) - sel.var(ddof=1)) < 1e-7
    assert abs(float(OF.masked_var(x, m, unbiased=False)) - sel.var(ddof=0)) < 1e-7


def test_masked_var_errors():
    x = torch.ones(2, 3)
    with pytest.raises(ValueError):
        OF.masked_var(x, torch.zeros(2, 3, dtype=torch.int64))
    one = torch.zeros(2, 3, dtype=torch.int64)
    one[1, 2] = 1
    with pytest.raises(ValueError):
        OF.masked_var(x, one)


# ----------------------------------------------------------------------------------------- value loss


def test_value_loss_hand_cases():
    m = torch.ones(1, 4)
    values = torch.zeros(1, 4, dtype=torch.float64)
    #            inside the range | beyond, target on the near side | beyond, target beyond too | below the range
    vpreds = torch.tensor([[0.1, 1.0, 1.0, -1.0]], dtype=torch.float64)
    returns = torch.tensor([[0.5, 0.0, 2.0, -3.0]], dtype=torch.float64)
    tok = [0.16, 1.0, (0.2 - 2.0) ** 2, (-0.2 + 3.0) ** 2]
    loss, frac = O.compute_value_loss(vpreds, returns, values, m, 0.2, "token-mean")
    assert abs(float(loss) - 0.5 * sum(tok) / 4) < 1e-9
    assert abs(float(frac) - 0.5) < 1e-9
    loss, _ = O.compute_value_loss(vpreds, returns, values, m, 0.2, "seq-mean-token-sum")
    assert abs(float(loss) - 0.5 * sum(tok)) < 1e-9


def test_value_loss_gradient_is_zero_where_clipped():
    vpreds = torch.tensor([[0.1, 1.0, 1.0]], dtype=torch.float64, requires_grad=True)
    returns = torch.tensor([[0.5, 0.0, 2.0]], dtype=torch.float64)
    loss, _ = O.compute_value_loss(vpreds, returns, torch.zeros(1, 3, dtype=torch.float64), torch.ones(1, 3), 0.2)
    (g,) = torch.autograd.grad(loss, vpreds)
    assert torch.allclose(g, torch.tensor([[(0.1 - 0.5) / 3, 1.0 / 3, 0.0]], dtype=torch.float64), atol=1e-12)


# ------------------------------------------------------------------------------- CPGD / GPG / GMPO


def test_cpgd_hand_cases():
    cfg = O.LossConfig(clip_ratio=0.2, clip_ratio_low=0.2, clip_ratio_high=0.2, clip_ratio_c=3.0)
    old = torch.tensor([[-1.0, -1.0, -1.0, -1.0, -1.0]], dtype=torch.float64)
    lp = torch.tensor([[-0.5, -0.9, -1.5, -1.1, 0.5]], dtype=torch.float64, requires_grad=True)
    A = torch.tensor([[2.0, 2.0, -1.0, -1.0, -1.0]], dtype=torch.float64)
    m = torch.ones(1, 5)
    hi, lo = math.log(1.2), math.log(0.8)
    tok = [-(-1.0 + hi) * 2.0, 0.9 * 2.0, (-1.0 + lo) * 1.0, -1.1, 0.5]
    loss, frac, kl, lower = O.compute_policy_loss_cpgd(old, lp, A, m, "token-mean", cfg)
    assert abs(float(loss) - sum(tok) / 5) < 1e-12
    assert abs(float(frac) - 2 / 5) < 1e-12           # tokens 0 and 2
    assert abs(float(lower) - 1 / 5) < 1e-12          # token 4: ratio e^1.5 > 3 with a negative advantage
    assert abs(float(kl) - float(-(lp - old).mean())) < 1e-12
    (g,) = torch.autograd.grad(loss, lp)
    assert torch.allclose(g, torch.tensor([[0.0, -2.0, 0.0, 1.0, 1.0]], dtype=torch.float64) / 5, atol=1e-12)


def test_cpgd_clip_flag_agrees_with_the_clamp():
    g = torch.Generator().manual_seed(8)
    old = torch.randn(6, 9, generator=g, dtype=torch.float64)
    lp = old + 0.4 * torch.randn(6, 9, generator=g, dtype=torch.float64)
    A = torch.randn(6, 9, generator=g, dtype=torch.float64)
    cfg = O.LossConfig(clip_ratio=0.2, clip_ratio_low=0.15, clip_ratio_high=0.3, clip_ratio_c=3.0)
    m = torch.ones(6, 9)
    lp.requires_grad_(True)
    loss, frac, _, _ = O.compute_policy_loss_cpgd(old, lp, A, m, "seq-mean-token-sum", cfg)
    (gr,) = torch.autograd.grad(loss, lp)
    # the gradient vanishes exactly on the clipped tokens (and where A == 0, which randn never gives)
    assert abs(float((gr == 0).double().mean()) - float(frac)) < 1e-12


def test_policy_drift_hand_case():
    old = torch.tensor([[-1.0, -1.0]], dtype=torch.float64)
    lp = torch.tensor([[-0.5, 1.0]], dtype=torch.float64, requires_grad=True)
    loss = O.policy_drift_loss(old, lp, torch.ones(1, 2), "token-mean")
    w = [math.exp(0.5) - 1.0, 2.0]  # exp(2) - 1 > 2 is clamped
    assert abs(float(loss) - (w[0] * -0.5 + w[1] * 1.0) / 2) < 1e-12
    (g,) = torch.autograd.grad(loss, lp)
    assert torch.allclose(g, torch.tensor([w], dtype=torch.float64) / 2, atol=1e-12)  # the weight is detached


def test_gpg_is_aggregated_minus_logprob_times_advantage():
    g = torch.Generator().manual_seed(9)
    lp, A = torch.randn(3, 7, generator=g, dtype=torch.float64), torch.randn(3, 7, generator=g, dtype=torch.float64)
    m = (torch.rand(3, 7, generator=g) > 0.3).double()
    w = torch.rand(3, 7, generator=g, dtype=torch.float64)
    for mode in O.AGG_MODES:
        loss, a, b, c = O.compute_policy_loss_gpg(None, lp, A, m, mode)
        assert torch.allclose(loss, O.agg_loss(-(lp * A), m, mode))
        assert float(a) == 0 and float(b) == 0 and float(c) == 0
    loss, *_ = O.compute_policy_loss_gpg(None, lp, A, m, "token-mean", None, w)
    assert torch.allclose(loss, O.agg_loss(-(lp * A * w), m, "token-mean"))


def test_geo_mean_is_geometric_mean_of_token_ratios():
    g = torch.Generator().manual_seed(10)
    B, L = 4, 6
    old = torch.randn(B, L, generator=g, dtype=torch.float64)
    lp = old + 0.05 * torch.randn(B, L, generator=g, dtype=torch.float64)  # inside the clip range
    A = torch.tensor([1.5, -0.5, 2.0, -1.0], dtype=torch.float64).unsqueeze(1).expand(B, L)
    m = torch.ones(B, L)
    cfg = O.LossConfig(clip_ratio=0.4, clip_ratio_low=0.4, clip_ratio_high=0.4)
    loss, frac, kl, lower = O.compute_policy_loss_geo_mean(old, lp, A, m, "token-mean", cfg)
    geo = torch.exp(lp - old).prod(dim=1) ** (1.0 / L)
    assert abs(float(loss) - float((-A[:, 0] * geo).mean())) < 1e-7  # 1e-8 in the denominators
    assert float(frac) == 0 and float(lower) == 0


def test_geo_mean_clipping_single_token_sequences():
    # L = 1: the loss of a sequence is -A * exp(x) with x the clipped log-ratio
    cfg = O.LossConfig(clip_ratio=0.2, clip_ratio_low=0.2, clip_ratio_high=0.3)
    d = torch.tensor([[0.5], [-0.5], [0.5], [-0.5], [0.1]], dtype=torch.float64)
    A = torch.tensor([[1.0], [1.0], [-2.0], [-2.0], [1.0]], dtype=torch.float64)
    x = [0.3, -0.5, 0.5, -0.2, 0.1]  # A>0 clips above, A<0 clips below, the pessimistic side stays
    old = torch.zeros(5, 1, dtype=torch.float64)
    lp = d.clone().requires_grad_(True)
    loss, frac, kl, lower = O.compute_policy_loss_geo_mean(old, lp, A, torch.ones(5, 1), "token-mean", cfg)
    want = sum(-float(A[i]) * math.exp(x[i]) for i in range(5)) / 5
    assert abs(float(loss) - want) < 1e-7
    # d != clamp(d) on tokens 0..3; split by the advantage's sign
    assert abs(float(frac) - 2 / 5) < 1e-9 and abs(float(lower) - 2 / 5) < 1e-9
    (gr,) = torch.autograd.grad(loss, lp)
    want_g = [0.0, -math.exp(-0.5), 2.0 * math.exp(0.5), 0.0, -math.exp(0.1)]
    assert torch.allclose(gr.flatten(), torch.tensor(want_g, dtype=torch.float64) / 5, atol=1e-7)


def test_geo_mean_importance_weights_enter_as_their_geometric_mean():
    cfg = O.LossConfig(clip_ratio=0.2)
    old = torch.zeros(1, 2, dtype=torch.float64)
    lp = torch.tensor([[0.1, -0.1]], dtype=torch.float64)
    A = torch.ones(1, 2, dtype=torch.float64)
    w = torch.tensor([[4.0, 1.0]], dtype=torch.float64)
    loss, *_ = O.compute_policy_loss_geo_mean(old, lp, A, torch.ones(1, 2), "token-mean", cfg, w)
    assert abs(float(loss) - (-1.0 * math.exp(0.0) * 2.0)) < 1e-6


# ------------------------------------------------------------------------------------ PF-PPO resampling


def test_pf_ppo_weights_by_hand():
    import math

    import torch

    from oracle import core_algos as OC

    s = torch.tensor([2.0, -3.0, 0.0, 2.0, 0.5])
    w = OC.pf_ppo_weights(s, "pow", 2.0)
    assert w.tolist() == pytest.approx([4.0, 9.0, 1e-8, 4.0, 0.25], rel=1e-6)
    w = OC.pf_ppo_weights(s, "pow", 0.5)
    assert w.tolist() == pytest.approx([math.sqrt(2), math.sqrt(3), 1e-8, math.sqrt(2), math.sqrt(0.5)], rel=1e-6)
    w = OC.pf_ppo_weights(s, "max_min", 2.0)  # both sequences at the maximum, the one at the minimum
    assert w.tolist() == pytest.approx([1.0, 1.0, 1e-8, 1.0, 1e-8], rel=1e-6)
    w = OC.pf_ppo_weights(s, "max_random", 2.0)
    assert w.tolist() == pytest.approx([0.4, 0.1, 0.1, 0.4, 0.1], rel=1e-6)
    with pytest.raises(ValueError, match="Unsupported reweight_method"):
        OC.pf_ppo_weights(s, "median", 2.0)


def _pf_ppo_batch(B=12, L=5, seed=0):
    from types import SimpleNamespace

    import numpy as np
    import torch

    g = torch.Generator().manual_seed(seed)
    batch = {"token_level_scores": torch.randn(B, L, generator=g), "responses": torch.randint(0, 99, (B, L), generator=g),
             "advantages": torch.randn(B, L, generator=g), "flag": torch.arange(B, dtype=torch.uint8)}
    extra = {"uid": np.array([f"u{i}" for i in range(B)], dtype=object), "names": [f"n{i}" for i in range(B)]}
    meta = {"per_row": list(range(B)), "temperature": 0.7, "short_list": [1, 2]}
    return SimpleNamespace(batch=batch, non_tensor_batch=extra, meta_info=meta)


def test_pf_ppo_resampling_is_one_draw_applied_everywhere():
    import torch

    from oracle import core_algos as OC

    data = _pf_ppo_batch()
    before = {k: v.clone() for k, v in data.batch.items()}
    torch.manual_seed(5)
    out = OC.compute_pf_ppo_reweight_data(data, "pow", 2.0)
    # the draw: torch.multinomial on the global host generator, from the hand-checked weights
    torch.manual_seed(5)
    picks = torch.multinomial(OC.pf_ppo_weights(before["token_level_scores"].sum(-1), "pow", 2.0), 12, replacement=True)
    for k, v in before.items():
        assert torch.equal(out.batch[k], v[picks]) and torch.equal(data.batch[k], v)  # the input is left alone
    assert list(out.non_tensor_batch["uid"]) == [f"u{i}" for i in picks.tolist()]
    assert out.non_tensor_batch["names"] == [f"n{i}" for i in picks.tolist()]
    assert out.meta_info == {"per_row": picks.tolist(), "temperature": 0.7, "short_list": [1, 2]}
    # "max_min": only the best and the worst sequence are ever drawn (their weight is 1 against 1e-8)
    torch.manual_seed(1)
    out = OC.compute_pf_ppo_reweight_data(data, "max_min")
    s = before["token_level_scores"].sum(-1)
    assert set(out.meta_info["per_row"]) <= {int(s.argmax()), int(s.argmin())}
