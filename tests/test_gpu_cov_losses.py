"""The covariance losses (Clip-Cov, KL-Cov) and CPGD's outcome advantage on the GPU against the oracle
(reference ``siirl/dag_worker/core_algos.py:461-517,898-1071``).

Tolerances: scalars 1e-6 + 1e-5 relative and gradients 1e-7 + 1e-5 relative against the float64 oracle; the picked
tokens (an index set) must be identical to the float32 oracle's, the reference's own dtype."""
from types import SimpleNamespace

import pytest
import torch

pytestmark = pytest.mark.gpu

from oracle import core_algos as O  # noqa: E402

DEV = "cuda:0"


def _cfg(**pl):
    return SimpleNamespace(clip_ratio=0.2, clip_ratio_low=0.2, clip_ratio_high=0.28, clip_ratio_c=3.0,
                           policy_loss=O.CovLossConfig(**pl))


def _case(seed, B, L, mask_dtype=torch.int64, spread=0.05):
    g = torch.Generator().manual_seed(seed)
    A = torch.randn(B, L, generator=g) * 1.5
    old = -torch.rand(B, L, generator=g) * 3
    lp = old + spread * torch.randn(B, L, generator=g)
    lens = torch.randint(1, L + 1, (B,), generator=g)
    m = (torch.arange(L)[None, :] < lens[:, None]) & (torch.rand(B, L, generator=g) < 0.9)
    m[0, 0] = True
    w = torch.rand(B, L, generator=g) + 0.5
    return old, lp, A, m.to(mask_dtype), w


def _close(a, b, rtol=1e-5, atol=1e-6, what=None):
    assert abs(float(a) - float(b)) <= atol + rtol * abs(float(b)), (float(a), float(b), what)


def _cancel_slack(A, m, agg, w=None):
    """Float32 accumulation of a policy loss is accurate relative to the sum of the magnitudes of its signed terms
    (|tok| <= |A| * ratio * weight, ratio < 3 in these cases), not relative to what cancellation leaves of them."""
    mag = 3.0 * A.double().abs() * (w.double() if w is not None else 1.0)
    return 2.0 ** -24 / 8 * float(O.agg_loss(mag, m.double(), agg))


@pytest.mark.parametrize("agg", O.AGG_MODES)
@pytest.mark.parametrize("B,L,mask_dtype,with_w", [(6, 64, torch.int64, False), (5, 37, torch.bool, True),
                                                   (33, 2052, torch.float32, True), (1, 5, torch.int64, False)])
def test_kl_cov_matches_oracle(agg, B, L, mask_dtype, with_w):
    import siirl_amd.core_algos as CA

    old, lp, A, m, w = _case(100 + B + L, B, L, mask_dtype)
    cfg = _cfg(kl_cov_ratio=0.05, ppo_kl_coef=0.8)
    mf = m.to(torch.float64)
    # selection: float32 on the host, as the reference computes it
    want_idx, _ = O.kl_cov_selection(lp, A, m.to(torch.float32), 0.05)
    aux = CA._kl_cov_weights(lp.to(DEV), A.to(DEV), m.to(DEV), 0.05, 0.8)
    got_idx = torch.nonzero(aux.reshape(-1)).reshape(-1).cpu()
    assert sorted(got_idx.tolist()) == sorted(want_idx.tolist())
    assert torch.all(aux.reshape(-1)[got_idx.to(DEV)] == 0.8)

    lp64 = lp.double().requires_grad_(True)
    want = O.compute_policy_loss_kl_cov(old.double(), lp64, A.double(), mf, agg, cfg, w.double() if with_w else None,
                                        chosen=want_idx)
    (gwant,) = torch.autograd.grad(want[0], lp64)
    lpd = lp.to(DEV).requires_grad_(True)
    got = CA.compute_policy_loss_kl_cov(old.to(DEV), lpd, A.to(DEV), m.to(DEV), agg, cfg, w.to(DEV) if with_w else None)
    got[0].backward()
    for a, b in zip(got, want):
        _close(a, b)
    assert float(got[1]) == 0.0 and float(got[3]) == 0.0 and got[1].is_cuda
    assert torch.allclose(lpd.grad.cpu().double(), gwant, rtol=1e-5, atol=1e-7)


def _oracle_dropped(old, lp, A, m, cfg, lo, hi, seed):
    pl = cfg.policy_loss
    _, cand = O.clip_cov_candidates(old, lp, A, m.to(torch.float32), lo, hi, pl.clip_cov_lb, pl.clip_cov_ub)
    clip_num = max(int(pl.clip_cov_ratio * float(m.sum())), 1)
    torch.manual_seed(seed)
    perm = torch.randperm(len(cand)) if len(cand) else torch.empty(0, dtype=torch.long)
    return cand, cand[perm[: min(clip_num, len(cand))]]


@pytest.mark.parametrize("agg", O.AGG_MODES)
@pytest.mark.parametrize("B,L,mask_dtype,with_w", [(6, 64, torch.int64, False), (5, 37, torch.bool, True),
                                                   (33, 2052, torch.float32, True)])
def test_clip_cov_matches_oracle(agg, B, L, mask_dtype, with_w):
    import siirl_amd.core_algos as CA

    old, lp, A, m, w = _case(300 + B + L, B, L, mask_dtype, spread=0.15)
    cfg = _cfg(clip_cov_ratio=0.02, clip_cov_lb=0.3, clip_cov_ub=4.0)
    cand, dropped = _oracle_dropped(old, lp, A, m, cfg, 0.2, 0.28, seed=9)
    assert len(cand) > len(dropped) >= 1

    torch.manual_seed(9)
    lpd = lp.to(DEV).requires_grad_(True)
    got = CA.compute_policy_loss_clip_cov(old.to(DEV), lpd, A.to(DEV), m.to(DEV), agg, cfg, w.to(DEV) if with_w else None)
    after = torch.rand(2)  # the call drew one host randperm(len(candidates)) and nothing else
    torch.manual_seed(9)
    torch.randperm(len(cand))
    assert torch.equal(after, torch.rand(2))
    got[0].backward()

    lp64 = lp.double().requires_grad_(True)
    want = O.compute_policy_loss_clip_cov(old.double(), lp64, A.double(), m.double(), agg, cfg,
                                          w.double() if with_w else None, dropped=dropped)
    (gwant,) = torch.autograd.grad(want[0], lp64)
    for a, b in zip(got, want):
        _close(a, b)
    assert torch.allclose(lpd.grad.cpu().double(), gwant, rtol=1e-5, atol=1e-7)
    # the dropped tokens themselves: no gradient there, and their count is what the clip fraction reports
    assert torch.all(lpd.grad.cpu()[dropped[:, 0], dropped[:, 1]] == 0)
    _close(got[1], len(dropped) / (float(m.sum()) + 1e-8))


def test_clip_cov_candidates_match_oracle():
    import siirl_amd.core_algos as CA

    old, lp, A, m, _ = _case(41, 9, 130, spread=0.2)
    cov, stats = torch.ops.siirl_hip.cov_scores(old.to(DEV), lp.to(DEV), A.to(DEV), m.to(DEV), CA.LOSS_CLIP_COV, 0.2, 0.28)
    want, cand = O.clip_cov_candidates(old, lp, A, m.to(torch.float32), 0.2, 0.28, 0.3, 4.0)
    cov = cov.cpu()
    assert torch.equal(torch.isinf(cov), torch.isinf(want)) and bool(torch.isinf(want).any())
    fin = ~torch.isinf(want)
    assert torch.allclose(cov[fin], want[fin], rtol=1e-5, atol=1e-6)
    got_cand = torch.nonzero((cov < 4.0) & (cov > 0.3))
    assert torch.equal(got_cand, cand)
    assert float(stats[0]) == float((m > 0).sum()) and float(stats[1]) == float(m.sum())
    # kl_cov scores: plain means over the valid tokens, -inf outside the mask
    cov, stats = torch.ops.siirl_hip.cov_scores(None, lp.to(DEV), A.to(DEV), m.to(DEV), CA.LOSS_KL_COV, 0.0, 0.0)
    v = m > 0
    want = (A - A[v].double().mean().float()) * (lp - lp[v].double().mean().float())
    assert torch.all(torch.isinf(cov.cpu()[~v])) and torch.allclose(cov.cpu()[v], want[v], rtol=1e-5, atol=1e-6)


def test_cov_losses_edge_cases():
    import siirl_amd.core_algos as CA

    old, lp, A, m, _ = _case(77, 4, 16)
    zero = torch.zeros_like(m)
    # nothing valid: KL-Cov selects nothing and the loss is the aggregate of nothing (0 for token-mean)
    aux = CA._kl_cov_weights(lp.to(DEV), A.to(DEV), zero.to(DEV), 0.1, 1.0)
    assert float(aux.abs().sum()) == 0.0
    got = CA.compute_policy_loss_kl_cov(old.to(DEV), lp.to(DEV), A.to(DEV), zero.to(DEV), "token-mean", _cfg())
    assert float(got[0]) == 0.0
    # no candidate (bounds far away): Clip-Cov is the plain clip loss and draws nothing from the generator
    torch.manual_seed(4)
    cfg = _cfg(clip_cov_lb=1e3, clip_cov_ub=2e3)
    got = CA.compute_policy_loss_clip_cov(old.to(DEV), lp.to(DEV), A.to(DEV), m.to(DEV), "token-mean", cfg)
    after = torch.rand(2)
    torch.manual_seed(4)
    assert torch.equal(after, torch.rand(2))
    legacy = CA.compute_policy_loss(old.to(DEV), lp.to(DEV), A.to(DEV), m.to(DEV), cliprange=0.2, cliprange_low=0.2,
                                    cliprange_high=0.28, clip_ratio_c=1e30)
    _close(got[0], legacy[0], rtol=1e-6)
    assert float(got[1]) == 0.0
    # a ratio above 1 asks torch.topk for more than there is: an error, as in the reference
    with pytest.raises(RuntimeError):
        CA._kl_cov_weights(lp.to(DEV), A.to(DEV), m.to(DEV), 1.5, 1.0)
    # missing policy_loss block
    with pytest.raises(AssertionError):
        CA.compute_policy_loss_kl_cov(old.to(DEV), lp.to(DEV), A.to(DEV), m.to(DEV), "token-mean",
                                      SimpleNamespace(clip_ratio=0.2, policy_loss=None))
    assert CA.get_policy_loss_fn("kl_cov") is CA.compute_policy_loss_kl_cov
    assert CA.get_policy_loss_fn("clip_cov") is CA.compute_policy_loss_clip_cov


@pytest.mark.parametrize("mode", ["kl_cov", "clip_cov"])
def test_actor_loss_with_covariance_losses(mode):
    """The fused composition (policy term + entropy bonus + KL loss, scaled) with the covariance losses as the
    policy term, against the oracle's micro-batch arithmetic composed from the same picks."""
    import siirl_amd.core_algos as CA

    B, L = 7, 96
    old, lp, A, m, w = _case(55, B, L, spread=0.15)
    g = torch.Generator().manual_seed(1)
    ent = torch.rand(B, L, generator=g) * 2
    ref = lp + 0.1 * torch.randn(B, L, generator=g)
    pl = O.CovLossConfig(kl_cov_ratio=0.03, ppo_kl_coef=1.2, clip_cov_ratio=0.02, clip_cov_lb=0.3, clip_cov_ub=4.0)
    pl.loss_mode = mode
    cfg = SimpleNamespace(clip_ratio=0.2, clip_ratio_low=0.2, clip_ratio_high=0.28, clip_ratio_c=3.0, entropy_coeff=0.01,
                          use_kl_loss=True, kl_loss_coef=0.02, kl_loss_type="low_var_kl", loss_agg_mode="seq-mean-token-mean",
                          policy_loss=pl)
    lpd, entd = lp.to(DEV).requires_grad_(True), ent.to(DEV).requires_grad_(True)
    torch.manual_seed(21)
    out = CA.actor_loss(old.to(DEV), lpd, A.to(DEV), m.to(DEV), cfg, entropy=entd, ref_log_prob=ref.to(DEV),
                        loss_scale_factor=0.25, rollout_is_weights=w.to(DEV))
    out.loss.backward()

    lp64, ent64 = lp.double().requires_grad_(True), ent.double().requires_grad_(True)
    kw = {}
    if mode == "clip_cov":
        _, kw["dropped"] = _oracle_dropped(old, lp, A, m, cfg, 0.2, 0.28, seed=21)
    else:
        kw["chosen"], _ = O.kl_cov_selection(lp, A, m.to(torch.float32), 0.03)
    fn = O.compute_policy_loss_clip_cov if mode == "clip_cov" else O.compute_policy_loss_kl_cov
    pg, frac, kl, _ = fn(old.double(), lp64, A.double(), m.double(), cfg.loss_agg_mode, cfg, w.double(), **kw)
    total = (pg - 0.01 * O.agg_loss(ent64, m.double(), cfg.loss_agg_mode)
             + 0.02 * O.agg_loss(O.kl_penalty(lp64, ref.double(), "low_var_kl"), m.double(), cfg.loss_agg_mode)) * 0.25
    glp, gent = torch.autograd.grad(total, (lp64, ent64))
    _close(out.loss, total)
    mt = out.metrics()
    _close(mt["actor/pg_loss"], float(pg) * 0.25)
    _close(mt["actor/pg_clipfrac"], frac)
    _close(mt["actor/ppo_kl"], kl)
    assert torch.allclose(lpd.grad.cpu().double(), glp, rtol=1e-5, atol=1e-8)
    assert torch.allclose(entd.grad.cpu().double(), gent, rtol=1e-5, atol=1e-9)


def test_cov_selection_at_batch_scale():
    """[2048, 8192] (16.8 M tokens): the picks have the size the reference's arithmetic gives and are the largest
    scores; checked through properties, the oracle's loops being too slow here."""
    import siirl_amd.core_algos as CA

    B, L = 2048, 8192
    g = torch.Generator(device=DEV).manual_seed(8)
    A = torch.randn(B, 1, device=DEV, generator=g).expand(B, L).contiguous()
    old = -torch.rand(B, L, device=DEV, generator=g) * 3
    lp = old + 0.1 * torch.randn(B, L, device=DEV, generator=g)
    lens = torch.randint(256, L + 1, (B,), device=DEV, generator=g)
    m = (torch.arange(L, device=DEV)[None, :] < lens[:, None]).to(torch.int64)
    n = int(m.sum())
    aux = CA._kl_cov_weights(lp, A, m, 0.0002, 1.0)
    k = max(1, int(n * 0.0002))
    assert int((aux != 0).sum()) == k
    _, st = torch.ops.siirl_hip.cov_scores(None, lp, A, m, CA.LOSS_KL_COV, 0.0, 0.0)
    st = st.double().cpu()
    assert int(st[0] + st[4]) == n and int(st[1] + st[5]) == n
    cov, _ = torch.ops.siirl_hip.cov_scores(None, lp, A, m, CA.LOSS_KL_COV, 0.0, 0.0)
    assert float(cov[aux != 0].min()) >= float(cov[aux == 0].max())
    assert bool((m[aux != 0] > 0).all())
    torch.manual_seed(3)
    dropped = CA._clip_cov_dropped(old, lp, A, m, 0.2, 0.28, 0.0002, 1.0, 5.0)
    cov, stats = torch.ops.siirl_hip.cov_scores(old, lp, A, m, CA.LOSS_CLIP_COV, 0.2, 0.28)
    cand = (cov < 5.0) & (cov > 1.0)
    assert int((dropped != 0).sum()) == min(max(int(0.0002 * n), 1), int(cand.sum()))
    assert bool(cand[dropped != 0].all())


@pytest.mark.parametrize("mode", ["STD_weight", "naive", "clip_filter_like_weight"])
@pytest.mark.parametrize("on_host", [False, True])
def test_cpgd_outcome_advantage(mode, on_host):
    import numpy as np

    import siirl_amd.core_algos as CA

    g = torch.Generator().manual_seed(12)
    B, L = 40, 33
    lens = torch.randint(1, L + 1, (B,), generator=g)
    mask = (torch.arange(L)[None, :] < lens[:, None]).to(torch.int64)
    rewards = torch.zeros(B, L)
    rewards[torch.arange(B), lens - 1] = torch.randint(0, 3, (B,), generator=g).float()
    uid = np.array([f"prompt-{i // 4}" for i in range(B)], dtype=object)
    uid[36:] = [f"solo-{i}" for i in range(4)]     # four groups of one
    rewards[8:12] = 0.0
    rewards[8:12, 0] = 2.0                          # one group whose scores are all equal
    want, _ = O.compute_cpgd_outcome_advantage(rewards.double(), mask.double(), list(uid), weight_factor_in_cpgd=mode)
    r, mk = (rewards, mask) if on_host else (rewards.to(DEV), mask.to(DEV))
    got, got2 = CA.compute_cpgd_outcome_advantage(r, mk, uid, weight_factor_in_cpgd=mode)
    assert got is got2 and got.device == r.device and got.dtype == torch.float32
    assert torch.allclose(got.cpu().double(), want, rtol=1e-5, atol=1e-6)
    with pytest.raises(NotImplementedError):
        CA.compute_cpgd_outcome_advantage(r, mk, uid, weight_factor_in_cpgd="other")


def test_sweep_covariance_losses():
    """Seeded random shapes, mask dtypes (weighted float masks included), aggregation modes, bounds and quotas through
    both losses; the picks must equal the float32 oracle's, loss and gradient the float64 oracle's.
    ``SIIRL_TEST_SEED=<int>`` shifts the seeds."""
    import os
    import random

    import siirl_amd.core_algos as CA

    shift = 100003 * int(os.environ.get("SIIRL_TEST_SEED", "0"))
    for case in range(60):
        rnd = random.Random(7000 + case + shift)
        B, L = rnd.randint(1, 24), rnd.choice((1, 3, 4, 17, 64, 129, 256, 2049))
        mdt = rnd.choice((torch.int64, torch.bool, torch.int32, torch.float32, torch.bfloat16))
        old, lp, A, m, w = _case(9000 + case + shift, B, L, torch.float32, spread=rnd.choice((0.02, 0.1, 0.3)))
        if mdt in (torch.float32, torch.bfloat16) and case % 2:
            m = m * torch.tensor([0.5, 1.0, 2.0])[torch.randint(0, 3, m.shape, generator=torch.Generator().manual_seed(case))]
        m = m.to(mdt)
        agg = rnd.choice(O.AGG_MODES)
        with_w = rnd.random() < 0.5
        mf = m.to(torch.float64)
        # KL-Cov
        ratio, coef = rnd.choice((0.0002, 0.01, 0.2)), rnd.choice((1.0, 0.3))
        cfg = _cfg(kl_cov_ratio=ratio, ppo_kl_coef=coef)
        want_idx, cov32 = O.kl_cov_selection(lp, A, m.to(torch.float32), ratio)
        aux = CA._kl_cov_weights(lp.to(DEV), A.to(DEV), m.to(DEV), ratio, coef)
        got_idx = sorted(torch.nonzero(aux.reshape(-1)).reshape(-1).tolist())
        if sorted(want_idx.tolist()) != got_idx:
            # allowed only when the cut falls between two covariances that float32 rounding cannot tell apart
            k = len(want_idx)
            top = torch.sort(cov32, descending=True).values
            assert k < len(top) and abs(float(top[k - 1] - top[k])) <= 1e-6 * max(1.0, abs(float(top[k]))), (case, B, L)
            want_idx = torch.tensor(got_idx)  # the device's side of the tie, for the arithmetic below
        lp64 = lp.double().requires_grad_(True)
        want = O.compute_policy_loss_kl_cov(old.double(), lp64, A.double(), mf, agg, cfg, w.double() if with_w else None,
                                            chosen=want_idx)
        lpd = lp.to(DEV).requires_grad_(True)
        got = CA.compute_policy_loss_kl_cov(old.to(DEV), lpd, A.to(DEV), m.to(DEV), agg, cfg, w.to(DEV) if with_w else None)
        if torch.isnan(want[0]):  # seq-mean-token-mean with an empty row
            assert torch.isnan(got[0]), (case, agg)
        else:
            (gwant,) = torch.autograd.grad(want[0], lp64)
            got[0].backward()
            info = (case, B, L, str(mdt), agg, with_w, ratio, coef)
            _close(got[0], want[0], atol=1e-6 + _cancel_slack(A, m, agg, w if with_w else None), what=info)
            _close(got[2], want[2], what=info)
            assert torch.allclose(lpd.grad.cpu().double(), gwant, rtol=1e-5, atol=1e-7), (case, "kl_cov grad")
        # Clip-Cov
        pl = dict(clip_cov_ratio=rnd.choice((0.0002, 0.05, 1.0)), clip_cov_lb=rnd.choice((0.1, 1.0)), clip_cov_ub=rnd.choice((2.0, 5.0)))
        cfg = _cfg(**pl)
        cov_d, _ = torch.ops.siirl_hip.cov_scores(old.to(DEV), lp.to(DEV), A.to(DEV), m.to(DEV), CA.LOSS_CLIP_COV, 0.2, 0.28)
        cand_d = torch.nonzero((cov_d < pl["clip_cov_ub"]) & (cov_d > pl["clip_cov_lb"]) & (m.to(DEV) > 0)).cpu()
        cand, dropped = _oracle_dropped(old, lp, A, m.to(torch.float32), cfg, 0.2, 0.28, seed=case)
        if not torch.equal(cand, cand_d):
            continue  # a covariance within rounding of a bound: the two candidate lists differ, so would the draw
        torch.manual_seed(case)
        lpd = lp.to(DEV).requires_grad_(True)
        got = CA.compute_policy_loss_clip_cov(old.to(DEV), lpd, A.to(DEV), m.to(DEV), agg, cfg, w.to(DEV) if with_w else None)
        lp64 = lp.double().requires_grad_(True)
        want = O.compute_policy_loss_clip_cov(old.double(), lp64, A.double(), mf, agg, cfg,
                                              w.double() if with_w else None, dropped=dropped)
        if torch.isnan(want[0]):
            assert torch.isnan(got[0]), (case, agg)
            continue
        (gwant,) = torch.autograd.grad(want[0], lp64)
        got[0].backward()
        _close(got[0], want[0], atol=1e-6 + _cancel_slack(A, m, agg, w if with_w else None),
               what=(case, B, L, str(mdt), agg, with_w, pl))
        # What hangs on a strict comparison of float32 numbers -- the clip fractions, the side of `maximum` a token's
        # gradient takes when its ratio rounds onto a clip bound (a tie in float32, none in float64) -- may instead
        # agree with the oracle run in float32, the reference's own dtype.
        lp32 = lp.clone().requires_grad_(True)
        want32 = O.compute_policy_loss_clip_cov(old, lp32, A, m.to(torch.float32), agg, cfg, w if with_w else None,
                                                dropped=dropped)
        (gwant32,) = torch.autograd.grad(want32[0], lp32)
        for a, b, b32 in zip(got[1:], want[1:], want32[1:]):
            if abs(float(a) - float(b32)) > 1e-6 + 1e-5 * abs(float(b32)):
                _close(a, b, what=(case, B, L, str(mdt), agg, with_w, pl))
        g = lpd.grad.cpu().double()
        ok = torch.isclose(g, gwant, rtol=1e-5, atol=1e-7) | torch.isclose(g, gwant32.double(), rtol=1e-5, atol=1e-7)
        assert bool(ok.all()), (case, "clip_cov grad", torch.nonzero(~ok).tolist()[:5])


@pytest.mark.parametrize("mode", ["kl_cov", "clip_cov"])
def test_cov_losses_accept_other_ranks_and_dtypes(mode):
    """1-D and 3-D operands, a bf16 log-prob (its gradient comes back in bf16), a bool mask that is a non-contiguous
    view: same value as the 2-D float32 call on the same numbers."""
    import siirl_amd.core_algos as CA

    old, lp, A, m, w = _case(91, 6, 40, torch.bool, spread=0.2)
    lp = lp.to(torch.bfloat16).float()  # representable in bf16, so both calls see the same numbers
    cfg = _cfg(kl_cov_ratio=0.05, ppo_kl_coef=0.5, clip_cov_ratio=0.03, clip_cov_lb=0.2, clip_cov_ub=4.0)
    fn = CA.compute_policy_loss_kl_cov if mode == "kl_cov" else CA.compute_policy_loss_clip_cov

    def call(o, l, a, k):
        torch.manual_seed(13)
        l = l.clone().requires_grad_(True)
        out = fn(o, l, a, k, "token-mean", cfg)
        out[0].backward()
        return [float(v) for v in out], l.grad

    base, g2 = call(old.to(DEV), lp.to(DEV), A.to(DEV), m.to(DEV))
    # 3-D: [2, 3, 40] is the same six rows
    v3, g3 = call(old.reshape(2, 3, 40).to(DEV), lp.reshape(2, 3, 40).to(DEV), A.reshape(2, 3, 40).to(DEV),
                  m.reshape(2, 3, 40).to(DEV))
    assert v3 == base and g3.shape == (2, 3, 40) and torch.equal(g3.reshape(6, 40), g2)
    # bf16 log-prob
    vb, gb = call(old.to(DEV), lp.to(DEV).to(torch.bfloat16), A.to(DEV), m.to(DEV))
    assert vb == base and gb.dtype == torch.bfloat16
    assert torch.allclose(gb.float(), g2, rtol=2 ** -7, atol=1e-9)
    # the mask as a non-contiguous view
    wide = torch.zeros(6, 80, dtype=torch.bool, device=DEV)
    wide[:, ::2] = m.to(DEV)
    vn, gn = call(old.to(DEV), lp.to(DEV), A.to(DEV), wide[:, ::2])
    assert vn == base and torch.equal(gn, g2)
    # one row (token-mean does not care how the tokens are cut into rows... but the covariance means do not either)
    v1, g1 = call(old.reshape(-1).to(DEV), lp.reshape(-1).to(DEV), A.reshape(-1).to(DEV), m.reshape(-1).to(DEV))
    assert g1.shape == (240,)
    for a, b in zip(v1, base):
        assert abs(a - b) <= 1e-6 + 1e-5 * abs(b)
