"""GPU parity: GAE + whitening, value loss, CPGD / GPG / GMPO losses and the CPGD drift term (through the C ABI)
vs the CPU oracle.

Tolerances: GAE `returns` and the un-whitened scan bit-exact against the fp32 oracle (same float32 operation
order); whitened advantages within 1e-5 relative (+1e-6 absolute); loss scalars within 1e-3 absolute of the
fp32 oracle and 2e-5 (+1e-5 relative) of the fp64 oracle on the same inputs; per-token gradients within
1e-6 + 1e-5 relative of autograd through the fp64 oracle."""

from types import SimpleNamespace

import pytest
import torch

from oracle import core_algos as OC
from oracle import torch_functional as OF

pytestmark = pytest.mark.gpu

AGGS = ["token-mean", "seq-mean-token-sum", "seq-mean-token-mean", "seq-mean-token-sum-norm"]


def _scalar(v):
    return float(v.detach()) if isinstance(v, torch.Tensor) else float(v)


def _close(got, want64, tol=2e-5):
    got, want64 = _scalar(got), _scalar(want64)
    return abs(got - want64) <= tol + 1e-5 * abs(want64)


def _grad_close(got, want64):
    err = (got.double() - want64).abs()
    return bool((err <= 1e-6 + 1e-5 * want64.abs()).all()), err.max().item()


def _cfg(lo=0.2, hi=0.28, c=3.0):
    return SimpleNamespace(clip_ratio=0.2, clip_ratio_low=lo, clip_ratio_high=hi, clip_ratio_c=c)


def _mask(B, L, g, kind, dtype):
    if kind == "full":
        m = torch.ones(B, L)
    elif kind == "tail":  # right padding
        lens = torch.randint(1, L + 1, (B,), generator=g)
        m = (torch.arange(L)[None, :] < lens[:, None]).float()
    else:  # observation tokens inside the response as well
        m = (torch.rand(B, L, generator=g) > 0.3).float()
        m[0, 0] = 1
        m[-1, -1] = 1
    return m.to(dtype)


# ------------------------------------------------------------------------------------------------ GAE


@pytest.mark.parametrize("B,L", [(1, 2), (3, 1), (8, 256), (70, 130), (2, 5000), (129, 64), (40, 1024), (17, 260),
                                 (16, 4)])
@pytest.mark.parametrize("kind,mdt", [("full", torch.int64), ("tail", torch.int64), ("holes", torch.bool),
                                      ("holes", torch.float32), ("tail", torch.int32)])
@pytest.mark.parametrize("gamma,lam", [(1.0, 1.0), (0.99, 0.95)])
def test_gae(dev, B, L, kind, mdt, gamma, lam):
    import siirl_amd.core_algos as CA

    g = torch.Generator().manual_seed(B * 1000 + L)
    r = torch.randn(B, L, generator=g)
    v = torch.randn(B, L, generator=g)
    m = _mask(B, L, g, kind, mdt)
    if int(m.sum()) < 2:
        m[:] = 1
    adv, ret = CA.compute_gae_advantage_return(r.to(dev), v.to(dev), m.to(dev), gamma, lam)
    m_o = m.float() if mdt == torch.bool else m
    raw_o, ret_o = OC.gae_unwhitened(r, v, m_o, gamma, lam)
    assert torch.equal(ret.cpu(), ret_o), (ret.cpu() - ret_o).abs().max()
    adv_o = OF.masked_whiten(raw_o.double(), m_o.double() if m_o.dtype != torch.int64 else m_o)
    err = (adv.cpu().double() - adv_o).abs()
    assert bool((err <= 1e-6 + 1e-5 * adv_o.abs()).all()), err.max()
    adv32, _ = OC.compute_gae_advantage_return(r, v, m_o, gamma, lam)
    assert (adv.cpu() - adv32).abs().max() < 1e-3


def test_gae_host_tensors_errors_and_dispatch(dev):
    import siirl_amd.core_algos as CA

    g = torch.Generator().manual_seed(5)
    r, v = torch.randn(4, 9, generator=g), torch.randn(4, 9, generator=g)
    m = torch.ones(4, 9, dtype=torch.int64)
    adv, ret = CA.compute_gae_advantage_return(r, v, m, 1.0, 0.95)  # host tensors are staged and returned on the host
    assert not adv.is_cuda and not ret.is_cuda
    _, ret_o = OC.gae_unwhitened(r, v, m, 1.0, 0.95)
    assert torch.equal(ret, ret_o)
    data = {"token_level_rewards": r, "values": v, "response_mask": m}
    out = CA.compute_advantage(data, CA.AdvantageEstimator.GAE, gamma=1.0, lam=0.95)
    assert torch.equal(out["returns"], ret_o) and torch.equal(out["advantages"], adv)
    assert CA.get_adv_estimator_fn("gae") is CA.compute_gae_advantage_return
    one = torch.zeros(4, 9, dtype=torch.int64)
    with pytest.raises(ValueError, match="At least one element"):
        CA.compute_gae_advantage_return(r, v, one, 1.0, 1.0)
    one[2, 3] = 1
    with pytest.raises(ValueError, match="division by zero"):
        CA.compute_gae_advantage_return(r, v, one, 1.0, 1.0)
    with pytest.raises(AttributeError):  # PF-PPO resamples a batch object (.batch, .non_tensor_batch, .meta_info)
        CA.compute_advantage(dict(data), "gae", use_pf_ppo=True)


class _Proto(SimpleNamespace):
    """The parts of the reference's batch object the dispatcher and the PF-PPO resampling touch."""

    def keys(self):
        return self.batch.keys()

    def __getitem__(self, key):
        return self.batch[key]

    def __setitem__(self, key, value):
        self.batch[key] = value


@pytest.mark.parametrize("where", ["host", "gpu"])
@pytest.mark.parametrize("method", ["pow", "max_min", "max_random"])
def test_pf_ppo_resampling(dev, where, method):
    """Same seed, same draw as the oracle (on the host, where the reference keeps the batch); on the GPU the draw
    comes from the device generator, so the check there is that one draw indexes everything consistently."""
    import numpy as np

    import siirl_amd.core_algos as CA
    from tests.test_oracle_estimators import _pf_ppo_batch

    src = _pf_ppo_batch(B=40, L=8, seed=3)
    data = _Proto(batch={k: (v.to(dev) if where == "gpu" else v) for k, v in src.batch.items()},
                  non_tensor_batch=src.non_tensor_batch, meta_info=src.meta_info)
    torch.manual_seed(11)
    got = CA.compute_pf_ppo_reweight_data(data, method, 2.0)
    picks = got.meta_info["per_row"]
    assert len(picks) == 40 and got.meta_info["temperature"] == 0.7 and got.meta_info["short_list"] == [1, 2]
    for k, v in src.batch.items():
        assert got.batch[k].is_cuda == (where == "gpu")
        assert torch.equal(got.batch[k].cpu(), v[picks]), k
        assert torch.equal(data.batch[k].cpu(), v)  # the input is left alone
    assert list(got.non_tensor_batch["uid"]) == [f"u{i}" for i in picks]
    assert got.non_tensor_batch["names"] == [f"n{i}" for i in picks]
    if where == "host":
        torch.manual_seed(11)
        want = OC.compute_pf_ppo_reweight_data(src, method, 2.0)
        assert want.meta_info["per_row"] == picks
    scores = src.batch["token_level_scores"].sum(-1)
    if method == "max_min":
        assert set(picks) <= {int(scores.argmax()), int(scores.argmin())}
    with pytest.raises(ValueError, match="Unsupported reweight_method"):
        CA.compute_pf_ppo_reweight_data(data, "median")


def test_gae_dispatch_with_pf_ppo(dev):
    import numpy as np

    import siirl_amd.core_algos as CA

    g = torch.Generator().manual_seed(8)
    B, L = 16, 12
    batch = {"token_level_scores": torch.randn(B, L, generator=g), "token_level_rewards": torch.randn(B, L, generator=g),
             "values": torch.randn(B, L, generator=g), "response_mask": torch.ones(B, L, dtype=torch.int64)}
    data = _Proto(batch=dict(batch), non_tensor_batch={"uid": np.arange(B)}, meta_info={"rows": list(range(B))})
    torch.manual_seed(2)
    out = CA.compute_advantage(data, "gae", gamma=1.0, lam=0.95, use_pf_ppo=True, pf_ppo_reweight_method="pow",
                               pf_ppo_weight_pow=2.0)
    assert out is not data and "advantages" in data.batch  # GAE wrote into the input, the resampled copy is returned
    picks = out.meta_info["rows"]
    torch.manual_seed(2)
    want = torch.multinomial(OC.pf_ppo_weights(batch["token_level_scores"].sum(-1), "pow", 2.0), B, replacement=True)
    assert picks == want.tolist()
    _, ret_o = OC.gae_unwhitened(batch["token_level_rewards"], batch["values"], batch["response_mask"], 1.0, 0.95)
    assert torch.equal(out.batch["returns"], ret_o[picks])
    assert list(out.non_tensor_batch["uid"]) == picks


@pytest.mark.parametrize("shape", [(7,), (5, 13), (2, 3, 700), (300000,)])
@pytest.mark.parametrize("mdt", [torch.int64, torch.bool, torch.float32])
def test_masked_whiten_and_var(dev, shape, mdt):
    import siirl_amd.torch_functional as F

    g = torch.Generator().manual_seed(len(shape) * 17 + shape[-1])
    x = torch.randn(*shape, generator=g) * 3 + 2
    m = (torch.rand(*shape, generator=g) > 0.4).to(mdt)
    m.view(-1)[:2] = 1
    m_o = m.double() if mdt != torch.int64 else m
    for shift in (True, False):
        got = F.masked_whiten(x.to(dev), m.to(dev), shift_mean=shift)
        want = OF.masked_whiten(x.double(), m_o, shift_mean=shift)
        assert got.shape == x.shape
        err = (got.cpu().double() - want).abs()
        assert bool((err <= 1e-6 + 1e-5 * want.abs()).all()), err.max()
    for unbiased in (True, False):
        got = F.masked_var(x.to(dev), m.to(dev), unbiased=unbiased)
        want = OF.masked_var(x.double(), m_o, unbiased=unbiased)
        assert abs(float(got) - float(want)) <= 1e-5 * abs(float(want)) + 1e-7
    assert torch.equal(F.clip_by_value(x, x - 1, x + 1), OF.clip_by_value(x, x - 1, x + 1))


# ----------------------------------------------------------------------------------------- value loss


@pytest.mark.parametrize("mode", AGGS)
@pytest.mark.parametrize("B,L", [(1, 1), (8, 256), (3, 4100)])
def test_value_loss(dev, mode, B, L):
    import siirl_amd.core_algos as CA

    g = torch.Generator().manual_seed(B + L)
    values = torch.randn(B, L, generator=g)
    vpreds = values + 0.5 * torch.randn(B, L, generator=g)
    returns = values + torch.randn(B, L, generator=g)
    m = _mask(B, L, g, "tail", torch.int64)
    clip = 0.3
    x = vpreds.to(dev).requires_grad_(True)
    loss, frac = CA.compute_value_loss(x, returns.to(dev), values.to(dev), m.to(dev), clip, mode)
    x64 = vpreds.double().requires_grad_(True)
    loss_o, frac_o = OC.compute_value_loss(x64, returns.double(), values.double(), m, clip, mode)
    assert _close(loss, loss_o) and _close(frac, frac_o), (float(loss.detach()), float(loss_o), float(frac), float(frac_o))
    l32, f32 = OC.compute_value_loss(vpreds, returns, values, m, clip, mode)
    assert abs(float(loss.detach()) - float(l32)) < 1e-3 and abs(float(frac) - float(f32)) < 1e-3
    loss.backward()
    loss_o.backward()
    ok, err = _grad_close(x.grad.cpu(), x64.grad)
    assert ok, err


def test_value_loss_ties_follow_autograd(dev):
    # float32 ties: a prediction exactly on a clip bound (min / max split the gradient), and equal to its target
    import siirl_amd.core_algos as CA

    clip = 0.3
    values = torch.tensor([[0.5, -1.25, 2.0, 0.75, 0.1]])
    returns = torch.tensor([[1.0, -2.0, 2.5, 0.25, 0.1]])
    vpreds = torch.stack([values[0, 0] + clip, values[0, 1] - clip, returns[0, 2], values[0, 3] + clip, values[0, 4]]).unsqueeze(0)
    m = torch.ones(1, 5, dtype=torch.int64)
    x = vpreds.to(dev).requires_grad_(True)
    loss, frac = CA.compute_value_loss(x, returns.to(dev), values.to(dev), m.to(dev), clip, "token-mean")
    x32 = vpreds.clone().requires_grad_(True)
    loss_o, frac_o = OC.compute_value_loss(x32, returns, values, m, clip, "token-mean")
    assert abs(float(loss.detach()) - float(loss_o)) < 1e-6 and float(frac) == float(frac_o)
    loss.backward()
    loss_o.backward()
    assert torch.allclose(x.grad.cpu(), x32.grad, rtol=1e-5, atol=1e-7), (x.grad.cpu(), x32.grad)


# ------------------------------------------------------------------------------- CPGD / GPG / GMPO


def _lossbatch(B, L, seed):
    g = torch.Generator().manual_seed(seed)
    old = torch.randn(B, L, generator=g) - 1.5
    lp = old + 0.3 * torch.randn(B, L, generator=g)
    adv = torch.randn(B, L, generator=g)
    adv[:, ::7] = 0.0  # zero advantages: sign() = 0 in GMPO
    m = _mask(B, L, g, "tail", torch.int64)
    w = torch.rand(B, L, generator=g) + 0.5
    return old, lp, adv, m, w, g


def _check_policy(dev, fn_gpu, fn_o, old, lp, adv, m, mode, cfg, w=None):
    x = lp.to(dev).requires_grad_(True)
    got = fn_gpu(old.to(dev), x, adv.to(dev), m.to(dev), mode, cfg, None if w is None else w.to(dev))
    x64 = lp.double().requires_grad_(True)
    want = fn_o(old.double(), x64, adv.double(), m, mode, cfg, None if w is None else w.double())
    want32 = fn_o(old, lp, adv, m, mode, cfg, w)
    for k in range(4):
        assert got[k].is_cuda and got[k].dim() == 0
        assert _close(got[k], want[k]), (k, float(got[k]), float(want[k]))
        assert abs(float(got[k]) - float(want32[k])) < 1e-3
    got[0].backward()
    want[0].backward()
    ok, err = _grad_close(x.grad.cpu(), x64.grad)
    assert ok, err


@pytest.mark.parametrize("mode", AGGS)
@pytest.mark.parametrize("B,L", [(1, 1), (8, 256), (3, 4100)])
def test_cpgd(dev, mode, B, L):
    import siirl_amd.core_algos as CA

    old, lp, adv, m, w, _ = _lossbatch(B, L, B * 7 + L)
    cfg = _cfg()
    _check_policy(dev, CA.compute_policy_loss_cpgd, OC.compute_policy_loss_cpgd, old, lp, adv, m, mode, cfg)
    assert CA.get_policy_loss_fn("cpgd") is CA.compute_policy_loss_cpgd


def test_cpgd_legacy_entry_and_errors(dev):
    import siirl_amd.core_algos as CA

    old, lp, adv, m, _, _ = _lossbatch(4, 33, 3)
    got = CA.compute_policy_loss(old.to(dev), lp.to(dev), adv.to(dev), m.to(dev), cliprange=0.2, cliprange_high=0.3,
                                 clip_ratio_c=3.0, loss_agg_mode="token-mean", use_cpgd_loss=True)
    want = OC.compute_policy_loss_cpgd(old.double(), lp.double(), adv.double(), m, "token-mean", _cfg(0.2, 0.3))
    for k in range(4):
        assert _close(got[k], want[k])
    with pytest.raises(ValueError):  # math.log(1 - 1.0)
        CA.compute_policy_loss_cpgd(old.to(dev), lp.to(dev), adv.to(dev), m.to(dev), "token-mean", _cfg(1.0, 0.2))
    with pytest.raises(AssertionError):
        CA.compute_policy_loss_cpgd(old.to(dev), lp.to(dev), adv.to(dev), m.to(dev), "token-mean", _cfg(c=1.0))
    with pytest.raises(AssertionError):
        CA.compute_policy_loss_cpgd(old.to(dev), lp.to(dev), adv.to(dev), m.to(dev), "token-mean", None)


@pytest.mark.parametrize("mode", AGGS)
@pytest.mark.parametrize("use_w", [False, True])
def test_gpg(dev, mode, use_w):
    import siirl_amd.core_algos as CA

    old, lp, adv, m, w, _ = _lossbatch(6, 300, 11)
    _check_policy(dev, CA.compute_policy_loss_gpg, OC.compute_policy_loss_gpg, old, lp, adv, m, mode, None,
                  w if use_w else None)
    assert CA.get_policy_loss_fn("gpg") is CA.compute_policy_loss_gpg


@pytest.mark.parametrize("B,L", [(1, 1), (8, 256), (3, 4100)])
@pytest.mark.parametrize("use_w", [False, True])
def test_geo_mean(dev, B, L, use_w):
    import siirl_amd.core_algos as CA

    old, lp, adv, m, w, _ = _lossbatch(B, L, B * 13 + L)
    cfg = _cfg(0.2, 0.28)
    _check_policy(dev, CA.compute_policy_loss_geo_mean, OC.compute_policy_loss_geo_mean, old, lp, adv, m,
                  "token-mean", cfg, w if use_w else None)
    assert CA.get_policy_loss_fn("geo_mean") is CA.compute_policy_loss_geo_mean


def test_cpgd_and_geo_mean_ties_follow_autograd(dev):
    # float32 values exactly on the clip bounds: clamp passes the gradient on the closed interval, min splits it
    import math

    import siirl_amd.core_algos as CA

    old = torch.tensor([[-1.0, -2.0, -0.5, -1.5]])
    adv = torch.tensor([[1.0, -1.0, 2.0, -0.5]])
    m = torch.ones(1, 4, dtype=torch.int64)
    cfg = _cfg(0.2, 0.28)
    lp_c = torch.stack([math.log(1 + 0.28) + old[0, 0], math.log(1 - 0.2) + old[0, 1], old[0, 2], old[0, 3]]).unsqueeze(0)
    lp_g = torch.stack([old[0, 0] + 0.28, old[0, 1] - 0.2, old[0, 2], old[0, 3] + 0.28]).unsqueeze(0)
    for fn_gpu, fn_o, lp in ((CA.compute_policy_loss_cpgd, OC.compute_policy_loss_cpgd, lp_c),
                             (CA.compute_policy_loss_geo_mean, OC.compute_policy_loss_geo_mean, lp_g)):
        x = lp.to(dev).requires_grad_(True)
        got = fn_gpu(old.to(dev), x, adv.to(dev), m.to(dev), "token-mean", cfg)
        x32 = lp.clone().requires_grad_(True)
        want = fn_o(old, x32, adv, m, "token-mean", cfg)
        for k in range(4):
            assert abs(float(got[k]) - float(want[k])) < 1e-6, (k, float(got[k]), float(want[k]))
        got[0].backward()
        want[0].backward()
        assert torch.allclose(x.grad.cpu(), x32.grad, rtol=1e-5, atol=1e-7), (x.grad.cpu(), x32.grad)


def test_geo_mean_empty_row(dev):
    # a fully masked row: 0 / (0 + 1e-8) = 0 -> ratio 1, advantage 0, loss 0 for that sequence
    import siirl_amd.core_algos as CA

    old, lp, adv, m, _, _ = _lossbatch(3, 17, 2)
    m[1] = 0
    _check_policy(dev, CA.compute_policy_loss_geo_mean, OC.compute_policy_loss_geo_mean, old, lp, adv, m,
                  "token-mean", _cfg())


# ------------------------------------------------------------------------- fused actor loss + drift


@pytest.mark.parametrize("loss_mode", ["vanilla", "cpgd", "gpg", "geo_mean"])
@pytest.mark.parametrize("agg", ["token-mean", "seq-mean-token-mean"])
def test_actor_loss_with_drift(dev, loss_mode, agg):
    import siirl_amd.core_algos as CA

    old, lp, adv, m, w, g = _lossbatch(8, 256, 99)
    ref = lp + 0.2 * torch.randn(8, 256, generator=g)
    ent = torch.rand(8, 256, generator=g) * 3
    cfg = SimpleNamespace(clip_ratio=0.2, clip_ratio_low=0.2, clip_ratio_high=0.28, clip_ratio_c=3.0,
                          entropy_coeff=0.01, use_kl_loss=True, kl_loss_coef=0.05, kl_loss_type="low_var_kl",
                          loss_agg_mode=agg, loss_mode=loss_mode, use_cpgd_loss=True, policy_drift_coeff=0.3)
    x = lp.to(dev).requires_grad_(True)
    e = ent.to(dev).requires_grad_(True)
    out = CA.actor_loss(old.to(dev), x, adv.to(dev), m.to(dev), cfg, entropy=e, ref_log_prob=ref.to(dev),
                        loss_scale_factor=0.25)
    x64 = lp.double().requires_grad_(True)
    e64 = ent.double().requires_grad_(True)
    fn = {"vanilla": OC.compute_policy_loss_vanilla, "cpgd": OC.compute_policy_loss_cpgd,
          "gpg": OC.compute_policy_loss_gpg, "geo_mean": OC.compute_policy_loss_geo_mean}[loss_mode]
    pg, *_ = fn(old.double(), x64, adv.double(), m, agg, cfg)
    drift = OC.policy_drift_loss(old.double(), x64, m, agg)
    want = (pg - 0.01 * OC.agg_loss(e64, m, agg) + 0.05 * OC.agg_loss(OC.kl_penalty(x64, ref.double(), "low_var_kl"), m, agg)
            + 0.3 * drift) * 0.25
    assert _close(out.loss, want), (float(out.loss.detach()), float(want))
    assert _close(out.policy_drift_loss, drift)
    out.loss.backward()
    want.backward()
    ok, err = _grad_close(x.grad.cpu(), x64.grad)
    assert ok, err
    ok, err = _grad_close(e.grad.cpu(), e64.grad)
    assert ok, err
    # the flag gates the term (reference dp_actor.py:488)
    cfg.use_cpgd_loss = False
    out2 = CA.actor_loss(old.to(dev), lp.to(dev), adv.to(dev), m.to(dev), cfg, entropy=ent.to(dev),
                         ref_log_prob=ref.to(dev), loss_scale_factor=0.25)
    assert _close(out2.loss, float(want) - 0.3 * 0.25 * float(drift)) and float(out2.policy_drift_loss) == 0.0


@pytest.mark.parametrize("B,L", [(5, 1024), (40, 4096), (3, 8192), (17, 2052), (2, 1000)])
@pytest.mark.parametrize("kind,mdt", [("tail", torch.int64), ("holes", torch.bool), ("holes", torch.float32)])
@pytest.mark.parametrize("gamma,lam", [(1.0, 1.0), (0.99, 0.95)])
def test_gae_chunked_scan(dev, B, L, kind, mdt, gamma, lam):
    """The chunked scan order against the fp64 oracle (float32 accuracy: 1e-5 of the largest magnitude in the row,
    the reference's own sequential float32 sum is no closer) and against the exact-order result."""
    import siirl_amd.core_algos as CA

    g = torch.Generator().manual_seed(B * 1000 + L)
    r = torch.randn(B, L, generator=g)
    v = torch.randn(B, L, generator=g)
    m = _mask(B, L, g, kind, mdt)
    m_o = m.float() if mdt == torch.bool else m
    raw64, ret64 = OC.gae_unwhitened(r.double(), v.double(), m_o.double(), gamma, lam)
    try:
        CA.set_gae_scan_order("chunked")
        adv_c, ret_c = CA.compute_gae_advantage_return(r.to(dev), v.to(dev), m.to(dev), gamma, lam)
    finally:
        CA.set_gae_scan_order("exact")
    adv_e, ret_e = CA.compute_gae_advantage_return(r.to(dev), v.to(dev), m.to(dev), gamma, lam)
    scale = raw64.abs().amax(dim=1, keepdim=True) + 1.0
    assert ((ret_c.cpu().double() - ret64).abs() <= 1e-5 * scale).all()
    assert ((ret_c - ret_e).abs().cpu().double() <= 2e-5 * scale).all()
    adv64 = OF.masked_whiten(raw64, m_o.double())
    assert ((adv_c.cpu().double() - adv64).abs() <= 1e-4 + 1e-4 * adv64.abs()).all()
    with pytest.raises(ValueError):
        CA.set_gae_scan_order("fastest")
