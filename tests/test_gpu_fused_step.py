"""GPU parity: the single-pass logits -> dlogits actor step and the forward+backward-in-one entry point (through
the C ABI) vs the CPU oracle's micro-batch step and vs the two-launch path.

Tolerances: log-prob / entropy / loss within 1e-3 absolute of the fp32 oracle (observed ~1e-5 against fp64);
dlogits within one unit in the last place of the logits dtype of the fp64 oracle's gradient (plus 1e-7 absolute)."""
from dataclasses import replace

import pytest
import torch

from oracle import actor_step as OA

pytestmark = pytest.mark.gpu

ULP = {torch.bfloat16: 2.0 ** -8, torch.float16: 2.0 ** -11, torch.float32: 2.0 ** -23}


def _inputs(B, L, V, dtype, seed):
    g = torch.Generator().manual_seed(seed)
    logits = (torch.randn(B, L, V, generator=g) * 3).to(dtype)
    resp = torch.randint(0, V, (B, L), generator=g)
    lens = torch.randint(1, L + 1, (B,), generator=g)
    mask = (torch.arange(L)[None] < lens[:, None]).long()
    with torch.no_grad():
        lp = torch.log_softmax(logits.float(), -1).gather(-1, resp[..., None])[..., 0]
    old = lp + 0.3 * torch.randn(B, L, generator=g)
    ref = lp + 0.2 * torch.randn(B, L, generator=g)
    adv = torch.randn(B, 1, generator=g).expand(B, L).contiguous()
    isw = torch.rand(B, L, generator=g) + 0.5
    return logits, resp, mask, old, ref, adv, isw


def _check(dev, logits, resp, mask, old, ref, adv, isw, cfg, T=1.0, scale=1.0, on_policy=False, use_isw=False,
           gpu_logits=None):
    import siirl_amd.core_algos as CA

    x = logits.to(dev) if gpu_logits is None else gpu_logits
    out = CA.fused_actor_step(x, resp.to(dev), None if on_policy else old.to(dev), adv.to(dev), mask.to(dev), cfg,
                              ref_log_prob=ref.to(dev) if cfg.use_kl_loss else None, temperature=T,
                              loss_scale_factor=scale, on_policy=on_policy,
                              rollout_is_weights=isw.to(dev) if use_isw else None)
    loss_o, d_o, met_o, lp_o, ent_o = OA.micro_batch_step(
        logits, resp, old.double(), adv.double(), mask, cfg, ref_log_prob=ref.double(), temperature=T,
        loss_scale_factor=scale, on_policy=on_policy, rollout_is_weights=isw.double() if use_isw else None,
        dtype=torch.float64)
    assert out.dlogits.shape == x.shape and out.dlogits.dtype == x.dtype
    assert abs(float(out.loss.detach()) - float(loss_o)) < 1e-3 * max(1.0, abs(float(loss_o)))
    valid = mask.bool()
    assert (out.log_prob.cpu()[valid].double() - lp_o[valid]).abs().max() < 1e-3
    if ent_o is not None:
        assert (out.entropy.cpu()[valid].double() - ent_o[valid]).abs().max() < 1e-3
    got = out.dlogits.cpu().double()
    err = (got - d_o).abs()
    tol = 1e-7 + 1.01 * ULP[logits.dtype] * d_o.abs()
    if logits.dtype == torch.float32:  # fp32 arithmetic: lse and E[z] carry about 2^-23 * |z| of rounding into p
        tol = tol + 2e-7 + 4e-6 * d_o.abs()
    # at a label whose probability is within 1e-4 of one, `g * (1 - p)` cancels in fp32 (here and in the reference's
    # autograd alike): a few fp32 ulps of the token's upstream gradient g, bounded through its advantage
    tol = tol + (2.0 ** -21 * scale * (1 + 5 * adv.double().abs())).unsqueeze(-1)
    assert bool((err <= tol).all()), (err.max().item(), (err / tol).max().item())
    m = out.metrics()
    for k in ("actor/pg_loss", "actor/pg_clipfrac", "actor/ppo_kl", "actor/pg_clipfrac_lower"):
        assert abs(m[k] - met_o[k]) < 1e-3, (k, m[k], met_o[k])
    return out


@pytest.mark.parametrize("B,L,V,dtype", [(2, 5, 1000, torch.float32), (3, 9, 50257, torch.bfloat16),
                                         (1, 4, 152064, torch.bfloat16), (2, 3, 32000, torch.float16),
                                         (1, 2, 200000, torch.bfloat16)])
@pytest.mark.parametrize("mode", ["vanilla", "cpgd", "gpg"])
def test_fused_step_matches_oracle(dev, B, L, V, dtype, mode):
    inp = _inputs(B, L, V, dtype, seed=B * 100 + L + V)
    cfg = OA.ActorConfig(clip_ratio_low=0.2, clip_ratio_high=0.28, clip_ratio_c=3.0, entropy_coeff=0.01,
                         use_kl_loss=True, kl_loss_coef=0.05, kl_loss_type="low_var_kl", loss_mode=mode,
                         use_cpgd_loss=(mode == "cpgd"), policy_drift_coeff=0.2)
    _check(dev, *inp, cfg, T=0.8, scale=0.5, use_isw=(mode != "cpgd"))


@pytest.mark.parametrize("agg", ["token-mean", "seq-mean-token-sum", "seq-mean-token-mean", "seq-mean-token-sum-norm"])
@pytest.mark.parametrize("on_policy", [False, True])
def test_fused_step_agg_modes_and_on_policy(dev, agg, on_policy):
    inp = _inputs(4, 17, 5000, torch.bfloat16, seed=7)
    cfg = OA.ActorConfig(clip_ratio_low=0.2, clip_ratio_high=0.28, loss_agg_mode=agg, entropy_coeff=0.0)
    out = _check(dev, *inp, cfg, on_policy=on_policy)
    assert out.entropy is None


def test_fused_step_strided_view_and_two_pass_agreement(dev):
    import siirl_amd.core_algos as CA
    import siirl_amd.torch_functional as F

    B, S, L, V = 3, 12, 6, 3000
    g = torch.Generator().manual_seed(3)
    full = (torch.randn(B, S, V, generator=g) * 2).to(torch.bfloat16).to(dev)
    view = full[:, -L - 1:-1]  # the actor's response window (dp_actor.py:231), B row blocks
    logits, resp, mask, old, ref, adv, isw = _inputs(B, L, V, torch.bfloat16, seed=4)
    cfg = OA.ActorConfig(entropy_coeff=0.02, use_kl_loss=True, kl_loss_coef=0.01)
    out = _check(dev, view.cpu(), resp, mask, old, ref, adv, isw, cfg, gpu_logits=view)
    # the same step through the two-launch path of this library
    x = view.contiguous().requires_grad_(True)
    lp = F.logprobs_from_logits(x, resp.to(dev), inplace_backward=False)
    ent = F.entropy_from_logits(x)
    two = CA.actor_loss(old.to(dev), lp, adv.to(dev), mask.to(dev), cfg, entropy=ent, ref_log_prob=ref.to(dev))
    two.loss.backward()
    diff = (x.grad.float() - out.dlogits.float()).abs()
    assert bool((diff <= 1e-7 + 2 ** -7 * x.grad.float().abs()).all()), diff.max()
    assert abs(float(two.loss.detach()) - float(out.loss.detach())) < 1e-5


def test_fused_step_masked_rows_are_zero_and_errors(dev):
    import siirl_amd.core_algos as CA

    logits, resp, mask, old, ref, adv, isw = _inputs(2, 6, 700, torch.bfloat16, seed=9)
    mask[0, 3:] = 0
    mask[1, :] = 0
    resp[1, 2] = -100  # a padding label under a zero mask must not poison anything
    cfg = OA.ActorConfig()
    out = CA.fused_actor_step(logits.to(dev), resp.to(dev), old.to(dev), adv.to(dev), mask.to(dev), cfg)
    assert float(out.dlogits[0, 3:].float().abs().max()) == 0.0 and float(out.dlogits[1].float().abs().max()) == 0.0
    assert float(out.dlogits[0, :3].float().abs().max()) > 0.0 and bool(torch.isfinite(out.dlogits.float()).all())
    with pytest.raises(ValueError, match="token-separable"):
        CA.fused_actor_step(logits.to(dev), resp.to(dev), old.to(dev), adv.to(dev), mask.to(dev),
                            replace(cfg, loss_mode="gspo"))
    with pytest.raises(RuntimeError):
        CA.fused_actor_step(logits, resp, old, adv, mask, cfg)


@pytest.mark.parametrize("T,V,dtype", [(5, 1000, torch.float32), (33, 50257, torch.bfloat16), (3, 152064, torch.bfloat16)])
def test_fwd_bwd_entry_equals_two_launches(dev, T, V, dtype):
    from siirl_amd import _lib

    h = _lib.lib()
    g = torch.Generator().manual_seed(T + V)
    x = (torch.randn(T, V, generator=g) * 3).to(dtype).to(dev)
    y = torch.randint(0, V, (T,), generator=g).to(dev)
    g1 = (torch.randn(T, generator=g) * 1e-2).to(dev)
    g2 = (torch.randn(T, generator=g) * 1e-2).to(dev)
    g1[0] = 0.0
    g2[0] = 0.0
    code = _lib.dtype_code(dtype)
    st = _lib.current_stream(dev)
    lp, ent, lse, ex, lp2, ent2 = (torch.empty(T, device=dev) for _ in range(6))
    d, d2 = torch.empty_like(x), torch.empty_like(x)
    _lib.check(h.siirl_logprob_entropy_fwd_bwd(_lib.ptr(x), code, T, V, V, _lib.ptr(y), 1.0, _lib.ptr(g1), _lib.ptr(g2),
                                               _lib.ptr(lp), _lib.ptr(ent), _lib.ptr(d), V, st), "fwd_bwd")
    _lib.check(h.siirl_logprob_entropy_fwd(_lib.ptr(x), code, T, V, V, _lib.ptr(y), 1.0, _lib.ptr(lp2), _lib.ptr(ent2),
                                           _lib.ptr(lse), _lib.ptr(ex), st), "fwd")
    _lib.check(h.siirl_logprob_entropy_bwd(_lib.ptr(x), code, T, V, V, _lib.ptr(y), 1.0, _lib.ptr(lse), _lib.ptr(ex),
                                           _lib.ptr(g1), _lib.ptr(g2), _lib.ptr(d2), V, 0, st), "bwd")
    assert (lp - lp2).abs().max() < 1e-5 and (ent - ent2).abs().max() < 1e-4
    diff = (d.float() - d2.float()).abs()
    assert bool((diff <= 1e-9 + 2 * ULP[dtype] * d2.float().abs()).all()), diff.max()
    assert float(d[0].float().abs().max()) == 0.0
    assert h.siirl_logprob_entropy_fwd_bwd(_lib.ptr(x), code, T, V, V, _lib.ptr(y), 1.0, _lib.ptr(g1), None, None, None,
                                           _lib.ptr(x), V, st) == -1  # no in-place mode


@pytest.mark.parametrize("V,dtype", [(1000, torch.float32), (50257, torch.bfloat16)])
def test_skip_labelled_rows_agree_between_the_paths(dev, V, dtype):
    """Rows labelled LABEL_SKIP_ROW (packed tokens outside the response window): the single-launch entry and the
    two-launch kernels give the same answer -- log-prob and entropy 0, a gradient of zeros whatever the upstream
    gradients are -- and neither reads the row (it holds NaN here)."""
    from siirl_amd import _lib
    from siirl_amd.padding import LABEL_SKIP_ROW

    h = _lib.lib()
    T = 9
    g = torch.Generator().manual_seed(V)
    x = (torch.randn(T, V, generator=g) * 3).to(dtype)
    y = torch.randint(0, V, (T,), generator=g)
    skipped = torch.tensor([1, 4, 8])
    y[skipped] = LABEL_SKIP_ROW
    x[skipped] = float("nan")
    x, y = x.to(dev), y.to(dev)
    g1 = (torch.randn(T, generator=g) * 1e-2).to(dev)  # non-zero on the skipped rows as well
    g2 = (torch.randn(T, generator=g) * 1e-2).to(dev)
    code, st = _lib.dtype_code(dtype), _lib.current_stream(dev)
    lp, ent, lse, ex, lp2, ent2 = (torch.full((T,), 7.0, device=dev) for _ in range(6))
    d, d2 = torch.full_like(x, 7.0), torch.full_like(x, 7.0)
    _lib.check(h.siirl_logprob_entropy_fwd_bwd(_lib.ptr(x), code, T, V, V, _lib.ptr(y), 1.0, _lib.ptr(g1), _lib.ptr(g2),
                                               _lib.ptr(lp), _lib.ptr(ent), _lib.ptr(d), V, st), "fwd_bwd")
    _lib.check(h.siirl_logprob_entropy_fwd(_lib.ptr(x), code, T, V, V, _lib.ptr(y), 1.0, _lib.ptr(lp2), _lib.ptr(ent2),
                                           _lib.ptr(lse), _lib.ptr(ex), st), "fwd")
    _lib.check(h.siirl_logprob_entropy_bwd(_lib.ptr(x), code, T, V, V, _lib.ptr(y), 1.0, _lib.ptr(lse), _lib.ptr(ex),
                                           _lib.ptr(g1), _lib.ptr(g2), _lib.ptr(d2), V, 1, st), "bwd")
    sk = skipped.to(dev)
    for t in (lp, ent, lp2, ent2):
        assert torch.count_nonzero(t[sk]) == 0
    assert torch.count_nonzero(d[sk]) == 0 and torch.count_nonzero(d2[sk]) == 0
    live = torch.ones(T, dtype=torch.bool, device=dev)
    live[sk] = False
    assert (lp[live] - lp2[live]).abs().max() < 1e-5 and (ent[live] - ent2[live]).abs().max() < 1e-4
    diff = (d[live].float() - d2[live].float()).abs()
    assert bool((diff <= 1e-9 + 2 * ULP[dtype] * d2[live].float().abs()).all()), diff.max()
    assert bool(torch.isfinite(d.float()).all()) and bool(torch.isfinite(d2.float()).all())


def test_fused_step_random_sweep(dev):
    """Seeded random shapes, dtypes, loss modes, aggregation modes, coefficients and temperatures through the
    single-pass step, each against the oracle's micro-batch step (tolerances of _check).  ``SIIRL_TEST_SEED=<int>`` in
    the environment shifts the seeds."""
    import os
    import random

    shift = 100003 * int(os.environ.get("SIIRL_TEST_SEED", "0"))
    rnd = random.Random(77 + shift)
    aggs = ["token-mean", "seq-mean-token-sum", "seq-mean-token-mean", "seq-mean-token-sum-norm"]
    for case in range(40):
        B, L = rnd.randint(1, 5), rnd.randint(1, 24)
        V = rnd.choice([2, 17, 255, 1000, 4097, 32000, 50257, rnd.randint(2, 70000)])
        dtype = rnd.choice([torch.bfloat16, torch.float32, torch.float16])
        mode = rnd.choice(["vanilla", "vanilla", "cpgd", "gpg"])
        cfg = OA.ActorConfig(clip_ratio_low=rnd.choice([0.1, 0.2]), clip_ratio_high=rnd.choice([0.2, 0.28]),
                             clip_ratio_c=rnd.choice([1.5, 3.0]), entropy_coeff=rnd.choice([0.0, 0.01]),
                             use_kl_loss=rnd.random() < 0.5, kl_loss_coef=0.05,
                             kl_loss_type=rnd.choice(["low_var_kl", "kl", "mse", "abs"]), loss_mode=mode,
                             loss_agg_mode=rnd.choice(aggs), use_cpgd_loss=(mode == "cpgd"), policy_drift_coeff=0.2)
        inp = _inputs(B, L, V, dtype, seed=1000 + case + shift)
        print(f"[sweep case {case}] B={B} L={L} V={V} {dtype} {mode} {cfg.loss_agg_mode} kl={cfg.use_kl_loss}", flush=True)
        _check(dev, *inp, cfg, T=rnd.choice([1.0, 0.8, 1.3]), scale=rnd.choice([1.0, 0.25]),
               on_policy=(mode == "vanilla" and rnd.random() < 0.2), use_isw=(mode != "cpgd" and rnd.random() < 0.5))
