"""GPU parity on the five baseline configurations.

Where the CPU oracle can process the configuration in seconds it is compared in full; at the full sizes of the
large ones (10 GB of logits, 18 TFLOP of GEMM) the HIP path runs on everything and the oracle checks a seeded
sample of rows, together with size-independent properties (gradient rows summing to zero, shift invariance,
group sums of advantages, bit-exact mask bookkeeping).  Tolerances are those of the task statement: logprob /
entropy / loss 1e-3 absolute, advantages 1e-5 relative, index and mask bookkeeping bit-exact."""

from types import SimpleNamespace

import numpy as np
import pytest
import torch

from grad_bar import check_fused_grad
from oracle import actor_step as OA
from oracle import core_algos as OC
from oracle import dapo_filter as OD
from oracle import fused_linear as OFL
from oracle import torch_functional as OF

pytestmark = pytest.mark.gpu


def _bf16_grad_close(got, want64):
    err = (got.double() - want64).abs()
    return bool((err <= 2.0 ** -7 * want64.abs() + 1e-9).all()), err.max().item()


# --------------------------------------------------------------------------------------------- config 1


def test_config1_grpo_step_fp32(dev):
    """64 prompts x 8 responses, L 256, V 32000, fp32; group-norm advantages over the whole batch, then two
    micro-batches of 8 sequences through logprob -> clipped loss (eps 0.2, token-mean) + low_var_kl * 0.001 ->
    backward to the logits, against the oracle's micro-batch step."""
    import siirl_amd.core_algos as CA
    import siirl_amd.torch_functional as SF

    P, n, L, V = 64, 8, 256, 32000
    B = P * n
    g = torch.Generator().manual_seed(101)
    lens = torch.randint(16, L + 1, (B,), generator=g)
    mask = (torch.arange(L)[None, :] < lens[:, None]).long()
    rewards = torch.zeros(B, L)
    rewards[torch.arange(B), lens - 1] = (torch.rand(B, generator=g) < 0.5).float()
    uid = OD.make_uid(P, n)
    adv, _ = CA.compute_grpo_outcome_advantage(rewards.to(dev), mask.to(dev), uid)
    adv_o, _ = OC.compute_grpo_outcome_advantage(rewards, mask, uid)
    assert ((adv.cpu() - adv_o).abs() <= 1e-5 * adv_o.abs() + 1e-7).all()
    assert torch.count_nonzero(adv.cpu()[mask == 0]) == 0

    cfg = OA.ActorConfig(clip_ratio=0.2, clip_ratio_low=0.2, clip_ratio_high=0.2, clip_ratio_c=3.0, entropy_coeff=0.0,
                         use_kl_loss=True, kl_loss_coef=0.001, kl_loss_type="low_var_kl", loss_agg_mode="token-mean")
    scale = 1.0 / (B // 8)
    for mb in range(2):
        rows = slice(mb * 8, mb * 8 + 8)
        logits = torch.randn(8, L, V, generator=g) * 2.0
        labels = torch.randint(0, V, (8, L), generator=g)
        lp_o = OF.logprobs_from_logits(logits, labels)
        old = lp_o + 0.05 * torch.randn(8, L, generator=g)
        ref = lp_o + 0.1 * torch.randn(8, L, generator=g)
        loss_o, dlog_o, met_o, lp_ref, _ = OA.micro_batch_step(logits, labels, old, adv_o[rows], mask[rows], cfg,
                                                               ref_log_prob=ref, loss_scale_factor=scale)
        leaf = logits.to(dev).requires_grad_(True)
        x = leaf * 1.0  # a non-leaf, as the model's logits are
        lp = SF.logprobs_from_logits(x, labels.to(dev), inplace_backward=True)  # entropy_coeff == 0: in-place allowed
        assert (lp.detach().cpu() - lp_ref).abs().max() < 1e-3
        # drop-in composition, call by call as dp_actor.py:455-500 does
        pg, cf, kl, cfl = CA.get_policy_loss_fn("vanilla")(old_log_prob=old.to(dev), log_prob=lp, advantages=adv[rows],
                                                           response_mask=mask[rows].to(dev), loss_agg_mode="token-mean",
                                                           config=cfg, rollout_is_weights=None)
        kld = CA.kl_penalty(logprob=lp, ref_logprob=ref.to(dev), kl_penalty="low_var_kl")
        kl_loss = CA.agg_loss(loss_mat=kld, loss_mask=mask[rows].to(dev), loss_agg_mode="token-mean")
        loss = (pg + kl_loss * cfg.kl_loss_coef) * scale
        # fused single-launch composition
        fused = CA.actor_loss(old.to(dev), lp, adv[rows], mask[rows].to(dev), cfg, ref_log_prob=ref.to(dev),
                              loss_scale_factor=scale)
        loss_v, fused_v = loss.detach().item(), fused.loss.detach().item()
        assert abs(loss_v - float(loss_o)) < 1e-3 and abs(fused_v - float(loss_o)) < 1e-3
        assert abs(loss_v - fused_v) < 1e-6
        m = fused.metrics()
        for k in ("actor/pg_loss", "actor/pg_clipfrac", "actor/ppo_kl", "actor/pg_clipfrac_lower", "actor/kl_loss",
                  "actor/pg_clip_mean", "actor/pg_clip_min", "actor/pg_clip_max"):
            assert abs(m[k] - met_o[k]) < 1e-3, (k, m[k], met_o[k])
        assert abs(float(cf) - met_o["actor/pg_clipfrac"]) < 1e-3 and abs(float(kl) - met_o["actor/ppo_kl"]) < 1e-3
        loss.backward()
        got = leaf.grad.cpu()
        err = (got.double() - dlog_o.double()).abs().max().item()
        assert err < 1e-8 + 1e-4 * dlog_o.abs().max().item(), err


# --------------------------------------------------------------------------------------------- config 2


@pytest.mark.parametrize("V", [152064])
def test_config2_full_size(dev, V):
    """bf16 logits [32768, 152064] ~ N(0,3), 1% spiked rows: the HIP path runs on all rows; the oracle checks 48
    seeded rows (forward and gradient); every gradient row sums to ~0; padded rows are exactly zero."""
    import siirl_amd.torch_functional as SF

    T = 32768
    gen = torch.Generator(device=dev).manual_seed(202)
    x = torch.empty(T, V, dtype=torch.bfloat16, device=dev)
    for lo in range(0, T, 2048):
        x[lo:lo + 2048] = (torch.randn(2048, V, device=dev, generator=gen) * 3).to(torch.bfloat16)
    rows = torch.randperm(T, device=dev, generator=gen)[: T // 100]
    cols = torch.randint(0, V, (T // 100,), device=dev, generator=gen)
    x[rows, cols] = (x[rows, cols].float() + 15).to(torch.bfloat16)
    y = torch.randint(0, V, (T,), device=dev, generator=gen)
    lens = torch.randint(512, 4097, (8,), device=dev, generator=gen)
    mask = (torch.arange(4096, device=dev)[None] < lens[:, None]).reshape(T).float()
    g_lp = torch.randn(T, device=dev, generator=gen) * 1e-2 * mask
    g_h = torch.randn(T, device=dev, generator=gen) * 1e-2 * mask
    x.requires_grad_(True)
    lp, ent = SF.logprobs_and_entropy_from_logits(x, y)
    (dx,) = torch.autograd.grad([lp, ent], [x], [g_lp, g_h])
    valid = torch.nonzero(mask).flatten()
    sample = torch.cat([valid[torch.randperm(valid.numel(), device=dev, generator=gen)[:36]], rows[:8],
                        torch.nonzero(mask == 0).flatten()[:4]])
    xs, ys = x.detach()[sample].cpu(), y[sample].cpu()
    lp_o, ent_o, _, _ = OF.logprob_entropy_forward(xs, ys, dtype=torch.float32)
    assert (lp[sample].cpu() - lp_o).abs().max() < 1e-3 and (ent[sample].cpu() - ent_o).abs().max() < 1e-3
    want = OF.logprob_entropy_backward(xs, ys, g_lp[sample].cpu(), g_h[sample].cpu(), dtype=torch.float64)
    ok, err = _bf16_grad_close(dx[sample].cpu(), want)
    assert ok, err
    sums = torch.empty(T, device=dev)
    for lo in range(0, T, 4096):
        sums[lo:lo + 4096] = dx[lo:lo + 4096].float().sum(-1)
    assert sums.abs().max() < 5e-3  # 152k bf16-rounded terms of magnitude <= 1e-2 * p
    pad = torch.nonzero(mask == 0).flatten()
    assert torch.count_nonzero(dx[pad[:64]]) == 0
    assert torch.isfinite(lp).all() and (ent > 0).all() and (ent < float(np.log(V)) + 1e-3).all()


# --------------------------------------------------------------------------------------------- config 3


def test_config3_dapo_loss_path(dev):
    """512 prompts x 16 responses, lengths in [256, 8192], rewards +-1, ~30% of the groups one-signed and removed
    by dynamic sampling (bit-exact); advantages; clip 0.2 / 0.28 (c = 10), token-mean over the whole batch."""
    import siirl_amd.core_algos as CA
    import siirl_amd.dapo_filter as DF

    P, n, L = 512, 16, 8192
    B = P * n
    rng = np.random.default_rng(303)
    r = rng.choice([-1.0, 1.0], size=(P, n)).astype(np.float32)
    forced = rng.choice(P, size=154, replace=False)
    r[forced] = r[forced, :1]
    r = r.reshape(-1)
    uid = OD.make_uid(P, n)
    gen = torch.Generator(device=dev).manual_seed(303)
    lens = torch.randint(256, L + 1, (B,), device=dev, generator=gen)
    mask = (torch.arange(L, device=dev)[None, :] < lens[:, None])
    rewards = torch.zeros(B, L, device=dev)
    rewards[torch.arange(B, device=dev), lens - 1] = torch.from_numpy(r).to(dev)

    cfgf = SimpleNamespace(algorithm=SimpleNamespace(filter_groups=SimpleNamespace(enable=True, metric="seq_final_reward")))
    out = DF.dynamic_sampling(cfgf, {"uid": uid, "token_level_rewards": rewards, "response_mask": mask})
    idx_o, kept_o, _ = OD.dynamic_sampling_keep_indices(r, uid)
    kept = out.metrics["dapo_sampling/filtered_indices"]
    assert kept == idx_o and out.metrics["dapo_sampling/kept_groups"] == len(kept_o)  # bit-exact bookkeeping
    assert np.array_equal(out.batch["uid"], uid[idx_o])
    Bk = len(kept)
    assert 0.6 * B < Bk < 0.75 * B

    rew_k, mask_k = out.batch["token_level_rewards"], out.batch["response_mask"]
    adv, _ = CA.compute_grpo_outcome_advantage(rew_k, mask_k, out.batch["uid"])
    adv_o, _ = OC.compute_grpo_outcome_advantage(rew_k[:, :].cpu(), mask_k.cpu().long(), uid[idx_o])
    assert ((adv.cpu() - adv_o).abs() <= 1e-5 * adv_o.abs() + 1e-7).all()

    lp = torch.randn(Bk, L, device=dev, generator=gen) - 1.5
    old = lp + 0.05 * torch.randn(Bk, L, device=dev, generator=gen)
    cfg = SimpleNamespace(clip_ratio=0.2, clip_ratio_low=0.2, clip_ratio_high=0.28, clip_ratio_c=10.0)
    x = lp.clone().requires_grad_(True)
    pg, cf, kl, cfl = CA.compute_policy_loss_vanilla(old, x, adv, mask_k, "token-mean", cfg)
    pg.backward()
    lp_c, old_c, mask_c = lp.cpu(), old.cpu(), mask_k.cpu().long()
    want = OC.compute_policy_loss_vanilla(old_c, lp_c, adv_o, mask_c, "token-mean", cfg)
    for a, b in zip((pg, cf, kl, cfl), want):
        assert abs(a.detach().item() - float(b)) < 1e-3, (a.detach().item(), float(b))
    # gradient: full fp64 autograd on the first 256 kept rows with the batch-wide token count as the normaliser
    sub = slice(0, 256)
    x64 = lp_c[sub].double().requires_grad_(True)
    pg_sub, *_ = OC.compute_policy_loss_vanilla(old_c[sub].double(), x64, adv_o[sub].double(), mask_c[sub], "seq-mean-token-sum", cfg)
    (pg_sub * 256 / mask_c.sum().double()).backward()  # token-mean over the whole batch = sum / total tokens
    g = x.grad[sub].cpu().double()
    assert ((g - x64.grad).abs() <= 1e-12 + 1e-5 * x64.grad.abs()).all()


# --------------------------------------------------------------------------------------------- config 4


def test_config4_gspo_long_context(dev):
    """One 32768-token sequence at V = 151936 (Qwen3), bf16: logprob -> GSPO loss (eps 3e-4 / 4e-4,
    seq-mean-token-mean) -> backward to the logits.  The loss-level oracle runs on the whole [1, 32768] row; the
    [T, V] oracle runs on 40 sampled tokens; a 2 x 512-token micro-batch is checked end to end."""
    import siirl_amd.core_algos as CA
    import siirl_amd.torch_functional as SF

    V = 151936
    cfg = SimpleNamespace(clip_ratio=0.2, clip_ratio_low=3e-4, clip_ratio_high=4e-4, clip_ratio_c=3.0)
    gen = torch.Generator(device=dev).manual_seed(404)
    # (a) full length, one sequence per micro-batch
    L = 32768
    x = torch.empty(L, V, dtype=torch.bfloat16, device=dev)
    for lo in range(0, L, 2048):
        x[lo:lo + 2048] = (torch.randn(2048, V, device=dev, generator=gen) * 3).to(torch.bfloat16)
    y = torch.randint(0, V, (L,), device=dev, generator=gen)
    n_valid = 30000
    mask = (torch.arange(L, device=dev) < n_valid).long()[None]
    adv = torch.full((1, L), 0.7, device=dev)
    xr = x.view(1, L, V).requires_grad_(True)
    lp = SF.logprobs_from_logits(xr, y[None], inplace_backward=False)
    old = lp.detach() - 0.02 * torch.randn(1, L, device=dev, generator=gen)
    pg, cf, kl, cfl = CA.compute_policy_loss_gspo(old, lp, adv, mask, "token-mean", cfg)
    want = OC.compute_policy_loss_gspo(old.cpu().double(), lp.detach().cpu().double(), adv.cpu().double(), mask.cpu(),
                                       "token-mean", cfg)
    for a, b in zip((pg, cf, kl, cfl), want):
        assert abs(a.detach().item() - float(b)) < 1e-3, (a.detach().item(), float(b))
    sample = torch.randperm(L, device=dev, generator=gen)[:40]
    lp_o = OF.logprobs_from_logits(x[sample].cpu(), y[sample].cpu())
    assert (lp.detach()[0, sample].cpu() - lp_o).abs().max() < 1e-3
    pg.backward()
    dx = xr.grad[0]
    # oracle gradient: d loss / d lp from autograd on the fp64 loss, pushed through the closed-form logprob backward
    lp64 = lp.detach().cpu().double().requires_grad_(True)
    OC.compute_policy_loss_gspo(old.cpu().double(), lp64, adv.cpu().double(), mask.cpu(), "token-mean", cfg)[0].backward()
    g_lp = lp64.grad[0, sample.cpu()]
    want_dx = OF.logprob_entropy_backward(x[sample].cpu(), y[sample].cpu(), g_lp, None, dtype=torch.float64)
    ok, err = _bf16_grad_close(dx[sample].cpu(), want_dx)
    assert ok, err
    assert torch.count_nonzero(dx[n_valid:n_valid + 64]) == 0  # masked tokens receive no gradient
    del x, xr, dx, lp
    # (b) a small micro-batch end to end against the oracle step
    Bm, Lm = 2, 512
    logits = (torch.randn(Bm, Lm, V, generator=torch.Generator().manual_seed(5)) * 3).to(torch.bfloat16)
    labels = torch.randint(0, V, (Bm, Lm), generator=torch.Generator().manual_seed(6))
    lens = torch.tensor([512, 300])
    m = (torch.arange(Lm)[None] < lens[:, None]).long()
    lp_ref = OF.logprobs_from_logits(logits, labels)
    oldm = lp_ref - 0.02 * torch.randn(Bm, Lm, generator=torch.Generator().manual_seed(7))
    advm = torch.tensor([[1.0], [-0.5]]).expand(Bm, Lm).contiguous()
    ocfg = OA.ActorConfig(clip_ratio=0.2, clip_ratio_low=3e-4, clip_ratio_high=4e-4, loss_agg_mode="seq-mean-token-mean",
                          loss_mode="gspo")
    loss_o, dlog_o, met_o, _, _ = OA.micro_batch_step(logits, labels, oldm, advm, m, ocfg, dtype=torch.float64)
    xd = logits.to(dev).requires_grad_(True)
    lpd = SF.logprobs_from_logits(xd, labels.to(dev))
    res = CA.actor_loss(oldm.to(dev), lpd, advm.to(dev), m.to(dev), ocfg)
    assert abs(float(res.loss.detach()) - float(loss_o)) < 1e-3
    assert abs(float(res.pg_clipfrac) - met_o["actor/pg_clipfrac"]) < 1e-3
    res.loss.backward()
    ok, err = _bf16_grad_close(xd.grad.cpu(), dlog_o)
    assert ok, err


# --------------------------------------------------------------------------------------------- config 5


def test_config5_fused_full_vocab_reduced_tokens(dev):
    """hidden [256, 3584], W [152064, 3584] (full hidden size and vocabulary, 256 tokens): complete oracle
    comparison, forward and both gradients."""
    from siirl_amd.fused_linear import fused_linear_logprob_entropy

    T, H, V = 256, 3584, 152064
    g = torch.Generator().manual_seed(505)
    h = torch.randn(T, H, generator=g).to(torch.bfloat16)
    w = (torch.randn(V, H, generator=g) * 0.02).to(torch.bfloat16)
    y = torch.randint(0, V, (T,), generator=g)
    g_lp, g_h = torch.randn(T, generator=g) * 1e-2, torch.randn(T, generator=g) * 1e-2
    hd, wd = h.to(dev).requires_grad_(True), w.to(dev).requires_grad_(True)
    lp, ent = fused_linear_logprob_entropy(hd, wd, y.to(dev))
    lp_o, ent_o = OFL.fused_linear_for_ppo_fwd(h, w, y, dtype=torch.float32)
    assert (lp.cpu() - lp_o).abs().max() < 1e-3 and (ent.cpu() - ent_o).abs().max() < 1e-3
    torch.autograd.backward([lp, ent], [g_lp.to(dev), g_h.to(dev)])
    dh_o, dw_o = OFL.fused_linear_for_ppo_bwd(g_lp, g_h, h, w, y, dtype=torch.float32)
    for got, want, name in ((hd.grad, dh_o, "d_hidden"), (wd.grad, dw_o, "d_weight")):
        check_fused_grad(got, want.double(), f"config 5, 256 tokens, {name}", floor=1e-9)


def test_config5_full_size_sampled(dev):
    """hidden [16384, 3584], W [152064, 3584]: the fused path runs in full; the oracle checks 24 sampled tokens
    (forward, d_hidden rows) and 16 sampled vocabulary rows of d_weight (using the per-token lse / ex that the
    forward produced, themselves checked on the sampled tokens)."""
    import siirl_amd.torch_functional as SF  # noqa: F401
    from siirl_amd.fused_linear import fused_linear_logprob_entropy

    T, H, V = 16384, 3584, 152064
    gen = torch.Generator(device=dev).manual_seed(506)
    h = torch.randn(T, H, device=dev, generator=gen).to(torch.bfloat16)
    w = torch.empty(V, H, dtype=torch.bfloat16, device=dev)
    for lo in range(0, V, 16384):
        n = min(16384, V - lo)
        w[lo:lo + n] = (torch.randn(n, H, device=dev, generator=gen) * 0.02).to(torch.bfloat16)
    y = torch.randint(0, V, (T,), device=dev, generator=gen)
    g_lp = torch.randn(T, device=dev, generator=gen) * 1e-2
    g_h = torch.randn(T, device=dev, generator=gen) * 1e-2
    hd, wd = h.clone().requires_grad_(True), w.clone().requires_grad_(True)
    lp, ent = fused_linear_logprob_entropy(hd, wd, y)
    torch.autograd.backward([lp, ent], [g_lp, g_h])
    ts = torch.randperm(T, device=dev, generator=gen)[:24]
    w_c = w.cpu()
    lp_o, ent_o = OFL.fused_linear_for_ppo_fwd(h[ts].cpu(), w_c, y[ts].cpu(), dtype=torch.float32)
    assert (lp[ts].cpu() - lp_o).abs().max() < 1e-3 and (ent[ts].cpu() - ent_o).abs().max() < 1e-3
    # d_hidden rows of the sampled tokens (each token's row depends on that token only)
    logits = h[ts].cpu().float() @ w_c.float().t()
    dlog = OF.logprob_entropy_backward(logits, y[ts].cpu(), g_lp[ts].cpu(), g_h[ts].cpu(), dtype=torch.float64)
    dh_o = dlog @ w_c.double()
    check_fused_grad(hd.grad[ts], dh_o, "config 5, full size, d_hidden rows of 24 tokens", floor=0.0)
    # d_weight rows of sampled vocabulary entries: sum over all tokens of dlogits[t, v] * hidden[t]
    vs = torch.cat([torch.randperm(V, device=dev, generator=gen)[:12], y[:4]])
    z = (h.float() @ w[vs].float().t())  # [T, 16] fp32 logits of the sampled columns (torch, as a checker)
    lse = (lp.detach() * 0)  # placeholders replaced below
    zy = (h.float() * w[y].float()).sum(-1)
    lse = zy - lp.detach()  # logprob = z_y - lse
    ex = lse - ent.detach()
    p = torch.exp(z - lse[:, None])
    onehot = (y[:, None] == vs[None, :]).float()
    d = g_lp[:, None] * (onehot - p) - g_h[:, None] * p * (z - ex[:, None])
    dw_o = (d.double().t() @ h.double()).cpu()
    check_fused_grad(wd.grad[vs], dw_o, "config 5, full size, d_weight rows of 16 vocabulary entries", floor=1e-9)
