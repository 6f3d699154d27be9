"""GPU checks at the baseline configurations' full sizes for the operations around the hot path (GAE, whitening,
value loss, data metrics, remove-padding bookkeeping, single-pass actor step), through size-independent properties:
closed forms, round trips, invariance to row order, agreement between two independent routes through the library."""
from types import SimpleNamespace

import pytest
import torch

pytestmark = pytest.mark.gpu


def test_config3_gae_closed_form_and_whitening(dev):
    # gamma = lam = 1, full mask: returns are the reward-to-go (exact for 0/1 rewards), advantages whiten to mean 0 / var 1
    import siirl_amd.core_algos as CA

    B, L = 2048, 8192
    g = torch.Generator(device=dev).manual_seed(0)
    r = (torch.rand(B, L, device=dev, generator=g) < 0.01).float()
    v = torch.randn(B, L, device=dev, generator=g)
    m = torch.ones(B, L, device=dev, dtype=torch.int64)
    adv, ret = CA.compute_gae_advantage_return(r, v, m, 1.0, 1.0)
    rtg = torch.flip(torch.cumsum(torch.flip(r.double(), [1]), 1), [1])
    assert (ret.double() - rtg).abs().max() < 1e-3  # |sum| <= ~120, float32 partial sums of integers and values
    a = adv.double()
    assert abs(float(a.mean())) < 1e-5 and abs(float(a.var(unbiased=True)) - 1.0) < 1e-4
    # trailing padding does not change the valid part (per-row truncation property), in bits
    m2 = m.clone()
    m2[:, L // 2:] = 0
    _, ret2 = CA.compute_gae_advantage_return(r[:, :L // 2].contiguous(), v[:, :L // 2].contiguous(),
                                              m[:, :L // 2].contiguous(), 1.0, 1.0)
    _, ret3 = CA.compute_gae_advantage_return(r, v, m2, 1.0, 1.0)
    assert torch.equal(ret3[:, :L // 2], ret2)


def test_config3_value_loss_two_routes(dev):
    # the fused value loss equals the library's own agg_loss over the token formula written with torch ops
    import siirl_amd.core_algos as CA

    B, L = 1024, 8192
    g = torch.Generator(device=dev).manual_seed(1)
    values = torch.randn(B, L, device=dev, generator=g)
    vpreds = (values + 0.5 * torch.randn(B, L, device=dev, generator=g)).requires_grad_(True)
    returns = values + torch.randn(B, L, device=dev, generator=g)
    lens = torch.randint(1, L + 1, (B,), device=dev, generator=g)
    m = (torch.arange(L, device=dev)[None] < lens[:, None]).long()
    loss, frac = CA.compute_value_loss(vpreds, returns, values, m, 0.3, "seq-mean-token-mean")
    (g1,) = torch.autograd.grad(loss, vpreds)
    vp2 = vpreds.detach().clone().requires_grad_(True)
    vc = torch.max(torch.min(vp2, values + 0.3), values - 0.3)
    tok = torch.max((vp2 - returns) ** 2, (vc - returns) ** 2)
    loss2 = 0.5 * CA.agg_loss(tok, m, "seq-mean-token-mean")
    (g2,) = torch.autograd.grad(loss2, vp2)
    assert abs(float(loss.detach()) - float(loss2.detach())) < 1e-5 * abs(float(loss2.detach())) + 1e-7
    assert (g1 - g2).abs().max() <= 1e-9 + 1e-5 * g2.abs().max()


def test_config3_metrics_row_order_invariance(dev):
    from siirl_amd.metric_utils import compute_data_metric

    B, P, L = 4096, 512, 8192
    g = torch.Generator(device=dev).manual_seed(2)
    lens = torch.randint(1, L + 1, (B,), device=dev, generator=g)
    rm = (torch.arange(L, device=dev)[None] < lens[:, None]).long()
    data = {"token_level_scores": torch.zeros(B, L, device=dev), "advantages": torch.randn(B, L, device=dev, generator=g),
            "returns": torch.randn(B, L, device=dev, generator=g), "values": torch.randn(B, L, device=dev, generator=g),
            "responses": torch.zeros(B, L, dtype=torch.long, device=dev),
            "attention_mask": torch.cat([torch.ones(B, P, dtype=torch.long, device=dev), rm], 1), "response_mask": rm}
    data["token_level_scores"][torch.arange(B, device=dev), lens - 1] = (torch.rand(B, device=dev, generator=g) < 0.5).float()
    data["token_level_rewards"] = data["token_level_scores"]
    a = compute_data_metric(data)
    perm = torch.randperm(B, device=dev, generator=g)
    b = compute_data_metric({k: v[perm] for k, v in data.items()})
    for k, v in a.items():
        if k.startswith("perf/"):
            continue
        assert abs(v - b[k]) <= 1e-6 + 1e-6 * abs(v), (k, v, b[k])
    assert a["response/length/max"] <= L and a["prompt/clip_ratio/mean"] == 1.0
    assert abs(a["critic/score/mean"] - float(data["token_level_scores"].sum(-1).mean())) < 1e-6
    assert a["response/length/mean"] == pytest.approx(float(lens.float().mean()), rel=1e-6)


def test_config4_unpad_round_trip_long_context(dev):
    import siirl_amd.padding as P

    B, S, L = 32, 32768 + 2048, 32768
    g = torch.Generator(device=dev).manual_seed(3)
    plen = torch.randint(1, S - L + 1, (B,), device=dev, generator=g)
    rlen = torch.randint(1, L + 1, (B,), device=dev, generator=g)
    pos = torch.arange(S, device=dev)[None]
    mask = ((pos >= (S - L - plen)[:, None]) & (pos < (S - L + rlen)[:, None])).long()
    ids = torch.randint(0, 151936, (B, S), device=dev, generator=g)
    rm, rolled, idx, cu, mx = P.unpad_ids_and_labels(ids, mask)
    nnz = int(mask.sum())
    assert idx.numel() == nnz and int(cu[-1]) == nnz and mx == int(mask.sum(1).max())
    assert bool((idx[1:] > idx[:-1]).all()) and bool(mask.flatten()[idx].all())
    assert torch.equal(rm[0], ids.flatten()[idx]) and torch.equal(rolled, torch.roll(rm[0], -1))
    vals = torch.randn(nnz, device=dev, generator=g)
    win = P.pad_and_slice_response(vals, idx, B, S, L)
    full = torch.zeros(B * S, device=dev)
    full[idx] = vals
    assert torch.equal(win, full.view(B, S)[:, -L - 1:-1])
    assert torch.equal(P.pad_input(P.index_first_axis(ids.flatten()[:, None].float(), idx), idx, B, S)[..., 0],
                       (ids * mask).float())


def test_config2_fused_step_equals_two_launch_path(dev):
    # 4096 rows of the headline vocabulary: the single-pass step against forward + actor_loss + backward
    import siirl_amd.core_algos as CA
    import siirl_amd.torch_functional as F

    B, L, V = 2, 2048, 152064
    g = torch.Generator(device=dev).manual_seed(4)
    x = (torch.randn(B, L, V, device=dev, generator=g) * 3).to(torch.bfloat16)
    y = torch.randint(0, V, (B, L), device=dev, generator=g)
    lens = torch.tensor([L, L // 3], device=dev)
    m = (torch.arange(L, device=dev)[None] < lens[:, None]).long()
    with torch.no_grad():
        lp0 = F.logprobs_from_logits(x, y)
    old = lp0 + 0.1 * torch.randn(B, L, device=dev, generator=g)
    ref = lp0 + 0.1 * torch.randn(B, L, device=dev, generator=g)
    adv = torch.randn(B, 1, device=dev, generator=g).expand(B, L).contiguous()
    cfg = SimpleNamespace(clip_ratio=0.2, clip_ratio_low=0.2, clip_ratio_high=0.28, clip_ratio_c=3.0, entropy_coeff=0.001,
                          use_kl_loss=True, kl_loss_coef=0.001, kl_loss_type="low_var_kl", loss_agg_mode="token-mean",
                          loss_mode="vanilla")
    out = CA.fused_actor_step(x, y, old, adv, m, cfg, ref_log_prob=ref, loss_scale_factor=0.25)
    xr = x.clone().requires_grad_(True)
    lp = F.logprobs_from_logits(xr, y, inplace_backward=False)
    ent = F.entropy_from_logits(xr)
    two = CA.actor_loss(old, lp, adv, m, cfg, entropy=ent, ref_log_prob=ref, loss_scale_factor=0.25)
    two.loss.backward()
    assert abs(float(two.loss.detach()) - float(out.loss.detach())) < 1e-6
    diff = (xr.grad.float() - out.dlogits.float()).abs()
    assert bool((diff <= 1e-12 + 2 ** -7 * xr.grad.float().abs()).all()), diff.max()
    # rows past the response lengths carry no gradient; rows sum to ~0 (softmax gradients)
    assert float(out.dlogits[1, L // 3:].float().abs().max()) == 0.0
    assert float(out.dlogits[0].float().sum(-1).abs().max()) < 1e-4
