"""The small-batch step under HIP graph capture, captured once and replayed with new data; every replay must equal the
eager result bit for bit (the library's entry points allocate nothing and never synchronise): the single-pass actor
step of a config-1 micro-batch ([8, 256] responses, 32000-entry fp32 vocabulary), and the actor's own sequence of the
reference-named functions with autograd inside the capture."""
import pytest
import torch

pytestmark = pytest.mark.gpu


def test_fused_step_replays_under_graph_capture(dev):
    from types import SimpleNamespace

    import siirl_amd.core_algos as CA

    B, L, V = 8, 256, 32000
    cfg = SimpleNamespace(clip_ratio=0.2, clip_ratio_low=0.2, clip_ratio_high=0.2, clip_ratio_c=3.0, entropy_coeff=0.001,
                          use_kl_loss=True, kl_loss_coef=0.001, kl_loss_type="low_var_kl", loss_agg_mode="token-mean",
                          loss_mode="vanilla")
    g = torch.Generator(device=dev).manual_seed(0)

    def fresh():
        x = torch.randn(B, L, V, device=dev, generator=g) * 2
        y = torch.randint(0, V, (B, L), device=dev, generator=g)
        lens = torch.randint(1, L + 1, (B,), device=dev, generator=g)
        m = (torch.arange(L, device=dev)[None] < lens[:, None]).long()
        old = -torch.rand(B, L, device=dev, generator=g) * 10
        ref = -torch.rand(B, L, device=dev, generator=g) * 10
        adv = torch.randn(B, 1, device=dev, generator=g).expand(B, L).contiguous()
        return [x, y, old, adv, m, ref]

    static = fresh()

    def run(t):
        out = CA.fused_actor_step(t[0], t[1], t[2], t[3], t[4], cfg, ref_log_prob=t[5], loss_scale_factor=0.125)
        return out.dlogits, out.log_prob, out.entropy, out.loss

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):  # warm-up on a side stream, as graph capture asks
        run(static)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        captured = run(static)
    for _ in range(4):  # replays with the program's own eager work and synchronisations in between
        new = fresh()
        for s, n in zip(static, new):
            s.copy_(n)
        graph.replay()
        torch.cuda.synchronize()
        got = [c.clone() for c in captured]
        want = run(new)
        torch.cuda.synchronize()
        for a, b in zip(got, want):
            assert torch.equal(a, b)


def test_reference_flow_replays_under_graph_capture(dev):
    """The actor's own sequence -- ``logprobs_from_logits``, ``entropy_from_logits`` on the same tensor,
    ``compute_policy_loss_vanilla``, ``agg_loss`` of the entropy, ``kl_penalty`` + ``agg_loss``, ``backward()``
    (dp_actor.py:179-195,455-500) -- captured with autograd inside the graph and replayed on new data: every replay
    equals the eager run bit for bit.  The operators allocate through torch's allocator only, never synchronise and
    record no memset nodes."""
    from types import SimpleNamespace

    import siirl_amd.core_algos as CA
    import siirl_amd.torch_functional as SF

    B, L, V = 4, 64, 5003
    cfg = SimpleNamespace(clip_ratio=0.2, clip_ratio_low=0.2, clip_ratio_high=0.28, clip_ratio_c=3.0)
    g = torch.Generator(device=dev).manual_seed(1)

    def fresh():
        x = (torch.randn(B, L, V, device=dev, generator=g) * 2).to(torch.bfloat16)
        y = torch.randint(0, V, (B, L), device=dev, generator=g)
        lens = torch.randint(1, L + 1, (B,), device=dev, generator=g)
        m = (torch.arange(L, device=dev)[None] < lens[:, None]).long()
        old = -torch.rand(B, L, device=dev, generator=g) * 10
        ref = -torch.rand(B, L, device=dev, generator=g) * 10
        adv = torch.randn(B, 1, device=dev, generator=g).expand(B, L).contiguous()
        return [x, y, old, adv, m, ref]

    def run(t):
        leaf = t[0].detach().requires_grad_(True)
        logits = leaf * 1.0
        lp = SF.logprobs_from_logits(logits, t[1])  # default in-place backward, as on the padded path
        ent = SF.entropy_from_logits(logits)
        pg, clipfrac, kl, _ = CA.compute_policy_loss_vanilla(old_log_prob=t[2], log_prob=lp, advantages=t[3],
                                                             response_mask=t[4], loss_agg_mode="token-mean", config=cfg)
        loss = pg - 0.01 * CA.agg_loss(loss_mat=ent, loss_mask=t[4], loss_agg_mode="token-mean")
        kld = CA.kl_penalty(logprob=lp, ref_logprob=t[5], kl_penalty="low_var_kl")
        loss = (loss + 0.05 * CA.agg_loss(loss_mat=kld, loss_mask=t[4], loss_agg_mode="token-mean")) * 0.25
        loss.backward()
        return leaf.grad, lp.detach(), ent.detach(), loss.detach(), clipfrac, kl

    static = fresh()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        for _ in range(2):
            run(static)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        captured = run(static)
    for _ in range(4):
        new = fresh()
        for s, n in zip(static, new):
            s.copy_(n)
        graph.replay()
        torch.cuda.synchronize()
        got = [c.clone() for c in captured]
        want = run(new)
        torch.cuda.synchronize()
        for i, (a, b) in enumerate(zip(got, want)):
            assert torch.equal(a, b), i
