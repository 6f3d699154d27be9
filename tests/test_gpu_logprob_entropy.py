"""GPU parity: HIP log-prob / entropy forward and backward (through the C ABI) vs the CPU oracle.

Tolerances (from the task statement): logprob / entropy within 1e-3 absolute of the fp32-math oracle
on the same (16-bit rounded) inputs; dlogits compared with the oracle's fp64 gradient after rounding
to the logits dtype: at most 1 ulp of that dtype or 1e-6 absolute."""

import pytest
import torch

from oracle import torch_functional as OF

pytestmark = pytest.mark.gpu

ABS_TOL = 1e-3


def _ulp_close(got, want64, dtype):
    """got: tensor in `dtype` (on cpu); want64: fp64 reference.  <= 1 ulp of dtype around the reference, or tiny."""
    want = want64.to(dtype)
    g, w = got.double(), want.double()
    if dtype == torch.float32:
        tol = 2e-6 * w.abs() + 2e-7
    else:
        eps = {torch.bfloat16: 2.0 ** -8, torch.float16: 2.0 ** -11}[dtype]
        tol = 2 * eps * torch.maximum(w.abs(), want64.abs()) + 1e-6
    bad = (g - want64).abs() > tol
    return not bool(bad.any()), (g - want64).abs().max().item()


def _make(T, V, dtype, seed, scale=3.0, spikes=True):
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(T, V, generator=g) * scale
    if spikes and T >= 4:
        rows = torch.randperm(T, generator=g)[: max(1, T // 8)]
        cols = torch.randint(0, V, (rows.numel(),), generator=g)
        x[rows, cols] += 15.0
    y = torch.randint(0, V, (T,), generator=g)
    return x.to(dtype), y


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32, torch.float16])
@pytest.mark.parametrize("T,V", [(1, 1), (3, 7), (5, 8), (4, 1000), (7, 4099), (16, 32000), (6, 152064), (3, 151936)])
def test_forward_backward_matches_oracle(dev, dtype, T, V):
    import siirl_amd.torch_functional as SF

    x, y = _make(T, V, dtype, seed=1000 + T * 7 + V)
    g = torch.Generator().manual_seed(5)
    g_lp = torch.randn(T, generator=g) * 1e-2
    g_h = torch.randn(T, generator=g) * 1e-2
    if T > 2:
        g_lp[1] = 0.0
        g_h[1] = 0.0  # a padded row

    xd = x.to(dev).requires_grad_(True)
    lp, ent = SF.logprobs_and_entropy_from_logits(xd, y.to(dev))
    assert lp.dtype == torch.float32 and ent.dtype == torch.float32 and lp.shape == (T,)
    lp_o, ent_o, _, _ = OF.logprob_entropy_forward(x, y, dtype=torch.float32)
    lp64, ent64, _, _ = OF.logprob_entropy_forward(x, y, dtype=torch.float64)
    assert (lp.cpu() - lp_o).abs().max() < ABS_TOL
    assert (ent.cpu() - ent_o).abs().max() < ABS_TOL
    # and much closer than the bar to the fp64 statement (fp32 accumulation over up to 152k terms)
    assert (lp.cpu().double() - lp64).abs().max() < 1e-4
    assert (ent.cpu().double() - ent64).abs().max() < 1e-4

    (dx,) = torch.autograd.grad([lp, ent], [xd], [g_lp.to(dev), g_h.to(dev)])
    assert dx.dtype == dtype and dx.shape == x.shape
    want = OF.logprob_entropy_backward(x, y, g_lp, g_h, dtype=torch.float64)
    ok, err = _ulp_close(dx.cpu(), want, dtype)
    assert ok, f"dlogits max abs err {err}"
    if T > 2:
        assert torch.count_nonzero(dx[1]) == 0


@pytest.mark.parametrize("temperature", [0.6, 1.0, 1.7])
def test_temperature_folded(dev, temperature):
    import siirl_amd.torch_functional as SF

    x, y = _make(9, 5003, torch.bfloat16, seed=3)
    xd = x.to(dev).requires_grad_(True)
    lp, ent = SF.logprobs_and_entropy_from_logits(xd, y.to(dev), temperature=temperature)
    lp64, ent64, _, _ = OF.logprob_entropy_forward(x, y, temperature, dtype=torch.float64)
    assert (lp.cpu().double() - lp64).abs().max() < 5e-5
    assert (ent.cpu().double() - ent64).abs().max() < 5e-5
    g = torch.Generator().manual_seed(1)
    g_lp, g_h = torch.randn(9, generator=g), torch.randn(9, generator=g)
    (dx,) = torch.autograd.grad([lp, ent], [xd], [g_lp.to(dev), g_h.to(dev)])
    want = OF.logprob_entropy_backward(x, y, g_lp, g_h, temperature, dtype=torch.float64)
    ok, err = _ulp_close(dx.cpu(), want, torch.bfloat16)
    assert ok, err


def test_reference_signatures_and_pairing(dev):
    import siirl_amd.torch_functional as SF

    x, y = _make(12, 3001, torch.bfloat16, seed=11)
    xd = x.to(dev).requires_grad_(True)
    # the actor's call order when entropy is wanted (dp_actor.py:179-195)
    lp = SF.logprobs_from_logits(logits=xd, labels=y.to(dev), inplace_backward=False)
    ent = SF.entropy_from_logits(xd)
    assert ent.grad_fn is lp.grad_fn  # one node: one backward pass writes both gradients
    lp64, ent64, _, _ = OF.logprob_entropy_forward(x, y, dtype=torch.float64)
    assert (lp.cpu().double() - lp64).abs().max() < 2e-5
    assert (ent.cpu().double() - ent64).abs().max() < 2e-5
    g_lp, g_h = torch.ones(12), torch.full((12,), -0.5)
    (dx,) = torch.autograd.grad([lp, ent], [xd], [g_lp.to(dev), g_h.to(dev)])
    want = OF.logprob_entropy_backward(x, y, g_lp, g_h, dtype=torch.float64)
    ok, err = _ulp_close(dx.cpu(), want, torch.bfloat16)
    assert ok, err
    # a different tensor never claims the parked entropy
    x2 = x.to(dev)
    lp2 = SF.logprobs_from_logits(x2, y.to(dev), inplace_backward=False)
    ent_other = SF.entropy_from_logits(x.to(dev) + 1.0)  # shifted logits: same entropy, separate pass
    assert (ent_other.cpu().double() - ent64).abs().max() < 2e-3
    ent2 = SF.entropy_from_logits(x2)
    assert (ent2.cpu().double() - ent64).abs().max() < 2e-5 and lp2.shape == (12,)
    # entropy alone, and the chunked spelling
    e3 = SF.entropy_from_logits_with_chunking(x.to(dev), 5)
    assert (e3.cpu().double() - ent64).abs().max() < 2e-5


def test_inplace_backward_overwrites_logits(dev):
    import siirl_amd.torch_functional as SF

    x, y = _make(10, 2049, torch.bfloat16, seed=21)
    leaf = x.to(dev).requires_grad_(True)
    xd = leaf * 1.0  # non-leaf, as the model's logits are
    ptr = xd.data_ptr()
    lp = SF.logprobs_from_logits(xd, y.to(dev), inplace_backward=True)
    g_lp = torch.linspace(-1, 1, 10)
    lp.backward(g_lp.to(dev))
    want = OF.logprob_entropy_backward(x, y, g_lp, None, dtype=torch.float64)
    ok, err = _ulp_close(leaf.grad.cpu(), want, torch.bfloat16)
    assert ok, err
    assert xd.data_ptr() == ptr
    ok2, _ = _ulp_close(xd.detach().cpu(), want, torch.bfloat16)  # the logits buffer now holds the gradient
    assert ok2


def test_strided_views_and_3d(dev):
    import siirl_amd.torch_functional as SF

    g = torch.Generator().manual_seed(8)
    full = (torch.randn(3, 11, 515, generator=g) * 2).to(torch.bfloat16)
    y = torch.randint(0, 515, (3, 6), generator=g)
    fd = full.to(dev).requires_grad_(True)
    view = fd[:, -7:-1, :]  # the actor's response slice (dp_actor.py:254): B blocks of strided rows
    lp = SF.logprobs_from_logits(view, y.to(dev), inplace_backward=False)
    ent = SF.entropy_from_logits(view)
    xs = full[:, -7:-1, :]
    lp64, ent64, _, _ = OF.logprob_entropy_forward(xs, y, dtype=torch.float64)
    assert lp.shape == (3, 6)
    assert (lp.cpu().double() - lp64).abs().max() < 2e-5
    assert (ent.cpu().double() - ent64).abs().max() < 2e-5
    g_lp, g_h = torch.randn(3, 6, generator=g), torch.randn(3, 6, generator=g)
    (lp * g_lp.to(dev)).sum().backward(retain_graph=True)
    want = OF.logprob_entropy_backward(xs, y, g_lp, None, dtype=torch.float64)
    got = fd.grad.cpu()
    ok, err = _ulp_close(got[:, -7:-1, :], want, torch.bfloat16)
    assert ok, err
    assert torch.count_nonzero(got[:, :4]) == 0 and torch.count_nonzero(got[:, -1]) == 0
    # odd row stride (rows not 16-byte aligned): scalar path
    wide = (torch.randn(5, 1003, generator=g)).to(torch.bfloat16)
    sub = wide[:, 1:1000]
    y2 = torch.randint(0, 999, (5,), generator=g)
    wd = wide.to(dev).requires_grad_(True)
    lp2, ent2 = SF.logprobs_and_entropy_from_logits(wd[:, 1:1000], y2.to(dev))
    a, b, _, _ = OF.logprob_entropy_forward(sub, y2, dtype=torch.float64)
    assert (lp2.cpu().double() - a).abs().max() < 2e-5 and (ent2.cpu().double() - b).abs().max() < 2e-5
    (lp2.sum() + ent2.sum()).backward()
    want2 = OF.logprob_entropy_backward(sub, y2, torch.ones(5), torch.ones(5), dtype=torch.float64)
    ok, err = _ulp_close(wd.grad.cpu()[:, 1:1000], want2, torch.bfloat16)
    assert ok, err


def test_special_rows(dev):
    import math

    import siirl_amd.torch_functional as SF

    V = 4096
    x = torch.zeros(4, V)
    x[1, 5] = 80.0  # one dominant logit
    x[2, :] = -1e4
    x[2, 7] = x[2, 9] = 3.0  # two equal logits, the rest negligible
    x[3] = torch.linspace(-30000, 30000, V)  # huge range
    y = torch.tensor([0, 5, 7, V - 1])
    lp, ent = SF.logprobs_and_entropy_from_logits(x.to(dev), y.to(dev))
    lp, ent = lp.cpu(), ent.cpu()
    assert abs(lp[0].item() + math.log(V)) < 1e-5 and abs(ent[0].item() - math.log(V)) < 1e-5
    assert abs(lp[1].item()) < 1e-5 and abs(ent[1].item()) < 1e-5
    assert abs(lp[2].item() + math.log(2)) < 1e-5 and abs(ent[2].item() - math.log(2)) < 1e-5
    lp64, ent64, _, _ = OF.logprob_entropy_forward(x, y, dtype=torch.float64)
    assert (lp.double() - lp64).abs().max() < 1e-3 and (ent.double() - ent64).abs().max() < 1e-3
    # label outside [0, V): NaN, no fault
    bad = SF.logprobs_from_logits(x.to(dev), torch.tensor([0, V, -1, 3]).to(dev))
    assert torch.isnan(bad[1]) and torch.isnan(bad[2]) and not torch.isnan(bad[0])


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_nan_in_a_row_without_upstream_gradient(dev, dtype):
    """By default the backward is dense, and ``0 * NaN`` reaches ``dlogits`` as it does through the reference's
    autograd (``torch_functional.py:99-132`` under ``backward()``); with ``set_skip_zero_rows(True)`` such a row is
    written as zeros unread.  Rows with a gradient are the same bits either way."""
    import siirl_amd.torch_functional as TF

    T, V = 37, 1000
    g = torch.Generator().manual_seed(5)
    x = (torch.randn(T, V, generator=g) * 2).to(dtype)
    x[3, 17] = float("nan")
    y = torch.randint(0, V, (T,), generator=g)
    g_lp, g_ent = torch.randn(T, generator=g), torch.randn(T, generator=g)
    g_lp[3] = 0.0
    g_ent[3] = 0.0
    grads = {}
    for skip in (False, True):
        TF.set_skip_zero_rows(skip)
        try:
            xd = x.to(dev).requires_grad_(True)
            lp, ent = TF.logprobs_and_entropy_from_logits(xd, y.to(dev))
            torch.autograd.backward([lp, ent], [g_lp.to(dev), g_ent.to(dev)])
        finally:
            TF.set_skip_zero_rows(False)
        grads[skip] = xd.grad
    assert torch.isnan(grads[False][3]).any() and not grads[True][3].any()
    keep = torch.arange(T) != 3
    assert torch.equal(grads[False][keep.to(dev)], grads[True][keep.to(dev)])
    assert torch.isfinite(grads[False][keep.to(dev)]).all()


def test_no_cpu_fallback():
    import siirl_amd.torch_functional as SF

    with pytest.raises(RuntimeError, match="GPU only"):
        SF.logprobs_from_logits(torch.zeros(2, 8), torch.zeros(2, dtype=torch.long))


def test_config2_slice_properties(dev):
    """Config-2 shape at a slice of its rows: shift invariance and gradient rows summing to zero hold at
    full vocabulary width (152064), plus parity on the rows the oracle checks."""
    import siirl_amd.torch_functional as SF

    T, V = 256, 152064
    gen = torch.Generator(device=dev).manual_seed(2)
    x = (torch.randn(T, V, device=dev, generator=gen) * 3).to(torch.bfloat16)
    y = torch.randint(0, V, (T,), device=dev, generator=gen)
    xr = x.clone().requires_grad_(True)
    lp, ent = SF.logprobs_and_entropy_from_logits(xr, y)
    lp_o, ent_o, _, _ = OF.logprob_entropy_forward(x[:32].cpu(), y[:32].cpu(), dtype=torch.float32)
    assert (lp[:32].cpu() - lp_o).abs().max() < ABS_TOL and (ent[:32].cpu() - ent_o).abs().max() < ABS_TOL
    # +4.0 is exact in bf16 for |x| < 128..: compare on logits quantised so the shift is lossless
    xq = (x.float() * 8).round().clamp(-127 * 8, 127 * 8) / 8
    a1, e1 = SF.logprobs_and_entropy_from_logits(xq.to(torch.bfloat16), y)
    a2, e2 = SF.logprobs_and_entropy_from_logits((xq + 4.0).to(torch.bfloat16), y)
    assert (a1 - a2).abs().max() < 1e-4 and (e1 - e2).abs().max() < 1e-4
    (dx,) = torch.autograd.grad([lp, ent], [xr], [torch.ones(T, device=dev), torch.ones(T, device=dev)])
    assert dx.float().sum(-1).abs().max() < 2e-2  # 152k bf16-rounded terms per row


def _actor_post_logits(SF, logits, labels, checkpointed, reentrant=False):
    """The actor's post-logits step (reference dp_actor.py:176-195): log-prob, then the entropy, optionally under
    torch.utils.checkpoint as with entropy_checkpointing."""
    import torch.utils.checkpoint as ckpt

    lp = SF.logprobs_from_logits(logits, labels, inplace_backward=False)
    if checkpointed:
        ent = ckpt.checkpoint(SF.entropy_from_logits, logits, use_reentrant=reentrant)
    else:
        ent = SF.entropy_from_logits(logits)
    return lp, ent


@pytest.mark.parametrize("pairing", [True, False])
@pytest.mark.parametrize("mode", ["plain", "checkpoint", "checkpoint_reentrant", "autocast", "autocast_checkpoint"])
def test_checkpoint_and_autocast_contexts(dev, mode, pairing):
    """The reference calls these functions under torch.autocast(bf16) (dp_actor.py:101) and wraps the entropy in
    torch.utils.checkpoint (:193-195): the forward must be re-runnable and every context must give the bits of the
    plain call."""
    import contextlib

    import siirl_amd.torch_functional as SF

    x, y = _make(37, 5003, torch.bfloat16, 11)
    g = torch.Generator().manual_seed(5)
    w_lp, w_ent = torch.randn(37, generator=g).to(dev), torch.randn(37, generator=g).to(dev)

    def run(mode):
        xd = x.to(dev).requires_grad_(True)
        ctx = torch.autocast("cuda", dtype=torch.bfloat16) if mode.startswith("autocast") else contextlib.nullcontext()
        with ctx:
            lp, ent = _actor_post_logits(SF, xd, y.to(dev), "checkpoint" in mode, reentrant=mode.endswith("reentrant"))
            loss = (lp * w_lp).sum() - (ent * w_ent).sum()
        loss.backward()
        return lp.detach(), ent.detach(), xd.grad

    SF.set_pairing(pairing)
    try:
        want = run("plain")
        got = run(mode)
    finally:
        SF.set_pairing(True)
    assert got[0].dtype == torch.float32 and got[1].dtype == torch.float32 and got[2].dtype == torch.bfloat16
    for a, b, what in zip(got, want, ("logprob", "entropy", "dlogits")):
        if what == "dlogits" and pairing and mode.endswith("reentrant"):
            # the reentrant checkpoint re-runs the entropy on a detached copy, so its gradient comes from its own
            # kernel and autograd adds the two bf16 results (as the reference's autograd does): each part carries
            # its own rounding, so compare with the fp64 oracle in units of the parts' magnitudes
            d1 = OF.logprob_entropy_backward(x, y, w_lp.cpu(), None, dtype=torch.float64)
            d2 = OF.logprob_entropy_backward(x, y, None, -w_ent.cpu(), dtype=torch.float64)
            tol = 2.0 ** -8 * (d1.abs() + d2.abs() + (d1 + d2).abs()) + 1e-7
            assert ((a.double().cpu() - (d1 + d2)).abs() <= tol).all(), (mode, what)
        else:
            assert torch.equal(a, b), (mode, what)
    lp_o = OF.logprobs_from_logits(x, y, dtype=torch.float32)
    assert (got[0].cpu() - lp_o).abs().max() < ABS_TOL


def test_no_grad_and_inference_mode(dev):
    import siirl_amd.torch_functional as SF

    x, y = _make(9, 777, torch.bfloat16, 2)
    xd, yd = x.to(dev), y.to(dev)
    ref = SF.logprobs_from_logits(xd, yd), SF.entropy_from_logits(xd)
    with torch.no_grad():  # reference dp_actor.py:330 (compute_log_prob)
        a = SF.logprobs_from_logits(xd.clone().requires_grad_(True), yd), SF.entropy_from_logits(xd)
    with torch.inference_mode():
        b = SF.logprobs_from_logits(xd, yd), SF.entropy_from_logits(xd)
    for t in (*a, *b):
        assert not t.requires_grad
    assert torch.equal(a[0], ref[0]) and torch.equal(a[1], ref[1]) and torch.equal(b[0], ref[0]) and torch.equal(b[1], ref[1])
