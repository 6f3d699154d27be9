"""Pins the oracle's log-prob / entropy / gradient functions (CPU only) against library identities, closed
forms and brute force, so that a dropped term, a wrong sign or a transposed index fails here."""

import math

import pytest
import torch
import torch.nn.functional as F

from oracle import torch_functional as OF


def _rand(T, V, seed, dtype=torch.float64, scale=3.0):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(T, V, generator=g, dtype=torch.float64) * scale).to(dtype), torch.randint(0, V, (T,), generator=g)


@pytest.mark.parametrize("T,V", [(1, 1), (4, 2), (7, 33), (5, 1000)])
def test_logprob_library_identities(T, V):
    x, y = _rand(T, V, 1)
    lp = OF.logprobs_from_logits(x, y)
    assert torch.allclose(lp, -F.cross_entropy(x, y, reduction="none"), atol=1e-12)
    assert torch.allclose(lp, F.log_softmax(x, -1).gather(-1, y[:, None]).squeeze(-1), atol=1e-12)
    # brute force in pure Python
    for r in range(T):
        row = [float(v) for v in x[r]]
        m = max(row)
        lse = m + math.log(sum(math.exp(v - m) for v in row))
        assert abs(float(lp[r]) - (row[int(y[r])] - lse)) < 1e-12


def test_logprob_invariants():
    x, y = _rand(6, 50, 2)
    assert torch.allclose(OF.logprobs_from_logits(x, y), OF.logprobs_from_logits(x + 7.25, y), atol=1e-12)
    allp = torch.stack([OF.logprobs_from_logits(x, torch.full((6,), k)) for k in range(50)], -1)
    assert torch.allclose(allp.exp().sum(-1), torch.ones(6, dtype=torch.float64), atol=1e-12)
    u = torch.zeros(3, 128, dtype=torch.float64)
    assert torch.allclose(OF.logprobs_from_logits(u, torch.tensor([0, 5, 127])), torch.full((3,), -math.log(128.0), dtype=torch.float64))
    # n-d input keeps its leading shape
    x3 = x.reshape(2, 3, 50)
    assert OF.logprobs_from_logits(x3, y.reshape(2, 3)).shape == (2, 3)


def test_entropy_identities_and_special_cases():
    x, _ = _rand(9, 77, 3)
    h = OF.entropy_from_logits(x)
    assert torch.allclose(h, torch.distributions.Categorical(logits=x).entropy(), atol=1e-12)
    assert (h >= 0).all() and (h <= math.log(77) + 1e-12).all()
    assert torch.allclose(OF.entropy_from_logits(torch.zeros(2, 64, dtype=torch.float64)), torch.full((2,), math.log(64.0), dtype=torch.float64))
    spike = torch.zeros(1, 100, dtype=torch.float64)
    spike[0, 3] = 200.0
    assert float(OF.entropy_from_logits(spike)) < 1e-12
    two = torch.full((1, 100), -1e4, dtype=torch.float64)
    two[0, 1] = two[0, 9] = 2.5
    assert abs(float(OF.entropy_from_logits(two)) - math.log(2)) < 1e-12
    assert torch.allclose(OF.entropy_from_logits(x), OF.entropy_from_logits(x - 3.0), atol=1e-12)
    # chunked spelling: fp32 result, same values
    xf = x.float()
    assert torch.allclose(OF.entropy_from_logits_with_chunking(xf, 4), OF.entropy_from_logits(xf), atol=1e-6)


def test_forward_with_temperature_matches_division():
    x, y = _rand(5, 40, 4)
    for T in (0.5, 1.0, 1.3):
        lp, ent, lse, ex = OF.logprob_entropy_forward(x, y, T)
        assert torch.allclose(lp, OF.logprobs_from_logits(x / T, y), atol=1e-12)
        assert torch.allclose(ent, OF.entropy_from_logits(x / T), atol=1e-12)
        assert torch.allclose(lse, torch.logsumexp(x / T, -1), atol=1e-12)
        assert torch.allclose(ex, (torch.softmax(x / T, -1) * x / T).sum(-1), atol=1e-12)


@pytest.mark.parametrize("temperature", [1.0, 0.7])
def test_backward_closed_form_vs_autograd(temperature):
    x, y = _rand(6, 29, 5)
    g = torch.Generator().manual_seed(6)
    g_lp = torch.randn(6, generator=g, dtype=torch.float64)
    g_h = torch.randn(6, generator=g, dtype=torch.float64)
    for a, b in ((g_lp, g_h), (g_lp, None), (None, g_h)):
        cf = OF.logprob_entropy_backward(x, y, a, b, temperature)
        ag = OF.logprob_entropy_backward_autograd(x, y, a, b, temperature)
        assert torch.allclose(cf, ag, atol=1e-12)
        assert cf.sum(-1).abs().max() < 1e-12  # both branches are orthogonal to the all-ones direction
    # the log-prob branch alone is g * (onehot - p)
    p = torch.softmax(x, -1)
    onehot = F.one_hot(y, 29).double()
    assert torch.allclose(OF.logprob_entropy_backward(x, y, g_lp, None), g_lp[:, None] * (onehot - p), atol=1e-12)


def test_backward_gradcheck_small_vocab():
    x, y = _rand(3, 11, 7)
    x = x.requires_grad_(True)
    assert torch.autograd.gradcheck(lambda t: OF.logprobs_from_logits(t, y), (x,), eps=1e-6, atol=1e-6)
    assert torch.autograd.gradcheck(lambda t: OF.entropy_from_logits(t), (x,), eps=1e-6, atol=1e-6)


def test_bf16_policy():
    """16-bit logits are upcast and the fp32 formula applied; the reference's literal 16-bit branch rounds its
    result to the input dtype and differs by up to a bf16 ulp of |logprob| (a side note, not the target)."""
    x, y = _rand(8, 3000, 8, dtype=torch.bfloat16)
    lp = OF.logprobs_from_logits(x, y)
    assert lp.dtype == torch.float32
    assert torch.allclose(lp.double(), OF.logprobs_from_logits(x.double(), y), atol=2e-6)
    lit = OF.logprobs_from_logits(x, y, literal_bf16=True)
    assert lit.dtype == torch.bfloat16 and (lit.float() - lp).abs().max() < 0.07
    assert OF.entropy_from_logits(x, literal_bf16=True).dtype == torch.bfloat16


def test_masked_reductions():
    v = torch.tensor([[1.0, 2.0, float("nan")], [4.0, 5.0, 6.0]])
    m = torch.tensor([[1, 1, 0], [0, 1, 1]])
    assert float(OF.masked_sum(v, m)) == 14.0
    assert abs(float(OF.masked_mean(v, m)) - 3.5) < 1e-6
    assert OF.masked_sum(v, m, axis=-1).tolist() == [3.0, 11.0]
    assert torch.allclose(OF.masked_mean(v, m, axis=-1), torch.tensor([1.5, 5.5]), atol=1e-6)
    assert float(OF.masked_mean(v, torch.zeros_like(m))) == 0.0  # 0 / 1e-8
    assert float(OF.gather_from_labels(v, torch.tensor([1, 2]))[1]) == 6.0


def test_flash_attn_dispatch_statement_ignores_minus_100():
    """oracle.logprobs_from_logits_flash_attn: equal to the v2 statement on ordinary labels; a label of -100 gives 0
    and a zero gradient row (the convention of the cross-entropy routine it calls)."""
    g = torch.Generator().manual_seed(4)
    x = torch.randn(5, 13, generator=g, dtype=torch.float64, requires_grad=True)
    y = torch.randint(0, 13, (5,), generator=g)
    a = OF.logprobs_from_logits_flash_attn(x, y)
    b = OF.logprobs_from_logits(x, y)
    assert torch.allclose(a, b, atol=1e-12)
    y[3] = -100
    c = OF.logprobs_from_logits_flash_attn(x, y)
    assert c[3].item() == 0.0 and torch.allclose(c[[0, 1, 2, 4]], b[[0, 1, 2, 4]].detach(), atol=1e-12)
    (gx,) = torch.autograd.grad(c.sum(), x)
    assert gx[3].abs().max().item() == 0.0 and gx[0].abs().max().item() > 0
