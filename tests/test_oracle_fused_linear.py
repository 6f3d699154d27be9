"""Pins the oracle of the fused lm_head + log-prob/entropy (CPU only): it must equal log-prob / entropy of
``(h @ W.T) / T`` in fp64, and its gradients must equal autograd through that expression."""

import pytest
import torch

from oracle import fused_linear as OFL
from oracle import torch_functional as OF


@pytest.mark.parametrize("temperature", [1.0, 0.8])
def test_fused_equals_unfused(temperature):
    g = torch.Generator().manual_seed(0)
    T, H, V = 37, 24, 211
    h = torch.randn(T, H, generator=g, dtype=torch.float64)
    w = torch.randn(V, H, generator=g, dtype=torch.float64) * 0.2
    ids = torch.randint(0, V, (T,), generator=g)
    lp, ent = OFL.fused_linear_for_ppo_fwd(h, w, ids, temperature, dtype=torch.float64, chunk_size=8)
    logits = (h @ w.t()) / temperature
    assert torch.allclose(lp, OF.logprobs_from_logits(logits, ids), atol=1e-12)
    assert torch.allclose(ent, OF.entropy_from_logits(logits), atol=1e-12)
    # 3-D hidden states keep their leading shape
    lp3, ent3 = OFL.fused_linear_for_ppo_fwd(h[:36].reshape(4, 9, H), w, ids[:36].reshape(4, 9), temperature, dtype=torch.float64)
    assert lp3.shape == (4, 9) and torch.allclose(lp3.reshape(-1), lp[:36], atol=1e-12)

    g_lp = torch.randn(T, generator=g, dtype=torch.float64)
    g_h = torch.randn(T, generator=g, dtype=torch.float64)
    hr, wr = h.clone().requires_grad_(True), w.clone().requires_grad_(True)
    lg = (hr @ wr.t()) / temperature
    total = (g_lp * OF.logprobs_from_logits(lg, ids)).sum() + (g_h * OF.entropy_from_logits(lg)).sum()
    total.backward()
    for a, b in ((g_lp, g_h),):
        dh, dw = OFL.fused_linear_for_ppo_bwd(a, b, h, w, ids, temperature, dtype=torch.float64, chunk_size=8)
        assert torch.allclose(dh, hr.grad, atol=1e-11) and torch.allclose(dw, wr.grad, atol=1e-11)
    dh, dw = OFL.fused_linear_for_ppo_bwd(g_lp, None, h, w, ids, temperature, dtype=torch.float64)
    hr.grad = wr.grad = None
    lg = (hr @ wr.t()) / temperature
    (g_lp * OF.logprobs_from_logits(lg, ids)).sum().backward()
    assert torch.allclose(dh, hr.grad, atol=1e-11) and torch.allclose(dw, wr.grad, atol=1e-11)


def test_literal_cast_rounds_outputs():
    g = torch.Generator().manual_seed(1)
    h = torch.randn(16, 32, generator=g).to(torch.bfloat16)
    w = (torch.randn(100, 32, generator=g) * 0.1).to(torch.bfloat16)
    ids = torch.randint(0, 100, (16,), generator=g)
    lp, ent = OFL.fused_linear_for_ppo_fwd(h, w, ids, literal_cast=True)
    assert lp.dtype == torch.bfloat16 and ent.dtype == torch.bfloat16  # the reference casts back (:32)
    lp32, _ = OFL.fused_linear_for_ppo_fwd(h, w, ids)
    assert lp32.dtype == torch.float32 and (lp.float() - lp32).abs().max() < 0.1


def _emulated_kernel_gradients(h, w, ids, g_lp, g_h):
    """The fused backward's arithmetic restated on the CPU: dlogits in float64 from the given upstream gradients,
    rounded to bf16, multiplied in float32, results rounded to bf16."""
    logits = h.double() @ w.double().t()
    d = OF.logprob_entropy_backward(logits, ids, g_lp, g_h, dtype=torch.float64).to(torch.bfloat16).float()
    return (d @ w.float()).to(torch.bfloat16), (d.t() @ h.float()).to(torch.bfloat16)


def test_gradient_bar_accepts_the_roundings_and_rejects_one_percent():
    """The bar of the fused lm_head gradients (``tests/grad_bar.py``) on the CPU side of the comparison: the two bf16
    roundings of the kernel pass; the same arithmetic fed an entropy gradient, a log-prob gradient or a temperature
    that is off by 1 % -- what a wrong c1, cy or 1/T in the dlogits epilogue would produce -- fails."""
    from grad_bar import REL_FROBENIUS, fused_grad_ok

    g = torch.Generator().manual_seed(11)
    T, H, V = 192, 128, 4096
    h = torch.randn(T, H, generator=g).to(torch.bfloat16)
    w = (torch.randn(V, H, generator=g) * (2.0 / H ** 0.5)).to(torch.bfloat16)
    ids = torch.randint(0, V, (T,), generator=g)
    g_lp = (torch.randn(T, generator=g) * 1e-2).double()
    g_h = (torch.randn(T, generator=g) * 1e-2).double()
    zero = torch.zeros_like(g_lp)
    for a, b, wrong_a, wrong_b in ((g_lp, g_h, g_lp * 1.01, g_h * 1.01),  # both coefficients (a wrong 1/T)
                                   (zero, g_h, zero, g_h * 1.01),          # entropy branch: c1 = -g_h / T^2
                                   (g_lp, zero, g_lp * 1.01, zero)):       # log-prob branch: cy = g_lp / T
        dh64, dw64 = OFL.fused_linear_for_ppo_bwd(a, b, h, w, ids, dtype=torch.float64)
        for got, want in zip(_emulated_kernel_gradients(h, w, ids, a, b), (dh64, dw64)):
            ok, max_ratio, rel_f, _, _ = fused_grad_ok(got, want)
            assert ok and 1e-3 < rel_f < REL_FROBENIUS, (max_ratio, rel_f)
        for got, want in zip(_emulated_kernel_gradients(h, w, ids, wrong_a, wrong_b), (dh64, dw64)):
            ok, max_ratio, rel_f, _, _ = fused_grad_ok(got, want)
            assert not ok and rel_f > REL_FROBENIUS, (max_ratio, rel_f)
    # a dropped slab of 1/50 of the vocabulary
    dh64, _ = OFL.fused_linear_for_ppo_bwd(g_lp, g_h, h, w, ids, dtype=torch.float64)
    logits = h.double() @ w.double().t()
    d = OF.logprob_entropy_backward(logits, ids, g_lp, g_h, dtype=torch.float64).to(torch.bfloat16).float()
    d[:, : V // 50] = 0
    ok, max_ratio, rel_f, _, _ = fused_grad_ok((d @ w.float()).to(torch.bfloat16), dh64)
    assert not ok and rel_f > 0.02, (max_ratio, rel_f)
