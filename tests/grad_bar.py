"""The error bar of the fused lm_head gradients, derived from the arithmetic (shared by the GPU tests; run on the CPU
by ``tests/test_oracle_fused_linear.py`` to show that it rejects a 1 % mistake).

``d_hidden[t, h] = sum_v D[t, v] W[v, h]`` and ``d_weight[v, h] = sum_t D[t, v] hidden[t, h]`` are computed from
``D = bf16(dlogits)`` with fp32 accumulation and leave as bf16.  Two roundings therefore separate a result from the
float64 oracle's (bf16 keeps 8 significant bits: half an ulp is between 2^-9 and 2^-8 of the value):

* each term carries the relative rounding error of its ``D`` entry, uniform within half an ulp: at most 2^-8 = 3.9e-3,
  root mean square r = 2^-8 / sqrt(3) * (0.5 .. 1 by where the mantissa sits) ~ 1.7e-3.  The errors of the terms are
  independent, so a sum's error has standard deviation r * sqrt(sum of squared terms): about r * |result| when the
  terms' signs are random, as they are for gradients, and exactly that for a single term;
* the result is rounded to bf16 once more: another relative error of at most 2^-8, rms ~ 1.7e-3.

fp32 accumulation (2^-24 per addition) and the recomputed logits (same products, other summation order) add nothing
that shows at this scale.  Expected relative Frobenius error: sqrt(2) * 1.7e-3 = 2.4e-3; with every mantissa at its
worst sqrt(2) * 2^-8 / sqrt(3) = 3.2e-3.  Largest element error: 2 * 2^-8 = 7.8e-3 of the element itself for a one-term
sum, ~ 2^-8 + 5 standard deviations of an element of typical size (~ 0.6 % of the largest magnitude) for long sums.
Observed on the GPU over the 160 comparisons of the fused lm_head tests: relative Frobenius 2.2e-3 .. 3.5e-3 (median
2.4e-3; the highest are tensors with one or a few non-zero rows), largest element error 2.5e-3 .. 6.2e-3 of the
largest magnitude.

The bars: ``REL_FROBENIUS = 5e-3`` (twice the expected figure, 1.4 times the worst seen) and ``MAX_OVER_SCALE = 1e-2``
(1.3 times the one-term bound, 1.6 times the worst seen).  What they reject: a dropped vocabulary slab of 1/50
(relative Frobenius error ~ 0.14, element errors of 3 % of the maximum), a K-step skipped in 56 (~ 0.13), upstream
gradients or a coefficient off by 1 % (1e-2 on the branch concerned).  ``floor`` absorbs results that are exact zeros in
the oracle and sums of cancelling fp32 terms on the GPU (a one-word vocabulary)."""

from __future__ import annotations

import torch

REL_FROBENIUS = 5e-3
MAX_OVER_SCALE = 1e-2


def fused_grad_errors(got: torch.Tensor, want64: torch.Tensor):
    """(largest element error / largest magnitude of the oracle, relative Frobenius error, largest magnitude)."""
    got = got.detach().cpu().double()
    want64 = want64.detach().cpu().double()
    scale = want64.abs().max().item()
    err = (got - want64).abs().max().item()
    rel_f = ((got - want64).norm() / want64.norm()).item() if scale > 0 else 0.0
    return (err / scale if scale > 0 else 0.0), rel_f, scale, err


def fused_grad_ok(got, want64, floor=1e-7):
    """True when ``got`` is within the bar of the float64 oracle ``want64``; also returns the observed figures."""
    max_ratio, rel_f, scale, err = fused_grad_errors(got, want64)
    norm_floor = floor * want64.numel() ** 0.5
    ok_max = err <= MAX_OVER_SCALE * scale + floor
    ok_f = scale == 0 or rel_f < REL_FROBENIUS or (got.detach().cpu().double() - want64.double().cpu()).norm().item() <= norm_floor
    return ok_max and ok_f, max_ratio, rel_f, scale, err


def check_fused_grad(got, want64, name, floor=1e-7):
    ok, max_ratio, rel_f, scale, err = fused_grad_ok(got, want64, floor)
    print(f"[grad-bar] {name}: max err / max |want| = {max_ratio:.3e} (err {err:.3e}, scale {scale:.3e}), "
          f"relative Frobenius = {rel_f:.3e}", flush=True)
    assert ok, (f"{name}: max err {err:.3e} vs {MAX_OVER_SCALE} * {scale:.3e} + {floor}, "
                f"relative Frobenius {rel_f:.3e} vs {REL_FROBENIUS}")
