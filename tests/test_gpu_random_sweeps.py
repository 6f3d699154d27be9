"""GPU parity, seeded random sweeps over shapes and contents for the bit-exact parts of the path: index and mask
bookkeeping, grouping by uid, keep masks.  Each test draws a few hundred small cases from one seed and compares every
one with the CPU oracle; a failure prints the case.  ``SIIRL_TEST_SEED=<int>`` in the environment shifts every seed, for
a run over cases other than the committed ones."""
import os

import numpy as np
import pytest
import torch

from oracle import core_algos as OC
from oracle import dapo_filter as OD
from oracle import padding as OP

pytestmark = pytest.mark.gpu

_SEED = 100003 * int(os.environ.get("SIIRL_TEST_SEED", "0"))


def test_sweep_response_mask_from_eos(dev):
    import siirl_amd.torch_functional as TF

    rng = np.random.default_rng(101 + _SEED)
    for case in range(150):
        B, L = int(rng.integers(1, 40)), int(rng.integers(1, 300))
        vocab = int(rng.integers(2, 12))
        ids = rng.integers(0, vocab, (B, L)).astype(np.int64)
        eos = rng.choice(20, size=int(rng.integers(1, 5)), replace=False).tolist()
        eos_arg = eos[0] if len(eos) == 1 and case % 2 else eos
        x = torch.from_numpy(ids).to(dev)
        if case % 3 == 0:
            x = x.to(torch.int32)
        got = TF.get_response_mask(x, eos_arg).cpu().numpy()
        assert np.array_equal(got, OP.get_response_mask(ids, eos)), (case, B, L, eos)


def test_sweep_unpad_arbitrary_masks(dev):
    """Masks with holes anywhere (not only left / right padding): indices are those of nonzero(mask.flatten())."""
    import siirl_amd.padding as P

    rng = np.random.default_rng(102 + _SEED)
    for case in range(120):
        B, S = int(rng.integers(1, 24)), int(rng.integers(1, 260))
        mask = (rng.random((B, S)) < rng.random()).astype(np.int64)
        if case % 7 == 0:
            mask[:] = 0
        ids = rng.integers(0, 99999, (B, S)).astype(np.int64)
        rm_o, idx_o, cu_o, mx_o, sl_o = OP.unpad_input(ids[..., None], mask)
        mdt = [torch.int64, torch.bool, torch.int32, torch.float32][case % 4]
        rm, rolled, idx, cu, mx = P.unpad_ids_and_labels(torch.from_numpy(ids).to(dev), torch.from_numpy(mask).to(dev).to(mdt))
        assert np.array_equal(idx.cpu().numpy(), idx_o) and np.array_equal(cu.cpu().numpy(), cu_o) and mx == mx_o, case
        assert np.array_equal(rm[0].cpu().numpy(), rm_o[:, 0]), case
        assert np.array_equal(rolled.cpu().numpy(), OP.rolled_labels(rm_o[:, 0])), case
        if idx_o.size and S >= 2:
            L = int(rng.integers(1, S))
            v = rng.standard_normal(idx_o.size).astype(np.float32)
            got = P.pad_and_slice_response(torch.from_numpy(v).to(dev), idx, B, S, L).cpu().numpy()
            assert np.array_equal(got, OP.pad_and_slice_response(v, idx_o, B, S, L)), (case, B, S, L)


def _random_groups(rng, case):
    G = int(rng.integers(1, 30))
    sizes = rng.integers(1, 20, G)
    if case % 5 == 0:
        sizes[:] = 1
    names = rng.choice(np.arange(-50, 50) * (2 ** 33 + 1), size=G, replace=False)
    uid = np.repeat(names, sizes).astype(np.int64)
    if case % 2:
        uid = uid[rng.permutation(uid.size)]
    return uid


def test_sweep_keep_mask_random_groups(dev):
    import siirl_amd.dapo_filter as DF

    rng = np.random.default_rng(103 + _SEED)
    pool = np.array([0.0, 1.0, -1.0, 0.1, 0.3, 1.0 / 3.0, 2.5, 1e-3])
    for case in range(200):
        uid = _random_groups(rng, case)
        B = uid.size
        dtype = [np.float32, np.float64][case % 2]
        vals = rng.choice(pool[: int(rng.integers(1, len(pool) + 1))], size=B).astype(dtype)
        for u in np.unique(uid)[::3]:  # a third of the groups hold one value throughout
            vals[uid == u] = vals[uid == u][0]
        want = OD.keep_mask(vals, uid)
        keep, gsz = DF.group_keep_mask(torch.from_numpy(vals).to(dev), torch.from_numpy(uid).to(dev), return_group_size=True)
        assert np.array_equal(keep.cpu().numpy().astype(bool), want), (case, B, dtype)
        sizes = {u: int((uid == u).sum()) for u in np.unique(uid)}
        assert gsz.cpu().tolist() == [sizes[u] for u in uid], case
        idx, _, _ = OD.dynamic_sampling_keep_indices(vals, uid)
        assert torch.nonzero(keep).flatten().cpu().tolist() == idx, case


def test_sweep_grpo_advantage_random_groups(dev):
    import siirl_amd.core_algos as CA

    rng = np.random.default_rng(104 + _SEED)
    for case in range(120):
        uid = _random_groups(rng, case)
        B, L = uid.size, int(rng.integers(1, 70))
        lens = rng.integers(1, L + 1, B)
        mask = (np.arange(L)[None] < lens[:, None]).astype(np.int64)
        score = rng.choice([0.0, 1.0, -1.0, 0.5, 3.25], size=B).astype(np.float32) if case % 2 else \
            rng.standard_normal(B).astype(np.float32)
        rewards = np.zeros((B, L), dtype=np.float32)
        rewards[np.arange(B), lens - 1] = score
        norm = bool(case % 3)
        want, _ = OC.compute_grpo_outcome_advantage(torch.from_numpy(rewards), torch.from_numpy(mask), uid,
                                                    norm_adv_by_std_in_grpo=norm)
        got, ret = CA.compute_grpo_outcome_advantage(torch.from_numpy(rewards).to(dev), torch.from_numpy(mask).to(dev),
                                                     uid, norm_adv_by_std_in_grpo=norm)
        assert got is ret or torch.equal(got, ret)
        err = (got.cpu().double() - want.double()).abs()
        tol = 1e-6 + 1e-5 * want.double().abs()
        if norm:
            # Conditioning: the reference takes mean and std in float32 (torch's two-pass std around its own float32
            # mean, whose summation order depends on the host's vector width), so a group whose spread is within a few
            # float32 ulps of its scores' magnitude gets an advantage that is off by ulp(|s|) / (std + eps) -- per cent,
            # not 1e-5 -- and not the same on every host.  The kernel takes the statistics in double; the two are
            # compared at four such units.
            amp = np.zeros(B)
            for u in np.unique(uid):
                rows = np.nonzero(uid == u)[0]
                if rows.size > 1:
                    sc = score[rows].astype(np.float64)
                    amp[rows] = np.spacing(np.float32(np.abs(sc).max())) / (sc.std(ddof=1) + 1e-6)
            tol = tol + torch.from_numpy(4.0 * amp)[:, None]
        assert bool((err <= tol).all()), (case, B, L, norm, err.max().item())
        assert bool((got.cpu()[mask == 0] == 0).all()), case


# ----------------------------------------------------------------------------------- floating-point parts

AGGS = ["token-mean", "seq-mean-token-sum", "seq-mean-token-mean", "seq-mean-token-sum-norm"]


def _loss_case(rng, case):
    from types import SimpleNamespace

    B, L = int(rng.integers(1, 20)), int(rng.integers(1, 600))
    g = torch.Generator().manual_seed(int(rng.integers(1 << 30)))
    lp = torch.randn(B, L, generator=g) - 1.5
    old = lp + float(rng.choice([0.0, 0.05, 0.5, 3.0])) * torch.randn(B, L, generator=g)
    adv = torch.randn(B, L, generator=g) * float(rng.choice([0.1, 1.0, 10.0]))
    if case % 4 == 0:
        adv[:, ::3] = 0.0
    lens = torch.from_numpy(rng.integers(0 if case % 5 == 0 else 1, L + 1, B))
    mask = (torch.arange(L)[None, :] < lens[:, None])
    if case % 3 == 0:  # holes inside the responses
        mask = mask & (torch.rand(B, L, generator=g) > 0.2)
    mdt = [torch.int64, torch.bool, torch.float32, torch.int32][case % 4]
    lo, hi = float(rng.choice([0.1, 0.2, 3e-4])), float(rng.choice([0.2, 0.28, 4e-4]))
    cfg = SimpleNamespace(clip_ratio=lo, clip_ratio_low=lo, clip_ratio_high=hi, clip_ratio_c=float(rng.choice([1.5, 3.0, 10.0])))
    isw = torch.rand(B, L, generator=g) + 0.5 if case % 6 == 0 else None
    return B, L, lp, old, adv, mask.to(mdt), cfg, isw


@pytest.mark.parametrize("loss", ["vanilla", "gspo"])
def test_sweep_policy_loss(dev, loss):
    """Random shapes, masks (empty rows, holes, every dtype), clip ranges and aggregation modes: the four returned
    loss and KL within 2e-5 + 1e-5 relative of the fp64 oracle; clip fractions within 1e-6 and d loss / d log_prob
    within 1e-6 + 1e-5 relative of the fp32 oracle."""
    import siirl_amd.core_algos as CA

    rng = np.random.default_rng((201 if loss == "vanilla" else 202) + _SEED)
    ofn = OC.compute_policy_loss_vanilla if loss == "vanilla" else OC.compute_policy_loss_gspo
    fn = CA.compute_policy_loss_vanilla if loss == "vanilla" else CA.compute_policy_loss_gspo
    for case in range(80):
        B, L, lp, old, adv, mask, cfg, isw = _loss_case(rng, case)
        mode = AGGS[case % 4]
        if mode == "seq-mean-token-mean" or loss == "gspo":
            mask = mask.clone()
            mask[:, 0] = 1  # an all-masked row makes this mode NaN in the reference too; covered elsewhere
        x64 = lp.double().requires_grad_(True)
        want = ofn(old.double(), x64, adv.double(), mask.double() if mask.dtype != torch.bool else mask, mode, cfg,
                   None if isw is None else isw.double())
        x32 = lp.clone().requires_grad_(True)
        want32 = ofn(old, x32, adv, mask, mode, cfg, isw)
        x = lp.to(dev).requires_grad_(True)
        got = fn(old.to(dev), x, adv.to(dev), mask.to(dev), mode, cfg, None if isw is None else isw.to(dev))
        # loss and KL are continuous in the inputs: against the float64 value.  The clip fractions and the branch a
        # token's gradient takes are comparisons of float32 quantities (a ratio that rounds onto `1 - eps` is a tie in
        # float32 and not in float64): against the oracle run in the reference's own dtype.
        # Float32 accumulation is accurate relative to the sum of the magnitudes of the signed terms it adds
        # (|token loss| <= |A| * ratio * weight, ratio < 3 here), not relative to what cancellation leaves of them:
        # 2^-27 of that sum on top of the bar (a row-sum mode at L in the hundreds adds up to ~1e-5).
        mag = 3.0 * adv.double().abs() * (isw.double() if isw is not None else 1.0)
        slack = 2.0 ** -27 * float(OC.agg_loss(mag, mask.double(), mode if loss == "vanilla" else "seq-mean-token-mean"))
        for k in (0, 2):
            a, b = float(got[k].detach()), float(want[k].detach())
            assert abs(a - b) <= 2e-5 + 1e-5 * abs(b) + (slack if k == 0 else 0.0), (case, loss, mode, k, a, b, slack)
        for k in (1, 3):
            a, b = float(got[k]), float(want32[k])
            assert abs(a - b) <= 1e-6, (case, loss, mode, k, a, b)
        if float(mask.double().sum()) > 0:
            got[0].backward()
            want32[0].backward()
            err = (x.grad.cpu() - x32.grad).abs()
            assert bool((err <= 1e-6 + 1e-5 * x32.grad.abs()).all()), (case, loss, mode, err.max().item())


def test_sweep_gae_and_value_loss(dev):
    import siirl_amd.core_algos as CA

    rng = np.random.default_rng(203 + _SEED)
    for case in range(60):
        B, L = int(rng.integers(1, 40)), int(rng.integers(1, 700))
        g = torch.Generator().manual_seed(case + _SEED)
        rewards, values = torch.randn(B, L, generator=g), torch.randn(B, L, generator=g)
        lens = torch.from_numpy(rng.integers(1, L + 1, B))
        mask = (torch.arange(L)[None, :] < lens[:, None]).long()
        if B * L < 3 or int(mask.sum()) < 2:
            continue
        gamma, lam = float(rng.choice([1.0, 0.99, 0.9])), float(rng.choice([1.0, 0.95, 0.5]))
        a_o, r_o = OC.compute_gae_advantage_return(rewards.double(), values.double(), mask, gamma, lam)
        a, r = CA.compute_gae_advantage_return(rewards.to(dev), values.to(dev), mask.to(dev), gamma, lam)
        scale = max(1.0, float(a_o.abs().max()))
        assert (a.cpu().double() - a_o).abs().max() <= 2e-4 * scale, (case, B, L, gamma, lam)
        assert (r.cpu().double() - r_o).abs().max() <= 1e-4 * max(1.0, float(r_o.abs().max())), (case, B, L)
        mode = AGGS[case % 4]
        vp64 = (values + 0.3 * torch.randn(B, L, generator=g)).double().requires_grad_(True)
        r32 = r_o.float()  # both sides get the same float32 returns: the clip fraction counts strict comparisons
        want = OC.compute_value_loss(vp64, r32.double(), values.double(), mask.double(), 0.2, mode)
        vp = vp64.detach().float().to(dev).requires_grad_(True)
        got = CA.compute_value_loss(vp, r32.to(dev), values.to(dev), mask.to(dev), 0.2, mode)
        # the loss against the float64 value; the clip fraction counts strict comparisons of float32 quantities (a
        # prediction within a rounding of `values + cliprange` falls on either side in float64), so it is compared
        # with the oracle run in the reference's own dtype
        vp32 = vp64.detach().float().requires_grad_(True)
        want32 = OC.compute_value_loss(vp32, r32, values, mask.float(), 0.2, mode)
        assert abs(float(got[0].detach()) - float(want[0].detach())) <= 2e-5 + 2e-5 * abs(float(want[0].detach())), \
            (case, mode, float(got[0].detach()), float(want[0].detach()))
        assert abs(float(got[1]) - float(want32[1])) <= 1e-6, (case, mode, float(got[1]), float(want32[1]))
        got[0].backward()
        want32[0].backward()  # which branch of the maximum a token's gradient takes is the same float32 comparison
        err = (vp.grad.cpu() - vp32.grad).abs()
        assert bool((err <= 1e-6 + 2e-5 * vp32.grad.abs()).all()), (case, mode, err.max().item())


def test_sweep_logprob_entropy(dev):
    """Random row counts, vocabulary sizes (odd, tiny, beyond one workgroup pass), dtypes, temperatures and row-strided
    views: log-prob and entropy within 1e-3 of the fp32 oracle, dlogits within 1 ulp of the logits dtype of the fp64
    oracle, plus the absolute error that fp32 rounding of lse and E[z] leaves (about 2^-23 * max|z| * |g|)."""
    import siirl_amd.torch_functional as SF
    from oracle import torch_functional as OF

    rng = np.random.default_rng(204 + _SEED)
    for case in range(90):
        T = int(rng.integers(1, 50))
        V = int(rng.choice([1, 2, 3, 7, 64, 255, 256, 257, 1000, 4097, 8191, 32000, 40001, int(rng.integers(1, 70000))]))
        dt = [torch.bfloat16, torch.float32, torch.float16][case % 3]
        temp = float(rng.choice([1.0, 0.6, 1.7]))
        g = torch.Generator().manual_seed(case + _SEED)
        pad = int(rng.choice([0, 0, 8, 5]))
        base = (torch.randn(T, V + pad, generator=g) * float(rng.choice([0.5, 3.0, 8.0]))).to(dt)
        x = base[:, :V]  # a row-strided view when pad > 0
        y = torch.randint(0, V, (T,), generator=g)
        g_lp, g_h = torch.randn(T, generator=g), torch.randn(T, generator=g)
        xd = base.to(dev)[:, :V].detach().requires_grad_(True)
        lp, ent = SF.logprobs_and_entropy_from_logits(xd, y.to(dev), temperature=temp)
        lp_o, ent_o, _, _ = OF.logprob_entropy_forward(x, y, temp, dtype=torch.float32)
        assert (lp.detach().cpu() - lp_o).abs().max() < 1e-3 and (ent.detach().cpu() - ent_o).abs().max() < 1e-3, (case, T, V, dt)
        torch.autograd.backward([lp, ent], [g_lp.to(dev), g_h.to(dev)])
        d64 = OF.logprob_entropy_backward(x, y, g_lp, g_h, temp, dtype=torch.float64)
        got = xd.grad.cpu()
        assert got.dtype == dt and got.shape == (T, V)
        eps = {torch.bfloat16: 2.0 ** -8, torch.float16: 2.0 ** -11, torch.float32: 2.0 ** -23}[dt]
        # fp32 arithmetic rounds lse and E[z] to about 2^-23 * max|z|; where the softmax is saturated that is an
        # absolute error of p, hence of the gradient, of that size times the upstream gradients
        zmax = (x.double().abs().max(dim=-1).values / temp).unsqueeze(-1)
        fp32_abs = 2.4e-7 * zmax * (g_lp.double().abs() + g_h.double().abs() * (1 + zmax)).unsqueeze(-1) / temp
        tol = 2 * eps * d64.abs() + 1e-6 + fp32_abs + (1e-5 * d64.abs() if dt == torch.float32 else 0)
        err = (got.double() - d64).abs()
        assert bool((err <= tol).all()), (case, T, V, dt, temp, float((err - tol).max()))


def test_sweep_logprob_entropy_over_random_views(dev):
    """Log-prob, entropy and their gradient over randomly sliced (..., V) views -- row-strided, outer-strided, with
    size-1 axes, rows that are not 16-byte aligned, an ignored label here and there -- in the three logits dtypes,
    against the fp64 oracle.  Tolerances: 2e-5 on the fp32 outputs against the fp64 value of the same (rounded)
    inputs; dlogits within 1 ulp of a 16-bit logits dtype (2^-7 relative for bf16, 2^-10 for fp16) and 5e-6 relative
    for fp32 (fp32 arithmetic with a hardware exp2 against the fp64 value), plus an absolute floor of a few fp32 ulps of
    the row's coefficients."""
    import random

    import siirl_amd.torch_functional as SF
    from oracle import torch_functional as OF

    rel = {torch.bfloat16: 2.0 ** -7, torch.float16: 2.0 ** -10, torch.float32: 5e-6}
    for case in range(160):
        rnd = random.Random(7000 + case + _SEED)
        g = torch.Generator().manual_seed(7000 + case + _SEED)
        dtype = (torch.bfloat16, torch.float32, torch.float16)[case % 3]
        nd = rnd.randint(1, 3)
        V = rnd.choice((1, 7, 8, 33, 250, 1031))
        lead = [rnd.choice((1, 2, 3, 5, 9)) for _ in range(nd)]
        pad = [rnd.randint(0, 3) for _ in range(nd)] + [rnd.choice((0, 0, 1, 8, 13))]
        base = (torch.randn(*[n + 2 * p for n, p in zip(lead, pad[:-1])], V + 2 * pad[-1], generator=g) * 2.5).to(dtype)
        idx = tuple(slice(p, p + n) for n, p in zip(lead, pad[:-1])) + (slice(pad[-1], pad[-1] + V),)
        xs = base[idx]
        y = torch.randint(0, V, lead, generator=g)
        if case % 9 == 0:
            y.view(-1)[0] = -100
        w1, w2 = torch.randn(lead, generator=g), torch.randn(lead, generator=g)
        leaf = base.to(dev).requires_grad_(True)
        view = leaf[idx]
        pairing = case % 2 == 0
        SF.set_pairing(pairing)
        try:
            lp = SF.logprobs_from_logits(view, y.to(dev), inplace_backward=False)
            ent = SF.entropy_from_logits(view)
            ((lp * w1.to(dev)).sum() + (ent * w2.to(dev)).sum()).backward()
        finally:
            SF.set_pairing(True)
        lp_o = OF.logprobs_from_logits_flash_attn(xs, y, dtype=torch.float64)
        ent_o = OF.entropy_from_logits(xs, dtype=torch.float64)
        assert (lp.detach().cpu().double() - lp_o).abs().max() < 2e-5, (case, "logprob")
        assert (ent.detach().cpu().double() - ent_o).abs().max() < 2e-5, (case, "entropy")
        xo = xs.double().requires_grad_(True)
        (OF.logprobs_from_logits_flash_attn(xo, y) * w1.double()).sum().backward()
        d_lp = xo.grad
        d_ent = OF.logprob_entropy_backward(xs, y.clamp(min=0), None, w2, dtype=torch.float64)
        want = d_lp + d_ent
        got = leaf.grad.cpu()
        mag = want.abs() if pairing else d_lp.abs() + d_ent.abs() + want.abs()
        err = (got[idx].double() - want).abs()
        # absolute floor: fp32 rounding of the row's coefficients, which scale with the upstream gradients and with
        # |x| (`p * (c0 + c1 * x)` cancels where x is near the row's mean logit), and of the probability itself, whose
        # exponent z - lse carries a rounding error proportional to |x| (it shows at the label of a confident row,
        # where g_lp * (1 - p) cancels)
        amax = xs.double().abs().amax(-1)
        floor = 1e-6 + 2e-7 * (w1.abs() * amax.clamp(min=1.0) + 2 * w2.abs() * amax).double().unsqueeze(-1)
        bound = rel[dtype] * mag + floor
        worst = int((err - bound).argmax())
        row = worst // xs.shape[-1]
        assert bool((err <= bound).all()), (
            f"case {case} {dtype} shape {tuple(xs.shape)} stride {xs.stride()}: worst element err "
            f"{err.flatten()[worst].item():.3e} > bound {bound.flatten()[worst].item():.3e}, want "
            f"{want.flatten()[worst].item():.3e}; its row: |x| max {amax.flatten()[row].item():.3e}, w1 "
            f"{w1.flatten()[row].item():.3e}, w2 {w2.flatten()[row].item():.3e}")
        outside = got.clone()
        outside[idx] = 0
        assert torch.count_nonzero(outside) == 0, (case, "gradient outside the view")


def test_sweep_loss_functions_over_shapes_dtypes_and_layouts(dev):
    """The [B, L] loss functions as callers may hand them operands: 1-D, 2-D and 3-D tensors, log-probs in fp32 /
    bf16 / fp64, masks in every dtype (and non-contiguous), operands that are transposed views; values against the
    fp64 oracle on the same (rounded) inputs to 1e-5 relative + 1e-6, gradients to 1e-5 relative + 1e-7 (the gradient
    of a 16-bit log-prob comes back in that dtype: 2^-7 relative), shapes and dtypes of the gradients as autograd
    expects them."""
    import random
    from types import SimpleNamespace

    import siirl_amd.core_algos as CA
    from oracle import core_algos as OC

    aggs = ["token-mean", "seq-mean-token-sum", "seq-mean-token-mean", "seq-mean-token-sum-norm"]
    for case in range(120):
        rnd = random.Random(9100 + case + _SEED)
        g = torch.Generator().manual_seed(9100 + case + _SEED)
        nd = rnd.choice((1, 2, 2, 3))
        shape = [rnd.choice((1, 2, 3, 7)) for _ in range(nd - 1)] + [rnd.choice((1, 5, 64, 300, 2500))]
        lp_dtype = (torch.float32, torch.bfloat16, torch.float64)[case % 3]
        lp0 = (torch.randn(shape, generator=g) * 0.7 - 1.5).to(lp_dtype)
        old = lp0.float() + torch.randn(shape, generator=g) * 0.15
        ref = lp0.float() + torch.randn(shape, generator=g) * 0.3
        adv = torch.randn(shape, generator=g)
        mask_b = torch.rand(shape, generator=g) > 0.3
        mask_b.view(-1)[0] = True
        mask = {0: mask_b, 1: mask_b.long(), 2: mask_b.float(), 3: mask_b.to(torch.int32), 4: mask_b.to(torch.bfloat16)}[case % 5]
        agg = aggs[case % 4]
        if agg == "seq-mean-token-mean":  # keep every row non-empty: an empty one is NaN by definition
            m2 = mask_b.reshape(-1, shape[-1])
            m2[:, 0] = True
            mask = m2.reshape(shape).to(mask.dtype)
            mask_b = mask.bool()
        cfg = SimpleNamespace(clip_ratio=0.2, clip_ratio_low=rnd.choice((0.1, 0.2)), clip_ratio_high=rnd.choice((0.2, 0.28)),
                              clip_ratio_c=rnd.choice((1.5, 3.0)))
        ocfg = OC.LossConfig(0.2, cfg.clip_ratio_low, cfg.clip_ratio_high, cfg.clip_ratio_c)
        transposed = nd == 2 and case % 4 == 1  # hand over non-contiguous views of contiguous transposes
        to_dev = (lambda t: t.t().contiguous().to(dev).t()) if transposed else (lambda t: t.to(dev))
        lp = to_dev(lp0).requires_grad_(True)
        which = case % 3
        if which == 0:
            pg, cf, kl, cfl = CA.compute_policy_loss_vanilla(to_dev(old), lp, to_dev(adv), to_dev(mask), agg, cfg)
            total = pg
        elif which == 1:
            kld = CA.kl_penalty(lp, to_dev(ref), "low_var_kl")
            total = CA.agg_loss(kld, to_dev(mask), agg)
        else:
            total = CA.agg_loss(lp * 1.0, to_dev(mask), agg)
        total.backward()
        assert lp.grad.shape == lp.shape and lp.grad.dtype == lp_dtype
        # oracle on the same rounded inputs, 2-D view
        L = shape[-1]
        x64 = lp0.double().reshape(-1, L).requires_grad_(True)
        m64 = mask_b.reshape(-1, L).double()
        if which == 0:
            want, cf_o, kl_o, cfl_o = OC.compute_policy_loss_vanilla(old.double().reshape(-1, L), x64,
                                                                     adv.double().reshape(-1, L), m64, agg, ocfg)
            assert abs(kl.item() - float(kl_o)) < 1e-5 + 1e-5 * abs(float(kl_o)), (case, "ppo_kl")
            # clip fractions and the branch a token's gradient takes are comparisons of float32 quantities (a ratio
            # that rounds onto a clip bound ties in float32 only): against the oracle in the reference's own dtype
            x32 = lp0.float().reshape(-1, L).requires_grad_(True)
            w32, cf_32, _, cfl_32 = OC.compute_policy_loss_vanilla(old.reshape(-1, L), x32, adv.reshape(-1, L),
                                                                   m64.float(), agg, ocfg)
            assert abs(cf.item() - float(cf_32)) < 1e-6 and abs(cfl.item() - float(cfl_32)) < 1e-6, (case, "clipfrac")
            w32.backward()
        elif which == 1:
            want = OC.agg_loss(OC.kl_penalty(x64, ref.double().reshape(-1, L), "low_var_kl"), m64, agg)
        else:
            want = OC.agg_loss(x64, m64, agg)
        want.backward()
        # a 16-bit log-prob makes kl_penalty return 16-bit values (as the reference's arithmetic would): bf16 accuracy
        vtol = 2.0 ** -7 if (lp_dtype == torch.bfloat16 and which == 1) else 1e-5
        tol = 1e-6 + vtol * abs(want.item())
        if which == 0:
            # the policy loss sums terms of both signs: float32 accumulation is accurate relative to the sum of their
            # magnitudes (|tok| <= |A| * ratio, ratio < 2 here), not relative to what is left after they cancel
            mag = OC.agg_loss(2.0 * adv.double().abs().reshape(-1, L), m64, agg).item()
            tol += 2.0 ** -24 * mag / 8
        assert abs(total.item() - want.item()) < tol, (case, which, agg, total.item(), want.item())
        gw = (x32.grad.double() if which == 0 else x64.grad).reshape(shape)
        rel = 2.0 ** -6 if lp_dtype == torch.bfloat16 else 1e-5
        err = (lp.grad.cpu().double() - gw).abs()
        assert bool((err <= rel * gw.abs() + 1e-7).all()), (case, which, agg, lp_dtype, tuple(shape), err.max().item())


def test_sweep_marft_gae(dev):
    """Random requests, agents, row lengths, token counts (zero included) and mask dtypes: the multi-agent token walk
    equals the oracle's bit for bit, in float and in the mask's dtype."""
    import siirl_amd.core_algos as CA

    rng = np.random.default_rng(110 + _SEED)
    for case in range(40):
        n_agents = int(rng.integers(1, 6))
        lens = rng.integers(1, 5, size=int(rng.integers(1, 6))).tolist()
        B = int(sum(lens))
        widths = rng.integers(1, 140, size=n_agents).tolist()
        mdt = [torch.int64, torch.int32, torch.uint8, torch.bool][case % 4]
        rews = [torch.from_numpy(rng.standard_normal((B, w)).astype(np.float32) * 4) for w in widths]
        vals = [torch.from_numpy(rng.standard_normal((B, w)).astype(np.float32) * 4) for w in widths]
        masks = [torch.from_numpy((np.arange(w)[None] < rng.integers(0, w + 1, (B, 1))).astype(np.int64)).to(mdt)
                 for w in widths]
        chains, row = [], 0
        for n in lens:
            chains.append((row, int(n)))
            row += int(n)
        gamma, lam = float(rng.choice([1.0, 0.99, 0.9])), float(rng.choice([1.0, 0.95, 0.5]))
        out_dtype = torch.float32 if case % 2 else None
        want_a, want_r = OC.marft_gae_unwhitened(rews, vals, masks, chains, gamma, lam, out_dtype=out_dtype)
        got_a, got_r = CA.marft_gae_unwhitened([t.to(dev) for t in rews], [t.to(dev) for t in vals],
                                               [t.to(dev) for t in masks], chains, gamma, lam, out_dtype=out_dtype)
        for a in range(n_agents):
            assert torch.equal(got_a[a].cpu(), want_a[a]) and torch.equal(got_r[a].cpu(), want_r[a]), (case, a, widths, lens)
