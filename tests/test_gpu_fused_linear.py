"""GPU parity: fused lm_head + log-prob/entropy (MFMA kernels through the C ABI) vs the CPU oracle.

Tolerances: logprob / entropy within 1e-3 absolute of the fp32 oracle (exact products of the bf16 inputs);
d_hidden / d_weight are bf16 outputs of fp32-accumulated GEMMs over bf16-rounded dlogits: compared with the fp64
oracle at the bar that those two roundings give (``tests/grad_bar.py``: 1 % of the tensor's largest magnitude per
element, 5e-3 relative in Frobenius norm; the observed figures are printed)."""

import os

import numpy as np
import pytest
import torch

from grad_bar import check_fused_grad
from oracle import fused_linear as OFL

pytestmark = pytest.mark.gpu


def _inputs(T, H, V, seed):
    g = torch.Generator().manual_seed(seed)
    h = torch.randn(T, H, generator=g).to(torch.bfloat16)
    w = (torch.randn(V, H, generator=g) * (2.0 / H ** 0.5)).to(torch.bfloat16)
    y = torch.randint(0, V, (T,), generator=g)
    g_lp = torch.randn(T, generator=g) * 1e-2
    g_h = torch.randn(T, generator=g) * 1e-2
    return h, w, y, g_lp, g_h


def _check_grad(got, want64, name, floor=1e-7):
    check_fused_grad(got, want64, name, floor)


@pytest.mark.parametrize("T,H,V", [(1, 64, 1), (5, 64, 33), (256, 64, 256), (300, 128, 1000), (513, 256, 8200),
                                   (64, 3584, 2048), (700, 192, 17000), (257, 64, 32769), (130, 128, 65537)])
@pytest.mark.parametrize("temperature", [1.0, 0.7])
def test_fused_matches_oracle(dev, T, H, V, temperature):
    from siirl_amd.fused_linear import FusedLinearForPPO

    h, w, y, g_lp, g_h = _inputs(T, H, V, seed=T + H + V)
    hd = h.to(dev).requires_grad_(True)
    wd = w.to(dev).requires_grad_(True)
    lp, ent = FusedLinearForPPO()(hd, wd, y.to(dev), temperature=temperature)
    assert lp.shape == (T,) and lp.dtype == torch.float32
    lp_o, ent_o = OFL.fused_linear_for_ppo_fwd(h, w, y, temperature, dtype=torch.float32)
    lp64, ent64 = OFL.fused_linear_for_ppo_fwd(h, w, y, temperature, dtype=torch.float64)
    assert (lp.cpu() - lp_o).abs().max() < 1e-3 and (ent.cpu() - ent_o).abs().max() < 1e-3
    assert (lp.cpu().double() - lp64).abs().max() < 1e-4 and (ent.cpu().double() - ent64).abs().max() < 1e-4
    torch.autograd.backward([lp, ent], [g_lp.to(dev), g_h.to(dev)])
    dh64, dw64 = OFL.fused_linear_for_ppo_bwd(g_lp, g_h, h, w, y, temperature, dtype=torch.float64)
    assert hd.grad.dtype == torch.bfloat16 and wd.grad.shape == w.shape
    _check_grad(hd.grad, dh64, "d_hidden")
    _check_grad(wd.grad, dw64, "d_weight")


def test_fused_random_shapes_sweep(dev):
    """Seeded random token counts, hidden sizes and vocabulary sizes (around the 256-row tile, the 8192-column slab and
    the 65536-column group boundaries as well as arbitrary ones), temperatures, and which of the two gradients flows,
    on both backward routes.  ``SIIRL_TEST_SEED=<int>`` in the environment shifts the seeds."""
    import random

    from siirl_amd import fused_linear as FL

    shift = 100003 * int(os.environ.get("SIIRL_TEST_SEED", "0"))
    edges = (1, 2, 255, 256, 257, 511, 513, 8191, 8192, 8193, 16385)
    try:
        for case in range(14):
            rnd = random.Random(4100 + case + shift)
            T = rnd.choice((1, 7, 63, 64, 65, 255, 256, 257, rnd.randint(1, 600)))
            H = 64 * rnd.choice((1, 2, 3, 5, 8))
            V = rnd.choice(edges) if case % 2 else rnd.randint(1, 24000)
            if case == 5:
                V = 65536 + rnd.choice((-1, 0, 1, 300))
                T, H = min(T, 130), 64
            temperature = rnd.choice((1.0, 0.6, 1.9))
            which = rnd.choice(("both", "both", "logprob", "entropy"))
            h, w, y, g_lp, g_h = _inputs(T, H, V, seed=4100 + case + shift)
            FL.set_saved_logits_limit((1 << 34) if case % 3 == 0 else 0)
            hd = h.to(dev).requires_grad_(True)
            wd = w.to(dev).requires_grad_(True)
            lp, ent = FL.FusedLinearForPPO()(hd, wd, y.to(dev), temperature=temperature)
            lp64, ent64 = OFL.fused_linear_for_ppo_fwd(h, w, y, temperature, dtype=torch.float64)
            what = (case, T, H, V, temperature, which)
            assert (lp.cpu().double() - lp64).abs().max() < 1e-4 and (ent.cpu().double() - ent64).abs().max() < 1e-4, what
            outs, grads = [], []
            if which != "entropy":
                outs.append(lp), grads.append(g_lp.to(dev))
            if which != "logprob":
                outs.append(ent), grads.append(g_h.to(dev))
            torch.autograd.backward(outs, grads)
            zero = torch.zeros_like(g_lp)
            dh64, dw64 = OFL.fused_linear_for_ppo_bwd(g_lp if which != "entropy" else zero,
                                                      g_h if which != "logprob" else zero, h, w, y, temperature,
                                                      dtype=torch.float64)
            # floor: a one-word vocabulary has a gradient of exactly zero, which fp32 sums over T tokens of 1e-2-sized
            # terms that cancel reach only to a few 1e-7
            _check_grad(hd.grad, dh64, f"d_hidden {what}", floor=1e-6)
            _check_grad(wd.grad, dw64, f"d_weight {what}", floor=1e-6)
    finally:
        FL.set_saved_logits_limit(0)


def test_single_branches_3d_and_linear_cross_entropy(dev):
    from siirl_amd.fused_linear import FusedLinearForPPO, linear_cross_entropy

    B, S, H, V = 3, 50, 128, 3000
    h, w, y, g_lp, g_h = _inputs(B * S, H, V, seed=9)
    h3, y3 = h.reshape(B, S, H), y.reshape(B, S)
    hd = h3.to(dev).requires_grad_(True)
    wd = w.to(dev).requires_grad_(True)
    lp, ent = FusedLinearForPPO(chunk_size=64)(hd, wd, y3.to(dev))
    assert lp.shape == (B, S) and ent.shape == (B, S)
    lp64, ent64 = OFL.fused_linear_for_ppo_fwd(h, w, y, dtype=torch.float64)
    assert (lp.cpu().double().reshape(-1) - lp64).abs().max() < 1e-4
    # log-prob branch only
    lp.backward(g_lp.reshape(B, S).to(dev))
    dh64, dw64 = OFL.fused_linear_for_ppo_bwd(g_lp, None, h, w, y, dtype=torch.float64)
    _check_grad(hd.grad.reshape(-1, H), dh64, "d_hidden(lp only)")
    _check_grad(wd.grad, dw64, "d_weight(lp only)")
    # entropy branch only, weight frozen
    hd2 = h.to(dev).requires_grad_(True)
    lp2, ent2 = linear_cross_entropy(hd2, w.to(dev), y.to(dev), 1.0, "none", None)
    assert (ent2.cpu().double() - ent64).abs().max() < 1e-4
    ent2.backward(g_h.to(dev))
    dh64, _ = OFL.fused_linear_for_ppo_bwd(None, g_h, h, w, y, dtype=torch.float64)
    _check_grad(hd2.grad, dh64, "d_hidden(entropy only)")
    s, _ = linear_cross_entropy(h.to(dev), w.to(dev), y.to(dev), 1.0, "sum", None)
    m, _ = linear_cross_entropy(h.to(dev), w.to(dev), y.to(dev), 1.0, "mean", None)
    assert abs(float(s) - float(lp64.sum())) < 1e-2 and abs(float(m) - float(lp64.mean())) < 1e-4
    with pytest.raises(ValueError, match="Invalid reduction"):
        linear_cross_entropy(h.to(dev), w.to(dev), y.to(dev), 1.0, "max", None)
    with pytest.raises(AssertionError):
        linear_cross_entropy(h.to(dev), w.to(dev), y.to(dev), 1, "none", None)
    cast = FusedLinearForPPO(cast_outputs=True)(h.to(dev), w.to(dev), y.to(dev))
    assert cast[0].dtype == torch.bfloat16
    with pytest.raises(ValueError, match="multiple of 64"):
        FusedLinearForPPO()(h[:, :100].contiguous().to(dev), w[:, :100].contiguous().to(dev), y.to(dev))


def test_fused_vs_fixtures(dev):
    from siirl_amd.fused_linear import fused_linear_logprob_entropy

    G = np.load(os.path.join(os.path.dirname(__file__), "golden", "oracle_small.npz"))
    h = torch.from_numpy(G["fl_hidden_bf16_bits"].copy()).view(torch.bfloat16)
    w = torch.from_numpy(G["fl_weight_bf16_bits"].copy()).view(torch.bfloat16)
    y = torch.from_numpy(G["fl_ids"])
    hd, wd = h.to(dev).requires_grad_(True), w.to(dev).requires_grad_(True)
    lp, ent = fused_linear_logprob_entropy(hd, wd, y.to(dev))
    assert np.abs(lp.detach().cpu().numpy() - G["fl_logprob"]).max() < 1e-3
    assert np.abs(ent.detach().cpu().numpy() - G["fl_entropy"]).max() < 1e-3
    torch.autograd.backward([lp, ent], [torch.from_numpy(G["fl_g_lp"]).to(dev), torch.from_numpy(G["fl_g_h"]).to(dev)])
    _check_grad(hd.grad, torch.from_numpy(G["fl_dhidden"]), "d_hidden")
    _check_grad(wd.grad, torch.from_numpy(G["fl_dweight"]), "d_weight")


@pytest.mark.parametrize("T,H,V", [(64, 64, 300), (257, 128, 32769), (1000, 192, 40000), (130, 128, 65537)])
@pytest.mark.parametrize("which", ["both", "logprob", "entropy"])
def test_saved_logits_route_equals_recompute(dev, T, H, V, which):
    """The backward that reads the logit tiles the forward parked gives the bits of the backward that recomputes
    them; the forward's outputs do not depend on whether it parks them."""
    import siirl_amd.fused_linear as FL

    g = torch.Generator().manual_seed(T + V)
    h = (torch.randn(T, H, generator=g) * 0.7).to(torch.bfloat16).to(dev)
    w = (torch.randn(V, H, generator=g) * 0.2).to(torch.bfloat16).to(dev)
    y = torch.randint(0, V, (T,), generator=g).to(dev)
    g_lp, g_h = torch.randn(T, generator=g).to(dev), torch.randn(T, generator=g).to(dev)
    out = {}
    try:
        for name, limit in (("saved", 1 << 40), ("recompute", 0)):
            FL.set_saved_logits_limit(limit)
            hd, wd = h.clone().requires_grad_(True), w.clone().requires_grad_(True)
            lp, ent = FL.fused_linear_logprob_entropy(hd, wd, y, 0.8)
            outs, grads = {"both": ([lp, ent], [g_lp, g_h]), "logprob": ([lp], [g_lp]), "entropy": ([ent], [g_h])}[which]
            torch.autograd.backward(outs, grads)
            out[name] = (lp.detach(), ent.detach(), hd.grad, wd.grad)
    finally:
        FL.set_saved_logits_limit(0)
    for a, b, what in zip(out["saved"], out["recompute"], ("logprob", "entropy", "d_hidden", "d_weight")):
        assert torch.equal(a, b), what


def test_saved_logits_limit_and_no_grad(dev):
    import siirl_amd.fused_linear as FL

    ns = torch.ops.siirl_hip
    h = torch.randn(70, 64, device=dev).to(torch.bfloat16)
    w = torch.randn(500, 64, device=dev).to(torch.bfloat16)
    y = torch.randint(0, 500, (70,), device=dev)
    lp, ent, lse, ex, sv = ns.fused_linear_logprob_entropy_fwd(h, w, y, 1.0, True)
    assert sv.numel() == 2 * 1 * 65536
    with pytest.raises(ValueError, match="saved"):
        ns.fused_linear_logprob_entropy_bwd(h, w, y, 1.0, lse, ex, torch.ones(70, device=dev), None, True, True, sv[:-1])
    with pytest.raises(ValueError):
        FL.set_saved_logits_limit(-1)
    assert FL._saved_logits_bytes(70, 500) == torch.ops.siirl_hip.fused_linear_logprob_entropy_fwd(
        h, w, y, 1.0, True)[4].numel() * 4


def test_parked_logits_allocation_failure_falls_back_to_recompute(dev):
    """When the buffer for the parked logits cannot be allocated the forward keeps nothing and the backward
    recomputes: same results, no error.  The failure is a real one: 65536 tokens x 1.2 M vocabulary entries need
    314 GB of parked tiles, more than the device has, while everything else about the problem is small (H = 64)."""
    import siirl_amd.fused_linear as FL

    T, H, V = 65536, 64, 1200128
    assert FL._saved_logits_bytes(T, V) > torch.cuda.get_device_properties(dev).total_memory
    g = torch.Generator(device=dev).manual_seed(1)
    h = (torch.randn(T, H, device=dev, generator=g) * 0.7).to(torch.bfloat16)
    w = (torch.randn(V, H, device=dev, generator=g) * 0.2).to(torch.bfloat16)
    y = torch.randint(0, V, (T,), device=dev, generator=g)

    def run():
        hd, wd = h.clone().requires_grad_(True), w.clone().requires_grad_(True)
        lp, ent = FL.fused_linear_logprob_entropy(hd, wd, y)
        (lp.sum() + ent.sum()).backward()
        return lp.detach(), ent.detach(), hd.grad, wd.grad

    try:
        FL.set_saved_logits_limit(0)
        want = run()
        FL.set_saved_logits_limit(1 << 50)
        assert torch.ops.siirl_hip.fused_linear_logprob_entropy_fwd(h, w, y, 1.0, True)[4].numel() == 0
        got = run()
    finally:
        FL.set_saved_logits_limit(0)
        torch.cuda.empty_cache()
    for a, b in zip(got, want):
        assert torch.equal(a, b)


@pytest.fixture
def rows_left_out():
    """The opt-in backward that leaves rows without upstream gradient out of its GEMMs (off by default)."""
    import siirl_amd.fused_linear as FL

    FL.set_skip_zero_rows(True)
    yield
    FL.set_skip_zero_rows(False)


def _live_rows(T, pattern, seed):
    g = torch.Generator().manual_seed(seed)
    if pattern == "packed":  # sequences of prompt + response tokens: only the response rows carry a gradient
        live = torch.zeros(T, dtype=torch.bool)
        t = 0
        while t < T:
            n = int(torch.randint(3, 40, (1,), generator=g))
            p = int(torch.randint(1, n, (1,), generator=g))
            live[t + p:t + n] = True
            t += n
        return live
    if pattern == "random":
        return torch.rand(T, generator=g) < 0.4
    if pattern == "one":
        live = torch.zeros(T, dtype=torch.bool)
        live[T // 2] = True
        return live
    if pattern == "none":
        return torch.zeros(T, dtype=torch.bool)
    return torch.ones(T, dtype=torch.bool)


@pytest.mark.parametrize("T,H,V", [(7, 64, 50), (300, 128, 1000), (513, 256, 8200), (1000, 192, 40000)])
@pytest.mark.parametrize("pattern", ["packed", "random", "one", "none", "all"])
def test_zero_gradient_rows_left_out_of_backward(dev, T, H, V, pattern):
    """Token rows whose two upstream gradients are zero are left out of the backward's GEMMs: d_hidden is exactly
    zero there (also where the hidden state holds NaN), both gradients match the oracle's, and they are, bit for
    bit, what the plain backward gives on the gathered rows."""
    import siirl_amd.fused_linear as FL

    h, w, y, g_lp, g_h = _inputs(T, H, V, seed=3 * T + V)
    live = _live_rows(T, pattern, seed=T + V)
    g_lp, g_h = g_lp * live, g_h * live
    if pattern == "packed":
        g_h = g_h * (torch.arange(T) % 3 != 0)  # rows with a log-prob gradient only
    rows = torch.nonzero((g_lp != 0) | (g_h != 0)).reshape(-1)
    dh64, dw64 = OFL.fused_linear_for_ppo_bwd(g_lp, g_h, h, w, y, 0.9, dtype=torch.float64)
    out = {}
    for skip in (True, False):
        FL.set_skip_zero_rows(skip)
        try:
            hd, wd = h.to(dev).requires_grad_(True), w.to(dev).requires_grad_(True)
            lp, ent = FL.fused_linear_logprob_entropy(hd, wd, y.to(dev), 0.9)
            torch.autograd.backward([lp, ent], [g_lp.to(dev), g_h.to(dev)])
        finally:
            FL.set_skip_zero_rows(False)
        _check_grad(hd.grad, dh64, f"d_hidden skip={skip}")
        _check_grad(wd.grad, dw64, f"d_weight skip={skip}")
        out[skip] = (hd.grad, wd.grad)
    dead = ~live
    assert not out[True][0][dead.to(dev)].any()
    assert torch.equal(out[True][0], out[False][0])  # a row of d_hidden does not depend on the other rows
    if len(rows) == T:
        assert torch.equal(out[True][1], out[False][1])
    elif len(rows):
        # the plain backward on the gathered operands
        ns = torch.ops.siirl_hip
        hc, yc = h[rows].to(dev), y[rows].to(dev)
        _, _, lse, ex, _ = ns.fused_linear_logprob_entropy_fwd(hc, w.to(dev), yc, 1 / 0.9, False)
        d_hc, d_w = ns.fused_linear_logprob_entropy_bwd(hc, w.to(dev), yc, 1 / 0.9, lse, ex, g_lp[rows].to(dev),
                                                        g_h[rows].to(dev), True, True)
        assert torch.equal(out[True][1], d_w)
        assert torch.equal(out[True][0][rows.to(dev)], d_hc)
    else:
        assert not out[True][1].any()


def test_zero_gradient_rows_hide_nan_hidden_states(dev, rows_left_out):
    import siirl_amd.fused_linear as FL

    T, H, V = 200, 64, 700
    h, w, y, g_lp, g_h = _inputs(T, H, V, seed=11)
    live = torch.arange(T) >= 60
    h[:60] = float("nan")
    hd, wd = h.to(dev).requires_grad_(True), w.to(dev).requires_grad_(True)
    lp, ent = FL.fused_linear_logprob_entropy(hd, wd, y.to(dev), 1.0)
    torch.autograd.backward([lp, ent], [(g_lp * live).to(dev), (g_h * live).to(dev)])
    assert torch.isfinite(hd.grad).all() and torch.isfinite(wd.grad).all()
    assert not hd.grad[:60].any()
    dh64, dw64 = OFL.fused_linear_for_ppo_bwd(g_lp[60:], g_h[60:], h[60:], w, y[60:], 1.0, dtype=torch.float64)
    _check_grad(hd.grad[60:], dh64, "d_hidden")
    _check_grad(wd.grad, dw64, "d_weight")


def test_default_backward_lets_nan_of_a_zero_gradient_row_through(dev):
    """Without the opt-in the backward is dense: a NaN hidden state in a row whose upstream gradients are zero reaches
    d_weight and that row of d_hidden, as ``0 * NaN`` does through the reference's autograd
    (``experimental/torch_functional.py:49-67``)."""
    import siirl_amd.fused_linear as FL

    T, H, V = 200, 64, 700
    h, w, y, g_lp, g_h = _inputs(T, H, V, seed=11)
    live = torch.arange(T) >= 60
    h[:60] = float("nan")
    hd, wd = h.to(dev).requires_grad_(True), w.to(dev).requires_grad_(True)
    lp, ent = FL.fused_linear_logprob_entropy(hd, wd, y.to(dev), 1.0)
    torch.autograd.backward([lp, ent], [(g_lp * live).to(dev), (g_h * live).to(dev)])
    assert torch.isnan(wd.grad).any() and torch.isnan(hd.grad[:60]).any()
    assert torch.isfinite(hd.grad[60:]).all()


def test_backward_rows_through_the_c_abi(dev):
    """siirl_fused_linear_logprob_entropy_bwd_rows called directly: rows in any order, an index outside [0, T)
    contributes nothing, a short workspace and a bad count are refused."""
    import ctypes as C

    from siirl_amd import _lib

    T, H, V = 260, 64, 900
    h, w, y, g_lp, g_h = _inputs(T, H, V, seed=5)
    hd, wd, yd = h.to(dev), w.to(dev), y.to(dev)
    ns = torch.ops.siirl_hip
    _, _, lse, ex, _ = ns.fused_linear_logprob_entropy_fwd(hd, wd, yd, 1.0, False)
    lib = _lib.lib()
    st = _lib.current_stream(dev)

    def call(rows, n=None, ws_short=0):
        rows_d = torch.tensor(rows, dtype=torch.int64, device=dev)
        n = len(rows) if n is None else n
        nws = lib.siirl_fused_linear_bwd_rows_workspace_bytes(max(n, 0), H, V, 1, 1)
        ws = torch.empty(max(nws - ws_short, 256), dtype=torch.uint8, device=dev)
        d_h = torch.full((T, H), 7.0, dtype=torch.bfloat16, device=dev)
        d_w = torch.full((V, H), 7.0, dtype=torch.bfloat16, device=dev)
        glp_d, gh_d = g_lp.to(dev), g_h.to(dev)
        rc = lib.siirl_fused_linear_logprob_entropy_bwd_rows(
            _lib.ptr(hd), _lib.ptr(wd), _lib.BF16, _lib.ptr(yd), T, H, V, 1.0, _lib.ptr(lse), _lib.ptr(ex),
            _lib.ptr(glp_d), _lib.ptr(gh_d), _lib.ptr(rows_d), n, _lib.ptr(d_h), _lib.ptr(d_w), _lib.ptr(ws),
            C.c_size_t(nws - ws_short), st)
        torch.cuda.synchronize()
        return rc, d_h, d_w

    picked = [259, 3, 100, 17, 256, 4]
    rc, d_h, d_w = call(picked)
    assert rc == 0
    sel = torch.zeros(T, dtype=torch.bool)
    sel[picked] = True
    dh64, dw64 = OFL.fused_linear_for_ppo_bwd(g_lp * sel, g_h * sel, h, w, y, 1.0, dtype=torch.float64)
    _check_grad(d_h, dh64, "d_hidden")
    _check_grad(d_w, dw64, "d_weight")
    assert not d_h[(~sel).to(dev)].any()
    rc, d_h2, d_w2 = call(picked + [T + 5, -1])
    assert rc == 0
    assert torch.equal(d_h2, d_h)
    _check_grad(d_w2, dw64, "d_weight with two rows outside the batch")
    rc, d_h0, d_w0 = call([])
    assert rc == 0 and not d_h0.any() and not d_w0.any()
    assert call(picked, ws_short=512)[0] == -4
    assert call(picked, n=T + 1)[0] == -1
    assert call(picked, n=-1)[0] == -1


def test_zero_gradient_rows_sweep(dev, rows_left_out):
    """Seeded random shapes and row patterns (``SIIRL_TEST_SEED`` shifts the seed): the backward that leaves rows out
    against the oracle, and zero rows of d_hidden exactly zero."""
    import siirl_amd.fused_linear as FL

    rng = np.random.default_rng(4242 + 100003 * int(os.environ.get("SIIRL_TEST_SEED", "0")))
    for case in range(10):
        T, H, V = int(rng.integers(1, 600)), 64 * int(rng.integers(1, 4)), int(rng.integers(2, 9000))
        h, w, y, g_lp, g_h = _inputs(T, H, V, seed=int(rng.integers(1 << 30)))
        live = torch.from_numpy(rng.random(T) < rng.random())
        g_lp, g_h = g_lp * live, g_h * (live & torch.from_numpy(rng.random(T) < 0.7))
        temperature = float(rng.choice([1.0, 0.6, 1.3]))
        dh64, dw64 = OFL.fused_linear_for_ppo_bwd(g_lp, g_h, h, w, y, temperature, dtype=torch.float64)
        hd, wd = h.to(dev).requires_grad_(True), w.to(dev).requires_grad_(True)
        lp, ent = FL.fused_linear_logprob_entropy(hd, wd, y.to(dev), temperature)
        torch.autograd.backward([lp, ent], [g_lp.to(dev), g_h.to(dev)])
        _check_grad(hd.grad, dh64, f"d_hidden case {case} {(T, H, V)}")
        _check_grad(wd.grad, dw64, f"d_weight case {case} {(T, H, V)}")
        assert not hd.grad[(~live).to(dev)].any(), (case, T, H, V)


@pytest.mark.parametrize("wrt", ["hidden", "weight"])
def test_zero_gradient_rows_with_one_gradient_requested(dev, wrt, rows_left_out):
    """The row-subset backward when only d_hidden or only d_weight is asked for."""
    import siirl_amd.fused_linear as FL

    T, H, V = 300, 128, 1000
    h, w, y, g_lp, g_h = _inputs(T, H, V, seed=77)
    live = _live_rows(T, "packed", seed=77)
    g_lp, g_h = g_lp * live, g_h * live
    dh64, dw64 = OFL.fused_linear_for_ppo_bwd(g_lp, g_h, h, w, y, 1.0, dtype=torch.float64)
    hd = h.to(dev).requires_grad_(wrt == "hidden")
    wd = w.to(dev).requires_grad_(wrt == "weight")
    lp, ent = FL.fused_linear_logprob_entropy(hd, wd, y.to(dev), 1.0)
    torch.autograd.backward([lp, ent], [g_lp.to(dev), g_h.to(dev)])
    if wrt == "hidden":
        assert wd.grad is None
        _check_grad(hd.grad, dh64, "d_hidden")
        assert not hd.grad[(~live).to(dev)].any()
    else:
        assert hd.grad is None
        _check_grad(wd.grad, dw64, "d_weight")


@pytest.mark.parametrize("dtype", [torch.float16, torch.float32])
@pytest.mark.parametrize("T,H,V", [(5, 64, 33), (300, 128, 1000), (513, 256, 8200), (64, 3584, 2048), (130, 128, 65537)])
def test_fp16_and_fp32_operands(dev, dtype, T, H, V):
    """hidden and W in float16 / float32 (the reference multiplies in whatever dtype they arrive,
    ``experimental/torch_functional.py:20-23``): log-prob and entropy against the oracle on the same values -- exact
    fp16 products on the half matrix instruction; three bf16 terms per fp32 element, good to 2^-16 per product --,
    gradients in the operands' dtype at the fused path's bar (bf16 dlogits times bf16-rounded operands, no more
    roundings than with bf16 operands once the outputs are fp16 / fp32).  Upstream gradients of order 1 here: a
    softmax gradient of order 1e-2 / V underflows an fp16 *result*, which is what loss scaling is for."""
    from siirl_amd.fused_linear import FusedLinearForPPO, linear_cross_entropy

    g = torch.Generator().manual_seed(7 * T + H + V)
    h = torch.randn(T, H, generator=g).to(dtype)
    w = (torch.randn(V, H, generator=g) * (2.0 / H ** 0.5)).to(dtype)
    y = torch.randint(0, V, (T,), generator=g)
    g_lp, g_h = torch.randn(T, generator=g), torch.randn(T, generator=g)
    hd, wd = h.to(dev).requires_grad_(True), w.to(dev).requires_grad_(True)
    lp, ent = FusedLinearForPPO()(hd, wd, y.to(dev), temperature=0.8)
    assert lp.dtype == torch.float32 and ent.dtype == torch.float32
    lp64, ent64 = OFL.fused_linear_for_ppo_fwd(h, w, y, 0.8, dtype=torch.float64)
    e_lp, e_ent = (lp.cpu().double() - lp64).abs().max().item(), (ent.cpu().double() - ent64).abs().max().item()
    print(f"[operands {dtype}] ({T}, {H}, {V}): logprob err {e_lp:.2e}, entropy err {e_ent:.2e}", flush=True)
    assert e_lp < 1e-4 and e_ent < 1e-4, (e_lp, e_ent)
    torch.autograd.backward([lp, ent], [g_lp.to(dev), g_h.to(dev)])
    assert hd.grad.dtype == dtype and wd.grad.dtype == dtype
    dh64, dw64 = OFL.fused_linear_for_ppo_bwd(g_lp, g_h, h, w, y, 0.8, dtype=torch.float64)
    _check_grad(hd.grad, dh64, f"d_hidden {dtype}", floor=1e-6)
    _check_grad(wd.grad, dw64, f"d_weight {dtype}", floor=1e-6)
    # the Triton-shaped interface and the row-subset backward take the same operands
    lp2, ent2 = linear_cross_entropy(h.to(dev), w.to(dev), y.to(dev), 0.8, "none", None)
    assert torch.equal(lp2, lp.detach()) and torch.equal(ent2, ent.detach())
    if T >= 64:
        live = (torch.arange(T) % 3 != 0).float()
        hd2, wd2 = h.to(dev).requires_grad_(True), w.to(dev).requires_grad_(True)
        lp3, ent3 = FusedLinearForPPO()(hd2, wd2, y.to(dev), temperature=0.8)
        torch.autograd.backward([lp3, ent3], [(g_lp * live).to(dev), (g_h * live).to(dev)])
        dh64s, dw64s = OFL.fused_linear_for_ppo_bwd(g_lp * live, g_h * live, h, w, y, 0.8, dtype=torch.float64)
        _check_grad(hd2.grad, dh64s, f"d_hidden {dtype}, rows without gradient left out", floor=1e-6)
        _check_grad(wd2.grad, dw64s, f"d_weight {dtype}, rows without gradient left out", floor=1e-6)
        assert torch.count_nonzero(hd2.grad[live == 0]) == 0


def test_fp16_and_fp32_random_shapes_sweep(dev):
    """Seeded random shapes with float16 / float32 operands on both backward routes (recompute and parked logits),
    around the same tile, slab and group boundaries as the bf16 sweep.  ``SIIRL_TEST_SEED=<int>`` shifts the seeds."""
    import random

    from siirl_amd import fused_linear as FL

    shift = 100003 * int(os.environ.get("SIIRL_TEST_SEED", "0"))
    edges = (1, 2, 255, 256, 257, 513, 8191, 8192, 8193, 16385)
    try:
        for case in range(12):
            rnd = random.Random(5200 + case + shift)
            dtype = (torch.float16, torch.float32)[case % 2]
            T = rnd.choice((1, 7, 63, 64, 65, 255, 256, 257, rnd.randint(1, 600)))
            H = 64 * rnd.choice((1, 2, 3, 5))
            V = rnd.choice(edges) if case % 3 else rnd.randint(1, 20000)
            if case == 7:
                T, H, V = 100, 64, 65536 + rnd.choice((-1, 0, 1, 300))
            temperature = rnd.choice((1.0, 0.6, 1.9))
            which = rnd.choice(("both", "both", "logprob", "entropy"))
            g = torch.Generator().manual_seed(5200 + case + shift)
            h = torch.randn(T, H, generator=g).to(dtype)
            w = (torch.randn(V, H, generator=g) * (2.0 / H ** 0.5)).to(dtype)
            y = torch.randint(0, V, (T,), generator=g)
            g_lp, g_h = torch.randn(T, generator=g), torch.randn(T, generator=g)
            FL.set_saved_logits_limit((1 << 34) if case % 4 < 2 else 0)
            hd, wd = h.to(dev).requires_grad_(True), w.to(dev).requires_grad_(True)
            lp, ent = FL.FusedLinearForPPO()(hd, wd, y.to(dev), temperature=temperature)
            lp64, ent64 = OFL.fused_linear_for_ppo_fwd(h, w, y, temperature, dtype=torch.float64)
            what = (case, dtype, T, H, V, temperature, which)
            assert (lp.cpu().double() - lp64).abs().max() < 1e-4 and (ent.cpu().double() - ent64).abs().max() < 1e-4, what
            outs, grads = [], []
            if which != "entropy":
                outs.append(lp), grads.append(g_lp.to(dev))
            if which != "logprob":
                outs.append(ent), grads.append(g_h.to(dev))
            torch.autograd.backward(outs, grads)
            zero = torch.zeros_like(g_lp)
            dh64, dw64 = OFL.fused_linear_for_ppo_bwd(g_lp if which != "entropy" else zero,
                                                      g_h if which != "logprob" else zero, h, w, y, temperature,
                                                      dtype=torch.float64)
            assert hd.grad.dtype == dtype and wd.grad.dtype == dtype
            _check_grad(hd.grad, dh64, f"d_hidden {what}", floor=1e-5)
            _check_grad(wd.grad, dw64, f"d_weight {what}", floor=1e-5)
    finally:
        FL.set_saved_logits_limit(0)


def test_mixed_operand_dtypes_are_refused(dev):
    from siirl_amd.fused_linear import fused_linear_logprob_entropy

    h = torch.randn(8, 64, device=dev)
    w = torch.randn(16, 64, device=dev).to(torch.bfloat16)
    y = torch.zeros(8, dtype=torch.int64, device=dev)
    with pytest.raises(TypeError, match="one dtype"):
        fused_linear_logprob_entropy(h, w, y)
    with pytest.raises(TypeError):
        fused_linear_logprob_entropy(h.double(), w.double(), y)
