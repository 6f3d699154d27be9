#!/usr/bin/env python3
"""Benchmark of the per-token RL loss hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--no-cpu-baseline]

A step is one pass of the hot path over one batch: log-prob + entropy forward over bf16 logits
``[32768, 152064]`` (8 sequences x 4096 tokens, Qwen2.5-7B vocabulary), then the backward pass that
writes ``dlogits`` -- the "logprob+entropy fwd+bwd" workload the headline metric is quoted on.  Inputs are
synthetic and resident in HBM before the timed region.  One JSON line is printed at the end.

``roofline`` describes the dominant kernel (the backward): algorithmic bytes per launch (read the row,
write the gradient: 4 * V bytes per token for bf16) over its average duration, measured with events on
the launch stream inside the timed region.  ``cpu_baseline`` times the CPU oracle (a torch restatement
of the reference's eager ops) on a bounded row sample of the same tensor on the host cores.
"""

from __future__ import annotations

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

METRIC = "logprob+entropy fwd+bwd tokens/sec @vocab152k bf16; % HBM roofline"
HBM_PEAK_GBS = 8000.0  # MI355X HBM3E, published peak

# Config 2 of the baseline: 8 sequences x 4096 tokens, vocab 152064, bf16 logits ~ N(0, 3) with one +15
# spike in 1% of the rows, uniform labels, upstream gradients ~ N(0, 1e-2) zeroed on padded rows
# (sequence lengths uniform in [512, 4096]).
SEQS, SEQ_LEN, VOCAB = 8, 4096, 152064
SEED = 20250602

# HBM bytes per launch of the dominant kernel (lpe_bwd_flat_kernel at the default workload) from two
# rocprofv3 --pmc runs, FETCH_SIZE and WRITE_SIZE in KiB per dispatch, each scaled by what the same
# counter reads for a plain 2 GiB device copy (FETCH_SIZE reads half the bytes fetched: factor 2.0;
# WRITE_SIZE factor 1.0).  Figures and commands: profiles/lpe_config2_hbm_traffic.md
MEASURED_TRAFFIC_BYTES = int((4872246.35 * 2.0 + 9733599.87) * 1024)
# The same for loss_partials_kernel + loss_bwd_kernel at config 3 with 5488 kept trajectories
# (profiles/loss_path_config3_hbm_traffic.md)
MEASURED_TRAFFIC_BYTES_CONFIG3 = int(((526927.5 + 527223.3) * 2.0 + 1372.0 + 176093.0) * 1024)


def cpu_model() -> str:
    """Model name of the host CPU the baseline leg runs on."""
    try:
        with open("/proc/cpuinfo") as f:
            for line in f:
                if line.lower().startswith("model name"):
                    return line.split(":", 1)[1].strip()
    except OSError:
        pass
    return "unknown"


def make_workload(dev, seqs=SEQS, seq_len=SEQ_LEN, vocab=VOCAB, seed=SEED):
    import torch

    T = seqs * seq_len
    gen = torch.Generator(device=dev).manual_seed(seed)
    logits = torch.empty(T, vocab, dtype=torch.bfloat16, device=dev)
    for lo in range(0, T, 2048):  # chunked so that the fp32 staging stays small
        n = min(2048, T - lo)
        logits[lo : lo + n] = (torch.randn(n, vocab, device=dev, generator=gen) * 3.0).to(torch.bfloat16)
    n_spike = max(1, T // 100)
    rows = torch.randperm(T, device=dev, generator=gen)[:n_spike]
    cols = torch.randint(0, vocab, (n_spike,), device=dev, generator=gen)
    logits[rows, cols] = (logits[rows, cols].float() + 15.0).to(torch.bfloat16)
    labels = torch.randint(0, vocab, (T,), device=dev, generator=gen)
    lengths = torch.randint(512, seq_len + 1, (seqs,), device=dev, generator=gen)
    mask = (torch.arange(seq_len, device=dev)[None, :] < lengths[:, None]).reshape(T).float()
    g_lp = torch.randn(T, device=dev, generator=gen) * 1e-2 * mask
    g_ent = torch.randn(T, device=dev, generator=gen) * 1e-2 * mask
    return logits, labels, g_lp, g_ent, mask


def cpu_baseline(logits, labels, g_lp, g_ent, rows=4096, iters=5):
    """Oracle (``kind: port``): the reference's eager ops on fp32-upcast rows, forward + autograd backward."""
    import torch

    from oracle import torch_functional as OF

    x = logits[:rows].float().cpu()
    y, a, b = labels[:rows].cpu(), g_lp[:rows].cpu(), g_ent[:rows].cpu()
    times = []
    for it in range(iters + 1):
        xr = x.clone().requires_grad_(True)
        t0 = time.perf_counter()
        lp = OF.logprobs_from_logits(xr, y)
        ent = OF.entropy_from_logits(xr)
        torch.autograd.grad([lp, ent], [xr], [a, b])
        dt = time.perf_counter() - t0
        if it:  # first pass is the warm-up
            times.append(dt)
    times.sort()
    med = times[len(times) // 2]
    return {"value": rows / med, "unit": "tokens/s", "cores": torch.get_num_threads(), "cpu": cpu_model(), "kind": "port",
            "sample": f"first {rows} of {logits.shape[0]} rows of the same tensor, upcast to fp32; "
                      f"median of {iters} fwd+bwd passes ({med:.2f} s each)"}


def gemm_rate(config5_line):
    """TFLOP/s of the forward GEMM of a config 5 line."""
    return next(v["TFLOP/s"] for k, v in config5_line["kernels"].items() if k.startswith("forward"))


def bench_config3(args, dev, quick=False):
    """DAPO [B, L] path at config 3: 512 prompts x 16 responses, L = 8192 fp32.  One step = dynamic-sampling keep
    mask over the 8192 trajectories, GRPO advantages on the kept ones, and the fused actor loss (asymmetric clip,
    low-variance KL term) forward + backward over the kept [~5.7k, 8192] tokens.  Not the headline."""
    import torch
    from types import SimpleNamespace

    import siirl_amd.core_algos as CA
    import siirl_amd.dapo_filter as DF

    P, n, L = 512, 16, 8192
    B = P * n
    gen = torch.Generator(device=dev).manual_seed(SEED)
    uid = torch.from_numpy(DF.make_uid(P, n)).to(dev)
    # ~30 % of the groups get one score for every member and are dropped by the filter
    solved = torch.rand(P, device=dev, generator=gen)
    acc = (torch.rand(B, device=dev, generator=gen) < 0.5).float()
    acc = torch.where(solved.repeat_interleave(n) < 0.3, torch.ones_like(acc), acc)
    lens = torch.randint(L // 16, L + 1, (B,), device=dev, generator=gen)
    mask = (torch.arange(L, device=dev)[None] < lens[:, None]).long()
    rewards = torch.zeros(B, L, device=dev)
    rewards[torch.arange(B, device=dev), lens - 1] = acc
    keep = DF.group_keep_mask(acc, uid)
    kept = torch.nonzero(keep).flatten()
    Bk = int(kept.numel())
    lp = torch.randn(Bk, L, device=dev, generator=gen) - 1.5
    old = lp + 0.05 * torch.randn(Bk, L, device=dev, generator=gen)
    ref = lp + 0.1 * torch.randn(Bk, L, device=dev, generator=gen)
    # the filter's index select of the kept trajectories (reference data_coordinator/sample.py:242-322)
    kept_list = kept.tolist()
    sel = DF.filter_tensordict({"response_mask": mask, "token_level_rewards": rewards, "uid": uid}, kept_list)
    mk, rk, uk = sel["response_mask"], sel["token_level_rewards"], sel["uid"]
    cfg = SimpleNamespace(clip_ratio=0.2, clip_ratio_low=0.2, clip_ratio_high=0.28, clip_ratio_c=10.0,
                          entropy_coeff=0.0, use_kl_loss=True, kl_loss_coef=0.001, kl_loss_type="low_var_kl",
                          loss_agg_mode="token-mean", loss_mode="vanilla")
    x = lp.requires_grad_(True)

    def step(ev=None):
        if ev:
            ev[0].record()
        DF.group_keep_mask(acc, uid)
        adv, _ = CA.compute_grpo_outcome_advantage(rk, mk, uk)
        if ev:
            ev[1].record()
        out = CA.actor_loss(old, x, adv, mk, cfg, ref_log_prob=ref)
        out.loss.backward()
        if ev:
            ev[2].record()
        x.grad = None

    steps, warm = args.steps, args.warmup
    for _ in range(warm):
        step()
    torch.cuda.synchronize()
    evs = [[torch.cuda.Event(enable_timing=True) for _ in range(3)] for _ in range(steps)]
    t0 = time.perf_counter()
    for k in range(steps):
        step(evs[k])
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    grp_ms = sum(e[0].elapsed_time(e[1]) for e in evs) / steps
    loss_ms = sum(e[1].elapsed_time(e[2]) for e in evs) / steps
    tokens = Bk * L
    loss_bytes = tokens * (2 * (4 * 4 + 8) + 4)  # forward and backward each read 4 fp32 operands + int64 mask; d_lp written

    # the path's smaller building blocks on the same [kept, L] tensors, each timed alone (not part of the step)
    import siirl_amd.torch_functional as SF

    block_ms = None
    gbs = loss_bytes / loss_ms / 1e6

    if not quick:
        def timed_ms(fn, iters=10):
            fn()
            torch.cuda.synchronize()
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            for _ in range(iters):
                fn()
            e1.record()
            torch.cuda.synchronize()
            return e0.elapsed_time(e1) / iters

        lpd = lp.detach()
        kl_ctrl = CA.FixedKLController(0.001)
        td = {"token_level_scores": rk, "old_log_probs": old, "ref_log_prob": ref, "response_mask": mk}
        lm = torch.randn(Bk, L, device=dev, generator=gen).requires_grad_(True)

        def agg_fb():
            CA.agg_loss(lm, mk, "seq-mean-token-mean").backward()
            lm.grad = None

        adv_b, _ = CA.compute_grpo_outcome_advantage(rk, mk, uk)
        cov_cfg = SimpleNamespace(clip_ratio=0.2, clip_ratio_low=0.2, clip_ratio_high=0.28, clip_ratio_c=10.0,
                                  policy_loss=SimpleNamespace(kl_cov_ratio=0.0002, ppo_kl_coef=1.0, clip_cov_ratio=0.0002,
                                                              clip_cov_lb=1.0, clip_cov_ub=5.0))

        def kl_cov_fb():
            CA.compute_policy_loss_kl_cov(old, x, adv_b, mk, "token-mean", cov_cfg)[0].backward()
            x.grad = None

        cov_scores, cov_stats = torch.ops.siirl_hip.cov_scores(None, lpd, adv_b, mk, CA.LOSS_KL_COV, 0.0, 0.0)
        k_cov = max(1, int(int(float(cov_stats[0]) + float(cov_stats[4])) * 0.0002))
        blocks = {
            "kl_cov policy loss forward + backward: scores, top-k pick, loss, gradient (108 B/token)": (kl_cov_fb, 108),
            f"siirl_topk_mark: the {k_cov} largest of the covariance scores marked (20 B/token: four reads, one write)":
                (lambda: torch.ops.siirl_hip.topk_mark(cov_scores, k_cov, 1.0), 20),
            "masked_mean(values, mask) -> scalar (12 B/token)": (lambda: SF.masked_mean(lpd, mk), 12),
            "masked_mean(values, mask, axis=-1) -> [B] (12 B/token)": (lambda: SF.masked_mean(lpd, mk, axis=-1), 12),
            "kl_penalty low_var_kl forward (12 B/token)": (lambda: CA.kl_penalty(lpd, ref, "low_var_kl"), 12),
            "apply_kl_penalty: rewards = scores - beta * kl * mask, batch KL, one host sync (24 B/token)":
                (lambda: CA.apply_kl_penalty(td, kl_ctrl, "low_var_kl"), 24),
            "agg_loss seq-mean-token-mean forward + backward (28 B/token)": (agg_fb, 28),
            # per kept token: the int64 mask and the fp32 rewards, read and written once each (the uids are B values)
            "filter_tensordict: the kept trajectories of response_mask, token_level_rewards and uid selected (24 B/token)":
                (lambda: DF.filter_tensordict({"response_mask": mask, "token_level_rewards": rewards, "uid": uid}, kept_list), 24),
        }
        block_ms = {}
        for name, (fn, bpt) in blocks.items():
            ms = timed_ms(fn)
            block_ms[name] = {"ms": ms, "GB/s": tokens * bpt / ms / 1e6}
    out = {
        "metric": "DAPO loss path (filter + GRPO advantage + clipped loss fwd+bwd) tokens/sec @[B,L] fp32",
        "value": tokens * steps / wall, "unit": "tokens/s", "n_gpus": 1, "steps": steps, "warmup": warm,
        "ms_per_step": wall * 1e3 / steps, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f32", "data": "synthetic",
        "config": {"workload": f"config3: {P} prompts x {n} responses, L = {L}; {Bk} trajectories kept by the filter",
                   "trajectories": B, "kept": Bk, "response_length": L, "seed": SEED},
        "kernels": {"keep mask + GRPO advantage": {"ms": grp_ms},
                    "actor loss forward + backward (loss_partials/finish/bwd kernels)": {"ms": loss_ms, "GB/s": gbs}},
        "building_blocks": block_ms,
        "roofline": {"bound": "hbm", "kernel": "loss_partials_kernel + loss_bwd_kernel", "achieved": gbs, "peak": 8000.0,
                     "unit": "GB/s", "frac": gbs / 8000.0,
                     "traffic": MEASURED_TRAFFIC_BYTES_CONFIG3 if Bk == 5488 else None},
        "cpu_baseline": None,
    }
    if not args.no_cpu_baseline:  # the oracle's eager ops on the host cores, a 512-trajectory sample of the same step
        from oracle import core_algos as OC
        from oracle import dapo_filter as OD

        n_s = 512
        acc_c, uid_c = acc[:n_s * 2].cpu().numpy(), uid[:n_s * 2].cpu().numpy()
        old_c, lp_c, ref_c = old[:n_s].cpu(), lp.detach()[:n_s].cpu(), ref[:n_s].cpu()
        mk_c, rk_c, uk_c = mk[:n_s].cpu(), rk[:n_s].cpu(), uk[:n_s].cpu().numpy()
        times = []
        for it in range(4):
            t1 = time.perf_counter()
            OD.dynamic_sampling_keep_indices(acc_c, uid_c)
            adv_c, _ = OC.compute_grpo_outcome_advantage(rk_c, mk_c, uk_c)
            xc = lp_c.clone().requires_grad_(True)
            pg, *_ = OC.compute_policy_loss_vanilla(old_c, xc, adv_c, mk_c, "token-mean", cfg)
            kl = OC.agg_loss(OC.kl_penalty(xc, ref_c, "low_var_kl"), mk_c, "token-mean")
            (pg + 0.001 * kl).backward()
            if it:
                times.append(time.perf_counter() - t1)
        med = sorted(times)[len(times) // 2]
        out["cpu_baseline"] = {"value": n_s * L / med, "unit": "tokens/s", "cores": torch.get_num_threads(), "cpu": cpu_model(), "kind": "port",
                               "sample": f"first {n_s} kept trajectories (of {Bk}) x {L} tokens, filter over {2 * n_s} "
                                         f"trajectories; median of 3 passes ({med:.2f} s each)"}
    return out


def bench_config5(args, dev, quick=False):
    """Fused lm_head + log-prob/entropy (MFMA path): hidden [16384, 3584] ~ N(0,1), W [152064, 3584] ~ N(0, 0.02),
    bf16, uniform labels, forward + backward to hidden and W.  Not the headline; same JSON shape."""
    import torch

    from siirl_amd.fused_linear import fused_linear_logprob_entropy

    T, H, V = 16384, 3584, 152064
    gen = torch.Generator(device=dev).manual_seed(SEED)
    h = torch.randn(T, H, device=dev, generator=gen).to(torch.bfloat16).requires_grad_(True)
    w = torch.empty(V, H, dtype=torch.bfloat16, device=dev)
    for lo in range(0, V, 16384):
        n = min(16384, V - lo)
        w[lo:lo + n] = (torch.randn(n, H, device=dev, generator=gen) * 0.02).to(torch.bfloat16)
    w.requires_grad_(True)
    y = torch.randint(0, V, (T,), device=dev, generator=gen)
    g_lp = torch.randn(T, device=dev, generator=gen) * 1e-2
    g_h = torch.randn(T, device=dev, generator=gen) * 1e-2

    def step(ev=None):
        if ev:
            ev[0].record()
        lp, ent = fused_linear_logprob_entropy(h, w, y)
        if ev:
            ev[1].record()
        torch.autograd.backward([lp, ent], [g_lp, g_h])
        if ev:
            ev[2].record()
        h.grad = w.grad = None

    import siirl_amd.fused_linear as FL

    steps, warm = min(args.steps, 10), min(args.warmup, 2)

    def timed():
        for _ in range(warm):
            step()
        torch.cuda.synchronize()
        evs = [[torch.cuda.Event(enable_timing=True) for _ in range(3)] for _ in range(steps)]
        t0 = time.perf_counter()
        for k in range(steps):
            step(evs[k])
        torch.cuda.synchronize()
        wall = time.perf_counter() - t0
        return (wall, sum(e[0].elapsed_time(e[1]) for e in evs) / steps,
                sum(e[1].elapsed_time(e[2]) for e in evs) / steps)

    # the route the configuration names (no [T, V] tensor kept: the backward recomputes the logits) is the headline;
    # the opt-in route that parks the fp32 logit tiles between forward and backward is reported beside it
    FL.set_saved_logits_limit(0)
    wall, fwd_ms, bwd_ms = timed()
    gemm = 2.0 * T * H * V
    tf_step = 3 * gemm / (wall / steps) / 1e12

    # yardstick: the vendor library's plain bf16 GEMMs (torch.mm -> hipBLASLt / rocBLAS) of the shapes and operand
    # layouts of the fused path's GEMMs, no epilogue, results written out; reported beside the fused kernels' rates,
    # never part of `value`
    def mm_ms(a, b, out_shape, n=5):
        with torch.no_grad():
            out_buf = torch.empty(out_shape, dtype=torch.bfloat16, device=dev)
            for _ in range(2):
                torch.mm(a, b, out=out_buf)
            torch.cuda.synchronize()
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            for _ in range(n):
                torch.mm(a, b, out=out_buf)
            e1.record()
            torch.cuda.synchronize()
            del out_buf
        return e0.elapsed_time(e1) / n

    Vg = 65536  # one group of dlogits columns, as the backward updates d hidden and d weight
    with torch.no_grad():
        dl = (torch.randn(T, Vg, device=dev, generator=gen) * 1e-3).to(torch.bfloat16)
        lib_ms = mm_ms(w.detach(), h.detach().t(), (V, T))                 # logits^T = W . hidden^T
        lib_dh_ms = mm_ms(dl, w.detach()[:Vg], (T, H))                     # d hidden += dlogits . W_group
        lib_dw_ms = mm_ms(dl.t(), h.detach(), (Vg, H))                     # d weight_group = dlogits^T . hidden
        del dl
    torch.cuda.empty_cache()
    extras = {}
    if not quick:
        FL.set_saved_logits_limit(16 << 30)
        p_wall, p_fwd_ms, p_bwd_ms = timed()
        FL.set_saved_logits_limit(0)
        saved_gb = FL._saved_logits_bytes(T, V) / 1e9
        # the same tensors as a packed batch of 8 sequences of 2048 tokens whose first 512 are prompt tokens: their
        # rows arrive with zero gradients and the backward leaves them out of its GEMMs
        live = (torch.arange(T, device=dev) % 2048 >= 512).float()
        dense_g = (g_lp, g_h)
        g_lp, g_h = dense_g[0] * live, dense_g[1] * live
        FL.set_skip_zero_rows(True)
        r_wall, r_fwd_ms, r_bwd_ms = timed()
        FL.set_skip_zero_rows(False)
        g_lp, g_h = dense_g
        n_live = int(live.sum().item())

        # the same forward launch on quiet operands (all zeros): identical instruction stream, fewer wires toggling.
        # The gap to the timing on the configuration's random operands is what the power limit costs.
        def forward_ms(hh, ww, n=5):
            with torch.no_grad():
                for _ in range(2):
                    fused_linear_logprob_entropy(hh, ww, y)
                torch.cuda.synchronize()
                e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                e0.record()
                for _ in range(n):
                    fused_linear_logprob_entropy(hh, ww, y)
                e1.record()
                torch.cuda.synchronize()
            return e0.elapsed_time(e1) / n

        fwd_random_ms = forward_ms(h.detach(), w.detach())
        hz, wz = torch.zeros_like(h), torch.zeros_like(w)
        fwd_zero_ms = forward_ms(hz, wz)
        del hz, wz
        extras = {
            "parked_variant": {"what": "set_saved_logits_limit(16 GiB): the forward parks its fp32 logit tiles "
                                       f"({saved_gb:.2f} GB) and the backward reads them back instead of recomputing; "
                                       "opt-in, NOT the configuration's route",
                               "ms_per_step": p_wall * 1e3 / steps, "tokens_per_s": T * steps / p_wall,
                               "forward_ms": p_fwd_ms, "backward_ms": p_bwd_ms,
                               "algorithmic_TFLOP/s": 3 * gemm / (p_wall / steps) / 1e12,
                               "frac_of_peak": 3 * gemm / (p_wall / steps) / 1e12 / 2500.0},
            "response_rows_variant": {"what": "8 packed sequences of 2048 tokens, the first 512 of each prompt tokens "
                                              "with zero upstream gradients: the backward runs its GEMMs over the "
                                              f"{n_live} response rows only (set_skip_zero_rows(True))",
                                      "ms_per_step": r_wall * 1e3 / steps, "tokens_per_s": T * steps / r_wall,
                                      "forward_ms": r_fwd_ms, "backward_ms": r_bwd_ms, "rows_with_gradient": n_live},
            "power_limit_probe": {"what": "the forward alone (no grad) on the configuration's random operands and on "
                                          "all-zero operands: same instructions, quieter data",
                                  "forward_ms_random_operands": fwd_random_ms, "TFLOP/s_random": gemm / fwd_random_ms / 1e9,
                                  "forward_ms_zero_operands": fwd_zero_ms, "TFLOP/s_zero": gemm / fwd_zero_ms / 1e9},
        }
    out = {
        "metric": "fused lm_head+logprob/entropy fwd+bwd tokens/sec @vocab152k bf16; % MFMA roofline",
        "value": T * steps / wall, "unit": "tokens/s", "n_gpus": 1, "steps": steps, "warmup": warm,
        "ms_per_step": wall * 1e3 / steps, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16", "data": "synthetic",
        "config": {"workload": f"config5: fused lm_head + logprob/entropy, hidden [{T}, {H}], W [{V}, {H}], fwd + bwd to "
                               "hidden and W, no [T, V] tensor kept (logits recomputed per 8192-column slab in the "
                               "backward)", "tokens": T, "hidden": H, "vocab": V, "seed": SEED},
        "kernels": {"forward (gemm_nt_kernel<SoftmaxPartialsEpi> + merge)": {"ms": fwd_ms, "TFLOP/s": gemm / fwd_ms / 1e9},
                    "backward (recompute + dlogits per slab, d hidden and d weight per 65536 columns)":
                        {"ms": bwd_ms, "TFLOP/s executed": 3 * gemm / bwd_ms / 1e9}},
        "library_gemm_yardstick": {"what": f"torch.mm in bf16 through the vendor library, no epilogue: W [{V}, {H}] . "
                                           f"hidden^T (the forward's and the recompute's GEMM), dlogits [{T}, {Vg}] . "
                                           f"W[:{Vg}] (d hidden of one 65536-column group), dlogits^T . hidden (d weight "
                                           "of one group)",
                                   "ms": lib_ms, "TFLOP/s": gemm / lib_ms / 1e9,
                                   "fused_forward_over_library": (gemm / fwd_ms / 1e9) / (gemm / lib_ms / 1e9),
                                   "d_hidden_shape_TFLOP/s": 2.0 * T * H * Vg / lib_dh_ms / 1e9,
                                   "d_weight_shape_TFLOP/s": 2.0 * T * H * Vg / lib_dw_ms / 1e9},
        **extras,
        "roofline": {"bound": "mfma", "kernel": "gemm_nt_kernel", "achieved": tf_step, "peak": 2500.0, "unit": "TFLOP/s",
                     "frac": tf_step / 2500.0, "traffic": None,
                     "note": "algorithmic flops = 3 GEMMs x 2*T*H*V per step (forward, d hidden, d weight); the "
                             "backward's recomputation of the logits (a fourth GEMM) is executed but not counted"},
        "cpu_baseline": None,
    }
    if not args.no_cpu_baseline:  # the oracle's chunked fp32 matmul + log-softmax on the host cores, 256 tokens
        from oracle import fused_linear as OFL

        n_s = 256
        hc, wc, yc = h.detach()[:n_s].float().cpu(), w.detach().float().cpu(), y[:n_s].cpu()
        gl, gh = g_lp[:n_s].cpu(), g_h[:n_s].cpu()
        times = []
        for it in range(3):
            t1 = time.perf_counter()
            OFL.fused_linear_for_ppo_fwd(hc, wc, yc)
            OFL.fused_linear_for_ppo_bwd(gl, gh, hc, wc, yc)
            if it:
                times.append(time.perf_counter() - t1)
        med = sorted(times)[len(times) // 2]
        out["cpu_baseline"] = {"value": n_s / med, "unit": "tokens/s", "cores": torch.get_num_threads(), "cpu": cpu_model(), "kind": "port",
                               "sample": f"first {n_s} of {T} tokens against the full [{V}, {H}] weight in fp32; "
                                         f"median of 2 fwd+bwd passes ({med:.2f} s each)"}
    return out


def bench_config1(args, dev, quick=False):
    """Config 1, the CPU-runnable GRPO step in fp32: 64 prompts x 8 responses, L = 256, V = 32000.  One step =
    group-normalised advantages over the 512 trajectories, then 64 micro-batches of 8 sequences, each
    logits [2048, 32000] fp32 -> log-prob -> clipped loss (eps 0.2, token-mean) + 0.001 * low_var_kl -> backward to
    the logits.  One logits buffer is reused by every micro-batch (the full tensor would be 16.8 GB); the labels,
    old / reference log-probs, advantages and masks are the micro-batch's own.  Not the headline."""
    import torch
    from types import SimpleNamespace

    import siirl_amd.core_algos as CA
    import siirl_amd.dapo_filter as DF
    import siirl_amd.torch_functional as SF

    SF.set_skip_zero_rows(False)  # dense rows, as the byte count assumes
    P, n, L, V, MB = 64, 8, 256, 32000, 8
    B = P * n
    gen = torch.Generator(device=dev).manual_seed(SEED)
    lens = torch.randint(16, L + 1, (B,), device=dev, generator=gen)
    mask = (torch.arange(L, device=dev)[None] < lens[:, None]).long()
    rewards = torch.zeros(B, L, device=dev)
    rewards[torch.arange(B, device=dev), lens - 1] = (torch.rand(B, device=dev, generator=gen) < 0.5).float()
    uid = torch.from_numpy(DF.make_uid(P, n)).to(dev)
    logits = (torch.randn(MB, L, V, device=dev, generator=gen) * 2.0).requires_grad_(True)
    labels = torch.randint(0, V, (B, L), device=dev, generator=gen)
    with torch.no_grad():
        lp0 = SF.logprobs_from_logits(logits, labels[:MB], inplace_backward=False)
    old = lp0.repeat(B // MB, 1) + 0.05 * torch.randn(B, L, device=dev, generator=gen)
    ref = lp0.repeat(B // MB, 1) + 0.1 * torch.randn(B, L, device=dev, generator=gen)
    cfg = SimpleNamespace(clip_ratio=0.2, clip_ratio_low=0.2, clip_ratio_high=0.2, clip_ratio_c=3.0, entropy_coeff=0.0,
                          use_kl_loss=True, kl_loss_coef=0.001, kl_loss_type="low_var_kl", loss_agg_mode="token-mean",
                          loss_mode="vanilla")
    scale = 1.0 / (B // MB)

    def step():
        adv, _ = CA.compute_grpo_outcome_advantage(rewards, mask, uid)
        for mb in range(B // MB):
            rows = slice(mb * MB, mb * MB + MB)
            lp = SF.logprobs_from_logits(logits, labels[rows], inplace_backward=False)
            out = CA.actor_loss(old[rows], lp, adv[rows], mask[rows], cfg, ref_log_prob=ref[rows], loss_scale_factor=scale)
            out.loss.backward()
            logits.grad = None

    steps, warm = args.steps, args.warmup
    for _ in range(warm):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        step()
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    tokens = B * L
    step_bytes = tokens * V * 4 * 3  # fp32 logits: forward reads the row, backward reads it and writes the gradient

    fused_wall, graph_ms = None, None
    if not quick:
        def fused_step():  # the same step with the single-pass logits -> loss -> dlogits kernel per micro-batch
            adv, _ = CA.compute_grpo_outcome_advantage(rewards, mask, uid)
            for mb in range(B // MB):
                rows = slice(mb * MB, mb * MB + MB)
                CA.fused_actor_step(logits.detach(), labels[rows], old[rows], adv[rows], mask[rows], cfg,
                                    ref_log_prob=ref[rows], loss_scale_factor=scale)

        for _ in range(warm):
            fused_step()
        torch.cuda.synchronize()
        t1 = time.perf_counter()
        for _ in range(steps):
            fused_step()
        torch.cuda.synchronize()
        fused_wall = time.perf_counter() - t1

        # the same 64 single-pass micro-batch steps recorded once into a HIP graph and replayed: one submission per step
        graph_ms = None
        try:
            losses = []

            def graph_body():
                adv, _ = CA.compute_grpo_outcome_advantage(rewards, mask, uid)
                for mb in range(B // MB):
                    rows = slice(mb * MB, mb * MB + MB)
                    losses.append(CA.fused_actor_step(logits.detach(), labels[rows], old[rows], adv[rows], mask[rows], cfg,
                                                      ref_log_prob=ref[rows], loss_scale_factor=scale).loss)

            side = torch.cuda.Stream()
            side.wait_stream(torch.cuda.current_stream())
            with torch.cuda.stream(side):
                graph_body()
            torch.cuda.current_stream().wait_stream(side)
            torch.cuda.synchronize()
            eager_total = float(torch.stack(losses).sum())
            losses.clear()
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph):
                graph_body()
            for _ in range(warm + 1):
                graph.replay()
            torch.cuda.synchronize()
            t2 = time.perf_counter()
            for _ in range(steps):
                graph.replay()
            torch.cuda.synchronize()
            graph_ms = (time.perf_counter() - t2) * 1e3 / steps
            replay_total = float(torch.stack(losses).sum())
            if replay_total != eager_total:
                raise RuntimeError(f"graph replay gives loss {replay_total}, eager {eager_total}")
        except Exception as e:  # reported, never hidden: the eager figures above stand by themselves
            graph_ms = f"failed: {type(e).__name__}: {e}"
    gbs = step_bytes * steps / wall / 1e9
    out = {
        "metric": "GRPO loss step (advantages + 64 micro-batches of logprob fwd, clipped loss + KL, bwd) tokens/sec @vocab32k fp32",
        "value": tokens * steps / wall, "unit": "tokens/s", "n_gpus": 1, "steps": steps, "warmup": warm,
        "ms_per_step": wall * 1e3 / steps, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f32", "data": "synthetic",
        "config": {"workload": f"config1: {P} prompts x {n} responses, L = {L}, V = {V}, fp32, micro-batches of {MB} "
                               f"sequences, eps 0.2, token-mean, low_var_kl x 0.001", "tokens": tokens, "seed": SEED},
        "roofline": {"bound": "hbm", "kernel": "lpe_fwd_kernel + lpe_bwd_flat_kernel (whole step, wall clock)",
                     "achieved": gbs, "peak": 8000.0, "unit": "GB/s", "frac": gbs / 8000.0, "traffic": None,
                     "note": "64 micro-batches of 262 MB each; per micro-batch two logits passes (0.12 ms at the "
                             "config 2 rates) and the [8, 256] loss kernels, issued through the C++ torch.library layer"},
        "fused_step_variant": None if quick else {
            "what": "siirl_actor_step_fused per micro-batch (one pass over the logits)",
            "ms_per_step": fused_wall * 1e3 / steps, "tokens_per_s": tokens * steps / fused_wall,
            "ms_per_step_as_one_hip_graph": graph_ms},
        "cpu_baseline": None,
    }
    if not args.no_cpu_baseline:  # the CPU-runnable case: the oracle on a sample of 8 of the 64 micro-batches
        from oracle import actor_step as OA
        from oracle import core_algos as OC

        n_mb = 8
        rw_c, m_c, uid_c = rewards.cpu(), mask.cpu(), uid.cpu().numpy()
        x_c, y_c, old_c, ref_c = logits.detach().cpu(), labels.cpu(), old.cpu(), ref.cpu()
        ocfg = OA.ActorConfig(clip_ratio=0.2, clip_ratio_low=0.2, clip_ratio_high=0.2, clip_ratio_c=3.0, entropy_coeff=0.0,
                              use_kl_loss=True, kl_loss_coef=0.001, kl_loss_type="low_var_kl", loss_agg_mode="token-mean")
        t1 = time.perf_counter()
        adv_c, _ = OC.compute_grpo_outcome_advantage(rw_c, m_c, uid_c)
        for mb in range(n_mb):
            rows = slice(mb * MB, mb * MB + MB)
            OA.micro_batch_step(x_c, y_c[rows], old_c[rows], adv_c[rows], m_c[rows], ocfg, ref_log_prob=ref_c[rows],
                                loss_scale_factor=scale)
        el = time.perf_counter() - t1
        out["cpu_baseline"] = {"value": n_mb * MB * L / el, "unit": "tokens/s", "cores": torch.get_num_threads(), "cpu": cpu_model(),
                               "kind": "port", "sample": f"advantages over all {B} trajectories + the first {n_mb} of "
                                                         f"{B // MB} micro-batches, one pass ({el:.1f} s)"}
    return out


def bench_config4(args, dev, quick=False):
    """Config 4, GSPO long context: sequences of 32768 response tokens, bf16 logits at V = 151936 (Qwen3), one
    sequence per micro-batch.  One step = one sequence: log-prob forward, GSPO loss (sequence-level ratio, clip
    3e-4 / 4e-4, seq-mean-token-mean, scaled by 1/32) forward + backward, log-prob backward to the logits.  The
    32 sequences of the configuration are 32 such steps over one reused 9.96 GB logits buffer.  Not the headline."""
    import torch
    from types import SimpleNamespace

    import siirl_amd.core_algos as CA
    import siirl_amd.torch_functional as SF

    SF.set_skip_zero_rows(False)  # dense rows, as the byte count assumes
    L, V, NSEQ = 32768, 151936, 32
    gen = torch.Generator(device=dev).manual_seed(SEED)
    x = torch.empty(1, L, V, dtype=torch.bfloat16, device=dev)
    for lo in range(0, L, 2048):
        x[0, lo:lo + 2048] = (torch.randn(2048, V, device=dev, generator=gen) * 3).to(torch.bfloat16)
    x.requires_grad_(True)
    y = torch.randint(0, V, (1, L), device=dev, generator=gen)
    mask = (torch.arange(L, device=dev) < 30000).long()[None]
    adv = torch.full((1, L), 0.7, device=dev)
    with torch.no_grad():
        lp0 = SF.logprobs_from_logits(x, y, inplace_backward=False)
    old = lp0 - 0.02 * torch.randn(1, L, device=dev, generator=gen)
    cfg = SimpleNamespace(clip_ratio=0.2, clip_ratio_low=3e-4, clip_ratio_high=4e-4, clip_ratio_c=3.0, entropy_coeff=0.0,
                          use_kl_loss=False, loss_agg_mode="seq-mean-token-mean", loss_mode="gspo")

    def step():
        lp = SF.logprobs_from_logits(x, y, inplace_backward=False)
        out = CA.actor_loss(old, lp, adv, mask, cfg, loss_scale_factor=1.0 / NSEQ)
        out.loss.backward()
        x.grad = None

    steps, warm = args.steps, args.warmup
    for _ in range(warm):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        step()
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    step_bytes = L * V * 2 * 3
    gbs = step_bytes * steps / wall / 1e9
    out = {
        "metric": "GSPO long-context step (logprob fwd + sequence-level clipped loss fwd+bwd + logprob bwd) tokens/sec @vocab151936 bf16",
        "value": L * steps / wall, "unit": "tokens/s", "n_gpus": 1, "steps": steps, "warmup": warm,
        "ms_per_step": wall * 1e3 / steps, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16", "data": "synthetic",
        "config": {"workload": f"config4: one of {NSEQ} sequences x {L} tokens per step, V = {V}, bf16 logits ~N(0,3), "
                               f"log-ratios ~N(0,0.02), clip 3e-4/4e-4, seq-mean-token-mean", "tokens": L, "seed": SEED},
        "roofline": {"bound": "hbm", "kernel": "lpe_fwd_kernel + lpe_bwd_flat_kernel (whole step, wall clock)",
                     "achieved": gbs, "peak": 8000.0, "unit": "GB/s", "frac": gbs / 8000.0, "traffic": None},
        "cpu_baseline": None,
    }
    if not args.no_cpu_baseline:
        from oracle import actor_step as OA

        rows = 2048
        ocfg = OA.ActorConfig(clip_ratio=0.2, clip_ratio_low=3e-4, clip_ratio_high=4e-4, loss_agg_mode="seq-mean-token-mean",
                              loss_mode="gspo")
        x_c = x.detach()[:, :rows].cpu()
        y_c, old_c, adv_c, m_c = y[:, :rows].cpu(), old[:, :rows].cpu(), adv[:, :rows].cpu(), mask[:, :rows].cpu()
        times = []
        for it in range(3):
            t1 = time.perf_counter()
            OA.micro_batch_step(x_c, y_c, old_c, adv_c, m_c, ocfg)
            if it:
                times.append(time.perf_counter() - t1)
        med = sorted(times)[len(times) // 2]
        out["cpu_baseline"] = {"value": rows / med, "unit": "tokens/s", "cores": torch.get_num_threads(), "cpu": cpu_model(), "kind": "port",
                               "sample": f"first {rows} of {L} tokens of the sequence, upcast to fp32; median of 2 "
                                         f"passes ({med:.2f} s each)"}
    return out


def bench_critic(args, dev):
    """The critic-side operations either side of the path at PPO shape [1024, 8192] fp32: outcome reward placement
    with the overlong penalty, GAE + whitening, the clipped value loss forward + backward, and the per-step data
    metrics.  Not the headline; one JSON line with a per-operation breakdown."""
    import torch
    from types import SimpleNamespace

    import siirl_amd.core_algos as CA
    import siirl_amd.metric_utils as MU
    import siirl_amd.reward as RW

    B, P, L = 1024, 1024, 8192
    gen = torch.Generator(device=dev).manual_seed(SEED)
    lens = torch.randint(L // 16, L + 1, (B,), device=dev, generator=gen)
    mask = (torch.arange(L, device=dev)[None] < lens[:, None]).long()
    amask = torch.cat([torch.ones(B, P, dtype=torch.long, device=dev), mask], 1).contiguous()
    scores = (torch.rand(B, device=dev, generator=gen) < 0.5).double()
    values = torch.randn(B, L, device=dev, generator=gen)
    vpreds = (values + 0.05 * torch.randn(B, L, device=dev, generator=gen)).requires_grad_(True)
    overlong = SimpleNamespace(enable=True, len=1024, penalty_factor=1.0, log=False)
    ops = ("reward placement", "GAE + whitening", "value loss fwd+bwd", "data metrics")

    def step(ev=None):
        rec = (lambda i: ev[i].record()) if ev else (lambda i: None)
        rec(0)
        rewards = RW.place_outcome_reward(scores, amask, L, overlong, max_resp_len=L)
        rec(1)
        adv, ret = CA.compute_gae_advantage_return(rewards, values, mask, 1.0, 0.95)
        rec(2)
        loss, _ = CA.compute_value_loss(vpreds, ret, values, mask, 0.5, "token-mean")
        loss.backward()
        vpreds.grad = None
        rec(3)
        MU.compute_data_metric({"token_level_scores": rewards, "token_level_rewards": rewards, "advantages": adv,
                                "returns": ret, "values": values, "responses": mask, "response_mask": mask,
                                "attention_mask": amask})
        rec(4)
        return rewards, adv, ret

    steps, warm = args.steps, args.warmup
    for _ in range(warm):
        step()
    torch.cuda.synchronize()
    evs = [[torch.cuda.Event(enable_timing=True) for _ in range(5)] for _ in range(steps)]
    t0 = time.perf_counter()
    for k in range(steps):
        step(evs[k])
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    ms = [sum(e[i].elapsed_time(e[i + 1]) for e in evs) / steps for i in range(4)]
    tokens = B * L
    # the same GAE with the chunked scan order (rows cut into 16 chunks scanned in parallel; float32-accurate, not
    # bit-identical to the sequential order above)
    rewards0 = RW.place_outcome_reward(scores, amask, L, overlong, max_resp_len=L)
    CA.set_gae_scan_order("chunked")
    try:
        for _ in range(warm):
            CA.compute_gae_advantage_return(rewards0, values, mask, 1.0, 0.95)
        g0, g1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        g0.record()
        for _ in range(steps):
            CA.compute_gae_advantage_return(rewards0, values, mask, 1.0, 0.95)
        g1.record()
        torch.cuda.synchronize()
        gae_chunked_ms = g0.elapsed_time(g1) / steps
    finally:
        CA.set_gae_scan_order("exact")
    # multi-agent GAE: 128 requests of 4 trajectory steps, 3 agents answering with 1024-2048 tokens each; one call
    # of the token walk (the reference's per-token Python loop), operands on the GPU
    m_req, m_steps, m_w = 128, 4, 2048
    m_rows = m_req * m_steps
    m_vals = [torch.randn(m_rows, m_w, device=dev, generator=gen) for _ in range(3)]
    m_rews = [torch.randn(m_rows, m_w, device=dev, generator=gen) for _ in range(3)]
    m_masks = [(torch.arange(m_w, device=dev)[None] <
                torch.randint(m_w // 2, m_w + 1, (m_rows, 1), device=dev, generator=gen)).long() for _ in range(3)]
    m_chains = [(i * m_steps, m_steps) for i in range(m_req)]
    m_tokens = sum(int(m.sum()) for m in m_masks)
    for _ in range(warm):
        CA.marft_gae_unwhitened(m_rews, m_vals, m_masks, m_chains, 0.99, 0.95)
    torch.cuda.synchronize()
    t1 = time.perf_counter()
    for _ in range(steps):
        CA.marft_gae_unwhitened(m_rews, m_vals, m_masks, m_chains, 0.99, 0.95)
    torch.cuda.synchronize()
    marft_ms = (time.perf_counter() - t1) * 1e3 / steps
    marft = {"ms": marft_ms, "tokens_walked": m_tokens, "tokens_per_s": m_tokens / marft_ms * 1e3}
    # GAE + whitening: the scan reads rewards, values, mask and writes advantages, returns (24 B + 8 B mask), the
    # whitening apply reads and writes the advantages once more
    gae_bytes = tokens * (4 + 4 + 8 + 4 + 4 + 4 + 4)
    out = {
        "metric": "PPO critic-side step (reward placement + GAE/whitening + value loss fwd+bwd + data metrics) tokens/sec @[B,L] fp32",
        "value": tokens * steps / wall, "unit": "tokens/s", "n_gpus": 1, "steps": steps, "warmup": warm,
        "ms_per_step": wall * 1e3 / steps, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f32", "data": "synthetic",
        "config": {"workload": f"critic: {B} trajectories, prompt {P} + response {L}, gamma 1.0, lam 0.95, "
                               f"cliprange_value 0.5, overlong buffer 1024", "seed": SEED},
        "kernels": {**{name: {"ms": t} for name, t in zip(ops, ms)},
                    "GAE + whitening, chunked scan order (not in the step above)": {"ms": gae_chunked_ms},
                    f"multi-agent GAE token walk, {m_req} requests x {m_steps} steps x 3 agents x <= {m_w} tokens "
                    "(not in the step above)": marft},
        "roofline": {"bound": "hbm", "kernel": "gae_scan_vec_kernel + whiten_apply_kernel", "achieved": gae_bytes / ms[1] / 1e6,
                     "peak": 8000.0, "unit": "GB/s", "frac": gae_bytes / ms[1] / 1e6 / 8000.0, "traffic": None,
                     "note": "the scan is a sequential recurrence per row: its duration is the latency of 8192 dependent "
                             "steps, not a bandwidth figure"},
        "cpu_baseline": None,
    }
    if not args.no_cpu_baseline:  # the oracle's eager ops on the host cores, first 64 trajectories
        from oracle import core_algos as OC
        from oracle import dapo_filter as OD
        from oracle import metric_utils as OM

        n_s = 64
        sc_c, am_c, m_c = scores[:n_s].cpu(), amask[:n_s].cpu(), mask[:n_s].cpu()
        v_c, vp_c = values[:n_s].cpu(), vpreds.detach()[:n_s].cpu()
        times = []
        for it in range(3):
            t1 = time.perf_counter()
            rw_c = OD.place_outcome_reward(sc_c.tolist(), am_c, L, True, L, 1024, 1.0)
            rw_c = torch.as_tensor(rw_c[0] if isinstance(rw_c, tuple) else rw_c, dtype=torch.float32)
            adv_c, ret_c = OC.compute_gae_advantage_return(rw_c, v_c, m_c, 1.0, 0.95)
            x = vp_c.clone().requires_grad_(True)
            l_c, _ = OC.compute_value_loss(x, ret_c, v_c, m_c, 0.5, "token-mean")
            l_c.backward()
            OM.compute_data_metric({"token_level_scores": rw_c, "token_level_rewards": rw_c, "advantages": adv_c,
                                    "returns": ret_c, "values": v_c, "responses": m_c, "response_mask": m_c,
                                    "attention_mask": am_c})
            if it:
                times.append(time.perf_counter() - t1)
        med = sorted(times)[len(times) // 2]
        out["cpu_baseline"] = {"value": n_s * L / med, "unit": "tokens/s", "cores": torch.get_num_threads(), "cpu": cpu_model(),
                               "kind": "port", "sample": f"first {n_s} of {B} trajectories x {L} tokens; median of 2 "
                                                         f"passes ({med:.2f} s each)"}
        # the oracle's multi-agent walk (the reference's loop over every token): two requests of the batch above
        cut = 2 * m_steps
        t1 = time.perf_counter()
        OC.marft_gae_unwhitened([t[:cut].cpu() for t in m_rews], [t[:cut].cpu() for t in m_vals],
                                [t[:cut].cpu() for t in m_masks], m_chains[:2], 0.99, 0.95)
        dt = time.perf_counter() - t1
        marft["cpu_oracle_tokens_per_s"] = sum(int(m[:cut].sum()) for m in m_masks) / dt
    print(json.dumps(out), flush=True)


def bench_glue(args, dev):
    """Remove-padding bookkeeping around the path at 64 sequences x 9216 tokens (prompt 1024 + response 8192):
    packed ids + rolled labels + indices + cu_seqlens from the attention mask, and the scatter of per-token values
    back into the [B, response_length] window, forward and backward.  Not the headline."""
    import torch

    import siirl_amd.padding as PD

    B, S, L = 64, 9216, 8192
    gen = torch.Generator(device=dev).manual_seed(SEED)
    lens = torch.randint(S // 8, S + 1, (B,), device=dev, generator=gen)
    am = (torch.arange(S, device=dev)[None] >= (S - lens)[:, None]).long()  # left padding
    ids = torch.randint(0, 150000, (B, S), device=dev, generator=gen)
    nnz = int(am.sum())
    vals = torch.randn(nnz, device=dev, generator=gen).requires_grad_(True)
    g = torch.randn(B, L, device=dev, generator=gen)

    def step(ev=None):
        rec = (lambda i: ev[i].record()) if ev else (lambda i: None)
        rec(0)
        _, _, indices, _, _ = PD.unpad_ids_and_labels(ids, am)
        rec(1)
        out = PD.pad_and_slice_response(vals, indices, B, S, L)
        out.backward(g)
        vals.grad = None
        rec(2)

    steps, warm = args.steps, args.warmup
    for _ in range(warm):
        step()
    torch.cuda.synchronize()
    evs = [[torch.cuda.Event(enable_timing=True) for _ in range(3)] for _ in range(steps)]
    t0 = time.perf_counter()
    for k in range(steps):
        step(evs[k])
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    ms = [sum(e[i].elapsed_time(e[i + 1]) for e in evs) / steps for i in range(2)]
    out = {
        "metric": "remove-padding bookkeeping (unpad ids/labels/indices + response-window scatter fwd+bwd) tokens/sec",
        "value": nnz * steps / wall, "unit": "tokens/s", "n_gpus": 1, "steps": steps, "warmup": warm,
        "ms_per_step": wall * 1e3 / steps, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "int64", "data": "synthetic",
        "config": {"workload": f"glue: {B} sequences x {S} (prompt {S - L} + response {L}), left padded, {nnz} tokens",
                   "seed": SEED},
        "kernels": {"unpad_ids_and_labels (one host sync)": {"ms": ms[0]},
                    "pad_and_slice_response forward + backward": {"ms": ms[1]}},
        "roofline": {"bound": "hbm", "kernel": "unpad kernels", "achieved": B * S * 16 / ms[0] / 1e6, "peak": 8000.0,
                     "unit": "GB/s", "frac": B * S * 16 / ms[0] / 1e6 / 8000.0, "traffic": None,
                     "note": "index work at a size where launches and the host sync dominate; no roofline claim"},
        "cpu_baseline": None,
    }
    if not args.no_cpu_baseline:
        from oracle import padding as OP

        am_c, ids_c, v_c = am.cpu().numpy(), ids.cpu().numpy(), vals.detach().cpu().numpy()
        times = []
        for it in range(4):
            t1 = time.perf_counter()
            rm, idx, cu, mx = OP.unpad_input(ids_c.reshape(B, S, 1), am_c)[:4]
            OP.rolled_labels(rm.reshape(-1))
            OP.pad_and_slice_response(v_c, idx, B, S, L)
            if it:
                times.append(time.perf_counter() - t1)
        med = sorted(times)[len(times) // 2]
        out["cpu_baseline"] = {"value": nnz / med, "unit": "tokens/s", "cores": 1, "cpu": cpu_model(), "kind": "port",
                               "sample": f"the whole batch, forward only, numpy; median of 3 passes ({med * 1e3:.1f} ms each)"}
    print(json.dumps(out), flush=True)


def bench_actor(args, dev):
    """One remove-padding micro-batch of the actor end to end (reference siirl/engine/actor/dp_actor.py:112-127,
    170-231,455-501 with the drop-in functions): 8 sequences of 1024 prompt + 3072 response tokens, right padded
    responses, bf16 logits [nnz, 152064].  Packed ids and rolled labels from the attention mask -> log-prob + entropy of
    the packed logits -> response windows [8, 3072] -> clipped loss - entropy bonus + low-variance KL -> backward to
    the logits.  Timed twice: as the reference composes it (every packed row goes through the log-prob kernels), and
    with the rolled labels of the rows outside the response window marked so that the kernels skip them.  Not the
    headline."""
    import torch
    from types import SimpleNamespace

    import siirl_amd.core_algos as CA
    import siirl_amd.padding as PD
    import siirl_amd.torch_functional as SF

    B, P, L, V = 8, 1024, 3072, VOCAB
    S = P + L
    gen = torch.Generator(device=dev).manual_seed(SEED)
    lens = torch.randint(L // 4, L + 1, (B,), device=dev, generator=gen)
    am = torch.ones(B, S, dtype=torch.long, device=dev)
    am[:, P:] = (torch.arange(L, device=dev)[None] < lens[:, None]).long()
    ids = torch.randint(0, V, (B, S), device=dev, generator=gen)
    nnz = int(am.sum())
    logits = torch.empty(nnz, V, dtype=torch.bfloat16, device=dev)
    for lo in range(0, nnz, 2048):
        n = min(2048, nnz - lo)
        logits[lo:lo + n] = (torch.randn(n, V, device=dev, generator=gen) * 3.0).to(torch.bfloat16)
    logits.requires_grad_(True)
    mask = am[:, P:].contiguous()
    adv = torch.randn(B, 1, device=dev, generator=gen).expand(B, L).contiguous()
    cfg = SimpleNamespace(clip_ratio=0.2, clip_ratio_low=0.2, clip_ratio_high=0.28, clip_ratio_c=3.0, entropy_coeff=0.001,
                          use_kl_loss=True, kl_loss_coef=0.001, kl_loss_type="low_var_kl", loss_agg_mode="token-mean",
                          policy_loss=SimpleNamespace(loss_mode="vanilla"))

    def windows(response_length):
        _, labels, indices, _, _ = PD.unpad_ids_and_labels(ids, am, response_length=response_length)
        lp, ent = SF.logprobs_and_entropy_from_logits(logits, labels, temperature=1.0, inplace_backward=False)
        return (PD.pad_and_slice_response(lp, indices, B, S, L), PD.pad_and_slice_response(ent, indices, B, S, L))

    with torch.no_grad():
        lp0, _ = windows(None)
    old = (lp0 + 0.05 * torch.randn(B, L, device=dev, generator=gen)) * mask
    ref = (lp0 + 0.1 * torch.randn(B, L, device=dev, generator=gen)) * mask

    def step(response_length):
        lp_w, ent_w = windows(response_length)
        out = CA.actor_loss(old, lp_w, adv, mask, cfg, entropy=ent_w, ref_log_prob=ref)
        out.loss.backward()
        g = logits.grad
        logits.grad = None
        return out.loss.detach(), g

    steps, warm = min(args.steps, 20), min(args.warmup, 3)
    res = {}
    for name, rl in (("every packed row", None), ("rows outside the response window skipped", L)):
        for _ in range(warm):
            step(rl)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(steps):
            loss, g = step(rl)
        torch.cuda.synchronize()
        res[name] = ((time.perf_counter() - t0) / steps, float(loss), g)
    (t_all, loss_all, g_all), (t_skip, loss_skip, g_skip) = res.values()
    n_resp = int(mask.sum())
    es = logits.element_size()
    out = {
        "metric": "remove-padding actor micro-batch (unpad -> log-prob + entropy -> response windows -> clipped loss + "
                  "entropy + KL -> backward to the logits) tokens/sec @vocab152k bf16",
        "value": nnz / t_all, "unit": "tokens/s", "n_gpus": 1, "steps": steps, "warmup": warm,
        "ms_per_step": t_all * 1e3, "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "bf16",
        "data": "synthetic",
        "config": {"workload": f"actor: {B} sequences x ({P} prompt + <= {L} response), {nnz} packed tokens of which "
                               f"{n_resp} response tokens, V = {V}", "seed": SEED},
        "response_rows_only": {"what": "unpad_ids_and_labels(..., response_length=L): the packed rows the response "
                                       "window drops are labelled SIIRL_LABEL_SKIP_ROW and read by the log-prob kernels "
                                       "in neither pass (their gradient rows are zero-filled)",
                               "ms_per_step": t_skip * 1e3, "tokens_per_s": nnz / t_skip,
                               "same_loss": loss_all == loss_skip, "same_gradient": bool(torch.equal(g_all, g_skip))},
        # the default flow reads every packed row once in the forward; its backward reads the rows with a gradient
        # and writes every row (zero rows unread, the library's default)
        "roofline": {"bound": "hbm", "kernel": "lpe_fwd_kernel + lpe_bwd_flat_kernel",
                     "achieved": es * V * (2 * nnz + n_resp) / t_all / 1e9, "peak": 8000.0, "unit": "GB/s",
                     "frac": es * V * (2 * nnz + n_resp) / t_all / 1e9 / 8000.0, "traffic": None},
        "cpu_baseline": None,
    }
    print(json.dumps(out), flush=True)


def bench_host(args, dev):
    """Host time per call of the drop-in functions (the cost of the boundary itself): operands small enough that
    the GPU is never the bottleneck, the host clock read before any synchronisation.  One line of JSON: microseconds
    per call, forward alone (no graph), forward in grad mode, and forward + ``backward()``; then the ten-call
    micro-batch body of the reference actor (siirl/engine/actor/dp_actor.py:403-501) as one figure.  Not a
    throughput benchmark and not the headline."""
    import torch
    from types import SimpleNamespace

    import siirl_amd.core_algos as CA
    import siirl_amd.torch_functional as SF

    g = torch.Generator(device=dev).manual_seed(SEED)
    B, L, V = 8, 256, 512
    lens = torch.randint(16, L + 1, (B,), device=dev, generator=g)
    mask = (torch.arange(L, device=dev)[None] < lens[:, None]).long()
    lp_leaf = (torch.randn(B, L, device=dev, generator=g) - 1.5).requires_grad_(True)
    old = lp_leaf.detach() + 0.05 * torch.randn(B, L, device=dev, generator=g)
    ref = lp_leaf.detach() + 0.1 * torch.randn(B, L, device=dev, generator=g)
    adv = torch.randn(B, L, device=dev, generator=g)
    logits = (torch.randn(B, L, V, device=dev, generator=g) * 2).requires_grad_(True)
    labels = torch.randint(0, V, (B, L), device=dev, generator=g)
    cfg = SimpleNamespace(clip_ratio=0.2, clip_ratio_low=0.2, clip_ratio_high=0.2, clip_ratio_c=3.0, entropy_coeff=0.01,
                          use_kl_loss=True, kl_loss_coef=0.001, kl_loss_type="low_var_kl", loss_agg_mode="token-mean",
                          loss_mode="vanilla")
    ns = torch.ops.siirl_hip
    f32 = lp_leaf.detach()
    calls = {
        "torch.ops.siirl_hip.logprob_entropy_fwd": lambda: ns.logprob_entropy_fwd(logits.detach(), labels, 1.0, True),
        "torch.ops.siirl_hip.policy_loss_fwd": lambda: ns.policy_loss_fwd(old, f32, adv, mask, None, None, ref, 0, 0.2,
                                                                          0.2, 3.0, 20.0, 0, 0.0, 3, False, 0.001, 0.0,
                                                                          1.0),
        "torch.ops.siirl_hip.kl_penalty_fwd": lambda: ns.kl_penalty_fwd(f32, ref, 3),
        "torch.ops.siirl_hip.agg_loss_fwd": lambda: ns.agg_loss_fwd(f32, mask, 0),
        "logprobs_from_logits": lambda: SF.logprobs_from_logits(logits, labels, inplace_backward=False),
        "entropy_from_logits (own pass)": lambda: SF.entropy_from_logits(logits),
        "compute_policy_loss_vanilla": lambda: CA.compute_policy_loss_vanilla(old, lp_leaf, adv, mask, "token-mean", cfg),
        "agg_loss": lambda: CA.agg_loss(lp_leaf, mask, "token-mean"),
        "kl_penalty": lambda: CA.kl_penalty(lp_leaf, ref, "low_var_kl"),
        "masked_mean": lambda: SF.masked_mean(lp_leaf, mask),
        "actor_loss (fused)": lambda: CA.actor_loss(old, lp_leaf, adv, mask, cfg, ref_log_prob=ref),
    }

    def host_us(fn, n=300):
        for _ in range(30):
            fn()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(n):
            fn()
        el = time.perf_counter() - t0
        torch.cuda.synchronize()
        return el / n * 1e6

    per_call = {}
    for name, fn in calls.items():
        with torch.no_grad():
            a = host_us(fn)
        per_call[name] = {"no_grad_us": round(a, 1), "grad_mode_us": round(host_us(fn), 1)}

    def fwd_bwd(make_loss, leaf):
        def run():
            make_loss().backward()
            leaf.grad = None
        return host_us(run)

    per_call["logprobs_from_logits"]["fwd_bwd_us"] = round(fwd_bwd(
        lambda: SF.logprobs_from_logits(logits, labels, inplace_backward=False).sum(), logits), 1)
    per_call["compute_policy_loss_vanilla"]["fwd_bwd_us"] = round(fwd_bwd(
        lambda: CA.compute_policy_loss_vanilla(old, lp_leaf, adv, mask, "token-mean", cfg)[0], lp_leaf), 1)
    per_call["actor_loss (fused)"]["fwd_bwd_us"] = round(fwd_bwd(
        lambda: CA.actor_loss(old, lp_leaf, adv, mask, cfg, ref_log_prob=ref).loss, lp_leaf), 1)

    def micro_batch():  # dp_actor.py:403-501 with the drop-in functions: the reference's own ten calls
        lp = SF.logprobs_from_logits(logits, labels, inplace_backward=False)
        ent = SF.entropy_from_logits(logits)
        pg, clipfrac, kl, lower = CA.compute_policy_loss_vanilla(old_log_prob=old, log_prob=lp, advantages=adv,
                                                                 response_mask=mask, loss_agg_mode="token-mean",
                                                                 config=cfg)
        ent_loss = CA.agg_loss(loss_mat=ent, loss_mask=mask, loss_agg_mode="token-mean")
        policy = pg - ent_loss * cfg.entropy_coeff
        kld = CA.kl_penalty(logprob=lp, ref_logprob=ref, kl_penalty="low_var_kl")
        kl_loss = CA.agg_loss(loss_mat=kld, loss_mask=mask, loss_agg_mode="token-mean")
        policy = policy + kl_loss * cfg.kl_loss_coef
        (policy * 0.125).backward()
        logits.grad = None

    def micro_batch_fused():  # the same arithmetic through actor_loss
        lp = SF.logprobs_from_logits(logits, labels, inplace_backward=False)
        ent = SF.entropy_from_logits(logits)
        CA.actor_loss(old, lp, adv, mask, cfg, entropy=ent, ref_log_prob=ref, loss_scale_factor=0.125).loss.backward()
        logits.grad = None

    out = {"metric": "host microseconds per call of the drop-in functions (GPU work negligible)", "unit": "us",
           "n_gpus": 1, "data": "synthetic", "config": {"workload": f"host: [B, L] = [{B}, {L}] fp32 operands, logits "
                                                                    f"[{B}, {L}, {V}] fp32, int64 mask"},
           "per_call": per_call,
           "micro_batch_drop_in_us": round(host_us(micro_batch, 200), 1),
           "micro_batch_actor_loss_us": round(host_us(micro_batch_fused, 200), 1),
           "cpu": cpu_model()}
    print(json.dumps(out), flush=True)


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-other-configs", action="store_true",
                    help="default workload only: leave out the short runs of configs 1, 3, 4 and 5")
    ap.add_argument("--with-row-skip", action="store_true",
                    help="also time the variant that writes zeros, unread, on rows whose gradients are zero")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="also run a plain 2 GiB device copy (for scaling rocprofv3 FETCH_SIZE / WRITE_SIZE)")
    ap.add_argument("--workload", default="config2", choices=["config1", "config2", "config3", "config4", "config5", "critic", "glue", "host", "actor"],
                    help="config2 (default): the headline logprob+entropy fwd+bwd; config1: fp32 GRPO step at V = 32000; "
                         "config4: GSPO long-context sequence; config3: DAPO [B, L] loss path; "
                         "config5: fused lm_head variant; critic: reward placement + GAE + value loss + metrics; "
                         "glue: remove-padding bookkeeping; actor: one remove-padding micro-batch end to end; "
                         "host: host time per call")
    ap.add_argument("--seqs", type=int, default=SEQS, help="sequences of 4096 tokens (8 = the baseline's config)")
    args = ap.parse_args()
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        print("bench.py: this build measures one GPU only (the hot path needs no collective; every row is "
              "independent); run with --gpus 1", file=sys.stderr)
        sys.exit(2)

    import torch

    import siirl_amd.torch_functional as SF

    if not torch.cuda.is_available():
        print("bench.py: no GPU visible; the HIP path has no CPU fallback", file=sys.stderr)
        sys.exit(1)
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    if args.copy_calibration:  # three plain 2 GiB device copies: what the traffic counters read for a known size
        src = torch.empty(1 << 30, dtype=torch.bfloat16, device=dev).normal_()
        dst = torch.empty_like(src)
        for _ in range(3):
            dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst
    by_name = {"config1": bench_config1, "config3": bench_config3, "config4": bench_config4, "config5": bench_config5}
    if args.workload in by_name:
        print(json.dumps(by_name[args.workload](args, dev)), flush=True)
        return
    if args.workload == "critic":
        return bench_critic(args, dev)
    if args.workload == "glue":
        return bench_glue(args, dev)
    if args.workload == "host":
        return bench_host(args, dev)
    if args.workload == "actor":
        return bench_actor(args, dev)
    SF.set_skip_zero_rows(False)  # dense: every row is read and written, as the algorithmic byte count assumes

    logits, labels, g_lp, g_ent, mask = make_workload(dev, seqs=args.seqs)
    T, V = logits.shape
    x = logits.requires_grad_(True)

    def step():
        lp, ent = SF.logprobs_and_entropy_from_logits(x, labels)
        (dx,) = torch.autograd.grad([lp, ent], [x], [g_lp, g_ent])
        return lp, ent, dx

    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()

    ev = [[torch.cuda.Event(enable_timing=True) for _ in range(3)] for _ in range(args.steps)]
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for k in range(args.steps):
        ev[k][0].record()
        lp, ent = SF.logprobs_and_entropy_from_logits(x, labels)
        ev[k][1].record()
        (dx,) = torch.autograd.grad([lp, ent], [x], [g_lp, g_ent])
        ev[k][2].record()
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0

    fwd_ms = sum(e[0].elapsed_time(e[1]) for e in ev) / args.steps
    bwd_ms = sum(e[1].elapsed_time(e[2]) for e in ev) / args.steps
    ms_per_step = wall * 1e3 / args.steps
    tokens_per_s = T * args.steps / wall

    es = logits.element_size()
    fwd_bytes, bwd_bytes = es * V * T, 2 * es * V * T
    bwd_gbs = bwd_bytes / (bwd_ms * 1e-3) / 1e9
    fwd_gbs = fwd_bytes / (fwd_ms * 1e-3) / 1e9
    step_gbs = (fwd_bytes + bwd_bytes) / (ms_per_step * 1e-3) / 1e9

    row_skip = None
    if args.with_row_skip:  # padding rows written as zeros unread; reported beside the dense headline
        SF.set_skip_zero_rows(True)
        for _ in range(2):
            step()
        torch.cuda.synchronize()
        t1 = time.perf_counter()
        for _ in range(args.steps):
            step()
        torch.cuda.synchronize()
        skip_wall = time.perf_counter() - t1
        SF.set_skip_zero_rows(False)
        n_valid = int(mask.sum().item())
        # forward reads every row; backward reads the valid rows and writes every row
        row_skip = {"tokens_per_s": T * args.steps / skip_wall, "ms_per_step": skip_wall * 1e3 / args.steps,
                    "valid_tokens": n_valid, "algorithmic_bytes": es * V * (2 * T + n_valid)}
        # and with the rows outside the mask labelled LABEL_SKIP_ROW, so that the forward does not read them either
        from siirl_amd.padding import LABEL_SKIP_ROW

        dense_labels = labels
        labels = torch.where(mask > 0, labels, torch.full_like(labels, LABEL_SKIP_ROW))
        for _ in range(2):
            step()
        torch.cuda.synchronize()
        t1 = time.perf_counter()
        for _ in range(args.steps):
            step()
        torch.cuda.synchronize()
        label_wall = time.perf_counter() - t1
        labels = dense_labels
        row_skip["labelled_rows_skipped_in_both_passes"] = {
            "tokens_per_s": T * args.steps / label_wall, "ms_per_step": label_wall * 1e3 / args.steps,
            "algorithmic_bytes": es * V * (T + 2 * n_valid)}  # both passes read the valid rows only

    # the same micro-batch as ONE launch from logits to dlogits (PPO clip loss, entropy bonus, low-variance KL loss
    # evaluated in-kernel from each row's log-prob and entropy); reported beside the headline, never as `value`
    from types import SimpleNamespace

    import siirl_amd.core_algos as CA

    Bq, Lq = args.seqs, T // args.seqs
    gen = torch.Generator(device=dev).manual_seed(SEED + 1)
    with torch.no_grad():
        lp_now, _ = SF.logprobs_and_entropy_from_logits(logits.detach(), labels)
    old_lp = (lp_now + 0.05 * torch.randn(T, device=dev, generator=gen)).view(Bq, Lq)
    ref_lp = (lp_now + 0.1 * torch.randn(T, device=dev, generator=gen)).view(Bq, Lq)
    adv = torch.randn(Bq, 1, device=dev, generator=gen).expand(Bq, Lq).contiguous()
    acfg = SimpleNamespace(clip_ratio=0.2, clip_ratio_low=0.2, clip_ratio_high=0.28, clip_ratio_c=3.0,
                           entropy_coeff=0.001, use_kl_loss=True, kl_loss_coef=0.001, kl_loss_type="low_var_kl",
                           loss_agg_mode="token-mean", loss_mode="vanilla")
    x3 = logits.detach().view(Bq, Lq, V)

    def fused_ms_with(m2d):
        def fused():
            return CA.fused_actor_step(x3, labels.view(Bq, Lq), old_lp, adv, m2d, acfg, ref_log_prob=ref_lp)

        for _ in range(2):
            fused()
        torch.cuda.synchronize()
        t2 = time.perf_counter()
        for _ in range(args.steps):
            fused()
        torch.cuda.synchronize()
        return (time.perf_counter() - t2) * 1e3 / args.steps

    # bytes of the one-launch kernel by its own count: every row is read once (es*V) and written once (es*V); a row
    # with a non-zero aggregation weight is read a second time except for the 8192 16-byte vectors (128 KiB) that stay
    # in LDS between the passes; a zero-weight row (padding) is written as zeros without the second read
    row_bytes = es * V
    refetch = max(0.0, 1.0 - 131072.0 / row_bytes)
    m2 = mask.view(Bq, Lq)
    f_valid = float(m2.float().mean().item())
    masked_ms = fused_ms_with(m2)
    dense_ms = fused_ms_with(torch.ones_like(m2))
    masked_bytes = T * row_bytes * (2.0 + refetch * f_valid)
    dense_bytes = T * row_bytes * (2.0 + refetch)
    fused_step = {"what": "siirl_actor_step_fused: logits -> log-prob, entropy, PPO-clip + KL + entropy loss -> dlogits "
                          "in one launch, plus the [B, L] scalar/metric pass",
                  "bytes_model": "per row es*V read + es*V written + es*V*(1 - 128 KiB / (es*V)) read again when the "
                                 "row's loss weight is non-zero (the rest of the row waits in LDS)",
                  "config2_mask": {"valid_row_fraction": f_valid, "ms_per_step": masked_ms,
                                   "tokens_per_s": T / masked_ms * 1e3, "bytes": masked_bytes,
                                   "GB/s": masked_bytes / masked_ms / 1e6},
                  "dense_mask": {"valid_row_fraction": 1.0, "ms_per_step": dense_ms, "tokens_per_s": T / dense_ms * 1e3,
                                 "bytes": dense_bytes, "GB/s": dense_bytes / dense_ms / 1e6},
                  "note": "the config 2 mask leaves part of the rows without a second read; compare the dense figure "
                          "with the two-launch headline, which is dense"}

    # what the actor's `logits.div_(temperature)` before the calls (siirl/engine/actor/dp_actor.py:176) costs: a pass
    # over [T, V] in the forward and autograd's division of the gradient in the backward, against the one call that
    # takes the temperature as a factor.  Reported beside the headline, never as `value`.
    temp = 0.7

    def temperature_flow(one_call):
        def run():
            if one_call:
                lp, ent = SF.logprobs_and_entropy_from_logits(x, labels, temperature=temp)
            else:
                z = x / temp  # stands for div_ on the model's output: the same read + write
                lp = SF.logprobs_from_logits(z, labels, inplace_backward=False)
                ent = SF.entropy_from_logits(z)
            torch.autograd.backward([lp, ent], [g_lp, g_ent])
            x.grad = None

        for _ in range(2):
            run()
        torch.cuda.synchronize()
        t3 = time.perf_counter()
        for _ in range(5):
            run()
        torch.cuda.synchronize()
        return (time.perf_counter() - t3) * 1e3 / 5

    division_ms, folded_ms = temperature_flow(False), temperature_flow(True)

    # The headline once more through the reference's two names, as the actor calls them when the entropy bonus is on
    # (siirl/engine/actor/dp_actor.py:182-195): logprobs_from_logits(logits, labels, inplace_backward=False), then
    # entropy_from_logits(logits), then backward through both.  The second call is served by the first one's pass, so
    # this must cost what the headline's one call costs.
    def named_flow():
        lp = SF.logprobs_from_logits(x, labels, inplace_backward=False)
        ent = SF.entropy_from_logits(x)
        torch.autograd.backward([lp, ent], [g_lp, g_ent])
        x.grad = None

    for _ in range(args.warmup):
        named_flow()
    torch.cuda.synchronize()
    t4 = time.perf_counter()
    for _ in range(args.steps):
        named_flow()
    torch.cuda.synchronize()
    named_ms = (time.perf_counter() - t4) * 1e3 / args.steps

    # A copy yardstick from the library's own row mover: siirl_gather_rows with the identity index over the same
    # tensor reads and writes the backward's bytes (16-byte non-temporal accesses, no arithmetic).
    from siirl_amd import _lib

    ident = torch.arange(T, device=dev, dtype=torch.int64)
    dst = torch.empty_like(logits)
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)

    def copy_rows():
        rc = _lib.lib().siirl_gather_rows(_lib.ptr(logits), _lib.ptr(ident), T, V * es, T, _lib.ptr(dst),
                                          _lib.current_stream(dev))
        _lib.check(rc, "siirl_gather_rows")

    for _ in range(2):
        copy_rows()
    torch.cuda.synchronize()
    e0.record()
    for _ in range(10):
        copy_rows()
    e1.record()
    torch.cuda.synchronize()
    copy_ms = e0.elapsed_time(e1) / 10
    copy_gbs = 2 * es * V * T / copy_ms / 1e6
    del dst, ident
    torch.cuda.empty_cache()

    out = {
        "metric": METRIC,
        "value": tokens_per_s,
        "unit": "tokens/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": ms_per_step,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "bf16",
        "data": "synthetic",
        "config": {"workload": f"config2: logprob+entropy fwd+bwd, bf16 logits [{args.seqs}x{SEQ_LEN}, {V}] ~N(0,3), "
                               "1% spiked rows, uniform labels, grads ~N(0,1e-2) zeroed on padding; dense rows",
                   "tokens": T, "vocab": V, "seed": SEED},
        "hbm_roofline_pct_step": 100.0 * step_gbs / HBM_PEAK_GBS,
        "step_algorithmic_bytes": fwd_bytes + bwd_bytes,
        "kernels": {"lpe_fwd_kernel": {"ms": fwd_ms, "GB/s": fwd_gbs, "bytes": fwd_bytes},
                    "lpe_bwd_flat_kernel": {"ms": bwd_ms, "GB/s": bwd_gbs, "bytes": bwd_bytes}},
        "roofline": {"bound": "hbm", "kernel": "lpe_bwd_flat_kernel", "achieved": bwd_gbs, "peak": HBM_PEAK_GBS,
                     "unit": "GB/s", "frac": bwd_gbs / HBM_PEAK_GBS,
                     "traffic": MEASURED_TRAFFIC_BYTES if args.seqs == SEQS else None,
                     "traffic_source": "rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE of this command in separate runs "
                                       "(profiles/lpe_config2_hbm_traffic.md); a constant here, not read in this process"},
        "row_skip_variant": row_skip,
        "fused_step_variant": fused_step,
        "reference_named_flow_ms": named_ms,
        "reference_named_flow": {"what": "logprobs_from_logits(logits, labels, inplace_backward=False) + "
                                         "entropy_from_logits(logits) + backward, the actor's own calls "
                                         "(dp_actor.py:182-195), timed like the headline",
                                 "ms_per_step": named_ms, "over_headline": named_ms / ms_per_step},
        "copy_yardstick_GBs": copy_gbs,
        "copy_yardstick": {"what": "siirl_gather_rows with the identity index over the same [T, V] tensor: the "
                                   "library's plain row mover reading and writing the backward's bytes",
                           "ms": copy_ms, "GB/s": copy_gbs, "backward_GB/s": bwd_gbs,
                           "backward_over_copy": bwd_gbs / copy_gbs},
        "temperature_flow": {"what": f"temperature {temp}: `logits / T`, logprobs_from_logits, entropy_from_logits, "
                                     "backward (the reference's lines) against logprobs_and_entropy_from_logits("
                                     "logits, labels, temperature=T), backward",
                             "division_then_calls_ms": division_ms, "one_call_ms": folded_ms},
    }
    if not args.no_cpu_baseline:
        out["cpu_baseline"] = cpu_baseline(logits.detach(), labels, g_lp, g_ent)
    else:
        out["cpu_baseline"] = None
    if not args.no_other_configs and args.seqs == SEQS:
        # the other four configurations of the baseline, each a short run of its own workload (`--workload configN`
        # gives the full line with its variants): step time, roofline fraction and the CPU oracle beside it
        del x, logits, labels, g_lp, g_ent, mask, x3, lp_now, old_lp, ref_lp, adv, m2, lp, ent, dx
        torch.cuda.empty_cache()
        quick_steps = {"config1": (5, 2), "config3": (10, 2), "config4": (5, 2), "config5": (8, 2)}
        fns = {"config1": bench_config1, "config3": bench_config3, "config4": bench_config4, "config5": bench_config5}
        out["configs"] = {}
        for name, fn in fns.items():
            sub = argparse.Namespace(**vars(args))
            sub.steps, sub.warmup = quick_steps[name]
            r = fn(sub, dev, quick=True)
            out["configs"][name] = {k: r[k] for k in ("metric", "value", "unit", "ms_per_step", "steps", "warmup", "dtype")}
            out["configs"][name]["workload"] = r["config"]["workload"]
            out["configs"][name]["roofline"] = {k: r["roofline"][k] for k in ("bound", "kernel", "achieved", "peak", "unit", "frac")}
            out["configs"][name]["cpu_baseline"] = r["cpu_baseline"]
            if "library_gemm_yardstick" in r:
                out["configs"][name]["library_gemm_yardstick_TFLOPs"] = r["library_gemm_yardstick"]["TFLOP/s"]
                out["configs"][name]["forward_TFLOPs"] = gemm_rate(r)
            del r
            torch.cuda.empty_cache()
    print(json.dumps(out), flush=True)


if __name__ == "__main__":
    main()
