#!/usr/bin/env python3
"""Writes tests/golden/oracle_small.npz: small seeded inputs and the oracle's outputs for every function on the
path, computed in fp64 on this machine's CPU.  The fixtures let the GPU tests check the HIP path against numbers
that do not move when the oracle's code is edited, and let the CPU tests notice if it does.

    python tests/golden/make_golden.py

The reference package itself is not imported (its dependencies are absent); the reference-held known answers
live in reference_vectors.json beside this file."""

import os
import sys

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))

from oracle import core_algos as OC  # noqa: E402
from oracle import dapo_filter as OD  # noqa: E402
from oracle import fused_linear as OFL  # noqa: E402
from oracle import torch_functional as OF  # noqa: E402


def main():
    g = torch.Generator().manual_seed(20250601)
    out = {}
    # --- log-prob / entropy: bf16-representable logits [12, 1536], spikes, temperature 1 and 0.7
    T, V = 8, 1024
    x = (torch.randn(T, V, generator=g) * 3).to(torch.bfloat16)
    x[3, 100] = 15.0
    y = torch.randint(0, V, (T,), generator=g)
    g_lp = torch.randn(T, generator=g) * 1e-2
    g_h = torch.randn(T, generator=g) * 1e-2
    out["lpe_logits_bf16_bits"] = x.view(torch.int16).numpy()
    out["lpe_labels"] = y.numpy()
    out["lpe_g_lp"], out["lpe_g_h"] = g_lp.numpy(), g_h.numpy()
    for name, temp in (("t1", 1.0), ("t07", 0.7)):
        lp, ent, lse, ex = OF.logprob_entropy_forward(x, y, temp, dtype=torch.float64)
        dx = OF.logprob_entropy_backward(x, y, g_lp, g_h, temp, dtype=torch.float64)
        out[f"lpe_{name}_logprob"], out[f"lpe_{name}_entropy"] = lp.numpy(), ent.numpy()
        out[f"lpe_{name}_dlogits"] = dx.numpy()
    # --- [B, L] losses
    B, L = 6, 37
    lp = torch.randn(B, L, generator=g) - 1.5
    old = lp + 0.3 * torch.randn(B, L, generator=g)
    ref = lp + 0.2 * torch.randn(B, L, generator=g)
    adv = torch.randn(B, 1, generator=g).expand(B, L).contiguous()
    lens = torch.randint(1, L + 1, (B,), generator=g)
    mask = (torch.arange(L)[None] < lens[:, None]).long()
    for k, v in (("lp", lp), ("old", old), ("ref", ref), ("adv", adv), ("mask", mask)):
        out[f"loss_{k}"] = v.numpy()
    cfg = OC.LossConfig(0.2, 0.2, 0.28, 3.0)
    for mode in OC.AGG_MODES:
        tag = mode.replace("-", "_")
        x64 = lp.double().requires_grad_(True)
        res = OC.compute_policy_loss_vanilla(old.double(), x64, adv.double(), mask, mode, cfg)
        res[0].backward()
        out[f"vanilla_{tag}"] = np.array([float(r) for r in res])
        out[f"vanilla_{tag}_grad"] = x64.grad.numpy()
        out[f"agg_{tag}"] = np.array(float(OC.agg_loss(lp.double(), mask, mode)))
    x64 = lp.double().requires_grad_(True)
    old_g = lp + 0.01 * (old - lp)
    out["loss_old_gspo"] = old_g.numpy()
    res = OC.compute_policy_loss_gspo(old_g.double(), x64, adv.double(), mask, "token-mean", OC.LossConfig(0.2, 3e-3, 4e-3, 3.0))
    res[0].backward()
    out["gspo"] = np.array([float(r) for r in res])
    out["gspo_grad"] = x64.grad.numpy()
    for kind in ("kl", "abs", "mse", "low_var_kl"):
        out[f"kl_{kind}"] = OC.kl_penalty(lp.double(), ref.double(), kind).numpy()
    # --- GRPO advantage and DAPO keep mask
    P, n = 9, 4
    uid = np.repeat(np.arange(P, dtype=np.int64) * 3 + 1, n)
    s = (torch.rand(P * n, generator=g) < 0.5).float()
    s[:4] = 1.0
    rewards = torch.zeros(P * n, L)
    rewards[:, 5] = s
    gm = (torch.rand(P * n, L, generator=g) > 0.2).long()
    out["grpo_rewards"], out["grpo_mask"], out["grpo_uid"] = rewards.numpy(), gm.numpy(), uid
    out["grpo_adv"] = OC.compute_grpo_outcome_advantage(rewards.double(), gm, uid)[0].numpy()
    out["grpo_adv_nonorm"] = OC.compute_grpo_outcome_advantage(rewards.double(), gm, uid, norm_adv_by_std_in_grpo=False)[0].numpy()
    out["dapo_keep"] = OD.keep_mask(s.numpy(), uid)
    # --- fused lm_head
    T, H, V = 16, 64, 512
    h = torch.randn(T, H, generator=g).to(torch.bfloat16)
    w = (torch.randn(V, H, generator=g) * 0.05).to(torch.bfloat16)
    ids = torch.randint(0, V, (T,), generator=g)
    f_glp, f_gh = torch.randn(T, generator=g) * 1e-2, torch.randn(T, generator=g) * 1e-2
    flp, fent = OFL.fused_linear_for_ppo_fwd(h, w, ids, 1.0, dtype=torch.float64)
    dh, dw = OFL.fused_linear_for_ppo_bwd(f_glp, f_gh, h, w, ids, 1.0, dtype=torch.float64)
    out["fl_hidden_bf16_bits"], out["fl_weight_bf16_bits"] = h.view(torch.int16).numpy(), w.view(torch.int16).numpy()
    out["fl_ids"], out["fl_g_lp"], out["fl_g_h"] = ids.numpy(), f_glp.numpy(), f_gh.numpy()
    out["fl_logprob"], out["fl_entropy"], out["fl_dhidden"], out["fl_dweight"] = flp.numpy(), fent.numpy(), dh.numpy(), dw.numpy()
    path = os.path.join(HERE, "oracle_small.npz")
    np.savez_compressed(path, **out)
    print(f"wrote {path}: {len(out)} arrays, {os.path.getsize(path)} bytes")


if __name__ == "__main__":
    main()
