"""The oracle reproduces the committed fixtures of tests/golden/oracle_small.npz (CPU only): editing the oracle
cannot silently move the numbers the GPU tests are held to."""

import os

import numpy as np
import torch

from oracle import core_algos as OC
from oracle import dapo_filter as OD
from oracle import fused_linear as OFL
from oracle import torch_functional as OF

G = np.load(os.path.join(os.path.dirname(__file__), "golden", "oracle_small.npz"))


def _bf16(bits):
    return torch.from_numpy(bits.copy()).view(torch.bfloat16)


def test_logprob_entropy_fixtures():
    x, y = _bf16(G["lpe_logits_bf16_bits"]), torch.from_numpy(G["lpe_labels"])
    g_lp, g_h = torch.from_numpy(G["lpe_g_lp"]), torch.from_numpy(G["lpe_g_h"])
    for name, temp in (("t1", 1.0), ("t07", 0.7)):
        lp, ent, _, _ = OF.logprob_entropy_forward(x, y, temp, dtype=torch.float64)
        assert np.allclose(lp.numpy(), G[f"lpe_{name}_logprob"], atol=1e-12)
        assert np.allclose(ent.numpy(), G[f"lpe_{name}_entropy"], atol=1e-12)
        dx = OF.logprob_entropy_backward(x, y, g_lp, g_h, temp, dtype=torch.float64)
        assert np.allclose(dx.numpy(), G[f"lpe_{name}_dlogits"], atol=1e-14)


def test_loss_fixtures():
    lp, old, ref = (torch.from_numpy(G[f"loss_{k}"]).double() for k in ("lp", "old", "ref"))
    adv, mask = torch.from_numpy(G["loss_adv"]).double(), torch.from_numpy(G["loss_mask"])
    cfg = OC.LossConfig(0.2, 0.2, 0.28, 3.0)
    for mode in OC.AGG_MODES:
        tag = mode.replace("-", "_")
        res = OC.compute_policy_loss_vanilla(old, lp, adv, mask, mode, cfg)
        assert np.allclose([float(r) for r in res], G[f"vanilla_{tag}"], atol=1e-12)
        assert np.allclose(float(OC.agg_loss(lp, mask, mode)), G[f"agg_{tag}"], atol=1e-12)
    res = OC.compute_policy_loss_gspo(torch.from_numpy(G["loss_old_gspo"]).double(), lp, adv, mask, "token-mean",
                                      OC.LossConfig(0.2, 3e-3, 4e-3, 3.0))
    assert np.allclose([float(r) for r in res], G["gspo"], atol=1e-12)
    for kind in ("kl", "abs", "mse", "low_var_kl"):
        assert np.allclose(OC.kl_penalty(lp, ref, kind).numpy(), G[f"kl_{kind}"], atol=1e-12)


def test_group_fixtures():
    rewards, mask, uid = torch.from_numpy(G["grpo_rewards"]).double(), torch.from_numpy(G["grpo_mask"]), G["grpo_uid"]
    assert np.allclose(OC.compute_grpo_outcome_advantage(rewards, mask, uid)[0].numpy(), G["grpo_adv"], atol=1e-12)
    s = G["grpo_rewards"][:, 5]
    assert np.array_equal(OD.keep_mask(s, uid), G["dapo_keep"])
    assert not G["dapo_keep"][:4].any()  # the all-ones first group is dropped


def test_fused_linear_fixtures():
    h, w = _bf16(G["fl_hidden_bf16_bits"]), _bf16(G["fl_weight_bf16_bits"])
    ids = torch.from_numpy(G["fl_ids"])
    lp, ent = OFL.fused_linear_for_ppo_fwd(h, w, ids, 1.0, dtype=torch.float64)
    assert np.allclose(lp.numpy(), G["fl_logprob"], atol=1e-12) and np.allclose(ent.numpy(), G["fl_entropy"], atol=1e-12)
