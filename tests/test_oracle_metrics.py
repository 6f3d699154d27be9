"""Pins the oracle's data-metric restatement (CPU only) with numpy on the selected elements and a hand case."""
import numpy as np
import torch

from oracle import metric_utils as OM


def make_data(B, P, L, seed, with_values=True):
    g = torch.Generator().manual_seed(seed)
    rlen = torch.randint(1, L + 1, (B,), generator=g)
    rlen[0] = L
    plen = torch.randint(1, P + 1, (B,), generator=g)
    plen[-1] = P
    rmask = (torch.arange(L)[None] < rlen[:, None]).long()
    pmask = (torch.arange(P)[None] >= (P - plen)[:, None]).long()  # prompts are left-padded
    scores = torch.zeros(B, L)
    scores[torch.arange(B), rlen - 1] = (torch.rand(B, generator=g) > 0.5).float()
    data = {
        "token_level_scores": scores, "token_level_rewards": scores - 0.01 * torch.rand(B, L, generator=g) * rmask,
        "advantages": torch.randn(B, L, generator=g), "returns": torch.randn(B, L, generator=g) + 1.0,
        "responses": torch.zeros(B, L, dtype=torch.long), "attention_mask": torch.cat([pmask, rmask], 1),
        "response_mask": rmask,
    }
    if with_values:
        data["values"] = data["returns"] + 0.3 * torch.randn(B, L, generator=g)
    return data


def test_hand_case():
    data = {
        "token_level_scores": torch.tensor([[0.0, 1.0, 0.0], [0.0, 0.0, 0.0]]),
        "token_level_rewards": torch.tensor([[0.0, 1.0, 0.0], [0.0, 0.25, 0.0]]),
        "advantages": torch.tensor([[1.0, 3.0, 100.0], [-2.0, 4.0, 6.0]]),
        "returns": torch.tensor([[0.5, 1.5, 100.0], [2.5, 3.5, 4.5]]),
        "values": torch.tensor([[0.0, 2.0, 100.0], [2.0, 3.0, 5.0]]),
        "responses": torch.zeros(2, 3, dtype=torch.long),
        "attention_mask": torch.tensor([[0, 1, 1, 1, 0], [1, 1, 1, 1, 1]]),
        "response_mask": torch.tensor([[1, 1, 0], [1, 1, 1]]),
    }
    m = OM.compute_data_metric(data)
    assert m["critic/score/mean"] == 0.5 and m["critic/rewards/max"] == 1.0 and m["critic/rewards/min"] == 0.25
    assert abs(m["critic/advantages/mean"] - 2.4) < 1e-6 and m["critic/advantages/max"] == 6.0 and m["critic/advantages/min"] == -2.0
    assert m["critic/returns/mean"] == 2.5 and m["critic/values/max"] == 5.0
    diff = np.array([0.5, -0.5, 0.5, 0.5, -0.5])
    ret = np.array([0.5, 1.5, 2.5, 3.5, 4.5])
    assert abs(m["critic/vf_explained_var"] - (1 - diff.var(ddof=1) / (ret.var(ddof=1) + 1e-5))) < 1e-6
    assert m["response/length/mean"] == 2.5 and m["response/clip_ratio/mean"] == 0.5
    assert m["response/correct_length/mean"] == 2.0 and m["response/wrong_length/max"] == 3.0
    assert m["prompt/length/mean"] == 1.5 and m["prompt/length/min"] == 1.0 and m["prompt/clip_ratio/mean"] == 0.5


def test_against_numpy_selection():
    data = make_data(16, 7, 33, 0)
    m = OM.compute_data_metric(data)
    sel = data["response_mask"].bool().numpy()
    for key, name in (("advantages", "advantages"), ("returns", "returns"), ("values", "values")):
        x = data[name].numpy()[sel]
        assert abs(m[f"critic/{key}/mean"] - x.mean()) < 1e-6
        assert m[f"critic/{key}/max"] == x.max() and m[f"critic/{key}/min"] == x.min()
    ret, val = data["returns"].numpy()[sel].astype(np.float64), data["values"].numpy()[sel].astype(np.float64)
    assert abs(m["critic/vf_explained_var"] - (1 - (ret - val).var(ddof=1) / (ret.var(ddof=1) + 1e-5))) < 1e-5
    rl = data["response_mask"].sum(-1).numpy()
    rs = data["token_level_rewards"].sum(-1).numpy()
    assert m["response/length/max"] == rl.max() and abs(m["response/length/mean"] - rl.mean()) < 1e-6
    assert abs(m["response/correct_length/mean"] - rl[rs > 0.5].mean()) < 1e-5
    assert m["response/wrong_length/min"] == rl[rs <= 0.5].min()
    assert "critic/values/mean" not in OM.compute_data_metric(make_data(4, 3, 5, 1, with_values=False))
