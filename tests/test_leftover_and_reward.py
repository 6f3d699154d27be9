"""Leftover-cache semantics against the reference's own test vectors (CPU), the oracle's reward placement against
hand-computed cases (CPU), and the HIP reward placement against the oracle (GPU, exact)."""
import json
import os
from types import SimpleNamespace

import numpy as np
import pytest
import torch

from oracle import dapo_filter as OD

GOLD = json.load(open(os.path.join(os.path.dirname(__file__), "golden", "reference_vectors.json")))["leftover_cache"]


def _batch(uids, sources, meta):
    return {"uid": torch.tensor(uids), "input_ids": torch.randn(len(uids), 10),
            "data_source": np.array(sources), "metadata_field": meta}


def test_leftover_cache_caching_golden():
    from siirl_amd.dapo_filter import SamplingLeftoverCache, filter_tensordict

    g = GOLD["caching"]
    batch = {"uid": torch.tensor(g["batch_uid"]), "input_ids": torch.randn(8, 10)}
    w = SamplingLeftoverCache()
    out = w.postprocess(filter_tensordict(batch, g["filtered_indices"]), g["target_total_samples"])
    assert len(out) == g["returned_len"] and w.sampling_leftover_cache is not None
    assert w.sampling_leftover_cache["uid"].tolist() == g["cached_uid"]


def test_leftover_cache_merging_golden():
    from siirl_amd.dapo_filter import SamplingLeftoverCache, filter_tensordict

    g = GOLD["merging"]
    w = SamplingLeftoverCache()
    w.sampling_leftover_cache = _batch(g["cache_uid"], g["cache_sources"], g["cache_metadata"])
    batch = _batch(g["batch_uid"], g["batch_sources"], g["batch_metadata"])
    new = filter_tensordict(batch, g["filtered_indices"])
    want = OD.merge_leftover(w.sampling_leftover_cache, OD.filter_by_indices(batch, g["filtered_indices"]))
    out = w.postprocess(new, g["target_total_samples"])
    assert w.sampling_leftover_cache is None
    assert out["uid"].tolist() == g["merged_uid"] == want["uid"].tolist()
    assert list(out["data_source"]) == g["merged_sources"] == list(want["data_source"])
    assert out["metadata_field"] == g["merged_metadata"] == want["metadata_field"]
    assert out["input_ids"].shape == (6, 10) and torch.equal(out["input_ids"], want["input_ids"])


def test_leftover_cache_accumulates_over_rounds():
    from siirl_amd.dapo_filter import SamplingLeftoverCache

    w = SamplingLeftoverCache()
    assert w.postprocess({"uid": torch.tensor([1, 2]), "tags": ["a", "b"]}, 5) == {}
    assert w.postprocess({"uid": torch.tensor([3]), "tags": ["c"]}, 5) == {}
    out = w.postprocess({"uid": torch.tensor([4, 5]), "tags": ["d", "e"]}, 5)
    assert out["uid"].tolist() == [1, 2, 3, 4, 5] and out["tags"] == list("abcde") and w.sampling_leftover_cache is None
    assert w.postprocess({}, 1) == {} and w.sampling_leftover_cache == {}


def test_oracle_reward_placement_hand_cases():
    # response window of 6 after a prompt of 2; max_resp_len 6, buffer 4 -> expected length 2
    am = torch.tensor([[1, 1, 1, 1, 0, 0, 0, 0], [0, 1, 1, 1, 1, 1, 1, 1], [1, 1, 1, 1, 1, 1, 0, 0]])
    r, pens = OD.place_outcome_reward([1.0, 1.0, 0.0], am, 6, True, 6, 4, 1.0)
    assert pens == [0.0, -1.0, -0.5]
    want = torch.zeros(3, 6)
    want[0, 1], want[1, 5], want[2, 3] = 1.0, 0.0, -0.5
    assert torch.equal(r, want)
    r, pens = OD.place_outcome_reward([1.0, 1.0, 0.0], am, 6)
    want[1, 5], want[2, 3] = 1.0, 0.0
    assert torch.equal(r, want) and pens == [0.0, 0.0, 0.0]


@pytest.mark.gpu
@pytest.mark.parametrize("B,P,L", [(1, 0, 1), (3, 2, 6), (64, 100, 4096), (300, 7, 513)])
@pytest.mark.parametrize("mdt", [torch.int64, torch.bool])
@pytest.mark.parametrize("enable", [False, True])
def test_place_outcome_reward(dev, B, P, L, mdt, enable):
    from siirl_amd.reward import place_outcome_reward

    g = torch.Generator().manual_seed(B + L)
    vl = torch.randint(1, L + 1, (B,), generator=g)
    vl[0] = L
    am = torch.cat([torch.ones(B, P, dtype=torch.int64), (torch.arange(L)[None] < vl[:, None]).long()], 1)
    scores = (torch.rand(B, generator=g, dtype=torch.float64) * 2 - 0.5).tolist()
    cfg = SimpleNamespace(enable=enable, len=max(L // 4, 1), penalty_factor=0.7, log=True)
    want, pens = OD.place_outcome_reward(scores, am, L, enable, L, cfg.len, cfg.penalty_factor)
    got = place_outcome_reward(scores, am.to(dev).to(mdt), L, cfg, L, return_dict=True)
    assert torch.equal(got["reward_tensor"].cpu(), want)
    if enable:
        assert got["reward_extra_info"]["overlong_reward"] == pens
        assert got["reward_extra_info"]["overlong"] == [p < 0 for p in pens]
    host = place_outcome_reward(scores, am, L, cfg, L)  # host mask: staged, result returned on the host
    assert not host.is_cuda and torch.equal(host, want)


@pytest.mark.gpu
def test_place_outcome_reward_empty_response_and_errors(dev):
    from siirl_amd.reward import place_outcome_reward

    am = torch.tensor([[1, 1, 0, 0, 0], [1, 1, 1, 1, 0]], device=dev)
    r = place_outcome_reward([2.0, 3.0], am, 3)
    assert r.cpu().tolist() == [[0.0, 0.0, 2.0], [0.0, 3.0, 0.0]]  # no valid token: Python's index -1
    with pytest.raises(AssertionError):
        place_outcome_reward([2.0, 3.0], am, 3, SimpleNamespace(enable=True, len=1, penalty_factor=1.0, log=False))
    with pytest.raises(ValueError):
        place_outcome_reward([2.0], am, 3)
