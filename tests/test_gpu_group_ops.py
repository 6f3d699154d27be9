"""GPU parity: GRPO outcome advantage and the DAPO keep mask (through the C ABI) vs the CPU oracle.

Advantages: within 1e-5 relative (plus 1e-6 absolute) of the oracle.  Keep mask, kept indices and group
sizes: bit-exact against numpy (``np.std(values) > 0``)."""

from types import SimpleNamespace

import numpy as np
import pytest
import torch

from oracle import core_algos as OC
from oracle import dapo_filter as OD

pytestmark = pytest.mark.gpu


def _rel_close(got, want, rtol=1e-5, atol=1e-6):
    err = (got.double() - want.double()).abs()
    return bool((err <= atol + rtol * want.double().abs()).all()), err.max().item()


def _grpo_inputs(P, n, L, seed, reward="bernoulli", shuffle=False, big_ids=False):
    g = torch.Generator().manual_seed(seed)
    B = P * n
    lens = torch.randint(1, L + 1, (B,), generator=g)
    mask = (torch.arange(L)[None, :] < lens[:, None]).long()
    if reward == "bernoulli":
        s = (torch.rand(B, generator=g) < 0.5).float()
    elif reward == "pm1":
        s = (torch.rand(B, generator=g) < 0.5).float() * 2 - 1
    else:
        s = torch.randn(B, generator=g) * 3
    rewards = torch.zeros(B, L)
    rewards[torch.arange(B), lens - 1] = s  # outcome reward at the last valid token
    uid = torch.arange(P).repeat_interleave(n)
    if big_ids:
        ids = torch.randint(-(2 ** 40), 2 ** 40, (P,), generator=g)
        uid = ids[uid]
    if shuffle:
        perm = torch.randperm(B, generator=g)
        rewards, mask, uid = rewards[perm], mask[perm], uid[perm]
    return rewards, mask, uid


@pytest.mark.parametrize("P,n,L", [(1, 1, 1), (1, 5, 3), (64, 8, 256), (7, 3, 50), (300, 5, 17), (512, 16, 64)])
@pytest.mark.parametrize("reward", ["bernoulli", "pm1", "gauss"])
@pytest.mark.parametrize("shuffle,big_ids", [(False, False), (True, True)])
def test_grpo_matches_oracle(dev, P, n, L, reward, shuffle, big_ids):
    import siirl_amd.core_algos as CA

    rewards, mask, uid = _grpo_inputs(P, n, L, seed=P * 100 + n, reward=reward, shuffle=shuffle, big_ids=big_ids)
    for norm in (True, False):
        adv, ret = CA.compute_grpo_outcome_advantage(token_level_rewards=rewards.to(dev), response_mask=mask.to(dev),
                                                     index=uid.numpy(), norm_adv_by_std_in_grpo=norm)
        assert adv is ret and adv.shape == rewards.shape and adv.dtype == torch.float32 and adv.is_cuda
        want, _ = OC.compute_grpo_outcome_advantage(rewards, mask, uid.numpy(), norm_adv_by_std_in_grpo=norm)
        ok, err = _rel_close(adv.cpu(), want)
        assert ok, err
        want64, _ = OC.compute_grpo_outcome_advantage(rewards.double(), mask, uid.numpy(), norm_adv_by_std_in_grpo=norm)
        ok, err = _rel_close(adv.cpu(), want64, rtol=1e-5, atol=2e-6)
        assert ok, err
        assert torch.count_nonzero(adv.cpu()[mask == 0]) == 0  # mask bookkeeping: exact


def test_grpo_known_answers_and_invariants(dev):
    import siirl_amd.core_algos as CA

    ones = torch.ones(5, 2)
    r = torch.zeros(5, 2)
    r[0, 1] = 1.0  # one success in five: the reference's quickstart log shows max 1.789
    a, _ = CA.compute_grpo_outcome_advantage(r.to(dev), ones.to(dev), np.zeros(5, dtype=np.int64))
    assert abs(a[0, 0].item() - 0.8 / (0.2 ** 0.5 + 1e-6)) < 1e-5 and abs(a[0, 0].item() - 1.78885) < 1e-4
    r[1, 1] = 1.0  # two in five: min -0.730
    a, _ = CA.compute_grpo_outcome_advantage(r.to(dev), ones.to(dev), np.zeros(5, dtype=np.int64))
    assert abs(a[4, 0].item() + 0.4 / (0.3 ** 0.5 + 1e-6)) < 1e-5 and abs(a[4, 0].item() + 0.73030) < 1e-4
    # all-equal group -> exactly zero; singleton -> s / (1 + eps); pair {0, 1} -> unbiased std sqrt(1/2)
    r = torch.tensor([[1.0], [1.0], [1.0], [3.0], [0.0], [1.0]])
    uid = ["7", "7", "7", "9", "11", "11"]  # numeric strings are accepted as in the reference (:326)
    a, _ = CA.compute_grpo_outcome_advantage(r.to(dev), torch.ones(6, 1).to(dev), uid)
    a = a.cpu().flatten()
    assert a[0] == 0 and a[1] == 0 and a[2] == 0
    assert abs(a[3].item() - 3.0 / (1 + 1e-6)) < 1e-6
    assert abs(a[5].item() - 0.5 / (0.5 ** 0.5 + 1e-6)) < 1e-6 and abs(a[4].item() + a[5].item()) < 1e-7
    # permutation equivariance and a tensor index
    rewards, mask, uid_t = _grpo_inputs(40, 6, 9, seed=4, reward="gauss")
    a1, _ = CA.compute_grpo_outcome_advantage(rewards.to(dev), mask.to(dev), uid_t.to(dev))
    perm = torch.randperm(240, generator=torch.Generator().manual_seed(0))
    a2, _ = CA.compute_grpo_outcome_advantage(rewards[perm].to(dev), mask[perm].to(dev), uid_t[perm])
    assert (a1.cpu()[perm] - a2.cpu()).abs().max() < 1e-6
    # group sums of the normalised scores vanish
    assert a1.cpu()[:, 0].reshape(40, 6).sum(1).abs().max() < 1e-5  # token 0 is always inside the mask
    # host tensors are staged through the GPU and come back on the host
    a3, _ = CA.compute_grpo_outcome_advantage(rewards, mask, uid_t.numpy())
    assert not a3.is_cuda and (a3 - a1.cpu()).abs().max() == 0


def test_uids_that_are_not_int64(dev):
    """The reference keys its groups with Python objects (core_algos.py:326 ``int(index[i])``; filter_interface/dapo.py:70
    the uid itself unless it is a tensor / numpy scalar): uuid strings and 128-bit integers work there, so they do
    here -- numbered on the host in order of first appearance, same groups."""
    import uuid

    import siirl_amd.core_algos as CA
    from siirl_amd import dapo_filter as DF

    g = torch.Generator().manual_seed(12)
    names = [uuid.UUID(int=int(torch.randint(0, 2 ** 62, (1,), generator=g)) << 64 | 7 * k) for k in range(5)]
    order = torch.randint(0, 5, (23,), generator=g).tolist()
    big = [names[k].int for k in order]            # 128-bit Python integers
    text = [str(names[k]) for k in order]          # uuid strings
    small = np.asarray(order, dtype=np.int64)
    rewards, mask, _ = _grpo_inputs(23, 1, 7, seed=5, reward="gauss")
    want, _ = OC.compute_grpo_outcome_advantage(rewards, mask, small)
    got_big, _ = CA.compute_grpo_outcome_advantage(rewards.to(dev), mask.to(dev), big)
    got_obj, _ = CA.compute_grpo_outcome_advantage(rewards.to(dev), mask.to(dev), np.asarray(big, dtype=object))
    assert (got_big.cpu() - want).abs().max() < 1e-5 and torch.equal(got_big, got_obj)
    metric = torch.randint(0, 2, (23,), generator=g).double().numpy()
    want_keep = OD.keep_mask(metric, small)
    for uids in (big, text, np.asarray(text), np.asarray(big, dtype=object)):
        if isinstance(uids, np.ndarray) and uids.dtype.kind == "U":
            with pytest.raises(ValueError):  # numpy strings have .item: the reference calls int() on them
                DF.group_keep_mask(metric, uids, device=dev)
            continue
        assert np.array_equal(DF.group_keep_mask(metric, uids, device=dev).cpu().numpy(), want_keep)
        assert np.array_equal(OD.keep_mask(metric, uids), want_keep)


def test_compute_advantage_dispatch(dev):
    import siirl_amd.core_algos as CA

    rewards, mask, uid = _grpo_inputs(8, 4, 12, seed=2)
    att = torch.cat([torch.ones(32, 5, dtype=torch.long), mask], dim=1)
    data = {"token_level_rewards": rewards.to(dev), "responses": torch.zeros(32, 12, dtype=torch.long, device=dev),
            "attention_mask": att.to(dev), "uid": uid.numpy()}
    out = CA.compute_advantage(data, CA.AdvantageEstimator.GRPO)
    want, _ = OC.compute_grpo_outcome_advantage(rewards, mask, uid.numpy())
    assert (out["advantages"].cpu() - want).abs().max() < 1e-5 and out["returns"] is out["advantages"]
    assert torch.equal(out["response_mask"].cpu(), mask)
    assert CA.get_adv_estimator_fn("grpo") is CA.compute_grpo_outcome_advantage
    assert CA.get_adv_estimator_fn(CA.AdvantageEstimator.GRPO) is CA.compute_grpo_outcome_advantage
    with pytest.raises(ValueError, match="Unknown advantage estimator"):
        CA.get_adv_estimator_fn("gae_marft")
    with pytest.raises(TypeError):  # the reference's CPGD branch passes a keyword GRPO does not take
        CA.compute_advantage(dict(data), "cpgd")
    with pytest.raises(KeyError):  # the multi-agent estimator reads its agent list from the keyword arguments
        CA.compute_advantage(dict(data), "gae_marft")
    with pytest.raises(NotImplementedError):
        CA.compute_advantage(dict(data), "reinforce_plus_plus")


# ------------------------------------------------------------------------------------ DAPO keep mask


def _check_keep(dev, metric, uid):
    import siirl_amd.dapo_filter as DF

    keep, gsz = DF.group_keep_mask(metric, uid, device=dev, return_group_size=True)
    want = OD.keep_mask(metric, uid)
    assert keep.dtype == torch.bool
    assert np.array_equal(keep.cpu().numpy(), want), "keep mask differs from np.std(values) > 0"
    counts = {}
    for u in np.asarray(uid).tolist():
        counts[u] = counts.get(u, 0) + 1
    assert gsz.cpu().tolist() == [counts[u] for u in np.asarray(uid).tolist()]
    return keep


def test_keep_mask_doc_example(dev):
    """The worked example of the reference's docs (docs/user_interface/filter_interface.rst:72-77)."""
    vals = [1.0, 1.0, 1.0, 1.0, 1.0, 0.0, 1.0, 0.0, 0.0, 0.0, 0.0, 0.0, 0.5, 0.8, 0.2, 0.9]
    uid = np.repeat(np.arange(4, dtype=np.int64), 4)
    keep = _check_keep(dev, np.asarray(vals), uid)
    assert torch.nonzero(keep).flatten().tolist() == [4, 5, 6, 7, 12, 13, 14, 15]


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
@pytest.mark.parametrize("n", [1, 2, 3, 7, 8, 9, 15, 16, 17, 64, 127, 128, 129, 200, 257, 1000])
def test_keep_mask_numpy_summation_order(dev, dtype, n):
    """Groups of equal non-dyadic values: whether np.std is exactly 0 depends on numpy's summation order
    (sequential below 8, eight accumulators up to 128, recursive halving above)."""
    rng = np.random.default_rng(n)
    consts = np.array([0.1, 0.3, 1.0 / 3.0, 0.7, 2.6, 1e-3, 123.456, 0.5], dtype=dtype)
    G = len(consts) + 4
    vals = np.concatenate([np.full(n, c, dtype=dtype) for c in consts] +
                          [rng.standard_normal(n).astype(dtype) for _ in range(2)] +
                          [np.full(n, 0.1, dtype=dtype) + (np.arange(n) == n - 1) * dtype(1e-7 if dtype == np.float32 else 1e-16)] +
                          [np.full(n, 1e-30, dtype=dtype)])
    uid = np.repeat(np.arange(G, dtype=np.int64) * 7 - 3, n)
    _check_keep(dev, vals, uid)
    perm = rng.permutation(len(uid))  # interleaved groups: members are summed in batch order
    _check_keep(dev, vals[perm], uid[perm])


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
def test_keep_mask_config3_shape(dev, dtype):
    """512 prompts x 16 responses, rewards +-1, ~30% of the groups forced to one sign."""
    rng = np.random.default_rng(3)
    P, n = 512, 16
    r = rng.choice([-1.0, 1.0], size=(P, n)).astype(dtype)
    same = rng.choice(P, size=154, replace=False)
    r[same] = r[same, :1]
    uid = np.repeat(np.arange(P, dtype=np.int64), n)
    keep = _check_keep(dev, r.reshape(-1), uid)
    dropped_groups = (~keep.cpu().reshape(P, n).any(1)).sum().item()
    assert dropped_groups >= 154  # the forced ones, plus any group that came out one-signed by chance
    # integer / bool metrics (the "acc" metric) are computed in float64, as numpy does
    acc = (r.reshape(-1) > 0)
    _check_keep(dev, acc, uid)
    _check_keep(dev, acc.astype(np.int64), uid)


def test_dynamic_sampling_end_to_end(dev):
    import siirl_amd.dapo_filter as DF

    P, n, L = 20, 4, 6
    g = torch.Generator().manual_seed(5)
    s = (torch.rand(P * n, generator=g) < 0.5).float()
    s[:8] = 1.0
    s[8:12] = 0.0
    rewards = torch.zeros(P * n, L)
    rewards[:, -1] = s
    uid = DF.make_uid(P, n)
    assert uid.dtype == np.int64 and uid[:5].tolist() == [0, 0, 0, 0, 1]
    batch = {"uid": uid, "token_level_rewards": rewards.to(dev), "input_ids": torch.arange(P * n).to(dev),
             "data_source": np.array([f"d{i}" for i in range(P * n)]), "tags": [i * 2 for i in range(P * n)],
             "eos_token_id": [1, 2], "pad_token_id": 151643}
    cfg = SimpleNamespace(algorithm=SimpleNamespace(filter_groups=SimpleNamespace(enable=True, metric="seq_final_reward")))
    out = DF.dynamic_sampling(cfg, batch)
    idx, kept_uids, n_groups = OD.dynamic_sampling_keep_indices(s.numpy(), uid)
    assert out.metrics["dapo_sampling/filtered_indices"] == idx
    assert out.metrics["dapo_sampling/kept_groups"] == len(kept_uids)
    assert out.metrics["dapo_sampling/total_groups"] == n_groups == P
    assert out.metrics["dapo_sampling/initial_trajectories"] == P * n
    assert out.metrics["dapo_sampling/final_trajectories"] == len(idx)
    assert abs(out.metrics["dapo_sampling/kept_trajectories_ratio"] - len(idx) / (P * n)) < 1e-12
    want = OD.filter_by_indices({k: (v.cpu() if isinstance(v, torch.Tensor) else v) for k, v in batch.items()}, idx)
    assert out.batch["input_ids"].cpu().tolist() == idx == want["input_ids"].tolist()
    assert out.batch["uid"].tolist() == want["uid"].tolist()
    assert out.batch["data_source"].tolist() == want["data_source"].tolist() and out.batch["tags"] == want["tags"]
    assert out.batch["eos_token_id"] == [1, 2] and out.batch["pad_token_id"] == 151643  # metadata untouched
    assert 0 not in out.batch["uid"] and 1 not in out.batch["uid"] and 2 not in out.batch["uid"]
    # disabled filter: batch passes through
    off = SimpleNamespace(algorithm=SimpleNamespace(filter_groups=SimpleNamespace(enable=False, metric="acc")))
    assert DF.dynamic_sampling(off, batch).batch is batch
    with pytest.raises(KeyError):
        bad = SimpleNamespace(algorithm=SimpleNamespace(filter_groups=SimpleNamespace(enable=True, metric="acc")))
        DF.dynamic_sampling(bad, batch)
    # all groups constant -> empty batch
    allsame = dict(batch, token_level_rewards=torch.ones(P * n, L, device=dev))
    res = DF.dynamic_sampling(cfg, allsame)
    assert res.metrics["dapo_sampling/filtered_indices"] == [] and res.batch == {}
