"""Pins the oracle's DAPO filter / uid helpers (CPU only) against the vectors the reference's own tests and docs
hold (tests/golden/reference_vectors.json), and pins the statement of numpy's summation order that the GPU
keep-mask kernel reproduces."""

import json
import os

import numpy as np
import pytest
import torch

from oracle import dapo_filter as OD

GOLD = json.load(open(os.path.join(os.path.dirname(__file__), "golden", "reference_vectors.json")))


def test_uid_layout_from_reference_test():
    v = GOLD["uid_layout"]
    uid = OD.make_uid(v["num_prompts"], v["n"])
    assert uid.dtype == np.int64 and uid.tolist() == v["expected_uid"]
    # the same repeat applied to the other fields, as the reference's test checks
    assert np.repeat(np.array(v["input_ids"]), v["n"], axis=0).tolist() == v["expected_input_ids"]
    assert torch.tensor(v["attention_mask"]).repeat_interleave(v["n"], dim=0).tolist() == v["expected_attention_mask"]


def test_filter_is_ordered_index_select_from_reference_test():
    v = GOLD["filter_index_select"]
    B = v["batch_size"]
    batch = {"input_ids": torch.arange(B * 3).reshape(B, 3), "uid": torch.arange(B) // 16,
             "data_source": np.array([f"s{i}" for i in range(B)]), "ability": ["math"] * B,
             "global_token_num": list(range(B)), "eos_token_id": v["metadata_eos_token_id"],
             "pad_token_id": v["metadata_pad_token_id"]}
    idx = list(range(*v["indices_range"]))
    out = OD.filter_by_indices(batch, idx)
    assert len(out["input_ids"]) == len(out["uid"]) == v["expected_len"] == len(idx)
    assert len(out["data_source"]) == len(out["ability"]) == len(out["global_token_num"]) == len(idx)
    assert out["eos_token_id"] == v["metadata_eos_token_id"] and out["pad_token_id"] == v["metadata_pad_token_id"]
    assert out["input_ids"][:, 0].tolist() == [3 * i for i in idx] and out["global_token_num"] == idx
    rev = OD.filter_by_indices(batch, [5, 2, 9])  # order of the index list is kept
    assert rev["uid"].tolist() == [0, 0, 0] and rev["global_token_num"] == [5, 2, 9]
    assert OD.filter_by_indices(batch, []) == {}


def test_filter_worked_example_from_reference_docs():
    v = GOLD["filter_worked_example"]
    vals, uids = [], []
    for u, g in v["groups"].items():
        vals += g
        uids += [int(u)] * len(g)
    idx, kept, n_groups = OD.dynamic_sampling_keep_indices(np.array(vals), np.array(uids))
    assert sorted(kept) == v["kept_uids"] and n_groups == 4
    assert idx == [4, 5, 6, 7, 12, 13, 14, 15]
    assert OD.keep_mask(np.array(vals), np.array(uids)).tolist() == [u in v["kept_uids"] for u in uids]


def test_keep_rules_bruteforce():
    rng = np.random.default_rng(0)
    uids = rng.integers(0, 12, size=60)
    vals = rng.choice([0.0, 1.0], size=60)
    vals[uids == 3] = 1.0
    idx, kept, _ = OD.dynamic_sampling_keep_indices(vals, uids)
    for u in range(12):
        members = vals[uids == u]
        if len(members) == 0:
            continue
        expect = len(members) == 1 or len(set(members.tolist())) > 1
        assert (u in kept) == expect
    assert idx == sorted(idx) and all(int(uids[i]) in kept for i in idx)
    single = OD.keep_mask(np.array([5.0, 1.0, 1.0]), np.array([9, 4, 4]))
    assert single.tolist() == [True, False, False]  # a group of one is kept, an all-equal pair is not


def _np_pairwise(a):
    """numpy's pairwise summation, restated: sequential below 8 values, eight accumulators up to 128,
    halves (left half rounded down to a multiple of 8) above.  All arithmetic in a's dtype."""
    n = len(a)
    t = a.dtype.type
    if n < 8:
        res = t(0)
        for v in a:
            res = t(res + v)
        return res
    if n <= 128:
        r = [t(a[i]) for i in range(8)]
        i = 8
        while i < n - (n % 8):
            for k in range(8):
                r[k] = t(r[k] + a[i + k])
            i += 8
        res = t(t(t(r[0] + r[1]) + t(r[2] + r[3])) + t(t(r[4] + r[5]) + t(r[6] + r[7])))
        while i < n:
            res = t(res + a[i])
            i += 1
        return res
    n2 = n // 2
    n2 -= n2 % 8
    return t(_np_pairwise(a[:n2]) + _np_pairwise(a[n2:]))


def _np_std_restated(a):
    t = a.dtype.type
    n = len(a)
    mean = t(_np_pairwise(a) / t(n))
    d = (a - mean).astype(a.dtype)
    return np.sqrt(t(_np_pairwise((d * d).astype(a.dtype)) / t(n)))


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
def test_numpy_std_summation_order_is_as_restated(dtype):
    """The GPU kernel hard-codes this order; if numpy's differed, these would differ in the last bit."""
    rng = np.random.default_rng(1)
    for n in [1, 2, 7, 8, 9, 16, 17, 100, 128, 129, 136, 255, 256, 257, 1000, 4097]:
        for a in (rng.standard_normal(n).astype(dtype), np.full(n, 0.1, dtype=dtype), np.full(n, 1 / 3, dtype=dtype),
                  (rng.standard_normal(n) * 1e-20).astype(dtype)):
            assert _np_std_restated(a) == np.std(a), (n, dtype)
    assert np.std(np.array([0.1, 0.1, 0.1])) > 0  # the fp64 quirk: an all-equal group that is kept
    assert np.std(np.array([0.1, 0.1, 0.1], dtype=np.float32)) == 0
    assert OD.keep_mask(np.array([0.1, 0.1, 0.1]), np.array([0, 0, 0])).all()
    assert not OD.keep_mask(np.array([0.1, 0.1, 0.1], dtype=np.float32), np.array([0, 0, 0])).any()
