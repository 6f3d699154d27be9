"""GPU parity, seeded random sweeps over shapes and contents for the bit-exact parts of the path: index and mask
bookkeeping, grouping by uid, keep masks.  Each test draws a few hundred small cases from one seed and compares every
one with the CPU oracle; a failure prints the case."""
import numpy as np
import pytest
import torch

from oracle import core_algos as OC
from oracle import dapo_filter as OD
from oracle import padding as OP

pytestmark = pytest.mark.gpu


def test_sweep_response_mask_from_eos(dev):
    import siirl_amd.torch_functional as TF

    rng = np.random.default_rng(101)
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

    rng = np.random.default_rng(102)
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

    rng = np.random.default_rng(103)
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

    rng = np.random.default_rng(104)
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
        assert bool((err <= 1e-6 + 1e-5 * want.double().abs()).all()), (case, B, L, norm, err.max().item())
        assert bool((got.cpu()[mask == 0] == 0).all()), case
