"""Host-side dynamic micro-batching (CPU): textbook answers of the largest differencing method, invariants,
hand-checked ordering, and the split -> restore round trip."""
import itertools
import random

import pytest
import torch

import siirl_amd.seqlen_balancing as SB


def _sums(vals, parts):
    return sorted(sum(vals[i] for i in p) for p in parts)


def test_ldm_textbook_examples():
    # the worked examples of the largest differencing method (en.wikipedia.org/wiki/Largest_differencing_method,
    # which the reference cites): S = {8,7,6,5,4}; two-way {8,6} / {7,5,4}; three-way {8} / {7,4} / {6,5}
    vals = [8, 7, 6, 5, 4]
    two = SB.karmarkar_karp(vals, 2, equal_size=False)
    assert sorted(sorted(vals[i] for i in p) for p in two) == [[4, 5, 7], [6, 8]]
    three = SB.karmarkar_karp(vals, 3, equal_size=False)
    assert sorted(sorted(vals[i] for i in p) for p in three) == [[4, 7], [5, 6], [8]]
    # parts come out in descending order of their sums
    assert [sum(vals[i] for i in p) for p in two] == [16, 14]


def test_ldm_beats_or_matches_greedy_bound_and_is_optimal_on_easy_cases():
    # four equal pairs: a perfect split exists and differencing finds it
    vals = [10, 10, 7, 7, 3, 3, 1, 1]
    assert _sums(vals, SB.karmarkar_karp(vals, 2, False)) == [21, 21]
    # k = n: every item alone
    assert _sums(vals, SB.karmarkar_karp(vals, 8, False)) == sorted(vals)


@pytest.mark.parametrize("seed", range(5))
@pytest.mark.parametrize("k,equal", [(2, False), (3, False), (4, True), (8, True)])
def test_partition_invariants(seed, k, equal):
    rnd = random.Random(seed)
    n = 24
    vals = [rnd.randint(1, 4000) for _ in range(n)]
    parts = SB.get_seqlen_balanced_partitions(vals, k, equal)
    assert len(parts) == k and sorted(itertools.chain.from_iterable(parts)) == list(range(n))
    assert all(p == sorted(p) and p for p in parts)
    if equal:
        assert all(len(p) == n // k for p in parts)
    s = _sums(vals, parts)
    # differencing keeps the spread below the largest item
    assert s[-1] - s[0] <= max(vals)
    # deterministic
    assert parts == SB.get_seqlen_balanced_partitions(vals, k, equal)


def test_partition_errors():
    with pytest.raises(AssertionError):
        SB.get_seqlen_balanced_partitions([1, 2], 3, False)
    with pytest.raises(AssertionError):
        SB.get_seqlen_balanced_partitions([1, 2, 3], 2, True)


def test_workload_and_small_helpers():
    assert SB.calculate_workload([0, 1, 10]).tolist() == [0, 24577, 245860]
    assert SB.ceildiv(7, 2) == 4 and SB.ceildiv(8, 2) == 4 and SB.roundup_divisible(5, 4) == 8
    assert SB.get_reverse_idx([2, 0, 3, 1]) == [1, 3, 0, 2]


def _batch(lens, S):
    B = len(lens)
    mask = (torch.arange(S)[None] < torch.tensor(lens)[:, None]).long()
    return {"attention_mask": mask, "input_ids": torch.arange(B * S).reshape(B, S), "tag": [f"t{i}" for i in range(B)]}


def test_rearrange_micro_batches_hand_case():
    lens = [10, 2, 9, 3, 8, 4]
    batch = _batch(lens, 10)
    mbs, idx = SB.rearrange_micro_batches(batch, max_token_len=12, use_dynamic_bsz_balance=False)
    assert len(idx) == 3 == SB.ceildiv(sum(lens), 12)
    assert sorted(itertools.chain.from_iterable(idx)) == list(range(6))
    for mb, p in zip(mbs, idx):
        assert int(mb["attention_mask"].sum()) <= 12 and mb["tag"] == [f"t{i}" for i in p]
        assert torch.equal(mb["input_ids"], batch["input_ids"][p])
    # balance ordering: sorted heaviest first, then [::2][::-1] + [1::2] puts the heaviest in the middle
    _, idx_b = SB.rearrange_micro_batches(batch, max_token_len=12, use_dynamic_bsz_balance=True)
    work = SB.calculate_workload(lens).tolist()
    loads = [sum(work[i] for i in p) for p in idx_b]
    order = sorted(loads, reverse=True)
    assert loads == order[::2][::-1] + order[1::2]
    with pytest.raises(AssertionError):
        SB.rearrange_micro_batches(batch, max_token_len=9)
    _, idx_m = SB.rearrange_micro_batches(batch, max_token_len=100, min_num_micro_batch=2, num_batches_divided_by=4)
    assert len(idx_m) == 4


@pytest.mark.parametrize("seed", range(3))
def test_split_then_restore_round_trip(seed):
    rnd = random.Random(seed)
    lens = [rnd.randint(1, 64) for _ in range(40)]
    batch = _batch(lens, 64)
    mbs, idx = SB.prepare_dynamic_batch(batch, max_token_len=256)
    assert all(m is mbs[0] for m in mbs) and len(mbs) == len(idx)  # the reference appends the whole list each time
    per_row = torch.cat([mb["input_ids"][:, 0] for mb in mbs[0]])
    restored = SB.restore_dynamic_batch(per_row, idx)
    assert torch.equal(restored, batch["input_ids"][:, 0])


def test_ties_follow_the_reference_heap_order_worked_by_hand():
    """Equal sums everywhere, so every decision is a tie-break.  Expected assignments are worked by hand from the
    reference's comparison keys (``siirl/utils/model_utils/seqlen_balancing.py:41-142``): a set compares by
    (sum, number of items, list of (index, value) items); a state's sets are kept in descending order; the heap pops
    the state with the largest spread first and, among equal spreads, the one whose largest set is larger; a merge
    pairs set i of the first popped state with set k - 1 - i of the second and re-sorts.

    [1, 1, 1, 1], k = 2.  Four singleton states of spread 1; among equal spreads the larger first set wins, and the
    sets differ only in their index, so index 3 pops first, then 2: {3} | {2}, spread 0.  Then 1 and 0: {1} | {0}.
    Both have spread 0; {3} > {1}, so {3} | {2} pops first and merges with {1} | {0} crosswise: {3, 0} | {2, 1}.
    Sums and sizes tie; the item lists [(3, 1), (0, 1)] > [(2, 1), (1, 1)] keep that order.

    [4, 3, 3, 2, 2, 2], k = 2 (indices 0..5).  Spreads 4, 3, 3, 2, 2, 2.  Pop index 0 (spread 4), then of the two
    3s the larger item list: index 2.  -> {0} | {2}, sums 4 | 3, spread 1.  Pop index 1 (spread 3), then of the 2s
    the largest index, 5 -> {1} | {5}, sums 3 | 2, spread 1.  Pop 4, then 3 -> {4} | {3}, spread 0.  The two spread-1
    states: first sets {0} (sum 4) > {1} (sum 3), so {0} | {2} pops first and takes {1} | {5} crosswise:
    {0, 5} (6) and {2, 1} (6); equal sums and sizes, item lists [(2, 3), (1, 3)] > [(0, 4), (5, 2)], so the order
    becomes {2, 1} | {0, 5}.  Last merge: its first set (sum 6) > {4} (sum 2), so it pops first and takes {4} | {3}
    crosswise: {2, 1, 3} (8) | {0, 5, 4} (8); [(2, 3), ...] > [(0, 4), ...] keeps the order."""
    assert SB.karmarkar_karp([1, 1, 1, 1], 2, False) == [[3, 0], [2, 1]]
    assert SB.karmarkar_karp([4, 3, 3, 2, 2, 2], 2, False) == [[2, 1, 3], [0, 5, 4]]
    assert SB.get_seqlen_balanced_partitions([4, 3, 3, 2, 2, 2], 2, False) == [[1, 2, 3], [0, 4, 5]]
    # equal_size seeds the heap with groups of k neighbours of the sorted list.
    # [2, 2, 1, 1], k = 2: groups (indices 2, 3) and (0, 1); inside a group the larger index sorts first:
    # {3} | {2} and {1} | {0}, both spread 0; {1} (sum 2) > {3} (sum 1) pops first and takes the other crosswise:
    # {1, 2} (3) | {0, 3} (3); (1, 2) > (0, 2) keeps the order.
    assert SB.karmarkar_karp([2, 2, 1, 1], 2, True) == [[1, 2], [0, 3]]
    # [5] * 6, k = 3: groups {2} | {1} | {0} and {5} | {4} | {3}; the second has the larger first set, pops first and
    # takes the first crosswise: {5, 0} | {4, 1} | {3, 2}, already in descending item order.
    assert SB.karmarkar_karp([5, 5, 5, 5, 5, 5], 3, True) == [[5, 0], [4, 1], [3, 2]]
