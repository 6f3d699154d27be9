"""Dynamic micro-batching by token count: split a batch into micro-batches of balanced workload and restore the
original order afterwards.

Mirror of the part of ``siirl/utils/model_utils/seqlen_balancing.py`` that the actor / critic call around the loss
path (``rearrange_micro_batches`` ``:265-338``, ``get_reverse_idx`` ``:341-356``, ``prepare_dynamic_batch``
``:359-392``, ``restore_dynamic_batch`` ``:395-417``) with the partitioner they rest on
(``calculate_workload`` ``:29-38``, ``karmarkar_karp`` ``:41-142``, ``get_seqlen_balanced_partitions``
``:165-206``).  Host-side integer bookkeeping, as in the reference; batches are plain mappings of tensors, numpy
arrays and lists (a TensorDict works too).  One process per GPU and one GPU here: the reference's optional
``all_reduce(MAX)`` of the micro-batch count over the data-parallel group is not part of this build, so
``dp_group`` must be None.
"""

from __future__ import annotations

import heapq
from itertools import chain
from typing import List, Sequence

import torch

from .dapo_filter import filter_tensordict

__all__ = ["calculate_workload", "karmarkar_karp", "get_seqlen_balanced_partitions", "ceildiv",
           "roundup_divisible", "rearrange_micro_batches", "get_reverse_idx", "prepare_dynamic_batch",
           "restore_dynamic_batch"]


def calculate_workload(seqlen_list):
    """FLOPs of a dense transformer block up to a constant, for hidden size 4096: ``24576 * s + s**2``
    (reference ``seqlen_balancing.py:29-38``)."""
    s = seqlen_list if isinstance(seqlen_list, torch.Tensor) else torch.tensor(seqlen_list, dtype=torch.int64)
    return 24576 * s + s ** 2


class _Bucket:
    """One part of a partial partition: its sum and its ``(index, value)`` members in insertion order.
    Ordered by sum, then member count, then the member list itself."""

    __slots__ = ("total", "members")

    def __init__(self, members=()):
        self.members = list(members)
        self.total = sum(v for _, v in self.members)

    def absorb(self, other: "_Bucket"):
        self.members.extend(other.members)
        self.total += other.total

    def key(self):
        return (self.total, len(self.members), self.members)

    def __lt__(self, other):
        return self.key() < other.key()


class _Partial:
    """k buckets kept in descending order.  In the heap the partial with the largest spread (largest bucket sum
    minus smallest) comes first; equal spreads are ordered by the largest bucket, larger first."""

    __slots__ = ("buckets",)

    def __init__(self, members, k):
        assert len(members) in (1, k), f"{len(members)} not in [1, {k}]"
        self.buckets = sorted([_Bucket([m]) for m in members] + [_Bucket() for _ in range(k - len(members))],
                              reverse=True)

    @property
    def spread(self):
        return self.buckets[0].total - self.buckets[-1].total

    def fold(self, other: "_Partial"):
        # largest with smallest: the differencing step
        for mine, theirs in zip(self.buckets, reversed(other.buckets)):
            mine.absorb(theirs)
        self.buckets.sort(reverse=True)

    def __lt__(self, other):
        if self.spread != other.spread:
            return self.spread > other.spread
        return other.buckets[0] < self.buckets[0]


def karmarkar_karp(seqlen_list: Sequence[int], k_partitions: int, equal_size: bool) -> List[List[int]]:
    """Largest differencing method for k-way number partitioning (reference ``seqlen_balancing.py:41-142``).
    Returns k index lists, in the order of descending part sums; ``equal_size`` seeds the heap with groups of k
    neighbours of the sorted list so that every part receives the same number of items."""
    values = [int(v) for v in seqlen_list]
    order = sorted((v, i) for i, v in enumerate(values))
    heap: list = []
    if equal_size:
        assert len(values) % k_partitions == 0, f"{len(values)} % {k_partitions} != 0"
        for lo in range(0, len(order), k_partitions):
            heapq.heappush(heap, _Partial([(i, v) for v, i in order[lo:lo + k_partitions]], k_partitions))
    else:
        for v, i in order:
            heapq.heappush(heap, _Partial([(i, v)], k_partitions))
    while len(heap) > 1:
        first = heapq.heappop(heap)
        second = heapq.heappop(heap)
        first.fold(second)
        heapq.heappush(heap, first)
    parts = [[i for i, _ in b.members] for b in heap[0].buckets]
    if equal_size:
        for p in parts:
            assert len(p) * k_partitions == len(values), f"{len(p)} * {k_partitions} != {len(values)}"
    return parts


def get_seqlen_balanced_partitions(seqlen_list: Sequence[int], k_partitions: int, equal_size: bool) -> List[List[int]]:
    """k index lists with balanced sums, each sorted ascending (reference ``seqlen_balancing.py:165-206``)."""
    n = len(seqlen_list)
    assert n >= k_partitions, f"number of items:[{n}] < k_partitions:[{k_partitions}]"
    parts = karmarkar_karp(seqlen_list, k_partitions, equal_size)
    assert len(parts) == k_partitions, f"{len(parts)} != {k_partitions}"
    seen = set()
    out = []
    for i, p in enumerate(parts):
        assert len(p) > 0, f"the {i}-th partition is empty"
        seen.update(p)
        out.append(sorted(p))
    assert seen == set(range(n))
    return out


def ceildiv(a, b):
    return -(a // -b)


def roundup_divisible(a, b):
    return ((a + b - 1) // b) * b


def rearrange_micro_batches(batch, max_token_len, dp_group=None, num_batches_divided_by=None,
                            same_micro_num_in_dp=True, min_num_micro_batch=None, use_dynamic_bsz_balance=True):
    """Micro-batches whose attended-token totals stay below ``max_token_len``, and the index lists that map them
    back (reference ``seqlen_balancing.py:265-338``).  ``batch`` holds ``attention_mask`` ``[B, S]``."""
    if dp_group is not None:
        raise NotImplementedError("synchronising the micro-batch count over a data-parallel group is outside this build")
    mask = batch["attention_mask"]
    max_seq_len = mask.shape[-1]
    seq_len = mask.sum(dim=1).to("cpu", torch.int64)
    assert max_token_len >= max_seq_len, (
        f"max_token_len must be greater than the sequence length. Got {max_token_len=} and {max_seq_len=}"
    )
    total = int(seq_len.sum())
    n_micro = min(len(seq_len), ceildiv(total, max_token_len))
    if min_num_micro_batch is not None:
        n_micro = max(min_num_micro_batch, n_micro)
    if num_batches_divided_by is not None:
        n_micro = roundup_divisible(n_micro, num_batches_divided_by)
    assert n_micro <= len(seq_len)
    work = calculate_workload(seq_len).tolist()
    parts = get_seqlen_balanced_partitions(work, n_micro, equal_size=False)
    if use_dynamic_bsz_balance:
        # heaviest first, then the light ones moved to both ends (shorter warm-up and cool-down bubbles)
        parts.sort(key=lambda p: (sum(work[i] for i in p), p[0] if p else 0), reverse=True)
        parts = parts[::2][::-1] + parts[1::2]
    return [filter_tensordict(batch, p) for p in parts], parts


def get_reverse_idx(idx_map):
    """The inverse permutation: ``out[idx_map[i]] = i`` (reference ``seqlen_balancing.py:341-356``)."""
    out = list(idx_map)
    for i, j in enumerate(idx_map):
        out[j] = i
    return out


def prepare_dynamic_batch(data, max_token_len: int, dp_group=None, num_batches_divided_by=None,
                          same_micro_num_in_dp=True, min_num_micro_batch=None, use_dynamic_bsz_balance=True):
    """``(micro_batches, batch_idx_list)`` for dynamic batching (reference ``seqlen_balancing.py:359-392``).  As in
    the reference (``:388-392``) every entry of ``micro_batches`` is the whole list of micro-batches."""
    batches, idx = rearrange_micro_batches(data, max_token_len=max_token_len, dp_group=dp_group,
                                           num_batches_divided_by=num_batches_divided_by,
                                           same_micro_num_in_dp=same_micro_num_in_dp,
                                           min_num_micro_batch=min_num_micro_batch,
                                           use_dynamic_bsz_balance=use_dynamic_bsz_balance)
    return [batches for _ in idx], idx


def restore_dynamic_batch(data: torch.Tensor, batch_idx_list: List[List[int]]) -> torch.Tensor:
    """Rows of the concatenated micro-batch outputs put back in the original order (reference
    ``seqlen_balancing.py:395-417``)."""
    indices = list(chain.from_iterable(batch_idx_list))
    assert len(indices) == data.shape[0], f"{len(indices)} vs. {data.shape[0]}"
    back = torch.tensor(get_reverse_idx(indices), dtype=torch.long, device=data.device)
    return data[back]
