"""Oracle (test infrastructure): DAPO dynamic-sampling filter and the uid layout.

Restates ``siirl/user_interface/filter_interface/dapo.py:48-104`` (which groups to keep) and
``siirl/data_coordinator/sample.py:109-136,242-322`` (uid creation, ordered index select)."""

from __future__ import annotations

from collections import OrderedDict

import numpy as np
import torch


def make_uid(num_prompts: int, n: int) -> np.ndarray:
    """uid of a batch of ``num_prompts`` prompts sampled ``n`` times each: ``[0]*n + [1]*n + ...``
    as int64 (reference ``sample.py:127-131``; pinned by
    ``tests/dag_worker/test_dapo_pipeline.py:35-36`` -> ``[0, 0, 1, 1]``)."""
    return np.repeat(np.arange(num_prompts, dtype=np.int64), n, axis=0)


def dynamic_sampling_keep_indices(metric_values, uids):
    """Indices (ascending) of the trajectories whose uid-group has ``np.std(values) > 0`` or has
    a single member (reference ``dapo.py:66-93``).  ``np.std`` is the population standard
    deviation computed *in the dtype of the values* with numpy's pairwise summation, so a group
    of equal non-dyadic fp64 values such as ``[0.1, 0.1, 0.1]`` has std 1.4e-17 > 0 and is kept,
    while the same values in fp32 give exactly 0.  Returns ``(indices, kept_uids, n_groups)``."""
    def key(u):  # reference ``dapo.py:70,91``: tensor / numpy scalars through int(), any other object as it is
        return int(u) if hasattr(u, "item") else u

    groups = OrderedDict()
    for i in range(len(uids)):
        groups.setdefault(key(uids[i]), []).append(metric_values[i])
    kept = {u for u, vals in groups.items() if np.std(vals) > 0 or len(vals) == 1}
    idx = [i for i in range(len(uids)) if key(uids[i]) in kept]
    return idx, kept, len(groups)


def keep_mask(metric_values, uids) -> np.ndarray:
    idx, _, _ = dynamic_sampling_keep_indices(metric_values, uids)
    out = np.zeros(len(uids), dtype=bool)
    out[idx] = True
    return out


def filter_by_indices(batch: dict, indices):
    """Ordered index select of every batched field (reference ``sample.py:242-322``): tensors
    are indexed with the list in the given order, numpy arrays / lists whose length equals the
    batch size likewise, anything else is metadata and passes through.  An empty index list
    returns an empty dict (the reference returns an empty TensorDict)."""
    if not indices:
        return {}
    bsz = None
    for v in batch.values():
        if isinstance(v, torch.Tensor):
            bsz = v.shape[0]
            break
    it = torch.tensor(indices, dtype=torch.long)
    inp = np.asarray(indices, dtype=np.int64)
    out = {}
    for k, v in batch.items():
        if isinstance(v, torch.Tensor):
            out[k] = v[it]
        elif isinstance(v, np.ndarray) and len(v) == bsz:
            out[k] = v[inp]
        elif isinstance(v, (list, tuple)) and len(v) == bsz:
            out[k] = [v[i] for i in indices]
        else:
            out[k] = v
    return out


def merge_leftover(cache: dict, new: dict) -> dict:
    """``cache || new`` as the reference's leftover-cache test states it
    (``tests/dag_worker/test_dapo_pipeline.py:72-126``): tensors and numpy arrays concatenated along the batch
    axis, lists appended, other values taken from the new batch, one-sided keys kept."""
    out = {}
    for key in set(cache) | set(new):
        c, n = cache.get(key), new.get(key)
        if c is None:
            out[key] = n
        elif n is None:
            out[key] = c
        elif isinstance(c, torch.Tensor):
            out[key] = torch.cat([c, n], dim=0)
        elif isinstance(c, np.ndarray):
            out[key] = np.concatenate([c, n], axis=0)
        elif isinstance(c, (list, tuple)):
            out[key] = list(c) + list(n)
        else:
            out[key] = n
    return out


def place_outcome_reward(scores, attention_mask, response_length, overlong_enable=False, max_resp_len=None,
                         overlong_buffer_len=None, overlong_penalty_factor=None):
    """The reward tensor of ``DAPORewardManager.__call__`` (reference ``siirl/engine/reward_manager/dapo.py:57-126``)
    for given scalar scores: zeros, with ``score + min(-(valid - (max_resp_len - buffer)) / buffer * factor, 0)``
    (the second term only when the overlong buffer is enabled) at ``[i, valid - 1]``, ``valid`` the attention
    mask's sum over the response columns.  Returns ``(reward_tensor, overlong_rewards)``."""
    B, S = attention_mask.shape
    prompt_length = S - response_length
    reward = torch.zeros(B, response_length, dtype=torch.float32)
    pens = []
    for i in range(B):
        valid = attention_mask[i][prompt_length:].sum()
        r = float(scores[i])
        pen = 0.0
        if overlong_enable:
            expected = max_resp_len - overlong_buffer_len
            exceed = valid - expected
            pen = min(-exceed / overlong_buffer_len * overlong_penalty_factor, 0)
            r += pen
        reward[i, valid - 1] = r
        pens.append(float(pen))
    return reward, pens
