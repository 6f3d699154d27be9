"""DAPO dynamic sampling: drop the prompt groups whose metric has no variance.

Mirror of ``siirl/user_interface/filter_interface/dapo.py:24-107`` (``dynamic_sampling``) and of the two
helpers it leans on in ``siirl/data_coordinator/sample.py``: the uid layout of ``preprocess_dataloader``
(``:109-136``) and ``filter_tensordict`` (``:242-322``).  The group test -- ``np.std(values) > 0`` or a group
of one -- runs on the GPU (``siirl_group_keep_mask``) and reproduces numpy's arithmetic bit for bit; the
batch is then index-selected in ascending order of the kept positions.
"""

from __future__ import annotations

from dataclasses import dataclass, field
from typing import Any, Dict, List

import numpy as np
import torch

from . import _lib  # noqa: F401
from . import ops as _ops_module  # noqa: F401  (registers torch.ops.siirl_hip.*)

__all__ = ["NodeOutput", "make_uid", "group_keep_mask", "filter_tensordict", "dynamic_sampling",
           "SamplingLeftoverCache"]


@dataclass
class NodeOutput:
    """What a DAG node hands back (reference ``siirl/dag_worker/data_structures.py``): the batch and a metrics dict."""

    batch: Any = None
    metrics: Dict[str, Any] = field(default_factory=dict)


def make_uid(num_prompts: int, n: int) -> np.ndarray:
    """int64 uids ``[0]*n + [1]*n + ...`` as ``preprocess_dataloader`` creates them (reference
    ``sample.py:127-131``)."""
    return np.repeat(np.arange(num_prompts, dtype=np.int64), n, axis=0)


def _metric_tensor(values, dev) -> torch.Tensor:
    """The metric as a device tensor in the dtype numpy's ``np.std`` would compute in: float32 stays float32,
    float64 / Python floats / integers / bools become float64."""
    if isinstance(values, (list, tuple)) and len(values) and isinstance(values[0], torch.Tensor):
        values = torch.stack([v.detach().reshape(()) for v in values])  # np.std of 0-d tensors keeps their dtype
    if isinstance(values, torch.Tensor):
        t = values.detach().reshape(-1)
        if t.dtype == torch.float32:
            return t.to(dev).contiguous()
        if t.dtype in (torch.float64, torch.int64, torch.int32, torch.int16, torch.int8, torch.uint8, torch.bool):
            return t.to(device=dev, dtype=torch.float64).contiguous()
        raise TypeError(f"metric dtype {t.dtype} is not supported (float32, float64, integers, bool)")
    arr = np.asarray(values)
    arr = arr.reshape(-1)
    if arr.dtype == np.float32:
        return torch.from_numpy(np.ascontiguousarray(arr)).to(dev)
    if arr.dtype.kind in "fiub" and arr.dtype != np.float16:
        return torch.from_numpy(np.ascontiguousarray(arr.astype(np.float64))).to(dev)
    raise TypeError(f"metric dtype {arr.dtype} is not supported (float32, float64, integers, bool)")


def _uid_tensor(uids, dev) -> torch.Tensor:
    """int64 group codes on ``dev``.  Integer uids (the reference's ``preprocess_dataloader`` makes int64 ones,
    ``sample.py:127-131``) are used as they are; anything else the reference's dict would accept as a key (strings,
    integers beyond 64 bits, ``filter_interface/dapo.py:68-72``: ``int(uid)`` for numpy / tensor scalars, the object
    itself otherwise) is numbered on the host in order of first appearance -- only equality matters downstream."""
    if isinstance(uids, torch.Tensor):
        return uids.detach().reshape(-1).to(device=dev, dtype=torch.int64).contiguous()
    arr = np.asarray(uids)
    if arr.dtype.kind in "iu" and (arr.dtype.kind == "i" or arr.size == 0 or int(arr.max()) < 2 ** 63):
        return torch.from_numpy(np.ascontiguousarray(arr.reshape(-1).astype(np.int64))).to(dev)
    seq = list(uids) if isinstance(uids, (list, tuple)) else list(arr.reshape(-1))
    codes: dict = {}
    out = np.fromiter((codes.setdefault(int(v) if hasattr(v, "item") else v, len(codes)) for v in seq),
                      dtype=np.int64, count=len(seq))
    return torch.from_numpy(out).to(dev)


def group_keep_mask(metric_values, uids, device=None, return_group_size: bool = False):
    """Boolean ``[B]`` device tensor: True where the trajectory's uid-group has ``np.std(metric) > 0`` or a
    single member (reference ``dapo.py:76-85``)."""
    if device is None:
        for t in (metric_values, uids):
            if isinstance(t, torch.Tensor) and t.is_cuda:
                device = t.device
                break
        else:
            if not torch.cuda.is_available():
                raise RuntimeError("siirl_amd: no GPU visible; there is no CPU fallback")
            device = torch.device("cuda", torch.cuda.current_device())
    uid = _uid_tensor(uids, device)
    met = _metric_tensor(metric_values, device)
    B = uid.numel()
    if met.numel() != B:
        raise ValueError(f"{met.numel()} metric values for {B} uids")
    keep, gsz = torch.ops.siirl_hip.group_keep_mask(met, uid)
    keep = keep.bool()
    return (keep, gsz) if return_group_size else keep


def _select_rows(t: torch.Tensor, indices) -> torch.Tensor:
    """``t[indices]`` along the first axis.  A tensor on the GPU whose rows are whole 4-byte words goes through the
    row gather of the un-padding path (``siirl_gather_rows``: 16-byte moves, 6.2 TB/s on [8192, 8192] float32 rows);
    host tensors, as the reference holds them here, and odd-sized rows are indexed by torch."""
    idx = indices if isinstance(indices, torch.Tensor) and indices.device == t.device and indices.dtype == torch.long \
        else torch.as_tensor(indices, dtype=torch.long, device=t.device)
    row_bytes = t[0].numel() * t.element_size() if t.dim() >= 1 and t.shape[0] else 0
    if t.is_cuda and row_bytes >= 4 and row_bytes % 4 == 0 and not t.requires_grad:
        from . import padding as _padding

        return _padding.index_first_axis(t, idx)
    return t[idx]


def filter_tensordict(batch, indices: List[int]):
    """Ordered index select of every batched field (reference ``sample.py:242-322``): tensors are indexed
    with ``indices`` in the given order; numpy arrays / lists whose length equals the batch size likewise;
    anything else is metadata and is kept.  An empty list gives an empty batch.  Works on a ``dict`` and on
    a ``TensorDict`` (returned as the same kind)."""
    is_td = hasattr(batch, "batch_size") and not isinstance(batch, dict)
    if not indices:
        if is_td:
            return type(batch)({}, batch_size=(0,))
        return {}
    bsz = batch.batch_size[0] if is_td else next(v.shape[0] for v in batch.values() if isinstance(v, torch.Tensor))
    idx_np = np.asarray(indices, dtype=np.int64)
    idx_on = {}  # the index list as a tensor, made once per device
    out = {}
    for key, value in batch.items():
        data = getattr(value, "data", value) if type(value).__name__ == "NonTensorData" else value
        if isinstance(value, torch.Tensor):
            if value.device not in idx_on:
                idx_on[value.device] = torch.from_numpy(idx_np).to(value.device)
            out[key] = _select_rows(value, idx_on[value.device])
        elif isinstance(data, np.ndarray) and len(data) == bsz:
            out[key] = data[idx_np]
        elif isinstance(data, (list, tuple)) and len(data) == bsz:
            out[key] = [data[i] for i in indices]
        else:
            out[key] = value
    if is_td:
        return type(batch)(out, batch_size=len(indices))
    return out


def _batch_len(batch) -> int:
    if batch is None:
        return 0
    if hasattr(batch, "batch_size") and not isinstance(batch, dict):
        return int(batch.batch_size[0]) if len(batch.batch_size) else 0
    for v in batch.values():
        if isinstance(v, torch.Tensor):
            return int(v.shape[0])
    return 0


class SamplingLeftoverCache:
    """Carries kept trajectories from one DAPO sampling round to the next until a full batch exists: the
    leftover-cache semantics pinned by the reference's ``tests/dag_worker/test_dapo_pipeline.py:52-195``
    (the worker attribute is ``sampling_leftover_cache``, ``siirl/dag_worker/dagworker.py:126``).

    ``postprocess(filtered_batch, target_total_samples)``: a non-empty cache is merged in front of the new
    batch (``cache || new``) -- tensors concatenated along the batch axis, numpy arrays concatenated, lists and
    tuples appended, any other value is metadata and the new batch's wins, a key present on one side only is
    taken from that side -- and the cache is cleared; then, if fewer than ``target_total_samples`` samples are
    at hand they are cached and an empty batch is returned, otherwise the merged batch is."""

    def __init__(self):
        self.sampling_leftover_cache = None

    @staticmethod
    def merge(cache, new):
        out = {}
        keys = list(cache.keys()) + [k for k in new.keys() if k not in cache.keys()]
        for key in keys:
            c = cache.get(key) if key in cache.keys() else None
            n = new.get(key) if key in new.keys() else None
            if c is None or n is None:
                out[key] = n if c is None else c
            elif isinstance(c, torch.Tensor):
                out[key] = torch.cat([c, n.to(c.device)], dim=0)
            elif isinstance(c, np.ndarray):
                out[key] = np.concatenate([c, np.asarray(n)], axis=0)
            elif isinstance(c, (list, tuple)):
                out[key] = list(c) + list(n)
            else:
                out[key] = n
        return out

    def postprocess(self, filtered_batch, target_total_samples: int):
        batch = dict(filtered_batch.items()) if filtered_batch is not None else {}
        if self.sampling_leftover_cache is not None:
            batch = self.merge(self.sampling_leftover_cache, batch)
            self.sampling_leftover_cache = None
        if _batch_len(batch) < target_total_samples:
            self.sampling_leftover_cache = batch
            return {}
        return batch


def dynamic_sampling(config, batch, **kwargs) -> NodeOutput:
    """Filter trajectory groups by metric variance (reference ``dapo.py:24-107``).  ``config`` needs
    ``config.algorithm.filter_groups.{enable, metric}``; ``batch`` is a mapping with ``uid`` and the metric
    (``acc``, or ``seq_final_reward`` / ``seq_reward`` derived from the token-level tensors when absent).
    Returns the filtered batch and the same metrics dict, ``dapo_sampling/filtered_indices`` included."""
    fc = config.algorithm.filter_groups
    if not fc.enable:
        return NodeOutput(batch=batch, metrics={"sampling/kept_trajectories_ratio": 1.0})
    name = fc.metric
    keys = list(batch.keys())
    initial = len(batch["uid"]) if batch is not None else 0
    if name in keys:
        metric = batch[name]
    elif name == "seq_final_reward" and "token_level_rewards" in keys:
        metric = batch["token_level_rewards"].sum(dim=-1)
    elif name == "seq_reward" and "token_level_scores" in keys:
        metric = batch["token_level_scores"].sum(dim=-1)
    else:
        raise KeyError(f"Metric '{name}' for group filtering not found in batch and could not be computed. "
                       f"Available non-tensor keys: {keys}")
    uids = batch["uid"]
    keep, gsz = group_keep_mask(metric, uids, return_group_size=True)
    kept = torch.nonzero(keep).flatten().tolist()
    inv = 1.0 / gsz.double()  # each group of n members contributes n * (1/n) = 1
    total_groups = int(torch.round(inv.sum()).item())
    kept_groups = int(torch.round((inv * keep).sum()).item())
    filtered = filter_tensordict(batch, kept)
    final = len(kept)
    metrics = {
        "dapo_sampling/kept_trajectories_ratio": final / initial if initial > 0 else 1.0,
        "dapo_sampling/initial_trajectories": initial,
        "dapo_sampling/final_trajectories": final,
        "dapo_sampling/kept_groups": kept_groups,
        "dapo_sampling/total_groups": total_groups,
        "dapo_sampling/filtered_indices": kept,
    }
    return NodeOutput(batch=filtered, metrics=metrics)
