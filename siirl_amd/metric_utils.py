"""The per-step data metrics with the reference's function name and metric keys.

Mirror of ``compute_data_metric`` (``siirl/utils/metrics/metric_utils.py:70-183``): the same dictionary keys,
computed by one pair of kernels and fetched with a single device-to-host copy instead of one ``.item()`` per
entry.  ``perf/process_cpu_mem_used_gb`` and the ``num_turns/*`` entries are host-side and added here as the
reference adds them."""

from __future__ import annotations

import os

import torch

from . import _lib
from .core_algos import _f32, _mask_arg, _staging_device

__all__ = ["compute_data_metric"]

_KEYS = (
    "critic/score/mean", "critic/score/max", "critic/score/min",
    "critic/rewards/mean", "critic/rewards/max", "critic/rewards/min",
    "critic/advantages/mean", "critic/advantages/max", "critic/advantages/min",
    "critic/returns/mean", "critic/returns/max", "critic/returns/min",
    "critic/values/mean", "critic/values/max", "critic/values/min", "critic/vf_explained_var",
    "response/length/mean", "response/length/max", "response/length/min", "response/clip_ratio/mean",
    "response/correct_length/max", "response/correct_length/min", "response/correct_length/mean",
    "response/wrong_length/max", "response/wrong_length/min", "response/wrong_length/mean",
    "prompt/length/mean", "prompt/length/max", "prompt/length/min", "prompt/clip_ratio/mean",
)
_VALUE_KEYS = _KEYS[12:16]


def compute_data_metric(data) -> dict:
    """``data`` is a mapping (TensorDict or dict) with ``token_level_scores``, ``token_level_rewards``,
    ``advantages``, ``returns``, ``responses``, ``attention_mask``, ``response_mask`` and optionally ``values``
    and ``__num_turns__`` (reference ``metric_utils.py:70-177``).  Host tensors are staged to the GPU."""
    scores = data["token_level_scores"]
    dev, _ = _staging_device(scores, data["advantages"])
    B, L = scores.shape
    if data["responses"].shape[-1] != L:
        raise ValueError(f"responses has length {data['responses'].shape[-1]}, the token tensors {L}")
    amask = data["attention_mask"]
    Pw = amask.shape[-1] - L
    has_values = "values" in data.keys()
    sc, rw = _f32(scores, dev), _f32(data["token_level_rewards"], dev)
    adv, ret = _f32(data["advantages"], dev), _f32(data["returns"], dev)
    val = _f32(data["values"], dev) if has_values else None
    rm, rcode = _mask_arg(data["response_mask"], dev)
    am, acode = _mask_arg(amask, dev)
    for name, t in (("token_level_rewards", rw), ("advantages", adv), ("returns", ret), ("values", val),
                    ("response_mask", rm)):
        if t is not None and tuple(t.shape) != (B, L):
            raise ValueError(f"{name} has shape {tuple(t.shape)}, expected {(B, L)}")
    out = torch.empty(32, dtype=torch.float32, device=dev)
    nws = _lib.lib().siirl_data_metrics_workspace_bytes(B, L)
    ws = torch.empty(nws, dtype=torch.uint8, device=dev)
    with torch.cuda.device(dev):
        rc = _lib.lib().siirl_data_metrics(_lib.ptr(sc), _lib.ptr(rw), _lib.ptr(adv), _lib.ptr(ret), _lib.ptr(val),
                                           _lib.ptr(rm), rcode, _lib.ptr(am), acode, B, L, Pw, _lib.ptr(out),
                                           _lib.ptr(ws), nws, _lib.current_stream(dev))
    _lib.check(rc, "siirl_data_metrics")
    v = out.tolist()  # one copy, one sync
    metrics = {k: v[i] for i, k in enumerate(_KEYS) if has_values or k not in _VALUE_KEYS}
    try:
        import psutil

        metrics["perf/process_cpu_mem_used_gb"] = psutil.Process(os.getpid()).memory_info().rss / (1024 ** 3)
    except ImportError:  # the gauge is optional
        pass
    if "__num_turns__" in data.keys():
        turns = data["__num_turns__"]
        metrics["num_turns/min"] = turns.min()
        metrics["num_turns/max"] = turns.max()
        metrics["num_turns/mean"] = turns.mean()
    return metrics
