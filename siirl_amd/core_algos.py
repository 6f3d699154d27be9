"""Advantages, policy losses, aggregation and KL penalty with the reference's Python signatures.

Mirror of the in-scope part of ``siirl/dag_worker/core_algos.py``: the two registries (``:51-86``,
``:127-164``), ``compute_gae_advantage_return`` (``:229-276``), ``compute_grpo_outcome_advantage``
(``:279-348``), ``agg_loss`` (``:536-569``), ``compute_policy_loss_cpgd`` (``:572-629``),
``compute_policy_loss`` (``:631-707``), ``compute_policy_loss_vanilla`` (``:710-792``),
``compute_policy_loss_gspo`` (``:795-862``), ``compute_policy_loss_gpg`` (``:865-895``),
``compute_policy_loss_geo_mean`` (``:1074-1153``), ``compute_value_loss`` (``:1173-1212``), ``kl_penalty``
(``:1215-1276``), the KL controllers (``:167-226``), ``apply_kl_penalty`` (``:1358-1397``) and the GAE and GRPO
branches of ``compute_advantage`` (``:1400-1471``).  Same names, keyword arguments, return order and exception types; the arithmetic
runs in ``libsiirl_hip.so``.  ``actor_loss`` is an addition: the whole loss of one micro-batch
(policy loss, entropy bonus, KL loss, scaling, logged metrics) in one fused launch.

Tensors must be on the GPU, except in ``compute_grpo_outcome_advantage`` / ``apply_kl_penalty`` /
``compute_advantage``, which the reference runs on host tensors: host inputs are staged to the
current GPU and the results returned on the host.
"""

from __future__ import annotations

import ctypes as C
from enum import Enum
from typing import Any, Callable, Optional

import numpy as np
import torch

from . import _lib
from . import ops as _ops_module  # noqa: F401  (registers torch.ops.siirl_hip.*)

_OPS = torch.ops.siirl_hip
_actor_loss_op = _OPS.actor_loss.default  # one C++ autograd node: fused forward, elementwise backward, 13 scalars out
from . import torch_functional as siirl_F

__all__ = [
    "register_policy_loss", "get_policy_loss_fn", "register_adv_est", "get_adv_estimator_fn", "AdvantageEstimator",
    "AdaptiveKLController", "FixedKLController", "get_kl_controller", "compute_response_mask",
    "compute_gae_advantage_return", "compute_grpo_outcome_advantage", "compute_rewards", "agg_loss",
    "compute_policy_loss", "compute_policy_loss_vanilla", "compute_policy_loss_gspo", "compute_policy_loss_cpgd",
    "compute_policy_loss_gpg", "compute_policy_loss_geo_mean", "compute_policy_loss_clip_cov",
    "compute_policy_loss_kl_cov", "compute_cpgd_outcome_advantage", "compute_entropy_loss", "compute_value_loss", "kl_penalty",
    "kl_penalty_forward",
    "apply_kl_penalty", "compute_advantage", "actor_loss", "ActorLossOutput", "fused_actor_step",
    "FusedActorStepOutput", "agg_weights",
]

AGG_MODES = {"token-mean": 0, "seq-mean-token-sum": 1, "seq-mean-token-mean": 2, "seq-mean-token-sum-norm": 3}
KL_MODES = {"kl": 0, "k1": 0, "abs": 1, "mse": 2, "k2": 2, "low_var_kl": 3, "k3": 3}
LOSS_VANILLA, LOSS_GSPO, LOSS_CPGD, LOSS_GPG, LOSS_GEO_MEAN, LOSS_KL_COV, LOSS_CLIP_COV = range(7)
_LOSS_CODES = {"vanilla": LOSS_VANILLA, "gspo": LOSS_GSPO, "cpgd": LOSS_CPGD, "gpg": LOSS_GPG, "geo_mean": LOSS_GEO_MEAN,
               "kl_cov": LOSS_KL_COV, "clip_cov": LOSS_CLIP_COV}
# indices into the 16-float result block (SIIRL_OUT_* of include/siirl_hip.h)
(O_LOSS, O_PG, O_CLIPFRAC, O_PPOKL, O_CLIPLOWER, O_ENT, O_KL, O_RMEAN, O_RMIN, O_RMAX, O_MTOTAL, O_POLICY,
 O_DRIFT) = range(13)


class AdvantageEstimator(str, Enum):
    """reference ``siirl/execution/scheduler/enums.py:20-30``"""

    GAE = "gae"
    GRPO = "grpo"
    CPGD = "cpgd"
    GAE_MARFT = "gae_marft"


# ------------------------------------------------------------------------------------ registries

PolicyLossFn = Callable[..., tuple]
POLICY_LOSS_REGISTRY: dict[str, PolicyLossFn] = {}
ADV_ESTIMATOR_REGISTRY: dict[str, Any] = {}


def register_policy_loss(name: str):
    """Decorator: file a policy-loss function under ``name`` (reference ``core_algos.py:54-68``)."""

    def decorator(func):
        POLICY_LOSS_REGISTRY[name] = func
        return func

    return decorator


def get_policy_loss_fn(name):
    """reference ``core_algos.py:71-86``: unknown names raise ``ValueError`` listing what exists."""
    if name not in POLICY_LOSS_REGISTRY:
        raise ValueError(f"Unsupported loss mode: {name}. Supported modes are: {list(POLICY_LOSS_REGISTRY.keys())}")
    return POLICY_LOSS_REGISTRY[name]


def register_adv_est(name_or_enum):
    """reference ``core_algos.py:130-148``: a taken name may only be re-registered with the same function."""

    def decorator(fn):
        name = name_or_enum.value if isinstance(name_or_enum, Enum) else name_or_enum
        if name in ADV_ESTIMATOR_REGISTRY and ADV_ESTIMATOR_REGISTRY[name] != fn:
            raise ValueError(f"Adv estimator {name} has already been registered: {ADV_ESTIMATOR_REGISTRY[name]} vs {fn}")
        ADV_ESTIMATOR_REGISTRY[name] = fn
        return fn

    return decorator


def get_adv_estimator_fn(name_or_enum):
    """reference ``core_algos.py:151-164``"""
    name = name_or_enum.value if isinstance(name_or_enum, Enum) else name_or_enum
    if name not in ADV_ESTIMATOR_REGISTRY:
        raise ValueError(f"Unknown advantage estimator simply: {name}")
    return ADV_ESTIMATOR_REGISTRY[name]


# ------------------------------------------------------------------------------------ plumbing


def _f32(t: torch.Tensor, dev) -> torch.Tensor:
    return t.detach().to(device=dev, dtype=torch.float32).contiguous()


def _mask_arg(mask: torch.Tensor, dev):
    m = mask.detach().to(device=dev)
    if m.dtype not in (torch.bool, torch.uint8, torch.int32, torch.int64, torch.float32, torch.bfloat16, torch.float16):
        m = m.to(torch.float32)
    m = m.contiguous()
    return m, _lib.dtype_code(m.dtype)


def _as_2d(t: torch.Tensor):
    if t.dim() == 2:
        return t
    if t.dim() == 1:
        return t.unsqueeze(0)
    return t.reshape(-1, t.shape[-1])


def _gpu_of(*tensors):
    for t in tensors:
        if isinstance(t, torch.Tensor) and t.is_cuda:
            return t.device
    raise RuntimeError("siirl_amd: these ops run on the GPU only (no CPU fallback); move the tensors to the device")


def _staging_device(*tensors):
    """Device to compute on for the ops the reference runs on host tensors, and whether to copy back."""
    for t in tensors:
        if isinstance(t, torch.Tensor) and t.is_cuda:
            return t.device, False
    if not torch.cuda.is_available():
        raise RuntimeError("siirl_amd: no GPU visible; there is no CPU fallback")
    return torch.device("cuda", torch.cuda.current_device()), True


def _workspace(B, L, dev):
    n = _lib.lib().siirl_loss_workspace_bytes(B, L)
    return torch.empty(n, dtype=torch.uint8, device=dev), n


def _agg_code(loss_agg_mode: str) -> int:
    if loss_agg_mode not in AGG_MODES:
        raise ValueError(f"Invalid loss_agg_mode: {loss_agg_mode}")
    return AGG_MODES[loss_agg_mode]


# ------------------------------------------------------------------------------------ KL controllers


class AdaptiveKLController:
    """reference ``core_algos.py:167-189`` (https://arxiv.org/pdf/1909.08593.pdf)"""

    def __init__(self, init_kl_coef, target_kl, horizon):
        self.value = init_kl_coef
        self.target = target_kl
        self.horizon = horizon

    def update(self, current_kl, n_steps):
        proportional_error = np.clip(current_kl / self.target - 1, -0.2, 0.2)
        self.value *= 1 + proportional_error * n_steps / self.horizon


class FixedKLController:
    """reference ``core_algos.py:192-206``"""

    def __init__(self, kl_coef):
        self.value = kl_coef

    def update(self, current_kl, n_steps):
        pass


def get_kl_controller(kl_ctrl):
    """reference ``core_algos.py:209-226``"""
    if kl_ctrl.type == "fixed":
        return FixedKLController(kl_coef=kl_ctrl.kl_coef)
    if kl_ctrl.type == "adaptive":
        assert kl_ctrl.horizon > 0, f"horizon must be larger than 0. Got {kl_ctrl.horizon}"
        return AdaptiveKLController(init_kl_coef=kl_ctrl.kl_coef, target_kl=kl_ctrl.target_kl, horizon=kl_ctrl.horizon)
    raise NotImplementedError


# ------------------------------------------------------------------------------------ advantages


def compute_response_mask(data):
    """``attention_mask[:, -response_length:]``, 3-D embodied responses flattened (reference
    ``core_algos.py:89-125``).  Pure indexing."""
    responses, attention_mask = data["responses"], data["attention_mask"]
    if responses.ndim == 3:
        if attention_mask.ndim == 3:
            return attention_mask[:, :, -responses.size(2):].reshape(responses.size(0), -1)
        return attention_mask[:, -(responses.size(1) * responses.size(2)):]
    if responses.ndim == 2:
        return attention_mask[:, -responses.size(1):]
    raise ValueError(f"Unexpected responses shape: {responses.shape}, ndim={responses.ndim}")


def _uid_tensor(index, n, dev) -> torch.Tensor:
    """int64 group codes: integer arrays as they are; anything else goes through ``int()`` per entry as in the
    reference (``core_algos.py:326``: numeric strings, floats, integers beyond 64 bits) and is numbered in order of
    first appearance -- only equality of the keys matters."""
    if isinstance(index, torch.Tensor):
        out = index.detach().reshape(-1).to(device=dev, dtype=torch.int64)
    else:
        arr = np.asarray(index)
        if arr.dtype.kind in "iu" and (arr.dtype.kind == "i" or arr.size == 0 or int(arr.max()) < 2 ** 63):
            arr = arr.reshape(-1).astype(np.int64)
        else:
            seq = list(index) if isinstance(index, (list, tuple)) else list(arr.reshape(-1))
            codes: dict = {}
            arr = np.fromiter((codes.setdefault(int(v), len(codes)) for v in seq), dtype=np.int64, count=len(seq))
        out = torch.from_numpy(np.ascontiguousarray(arr)).to(dev)
    if out.numel() != n:
        raise ValueError(f"index has {out.numel()} entries for a batch of {n}")
    return out.contiguous()


_GAE_ORDERS = {"exact": 0, "chunked": 1}
_gae_order = "exact"


def set_gae_scan_order(order: str) -> None:
    """``"exact"`` (default): each row is scanned in one sequential pass in the reference's float32 operation
    order, ``returns`` is bit-identical to the reference's.  ``"chunked"``: rows of 1024 tokens or more are cut into
    up to 16 chunks that are scanned in parallel and stitched through their composed affine maps -- a dependent
    chain 16 times shorter, results equal to float32 accuracy rather than bit for bit."""
    global _gae_order
    if order not in _GAE_ORDERS:
        raise ValueError(f"unknown GAE scan order {order!r}; choose from {sorted(_GAE_ORDERS)}")
    _gae_order = order


@register_adv_est(AdvantageEstimator.GAE)
def compute_gae_advantage_return(token_level_rewards: torch.Tensor, values: torch.Tensor, response_mask: torch.Tensor,
                                 gamma, lam):
    """Generalised advantage estimation with whitened advantages (reference ``core_algos.py:229-276``).
    Returns ``(advantages, returns)``, ``[B, L]`` fp32; ``returns`` is the un-whitened advantage plus the
    values.  Raises the reference's ``ValueError`` when the mask selects fewer than two tokens.  The order of
    evaluation is chosen by ``set_gae_scan_order``."""
    dev, back = _staging_device(token_level_rewards, values, response_mask)
    B, L = token_level_rewards.shape
    r = _f32(token_level_rewards, dev)
    v = _f32(values, dev)
    m, mcode = _mask_arg(response_mask, dev)
    if tuple(v.shape) != (B, L) or tuple(m.shape) != (B, L):
        raise ValueError(f"values {tuple(v.shape)} and response_mask {tuple(m.shape)} must have shape {(B, L)}")
    adv = torch.empty(B, L, dtype=torch.float32, device=dev)
    ret = torch.empty(B, L, dtype=torch.float32, device=dev)
    stats = torch.empty(3, dtype=torch.float32, device=dev)
    nws = _lib.lib().siirl_gae_workspace_bytes(B, L)
    ws = torch.empty(nws, dtype=torch.uint8, device=dev)
    with torch.cuda.device(dev):
        rc = _lib.lib().siirl_gae_advantage_return(_lib.ptr(r), _lib.ptr(v), _lib.ptr(m), mcode, B, L, float(gamma),
                                                   float(lam), _lib.ptr(adv), _lib.ptr(ret), _lib.ptr(stats),
                                                   _lib.ptr(ws), nws, _GAE_ORDERS[_gae_order],
                                                   _lib.current_stream(dev))
    _lib.check(rc, "siirl_gae_advantage_return")
    siirl_F._check_whiten_count(float(stats[2]))
    if back:
        adv, ret = adv.to(token_level_rewards.device), ret.to(token_level_rewards.device)
    return adv, ret


@register_adv_est(AdvantageEstimator.GRPO)
def compute_grpo_outcome_advantage(token_level_rewards: torch.Tensor, response_mask: torch.Tensor, index,
                                   epsilon: float = 1e-6, norm_adv_by_std_in_grpo: bool = True, config=None):
    """Group-normalised outcome advantage (reference ``core_algos.py:279-348``): the sequence score is
    normalised by the mean and unbiased std of its ``index`` group (a group of one: mean 0, std 1),
    broadcast over the tokens and masked.  Returns the same ``[B, L]`` fp32 tensor twice."""
    dev, back = _staging_device(token_level_rewards, response_mask)
    B, L = token_level_rewards.shape
    r = _f32(token_level_rewards, dev)
    m, mcode = _mask_arg(response_mask, dev)
    uid = _uid_tensor(index, B, dev)
    adv = _OPS.grpo_advantage(r, m, uid, float(epsilon), bool(norm_adv_by_std_in_grpo))
    if back:
        adv = adv.to(token_level_rewards.device)
    return adv, adv


def _group_codes(index, n, dev) -> torch.Tensor:
    """int64 group codes for keys that are compared as they are (``core_algos.py:495``: ``id2score[index[i]]``):
    integer tensors / arrays unchanged, anything else numbered in order of first appearance."""
    if isinstance(index, torch.Tensor) and not index.dtype.is_floating_point:
        return _uid_tensor(index, n, dev)
    arr = np.asarray(index)
    if arr.dtype.kind in "iu":
        return _uid_tensor(arr, n, dev)
    seq = [v.item() if hasattr(v, "item") else v for v in (index if isinstance(index, (list, tuple)) else arr.reshape(-1))]
    codes: dict = {}
    return _uid_tensor(np.fromiter((codes.setdefault(v, len(codes)) for v in seq), dtype=np.int64, count=len(seq)), n, dev)


def compute_cpgd_outcome_advantage(token_level_rewards: torch.Tensor, response_mask: torch.Tensor, index,
                                   epsilon: float = 1e-6, weight_factor_in_cpgd: str = "STD_weight"):
    """CPGD's outcome advantage (reference ``core_algos.py:461-517``; the reference's dispatcher cannot reach it,
    ``:1475-1480``, callers use it directly).  Group statistics as in the GRPO estimator (a group of one: mean 0,
    std 1); ``STD_weight``: ``(s - mean) / (std + eps)``; ``naive``: ``s - mean``; ``clip_filter_like_weight``:
    ``(s - mean) * min(B / #groups whose std is not zero, 3)``.  Returns the same ``[B, L]`` fp32 tensor twice."""
    if weight_factor_in_cpgd not in ("STD_weight", "clip_filter_like_weight", "naive"):
        raise NotImplementedError
    dev, back = _staging_device(token_level_rewards, response_mask)
    B, L = token_level_rewards.shape
    r = _f32(token_level_rewards, dev)
    m, mcode = _mask_arg(response_mask, dev)
    uid = _group_codes(index, B, dev)
    adv = _OPS.grpo_advantage(r, m, uid, float(epsilon), weight_factor_in_cpgd == "STD_weight")
    if weight_factor_in_cpgd == "clip_filter_like_weight" and B > 0:
        # a group is live when its scores are not all equal (or it has one member: std is set to 1); each member of
        # a live group of n contributes 1 / n to the count
        # (in float64 the mean of equal float32 scores is exact, so "all equal" and "std == 0" coincide as they do
        # for torch.std)
        keep, gsz = _OPS.group_keep_mask(r.sum(dim=-1).to(torch.float64), uid)
        live = torch.round((keep.to(torch.float64) / gsz.to(torch.float64)).sum())
        factor = torch.clamp((B / live).to(torch.float32), max=3.0)  # no live group: inf, clamped
        adv = adv * factor
    if back:
        adv = adv.to(token_level_rewards.device)
    return adv, adv


_MARFT_INT_MASKS = (torch.bool, torch.uint8, torch.int32, torch.int64)


def marft_gae_unwhitened(rewards, values, masks, chains, gamma, lam, out_dtype=None):
    """The token walk of the reference's multi-agent GAE (``core_algos.py:400-448``) for explicit operands: lists
    over the agents (the batch's own response last) of ``[B, L_a]`` tensors, ``chains`` = ``(first_row, n_rows)`` per
    request.  Returns ``(advantages, returns)``, lists of tensors of ``out_dtype`` (default: each mask's dtype, what
    the reference's ``zeros_like(response_mask)`` gives: integer masks keep the integer part of every result), on the
    device of the inputs (host inputs are staged to the GPU and the results copied back)."""
    adv, ret, _, back = _marft_walk(rewards, values, masks, chains, gamma, lam, out_dtype)
    if back:
        adv = [a.to(m.device) for a, m in zip(adv, masks)]
        ret = [a.to(m.device) for a, m in zip(ret, masks)]
    return adv, ret


def _marft_walk(rewards, values, masks, chains, gamma, lam, out_dtype=None):
    """``marft_gae_unwhitened`` with the results left on the GPU: ``(advantages, returns, masks on the GPU, whether
    the inputs were on the host)``."""
    n_agents = len(masks)
    if not (len(rewards) == len(values) == n_agents) or n_agents < 1:
        raise ValueError("rewards, values and masks must list the same agents")
    if n_agents > _lib.MARFT_MAX_AGENTS:
        raise NotImplementedError(f"siirl_amd: at most {_lib.MARFT_MAX_AGENTS} agents, got {n_agents}")
    dev, back = _staging_device(*rewards, *values, *masks)
    B = masks[0].shape[0]
    mdt = masks[0].dtype
    for r, v, m in zip(rewards, values, masks):
        if m.dim() != 2 or m.shape[0] != B or r.shape != m.shape or v.shape != m.shape:
            raise ValueError(f"every agent needs [B, L] rewards, values and mask with B = {B}; got {tuple(r.shape)}, "
                             f"{tuple(v.shape)}, {tuple(m.shape)}")
        if m.shape[1] < 1:
            raise IndexError("index 0 is out of bounds for dimension 1 with size 0")
        if m.dtype != mdt:
            raise NotImplementedError("siirl_amd: the agents' masks must share one dtype")
    chains = [(int(s), int(n)) for s, n in chains]
    walked = [c for c in chains if c[1] > 0]
    if walked and mdt not in _MARFT_INT_MASKS:
        # the reference's range(mask row sum) (:410-412)
        raise TypeError("only integer tensors of a single element can be converted to an index")
    _check_marft_chains(walked, B)
    out_dtypes = [out_dtype or m.dtype for m in masks]
    if any(d != out_dtypes[0] for d in out_dtypes):
        raise NotImplementedError("siirl_amd: the agents' outputs must share one dtype")
    if out_dtypes[0].is_floating_point:
        mode = _lib.MARFT_STORE_FLOAT
    else:
        mode = _lib.MARFT_STORE_NONZERO if out_dtypes[0] == torch.bool else _lib.MARFT_STORE_TRUNCATED
    r32 = [_f32(t, dev) for t in rewards]
    v32 = [_f32(t, dev) for t in values]
    m_dev = [m.detach().to(dev).contiguous() for m in masks]
    if mdt not in _MARFT_INT_MASKS:  # no request is walked: the masks are never read
        m_dev = [torch.zeros(m.shape, dtype=torch.int64, device=dev) for m in masks]
    mcode = _lib.dtype_code(m_dev[0].dtype)
    adv = [torch.empty(m.shape, dtype=torch.float32, device=dev) for m in masks]
    ret = [torch.empty(m.shape, dtype=torch.float32, device=dev) for m in masks]
    status = torch.empty(1, dtype=torch.int32, device=dev)
    starts = torch.tensor([c[0] for c in walked], dtype=torch.int64).to(dev)
    lens = torch.tensor([c[1] for c in walked], dtype=torch.int64).to(dev)
    ptrs = lambda ts: (C.c_void_p * n_agents)(*[t.data_ptr() for t in ts])  # noqa: E731
    widths = (C.c_int64 * n_agents)(*[m.shape[1] for m in masks])
    # gamma * lam as the reference forms it: the product of two Python floats, rounded to float32 once; of two
    # tensors, their float32 product
    if isinstance(gamma, torch.Tensor) or isinstance(lam, torch.Tensor):
        g32 = float(torch.as_tensor(gamma, dtype=torch.float32))
        gl32 = float(torch.as_tensor(gamma, dtype=torch.float32) * torch.as_tensor(lam, dtype=torch.float32))
    else:
        g32, gl32 = float(gamma), float(gamma) * float(lam)
    with torch.cuda.device(dev):
        rc = _lib.lib().siirl_marft_gae(ptrs(r32), ptrs(v32), ptrs(m_dev), mcode, widths, n_agents, B, _lib.ptr(starts),
                                        _lib.ptr(lens), len(walked), g32, gl32, mode, ptrs(adv), ptrs(ret),
                                        _lib.ptr(status), _lib.current_stream(dev))
    _lib.check(rc, "siirl_marft_gae")
    if int(status.item()) == 1:
        raise IndexError("a response_mask row sums to more than its length: the token walk would leave the row")
    adv = [a.to(d) for a, d in zip(adv, out_dtypes)]
    ret = [a.to(d) for a, d in zip(ret, out_dtypes)]
    return adv, ret, [m.detach().to(dev) for m in masks], back


def _check_marft_chains(walked, B):
    """The requests' row ranges ``(first row, trajectory length)`` must lie inside the batch (the reference's own
    ``IndexError``) and must not overlap: the reference walks requests one after the other, so where a ``traj_len``
    runs into the next request's rows the later walk overwrites the earlier one's results and reads its values
    (``core_algos.py:400-448``); here every request is walked by a wave of its own at the same time, which has no
    such order -- refused instead of answered differently from run to run."""
    for first, n in walked:
        if first < 0 or first + n > B:
            raise IndexError(f"index {first + n - 1} is out of bounds for dimension 0 with size {B}")
    ordered = sorted(walked)
    for (a, na), (b, _) in zip(ordered, ordered[1:]):
        if a + na > b:
            raise NotImplementedError(f"siirl_amd: the request that starts at row {a} with traj_len {na} runs into the "
                                      f"request that starts at row {b}; overlapping requests are walked one after "
                                      "the other by the reference and are not supported here")


def compute_marft_gae_advantage_return(data, pre_agent_group_ids, gamma, lam):
    """Multi-agent GAE over reversed trajectories (reference ``core_algos.py:351-458``).  ``data.batch`` holds
    ``agent_group_<id>_token_level_rewards`` / ``_values`` / ``_response_mask`` for every id of
    ``pre_agent_group_ids`` plus the unprefixed three of the last agent; ``data.non_tensor_batch`` holds
    ``request_id`` (the first row of each distinct id starts a request) and ``traj_len`` (read at that row).
    Writes ``advantages`` / ``returns`` and returns ``None``.  Kept from the reference, because callers see them:
    the id list grows by one id per call (``:395``); the ids index the agent list, so they must be ``0 .. n - 1``;
    every agent's advantages are whitened over its own mask (``:451``, with ``masked_var``'s two ``ValueError``s),
    but the results of all the earlier agents go to the keys of the LAST given id, each overwriting the one
    before (``:452-454``); outputs before whitening take the mask's dtype (``:386-392``), so with the integer masks
    the token walk requires every stored advantage and return is truncated to its integer part."""
    batch, extra = data.batch, data.non_tensor_batch
    prefix = "agent_group_"
    names = [prefix + str(g) + "_" for g in pre_agent_group_ids] + [""]
    rewards = [batch[n + "token_level_rewards"] for n in names]
    values = [batch[n + "values"] for n in names]
    masks = [batch[n + "response_mask"] for n in names]
    last_given = pre_agent_group_ids[-1]  # IndexError for an empty list, as in the reference
    pre_agent_group_ids.append(last_given + 1)
    if list(pre_agent_group_ids) != list(range(len(pre_agent_group_ids))):
        raise NotImplementedError("siirl_amd: agent group ids must be 0 .. n - 1 (the reference indexes its agent list "
                                  f"with them), got {pre_agent_group_ids[:-1]}")
    seen, chains = set(), []
    for row, rid in enumerate(extra["request_id"]):
        if rid not in seen:
            seen.add(rid)
            chains.append((row, int(extra["traj_len"][row])))
    adv, ret, masks_dev, back = _marft_walk(rewards, values, masks, chains, gamma, lam)
    for g, (a, r, m, m_src) in enumerate(zip(adv, ret, masks_dev, masks)):
        white = siirl_F.masked_whiten(a, m)
        if back:
            white, r = white.to(m_src.device), r.to(m_src.device)
        if g != len(adv) - 1:
            _td_set(data, prefix + str(last_given) + "_advantages", white)
            _td_set(data, prefix + str(last_given) + "_returns", r)
        else:
            _td_set(data, "advantages", white)
            _td_set(data, "returns", r)


def compute_rewards(token_level_scores, old_log_prob, ref_log_prob, kl_ratio):
    """reference ``core_algos.py:520-533``: ``scores - (old - ref) * kl_ratio`` (k1 estimator, no mask)."""
    dev = _gpu_of(token_level_scores, old_log_prob, ref_log_prob)
    ones = torch.ones(token_level_scores.shape, dtype=torch.uint8, device=dev)
    rewards, _ = _kl_in_reward(token_level_scores, old_log_prob, ref_log_prob, ones, "kl", float(kl_ratio), dev)
    return rewards


def _kl_in_reward(scores, old, ref, mask, kl_type, beta, dev):
    if kl_type not in KL_MODES:
        raise NotImplementedError
    s2 = _as_2d(_f32(scores, dev))
    B, L = s2.shape
    o2, r2 = _as_2d(_f32(old, dev)), _as_2d(_f32(ref, dev))
    m, mcode = _mask_arg(_as_2d(mask), dev)
    rewards = torch.empty_like(s2)
    row_kl = torch.empty(B, dtype=torch.float32, device=dev)
    cur = torch.empty(1, dtype=torch.float32, device=dev)
    with torch.cuda.device(dev):
        rc = _lib.lib().siirl_kl_in_reward(_lib.ptr(s2), _lib.ptr(o2), _lib.ptr(r2), _lib.ptr(m), mcode, B, L,
                                           KL_MODES[kl_type], float(beta), _lib.ptr(rewards), _lib.ptr(row_kl),
                                           _lib.ptr(cur), _lib.current_stream(dev))
    _lib.check(rc, "siirl_kl_in_reward")
    return rewards.reshape(scores.shape), cur


def _resample_rows(t: torch.Tensor, idx: torch.Tensor) -> torch.Tensor:
    """``t[idx]`` along the first axis (GPU tensors through the row gather of the un-padding path)."""
    from .dapo_filter import _select_rows

    return _select_rows(t, idx)


def compute_pf_ppo_reweight_data(data, reweight_method: str = "pow", weight_pow: float = 2.0):
    """PF-PPO resampling of a batch by its scores (reference ``core_algos.py:1279-1355``): per-sequence score =
    ``token_level_scores.sum(-1)``; weight ``|score| ** weight_pow`` ("pow"), 1 at the batch's maximum and minimum
    score and 0 elsewhere ("max_min"), or 0.4 at the maximum and 0.1 elsewhere ("max_random"), ``+ 1e-8``;
    ``batch_size`` indices are drawn with replacement by ``torch.multinomial`` on the scores' device (the reference's
    batch lives on the host, so the same seed gives the same draw) and every tensor of ``data.batch``, every array or
    list of ``data.non_tensor_batch`` and every ``batch_size``-long list of ``data.meta_info`` is indexed with them.
    Returns a deep copy of ``data`` holding the resampled parts; ``data`` itself is left alone."""
    from copy import deepcopy

    with torch.no_grad():
        scores = data.batch["token_level_scores"].sum(dim=-1)
        if reweight_method == "pow":
            weights = torch.pow(torch.abs(scores), weight_pow)
        elif reweight_method == "max_min":
            weights = torch.where((scores == torch.max(scores)) | (scores == torch.min(scores)), 1.0, 0.0)
        elif reweight_method == "max_random":
            weights = torch.where(scores == torch.max(scores), 0.4, 0.1)
        else:
            raise ValueError(f"Unsupported reweight_method: {reweight_method}")
        weights = torch.clamp(weights + 1e-8, min=1e-8)
        batch_size = scores.shape[0]
        picks = torch.multinomial(weights, batch_size, replacement=True)
        resampled = {key: _resample_rows(t, picks) for key, t in data.batch.items()}
    picks_np = picks.cpu().numpy()
    extra = {}
    for key, arr in data.non_tensor_batch.items():
        extra[key] = arr[picks_np] if isinstance(arr, np.ndarray) else [arr[i] for i in picks_np]
    meta = {}
    for key, val in data.meta_info.items():
        meta[key] = [val[i] for i in picks_np] if isinstance(val, list) and len(val) == batch_size else val
    out = deepcopy(data)
    out.batch = type(data.batch)(resampled)
    if hasattr(data.batch, "batch_size"):
        out.batch.batch_size = data.batch.batch_size
    out.non_tensor_batch = extra
    out.meta_info = meta
    return out


def _td_set(data, key, value):
    target = data.batch if hasattr(data, "batch") and not callable(getattr(data, "batch")) else data
    target[key] = value


def apply_kl_penalty(data, kl_ctrl, kl_penalty="kl", multi_turn=False):
    """KL-in-reward (reference ``core_algos.py:1358-1397``): ``token_level_rewards = token_level_scores -
    beta * kl_penalty(old_log_probs, ref_log_prob) * response_mask``; the controller is then updated with
    the batch mean of the per-sequence masked mean.  ``data`` is any mapping of tensors."""
    scores = data["token_level_scores"]
    dev, back = _staging_device(scores, data["old_log_probs"])
    beta = kl_ctrl.value
    rewards, cur = _kl_in_reward(scores, data["old_log_probs"], data["ref_log_prob"], data["response_mask"],
                                 kl_penalty, beta, dev)
    current_kl = cur.item()
    batch_size = data.batch_size[0] if hasattr(data, "batch_size") else scores.shape[0]
    kl_ctrl.update(current_kl=current_kl, n_steps=batch_size)
    _td_set(data, "token_level_rewards", rewards.to(scores.device) if back else rewards)
    return data, {"actor/reward_kl_penalty": current_kl, "actor/reward_kl_penalty_coeff": beta}


def compute_advantage(data, adv_estimator, gamma=1.0, lam=1.0, norm_adv_by_std_in_grpo=True,
                      weight_factor_in_cpgd="STD_weight", **kwargs):
    """Dispatcher (reference ``core_algos.py:1400-1492``).  The GAE (``:1424-1439``, with the PF-PPO resampling
    of ``use_pf_ppo``, ``:1434-1439``), GRPO (``:1440-1471``) and multi-agent GAE (``:1483-1489``, ``data`` then needs
    ``.batch`` and ``.non_tensor_batch``) branches are built; the CPGD branch fails with the reference's own
    ``TypeError`` (it hands ``compute_grpo_outcome_advantage`` a keyword it does not take, ``:1475-1480``);
    ``compute_cpgd_outcome_advantage`` is there to be called directly."""
    if "response_mask" not in data.keys():
        _td_set(data, "response_mask", compute_response_mask(data))
    est = adv_estimator.value if isinstance(adv_estimator, Enum) else adv_estimator
    if est == "gae":
        advantages, returns = compute_gae_advantage_return(
            token_level_rewards=data["token_level_rewards"], values=data["values"],
            response_mask=data["response_mask"], gamma=gamma, lam=lam)
        data["advantages"] = advantages
        data["returns"] = returns
        if kwargs.get("use_pf_ppo", False):
            data = compute_pf_ppo_reweight_data(data, kwargs.get("pf_ppo_reweight_method", "pow"),
                                                kwargs.get("pf_ppo_weight_pow", 2.0))
        return data
    if est == "grpo":
        if "finish_step" in data.keys() and data["responses"].ndim == 3:
            responses = data["responses"]
            length = responses.size(1) * responses.size(2)
            finish = data["finish_step"] * responses.size(2)
            steps = torch.arange(length, device=responses.device).unsqueeze(0).expand(responses.size(0), -1)
            calc_mask = steps < finish.unsqueeze(1)
        else:
            calc_mask = data["response_mask"]
        advantages, returns = compute_grpo_outcome_advantage(
            token_level_rewards=data["token_level_rewards"], response_mask=calc_mask, index=data["uid"],
            norm_adv_by_std_in_grpo=norm_adv_by_std_in_grpo)
        data["advantages"] = advantages
        data["returns"] = returns
        data["response_mask"] = calc_mask
        return data
    if est == "cpgd":
        compute_grpo_outcome_advantage(token_level_rewards=data["token_level_rewards"],
                                       response_mask=data["response_mask"], index=data["uid"],
                                       weight_factor_in_cpgd=weight_factor_in_cpgd)
    if est == "gae_marft":
        compute_marft_gae_advantage_return(data, pre_agent_group_ids=kwargs["agent_group_ids"], gamma=gamma, lam=lam)
        return data
    raise NotImplementedError


# ------------------------------------------------------------------------------------ aggregation


def agg_loss(loss_mat: torch.Tensor, loss_mask: torch.Tensor, loss_agg_mode: str):
    """Aggregate a ``[B, L]`` loss into a scalar (reference ``core_algos.py:536-569``); unknown modes raise
    ``ValueError``.  ``seq-mean-token-mean`` of a row with an empty mask is NaN, as in the reference."""
    code = _agg_code(loss_agg_mode)
    _gpu_of(loss_mat)
    return _OPS.agg_loss(loss_mat, loss_mask, code)


def compute_entropy_loss(logits: torch.Tensor, response_mask: torch.Tensor, loss_agg_mode: str = "token-mean"):
    """Aggregated categorical entropy of ``logits [B, L, V]`` (reference ``core_algos.py:1156-1170``, kept there
    for backward compatibility): ``agg_loss(entropy_from_logits(logits), response_mask, loss_agg_mode)``."""
    return agg_loss(loss_mat=siirl_F.entropy_from_logits(logits), loss_mask=response_mask,
                    loss_agg_mode=loss_agg_mode)


# ------------------------------------------------------------------------------------ policy loss


def _clip_params(config):
    clip_ratio = config.clip_ratio
    lo = config.clip_ratio_low if getattr(config, "clip_ratio_low", None) is not None else clip_ratio
    hi = config.clip_ratio_high if getattr(config, "clip_ratio_high", None) is not None else clip_ratio
    return float(lo), float(hi)


def _policy_only(loss_mode, old_log_prob, log_prob, advantages, response_mask, agg_code, lo, hi, c, dclamp,
                 rollout_is_weights):
    _gpu_of(log_prob)
    outs = _actor_loss_op(log_prob, None, old_log_prob, advantages, response_mask, rollout_is_weights, None, loss_mode,
                          lo, hi, float(c), float(dclamp), agg_code, 0.0, 0, False, 0.0, 0.0, 1.0, True)
    return outs[O_PG], outs[O_CLIPFRAC], outs[O_PPOKL], outs[O_CLIPLOWER]


@register_policy_loss("vanilla")
def compute_policy_loss_vanilla(old_log_prob: torch.Tensor, log_prob: torch.Tensor, advantages: torch.Tensor,
                                response_mask: torch.Tensor, loss_agg_mode: str = "token-mean", config=None,
                                rollout_is_weights: Optional[torch.Tensor] = None):
    """Clipped PPO / GRPO / DAPO objective with dual clip (reference ``core_algos.py:710-792``).
    ``config`` is any object with ``clip_ratio``, ``clip_ratio_low``, ``clip_ratio_high``, ``clip_ratio_c``.
    Returns ``(pg_loss, pg_clipfrac, ppo_kl, pg_clipfrac_lower)`` as 0-d device tensors; only ``pg_loss``
    carries a gradient (to ``log_prob``)."""
    assert config is not None
    assert type(config).__name__ != "AlgorithmArguments"  # reference :744
    lo, hi = _clip_params(config)
    clip_ratio_c = config.clip_ratio_c
    assert clip_ratio_c > 1.0, (
        "The lower bound of the clip_ratio_c for dual-clip PPO should be greater than 1.0,"
        + f" but get the value: {clip_ratio_c}."
    )
    return _policy_only(LOSS_VANILLA, old_log_prob, log_prob, advantages, response_mask, _agg_code(loss_agg_mode),
                        lo, hi, clip_ratio_c, 20.0, rollout_is_weights)


@register_policy_loss("gspo")
def compute_policy_loss_gspo(old_log_prob: torch.Tensor, log_prob: torch.Tensor, advantages: torch.Tensor,
                             response_mask: torch.Tensor, loss_agg_mode: str = "seq-mean-token-mean", config=None,
                             rollout_is_weights: Optional[torch.Tensor] = None):
    """GSPO (reference ``core_algos.py:795-862``): sequence-level importance ratio, token-level gradient,
    always aggregated ``seq-mean-token-mean`` whatever ``loss_agg_mode`` says (``:854``);
    ``pg_clipfrac_lower`` is zero."""
    assert config is not None
    assert all(hasattr(config, k) for k in ("clip_ratio", "clip_ratio_low", "clip_ratio_high"))  # reference :824
    lo, hi = _clip_params(config)
    return _policy_only(LOSS_GSPO, old_log_prob, log_prob, advantages, response_mask,
                        AGG_MODES["seq-mean-token-mean"], lo, hi, 3.0, 20.0, rollout_is_weights)


def _check_cpgd_bounds(lo, hi):
    import math

    math.log(1 + hi), math.log(1 - lo)  # raises the reference's ValueError ("math domain error") for eps >= 1


@register_policy_loss("cpgd")
def compute_policy_loss_cpgd(old_log_prob: torch.Tensor, log_prob: torch.Tensor, advantages: torch.Tensor,
                             response_mask: torch.Tensor, loss_agg_mode: str = "token-mean", config=None,
                             rollout_is_weights: Optional[torch.Tensor] = None):
    """CPGD (reference ``core_algos.py:572-629``): the log-probability is clipped at ``old + log(1 + eps_high)``
    for positive advantages and at ``old + log(1 - eps_low)`` otherwise; ``rollout_is_weights`` is accepted
    and not used, as in the reference."""
    assert config is not None, "Config must be provided for CPGD loss"
    lo, hi = _clip_params(config)
    c = config.clip_ratio_c if getattr(config, "clip_ratio_c", None) is not None else 3.0
    assert c > 1.0, f"clip_ratio_c ({c}) must be > 1.0"
    _check_cpgd_bounds(lo, hi)
    return _policy_only(LOSS_CPGD, old_log_prob, log_prob, advantages, response_mask, _agg_code(loss_agg_mode),
                        lo, hi, c, 20.0, None)


@register_policy_loss("gpg")
def compute_policy_loss_gpg(old_log_prob: torch.Tensor, log_prob: torch.Tensor, advantages: torch.Tensor,
                            response_mask: torch.Tensor, loss_agg_mode: str = "token-mean", config=None,
                            rollout_is_weights: Optional[torch.Tensor] = None):
    """GPG (reference ``core_algos.py:865-895``): ``agg_loss(-log_prob * advantages [* weights])``.  The three
    metrics are zeros -- on the device here, where the reference returns host scalars (``:895``)."""
    old = log_prob.detach() if old_log_prob is None else old_log_prob
    return _policy_only(LOSS_GPG, old, log_prob, advantages, response_mask, _agg_code(loss_agg_mode),
                        0.2, 0.2, 3.0, 20.0, rollout_is_weights)


@register_policy_loss("geo_mean")
def compute_policy_loss_geo_mean(old_log_prob: torch.Tensor, log_prob: torch.Tensor, advantages: torch.Tensor,
                                 response_mask: torch.Tensor, loss_agg_mode: str = "token-mean", config=None,
                                 rollout_is_weights: Optional[torch.Tensor] = None):
    """GMPO (reference ``core_algos.py:1074-1153``): per sequence ``-mean(A) * exp(mean clipped log-ratio)``, the
    log-ratio clipped to ``[-eps_low, eps_high]`` on the side that the advantage's sign makes optimistic;
    plain mean over sequences, ``loss_agg_mode`` is not used.  The reference additionally asserts that
    ``config`` is not its ``ActorArguments`` class (``:1104``), which every stock actor violates; that check on
    the reference's own type has no counterpart here."""
    assert config is not None
    lo, hi = _clip_params(config)
    _agg_code(loss_agg_mode)
    return _policy_only(LOSS_GEO_MEAN, old_log_prob, log_prob, advantages, response_mask,
                        AGG_MODES["token-mean"], lo, hi, 3.0, 20.0, rollout_is_weights)


def _cov_operands(old_log_prob, log_prob, advantages, response_mask):
    dev = _gpu_of(log_prob)
    lp = _as_2d(_f32(log_prob, dev))
    old = None if old_log_prob is None else _as_2d(_f32(old_log_prob, dev))
    adv = _as_2d(_f32(advantages, dev))
    m, _ = _mask_arg(_as_2d(response_mask), dev)
    if m.shape != lp.shape:
        m = m.expand(lp.shape).contiguous()
    return dev, old, lp, adv, m


def _kl_cov_weights(log_prob, advantages, response_mask, kl_cov_ratio: float, ppo_kl_coef: float) -> torch.Tensor:
    """``[B, L]`` fp32: ``ppo_kl_coef`` on the ``max(1, int(n * kl_cov_ratio))`` tokens of largest covariance among
    the ``n`` tokens with a positive mask (reference ``core_algos.py:1047-1060``), 0 elsewhere.  One host sync (the
    count ``n``), as the reference's ``len(all_valid_adv)``."""
    dev, _, lp, adv, m = _cov_operands(None, log_prob, advantages, response_mask)
    cov, stats = _OPS.cov_scores(None, lp, adv, m, LOSS_KL_COV, 0.0, 0.0)
    st = stats.tolist()  # one host sync, as the reference's len(all_valid_adv)
    n = int(st[0] + st[4])  # exact beyond 2^24 tokens: the count and what float32 rounding took from it
    k = 0
    if min(kl_cov_ratio, n) != 0:  # reference :1052-1054
        k = max(1, int(n * kl_cov_ratio))
        if k > n:
            raise RuntimeError(f"kl_cov_ratio {kl_cov_ratio} selects {k} of {n} valid tokens")  # torch.topk: k out of range
    return _OPS.topk_mark(cov, k, float(ppo_kl_coef))


def _clip_cov_dropped(old_log_prob, log_prob, advantages, response_mask, lo, hi, clip_cov_ratio, lb, ub) -> torch.Tensor:
    """``[B, L]`` fp32, 1 on the tokens Clip-Cov drops (reference ``core_algos.py:963-983``): candidates are the
    unmasked tokens the PPO clip leaves alone with ``lb < cov < ub``, in row-major order; of them
    ``max(int(ratio * sum(mask)), 1)`` are drawn with one ``torch.randperm`` on the host's global generator, the
    reference's own draw.  Two host syncs (mask sum, candidate count), as there."""
    dev, old, lp, adv, m = _cov_operands(old_log_prob, log_prob, advantages, response_mask)
    cov, stats = _OPS.cov_scores(old, lp, adv, m, LOSS_CLIP_COV, lo, hi)
    st = stats.tolist()
    clip_num = max(int(clip_cov_ratio * (st[1] + st[5])), 1)  # the mask sum, exact in double
    cand = _OPS.range_indices(cov, lb, ub)  # flat indices, ascending = row-major order; the second host sync
    aux = torch.zeros_like(cov)
    if len(cand) > 0:
        perm = torch.randperm(len(cand))
        aux.reshape(-1)[cand[perm[: min(clip_num, len(cand))].to(dev)]] = 1.0
    return aux


def _policy_loss_cfg(config):
    assert config is not None
    pl = getattr(config, "policy_loss", None)
    assert pl is not None
    return pl


def _clip_cov_params(config):
    pl = _policy_loss_cfg(config)
    ratio = pl.clip_cov_ratio if getattr(pl, "clip_cov_ratio", None) is not None else 0.0002
    ub = pl.clip_cov_ub if getattr(pl, "clip_cov_ub", None) is not None else 5.0
    lb = pl.clip_cov_lb if getattr(pl, "clip_cov_lb", None) is not None else 1.0
    assert ratio > 0, "clip_ratio should be larger than 0."
    return float(ratio), float(lb), float(ub)


def _kl_cov_params(config):
    pl = _policy_loss_cfg(config)
    ratio = pl.kl_cov_ratio if getattr(pl, "kl_cov_ratio", None) is not None else 0.0002
    coef = pl.ppo_kl_coef if getattr(pl, "ppo_kl_coef", None) is not None else 1.0
    assert ratio > 0, "kl_cov_ratio should be larger than 0."
    return float(ratio), float(coef)


def _cov_policy_only(loss_mode, old_log_prob, log_prob, advantages, response_mask, agg_code, lo, hi, rollout_is_weights,
                     aux):
    outs = _actor_loss_op(log_prob, None, old_log_prob, advantages, response_mask, rollout_is_weights, None, loss_mode,
                          lo, hi, 3.0, 20.0, agg_code, 0.0, 0, False, 0.0, 0.0, 1.0, True, aux)
    return outs


@register_policy_loss("clip_cov")
def compute_policy_loss_clip_cov(old_log_prob: torch.Tensor, log_prob: torch.Tensor, advantages: torch.Tensor,
                                 response_mask: torch.Tensor, loss_agg_mode: str = "token-mean", config=None,
                                 rollout_is_weights: Optional[torch.Tensor] = None):
    """Clip-Cov (reference ``core_algos.py:898-995``): the PPO clip surrogate (no dual clip, no clamp of the
    log-ratio) with the loss of a few randomly drawn high-covariance tokens set to zero.  ``config.policy_loss``
    carries ``clip_cov_ratio`` (0.0002), ``clip_cov_lb`` (1.0), ``clip_cov_ub`` (5.0).  The draw is the reference's
    own ``torch.randperm`` on the host generator: with the same seed and inputs the same tokens are dropped.
    Returns ``(pg_loss, pg_clipfrac = masked share of dropped tokens, ppo_kl, 0)``.  The reference's assertion that
    ``config`` is not its ``ActorArguments`` (``:940``) has no counterpart here."""
    ratio, lb, ub = _clip_cov_params(config)
    lo, hi = _clip_params(config)
    agg_code = _agg_code(loss_agg_mode)
    aux = _clip_cov_dropped(old_log_prob, log_prob, advantages, response_mask, lo, hi, ratio, lb, ub)
    outs = _cov_policy_only(LOSS_CLIP_COV, old_log_prob, log_prob, advantages, response_mask, agg_code, lo, hi,
                            rollout_is_weights, aux)
    return outs[O_PG], outs[O_CLIPFRAC], outs[O_PPOKL], outs[O_CLIPLOWER]


@register_policy_loss("kl_cov")
def compute_policy_loss_kl_cov(old_log_prob: torch.Tensor, log_prob: torch.Tensor, advantages: torch.Tensor,
                               response_mask: torch.Tensor, loss_agg_mode: str = "token-mean", config=None,
                               rollout_is_weights: Optional[torch.Tensor] = None):
    """KL-Cov (reference ``core_algos.py:998-1071``): the unclipped surrogate ``-A * ratio``; the
    ``max(1, int(n * kl_cov_ratio))`` valid tokens of largest covariance between advantage and log-prob additionally
    pay ``ppo_kl_coef * |log_prob - old_log_prob|``.  ``config.policy_loss`` carries ``kl_cov_ratio`` (0.0002) and
    ``ppo_kl_coef`` (1.0).  Returns ``(pg_loss, 0, masked_mean(|log_prob - old_log_prob|), 0)``.  Of tokens whose
    covariances are equal at the cut the ones with the lowest flat index are taken (``torch.topk`` promises no order
    there)."""
    ratio, coef = _kl_cov_params(config)
    agg_code = _agg_code(loss_agg_mode)
    aux = _kl_cov_weights(log_prob, advantages, response_mask, ratio, coef)
    outs = _cov_policy_only(LOSS_KL_COV, old_log_prob, log_prob, advantages, response_mask, agg_code, 0.2, 0.2,
                            rollout_is_weights, aux)
    return outs[O_PG], outs[O_CLIPFRAC], outs[O_PPOKL], outs[O_CLIPLOWER]


def compute_value_loss(vpreds: torch.Tensor, returns: torch.Tensor, values: torch.Tensor, response_mask: torch.Tensor,
                       cliprange_value: float, loss_agg_mode: str = "token-mean"):
    """Clipped value loss of the critic (reference ``core_algos.py:1173-1212``).  Returns ``(vf_loss,
    vf_clipfrac)`` as 0-d device tensors; ``vf_loss`` carries the gradient to ``vpreds``."""
    _gpu_of(vpreds)
    return _OPS.value_loss(vpreds, returns, values, response_mask, float(cliprange_value), _agg_code(loss_agg_mode))


def compute_policy_loss(old_log_prob, log_prob, advantages, response_mask, cliprange=None, cliprange_low=None,
                        cliprange_high=None, clip_ratio_c=3.0, loss_agg_mode: str = "token-mean", use_cpgd_loss=False):
    """The legacy entry (reference ``core_algos.py:631-707``): as ``vanilla`` but the log-ratio is not clamped
    to +-20; ``use_cpgd_loss=True`` gives the CPGD loss (``:682-691``)."""
    assert clip_ratio_c > 1.0, (
        "The lower bound of the clip_ratio_c for dual-clip PPO should be greater than 1.0,"
        + f" but get the value: {clip_ratio_c}."
    )
    lo = cliprange if cliprange_low is None else cliprange_low
    hi = cliprange if cliprange_high is None else cliprange_high
    if use_cpgd_loss:
        _check_cpgd_bounds(float(lo), float(hi))
        return _policy_only(LOSS_CPGD, old_log_prob, log_prob, advantages, response_mask, _agg_code(loss_agg_mode),
                            float(lo), float(hi), clip_ratio_c, float("inf"), None)
    return _policy_only(LOSS_VANILLA, old_log_prob, log_prob, advantages, response_mask, _agg_code(loss_agg_mode),
                        float(lo), float(hi), clip_ratio_c, float("inf"), None)


# ------------------------------------------------------------------------------------ KL penalty


def kl_penalty_forward(logprob: torch.Tensor, ref_logprob: torch.Tensor, kl_penalty) -> torch.Tensor:
    """Per-token KL estimator (reference ``core_algos.py:1241-1276``): ``kl``/``k1``, ``abs``, ``mse``/``k2``,
    ``low_var_kl``/``k3``; anything else, ``full`` included, raises ``NotImplementedError``."""
    if kl_penalty not in KL_MODES:
        raise NotImplementedError
    _gpu_of(logprob, ref_logprob)
    return _OPS.kl_penalty(logprob, ref_logprob, KL_MODES[kl_penalty], False)


def kl_penalty(logprob: torch.Tensor, ref_logprob: torch.Tensor, kl_penalty) -> torch.Tensor:
    """reference ``core_algos.py:1215-1238``.  The reference hands the name, ``+`` suffix included, to
    ``kl_penalty_forward`` first (``:1227``), which knows no suffixed name: ``k1+``, ``k3+`` ... therefore
    raise ``NotImplementedError`` there, and do so here.  The straight-through estimator those names were
    meant to select (value of the estimator, gradient of k2) is ``kl_penalty_straight_through``."""
    return kl_penalty_forward(logprob, ref_logprob, kl_penalty)


def kl_penalty_straight_through(logprob: torch.Tensor, ref_logprob: torch.Tensor, kl_penalty: str) -> torch.Tensor:
    """Value of estimator ``kl_penalty`` (without the ``+``) with the gradient of k2,
    ``0.5 * (logprob - ref)^2`` -- the intent of reference ``core_algos.py:1231-1238``."""
    name = kl_penalty[:-1] if kl_penalty.endswith("+") else kl_penalty
    if name not in KL_MODES:
        raise NotImplementedError
    _gpu_of(logprob, ref_logprob)
    return _OPS.kl_penalty(logprob, ref_logprob, KL_MODES[name], True)


# ------------------------------------------------------------------------------------ fused actor loss


class ActorLossOutput:
    """Result of ``actor_loss``: ``loss`` (0-d, differentiable) and the scalars the actor logs, all still on
    the device; ``metrics()`` fetches them with a single device-to-host copy."""

    _NAMES = ("loss", "pg_loss", "pg_clipfrac", "ppo_kl", "pg_clipfrac_lower", "entropy_loss", "kl_loss",
              "ratio_mean", "ratio_min", "ratio_max", "mask_total", "policy_loss", "policy_drift_loss")

    def __init__(self, outs, loss_scale, kl_coef, has_kl, has_entropy):
        self._outs = outs
        for i, n in enumerate(self._NAMES):
            setattr(self, n, outs[i])
        self._scale, self._kl_coef, self._has_kl, self._has_entropy = loss_scale, kl_coef, has_kl, has_entropy

    def metrics(self) -> dict:
        """The per-micro-batch metrics of reference ``dp_actor.py:485-513`` under the same names."""
        v = torch.stack([o.detach() for o in self._outs]).tolist()
        out = {
            "actor/pg_clip_mean": v[O_RMEAN], "actor/pg_clip_min": v[O_RMIN], "actor/pg_clip_max": v[O_RMAX],
            "actor/pg_loss": v[O_PG] * self._scale, "actor/pg_clipfrac": v[O_CLIPFRAC], "actor/ppo_kl": v[O_PPOKL],
            "actor/pg_clipfrac_lower": v[O_CLIPLOWER],
        }
        if self._has_kl:
            out["actor/kl_loss"] = v[O_KL] * self._scale
            out["actor/kl_coef"] = self._kl_coef
        if self._has_entropy:
            out["actor/entropy_loss"] = v[O_ENT]
        return out


def actor_loss(old_log_prob, log_prob, advantages, response_mask, config, entropy=None, ref_log_prob=None,
               loss_scale_factor: float = 1.0, rollout_is_weights=None) -> ActorLossOutput:
    """The loss of one micro-batch as ``DataParallelPPOActor.update_policy`` composes it (reference
    ``siirl/engine/actor/dp_actor.py:455-500``), fused:
    ``loss = (pg_loss - entropy_coeff * agg(entropy) + kl_loss_coef * agg(kl_penalty(log_prob, ref))) * scale``.
    ``config`` carries ``clip_ratio*``, ``entropy_coeff``, ``use_kl_loss``, ``kl_loss_coef``, ``kl_loss_type``,
    ``loss_agg_mode``, ``policy_loss.loss_mode`` (or ``loss_mode``; vanilla, gspo, cpgd, gpg, geo_mean, kl_cov or clip_cov) and
    ``use_cpgd_loss`` / ``policy_drift_coeff``.  The entropy term is used when ``entropy`` is given and
    ``entropy_coeff != 0``; the KL term when ``config.use_kl_loss``; the drift term
    ``policy_drift_coeff * agg(clamp(exp(lp - old) - 1, max=2) * lp)`` (``dp_actor.py:488-494``) when
    ``config.use_cpgd_loss`` and the coefficient is non-zero."""
    _gpu_of(log_prob)
    mode = getattr(getattr(config, "policy_loss", None), "loss_mode", None) or getattr(config, "loss_mode", "vanilla")
    if mode not in _LOSS_CODES:
        raise ValueError(f"Unsupported loss mode: {mode}. Supported modes are: {sorted(_LOSS_CODES)}")
    lo, hi = _clip_params(config)
    c = getattr(config, "clip_ratio_c", 3.0)
    c = 3.0 if c is None else float(c)
    if mode in ("vanilla", "cpgd"):
        assert c > 1.0, f"The lower bound of the clip_ratio_c for dual-clip PPO should be greater than 1.0, but get the value: {c}."
    if mode == "cpgd":
        _check_cpgd_bounds(lo, hi)
    drift = float(getattr(config, "policy_drift_coeff", 0.0) or 0.0) if getattr(config, "use_cpgd_loss", False) else 0.0
    agg_code = _agg_code(getattr(config, "loss_agg_mode", "token-mean"))
    ent_coef = float(getattr(config, "entropy_coeff", 0.0))
    use_ent = entropy is not None and ent_coef != 0
    use_kl = bool(getattr(config, "use_kl_loss", False))
    kl_code, kl_coef = 0, 0.0
    if use_kl:
        if ref_log_prob is None:
            raise ValueError("config.use_kl_loss is set but ref_log_prob is None")
        kl_type = getattr(config, "kl_loss_type", "low_var_kl")
        if kl_type not in KL_MODES:
            raise NotImplementedError
        kl_code, kl_coef = KL_MODES[kl_type], float(getattr(config, "kl_loss_coef", 0.001))
    aux = None
    if mode == "kl_cov":
        aux = _kl_cov_weights(log_prob, advantages, response_mask, *_kl_cov_params(config))
    elif mode == "clip_cov":
        aux = _clip_cov_dropped(old_log_prob, log_prob, advantages, response_mask, lo, hi, *_clip_cov_params(config))
    outs = _actor_loss_op(log_prob, entropy if use_ent else None, old_log_prob, advantages, response_mask,
                          None if mode == "cpgd" else rollout_is_weights, ref_log_prob if use_kl else None,
                          _LOSS_CODES[mode], lo, hi, c, 20.0, agg_code, ent_coef if use_ent else 0.0, kl_code, False,
                          kl_coef, drift, float(loss_scale_factor), False, aux)
    return ActorLossOutput(outs, float(loss_scale_factor), kl_coef, use_kl, use_ent)


# ------------------------------------------------------------------------------------ fused actor step


class FusedActorStepOutput:
    """Result of ``fused_actor_step``: ``dlogits`` (gradient of the scaled loss w.r.t. the unscaled logits, shape and
    dtype of the logits), ``log_prob`` / ``entropy`` (``[B, L]`` fp32, detached), and ``loss_output``, the
    ``ActorLossOutput`` with the loss value and the logged scalars.  Typical use: ``logits.backward(out.dlogits)``."""

    def __init__(self, dlogits, log_prob, entropy, loss_output):
        self.dlogits, self.log_prob, self.entropy, self.loss_output = dlogits, log_prob, entropy, loss_output
        self.loss = loss_output.loss

    def metrics(self) -> dict:
        return self.loss_output.metrics()


def agg_weights(response_mask: torch.Tensor, loss_agg_mode: str) -> torch.Tensor:
    """``d agg_loss / d loss_mat`` for a unit upstream gradient: a function of the mask and the mode alone
    (reference ``core_algos.py:536-569``).  ``[B, L]`` fp32."""
    dev = _gpu_of(response_mask)
    m, mcode = _mask_arg(_as_2d(response_mask), dev)
    B, L = m.shape
    w = torch.empty(B, L, dtype=torch.float32, device=dev)
    out16 = torch.empty(16, dtype=torch.float32, device=dev)
    row_msum = torch.empty(B, dtype=torch.float32, device=dev)
    ws, nws = _workspace(B, L, dev)
    with torch.cuda.device(dev):
        rc = _lib.lib().siirl_agg_weights(_lib.ptr(m), mcode, B, L, _agg_code(loss_agg_mode), _lib.ptr(w),
                                          _lib.ptr(out16), _lib.ptr(row_msum), _lib.ptr(ws), nws,
                                          _lib.current_stream(dev))
    _lib.check(rc, "siirl_agg_weights")
    return w


def fused_actor_step(logits: torch.Tensor, responses: torch.Tensor, old_log_prob, advantages: torch.Tensor,
                     response_mask: torch.Tensor, config, ref_log_prob=None, temperature: float = 1.0,
                     loss_scale_factor: float = 1.0, on_policy: bool = False,
                     rollout_is_weights=None) -> FusedActorStepOutput:
    """One micro-batch of the actor update from the response logits to their gradient in a single pass over the
    logits (reference ``siirl/engine/actor/dp_actor.py:170-231,403-501``: ``logits / T`` -> log-prob -> entropy ->
    policy loss - entropy bonus + KL loss (+ CPGD drift) -> ``backward()``), for the token-separable losses
    ``vanilla``, ``cpgd`` and ``gpg``.  ``logits`` is ``[B, L, V]`` (or ``[B * L, V]``; row-strided views are
    fine) and is not modified; ``responses`` are the labels.  ``on_policy`` uses ``old = log_prob.detach()``
    (``dp_actor.py:436-437``).  ``gspo`` and ``geo_mean`` need sequence statistics before any gradient exists: use
    ``logprobs_from_logits`` + ``actor_loss`` for them."""
    from .ops import row_blocks

    dev = _gpu_of(logits)
    mode = getattr(getattr(config, "policy_loss", None), "loss_mode", None) or getattr(config, "loss_mode", "vanilla")
    if mode not in ("vanilla", "cpgd", "gpg"):
        raise ValueError(f"fused_actor_step supports the token-separable losses vanilla, cpgd and gpg, not {mode!r}")
    if logits.dtype not in (torch.float32, torch.bfloat16, torch.float16):
        raise TypeError(f"logits dtype {logits.dtype} is not supported")
    m2 = _as_2d(response_mask)
    B, L = m2.shape
    V = logits.shape[-1]
    if logits.numel() != B * L * V:
        raise ValueError(f"logits {tuple(logits.shape)} do not match response_mask {tuple(response_mask.shape)}")
    lo, hi = _clip_params(config)
    c = getattr(config, "clip_ratio_c", 3.0)
    c = 3.0 if c is None else float(c)
    if mode in ("vanilla", "cpgd"):
        assert c > 1.0, f"The lower bound of the clip_ratio_c for dual-clip PPO should be greater than 1.0, but get the value: {c}."
    if mode == "cpgd":
        _check_cpgd_bounds(lo, hi)
    agg = getattr(config, "loss_agg_mode", "token-mean")
    ent_coef = float(getattr(config, "entropy_coeff", 0.0))
    use_kl = bool(getattr(config, "use_kl_loss", False))
    kl_code, kl_coef = 0, 0.0
    if use_kl:
        if ref_log_prob is None:
            raise ValueError("config.use_kl_loss is set but ref_log_prob is None")
        kl_type = getattr(config, "kl_loss_type", "low_var_kl")
        if kl_type not in KL_MODES:
            raise NotImplementedError
        kl_code, kl_coef = KL_MODES[kl_type], float(getattr(config, "kl_loss_coef", 0.001))
    drift = float(getattr(config, "policy_drift_coeff", 0.0) or 0.0) if getattr(config, "use_cpgd_loss", False) else 0.0

    w = agg_weights(m2, agg).reshape(-1)
    lab = responses.detach().to(device=dev, dtype=torch.int64).reshape(-1).contiguous()
    old = None if on_policy else _f32(old_log_prob, dev).reshape(-1)
    adv = _f32(advantages, dev).reshape(-1)
    ref = _f32(ref_log_prob, dev).reshape(-1) if use_kl else None
    isw = None if (rollout_is_weights is None or mode == "cpgd") else _f32(rollout_is_weights, dev).reshape(-1)
    for name, t in (("responses", lab), ("old_log_prob", old), ("advantages", adv), ("ref_log_prob", ref),
                    ("rollout_is_weights", isw)):
        if t is not None and t.numel() != B * L:
            raise ValueError(f"{name} has {t.numel()} elements, expected {B * L}")
    lp = torch.empty(B * L, dtype=torch.float32, device=dev)
    ent = torch.empty(B * L, dtype=torch.float32, device=dev) if ent_coef != 0 else None
    x = logits.detach()
    dlogits = torch.empty(logits.shape, dtype=logits.dtype, device=dev)
    d2 = dlogits.view(-1, V)
    code = _lib.dtype_code(logits.dtype)
    es = x.element_size()
    done = 0

    def at(t, k):
        return None if t is None else C.c_void_p(t.data_ptr() + 4 * k)

    with torch.cuda.device(dev):
        for off, rows, stride in row_blocks(x):
            rc = _lib.lib().siirl_actor_step_fused(
                C.c_void_p(x.data_ptr() + off * es), code, rows, V, stride, C.c_void_p(lab.data_ptr() + 8 * done),
                1.0 / float(temperature), at(old, done), at(adv, done), at(ref, done), at(isw, done), at(w, done),
                at(w, done), _LOSS_CODES[mode], lo, hi, c, 20.0, ent_coef, kl_code, 0, kl_coef, drift,
                float(loss_scale_factor), at(lp, done), at(ent, done), C.c_void_p(d2.data_ptr() + done * V * es), V,
                _lib.current_stream(dev))
            _lib.check(rc, "siirl_actor_step_fused")
            done += rows
    lp2 = lp.view(B, L)
    ent2 = None if ent is None else ent.view(B, L)
    with torch.no_grad():
        loss_out = actor_loss(lp2 if on_policy else old.view(B, L), lp2, adv.view(B, L), m2, config, entropy=ent2,
                              ref_log_prob=None if ref is None else ref.view(B, L),
                              loss_scale_factor=loss_scale_factor,
                              rollout_is_weights=None if isw is None else isw.view(B, L))
    return FusedActorStepOutput(dlogits, lp2, ent2, loss_out)
