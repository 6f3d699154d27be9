"""``torch.library`` registration of the HIP entry points as ``torch.ops.siirl_hip.*``.

Each op is a thin shim: it checks shapes, allocates outputs with torch, and hands raw device
pointers plus the current stream to the C ABI.  Fake (meta) kernels give shapes to FakeTensor
tracing; there is deliberately no CPU kernel."""

from __future__ import annotations

from typing import Optional, Tuple

import torch

from . import _lib

_NS = "siirl_hip"


def _require_gpu(t: torch.Tensor, name: str):
    if not t.is_cuda:
        raise RuntimeError(f"siirl_amd: `{name}` is on {t.device}; these ops run on the GPU only (no CPU fallback)")


def row_blocks(x: torch.Tensor):
    """Splits a ``(..., V)`` tensor with unit inner stride into blocks of uniformly strided rows:
    yields ``(element_offset, n_rows, row_stride)``.  A contiguous tensor, or a row-sliced 2-D view,
    is a single block; a ``[B, S, V]`` slice along ``S`` gives ``B`` blocks."""
    V = x.shape[-1]
    if x.stride(-1) != 1 and V > 1:
        raise ValueError("siirl_amd: the vocab axis of logits must have stride 1")
    lead_shape, lead_stride = list(x.shape[:-1]), list(x.stride()[:-1])
    # drop size-1 axes, then peel trailing leading-axes that collapse into one uniformly strided axis
    dims = [(n, s) for n, s in zip(lead_shape, lead_stride) if n != 1]
    if not dims:
        yield 0, 1 if x.numel() else 0, max(V, 1)
        return
    n_in, s_in = dims[-1]
    k = len(dims) - 1
    while k > 0 and dims[k - 1][1] == n_in * s_in:
        n_in *= dims[k - 1][0]
        k -= 1
    outer = dims[:k]
    if s_in < V:
        raise ValueError("siirl_amd: overlapping logits rows are not supported")

    def rec(level, off):
        if level == len(outer):
            yield off, n_in, s_in
            return
        n, s = outer[level]
        for i in range(n):
            yield from rec(level + 1, off + i * s)

    yield from rec(0, 0)


@torch.library.custom_op(f"{_NS}::logprob_entropy_fwd", mutates_args=())
def logprob_entropy_fwd(logits: torch.Tensor, labels: Optional[torch.Tensor], inv_temperature: float,
                        want_entropy: bool) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor, torch.Tensor]:
    """-> (logprob, entropy, lse, ex), fp32, shape ``logits.shape[:-1]``; tensors not requested are empty."""
    _require_gpu(logits, "logits")
    lead = logits.shape[:-1]
    V = logits.shape[-1]
    dev = logits.device
    want_lp = labels is not None
    if want_lp:
        if labels.shape != lead:
            raise ValueError(f"labels shape {tuple(labels.shape)} does not match logits {tuple(logits.shape)}")
        labels = labels.to(device=dev, dtype=torch.int64).contiguous()
    f32 = dict(dtype=torch.float32, device=dev)
    lp = torch.empty(lead if want_lp else (0,), **f32)
    ent = torch.empty(lead if want_entropy else (0,), **f32)
    ex = torch.empty(lead if want_entropy else (0,), **f32)
    lse = torch.empty(lead, **f32)
    L = _lib.lib()
    es = logits.element_size()
    code = _lib.dtype_code(logits.dtype)
    stream = _lib.current_stream(dev)
    base = logits.data_ptr()
    done = 0
    with torch.cuda.device(dev):
        for off, rows, stride in row_blocks(logits):
            if rows == 0:
                continue
            o4 = done * 4
            rc = L.siirl_logprob_entropy_fwd(
                base + off * es, code, rows, V, stride,
                labels.data_ptr() + done * 8 if want_lp else None, inv_temperature,
                lp.data_ptr() + o4 if want_lp else None,
                ent.data_ptr() + o4 if want_entropy else None,
                lse.data_ptr() + o4,
                ex.data_ptr() + o4 if want_entropy else None, stream)
            _lib.check(rc, "siirl_logprob_entropy_fwd")
            done += rows
    return lp, ent, lse, ex


@logprob_entropy_fwd.register_fake
def _(logits, labels, inv_temperature, want_entropy):
    lead = logits.shape[:-1]
    mk = lambda shape: logits.new_empty(shape, dtype=torch.float32)  # noqa: E731
    return (mk(lead if labels is not None else (0,)), mk(lead if want_entropy else (0,)), mk(lead),
            mk(lead if want_entropy else (0,)))


def _bwd_launch(logits, labels, inv_temperature, lse, ex, g_logprob, g_entropy, out, skip_zero_rows):
    _require_gpu(logits, "logits")
    dev = logits.device
    V = logits.shape[-1]
    es = logits.element_size()
    code = _lib.dtype_code(logits.dtype)
    L = _lib.lib()
    stream = _lib.current_stream(dev)
    f = lambda t: None if t is None else t.to(device=dev, dtype=torch.float32).contiguous()  # noqa: E731
    g_logprob, g_entropy, lse, ex = f(g_logprob), f(g_entropy), f(lse), f(ex)
    if labels is not None:
        labels = labels.to(device=dev, dtype=torch.int64).contiguous()
    in_blocks = list(row_blocks(logits))
    if out is logits:
        out_blocks = in_blocks
    else:  # a fresh contiguous tensor: rows follow one another whatever the blocking of the input
        if not out.is_contiguous() or out.shape != logits.shape:
            raise ValueError("siirl_amd: dlogits must be contiguous and shaped like logits")
        out_blocks, r = [], 0
        for _, rows, _ in in_blocks:
            out_blocks.append((r * V, rows, V))
            r += rows
    flags = _lib.BWD_SKIP_ZERO_ROWS if skip_zero_rows else 0
    done = 0
    with torch.cuda.device(dev):
        for (off, rows, stride), (ooff, _, ostride) in zip(in_blocks, out_blocks):
            if rows == 0:
                continue
            o4 = done * 4
            rc = L.siirl_logprob_entropy_bwd(
                logits.data_ptr() + off * es, code, rows, V, stride,
                labels.data_ptr() + done * 8 if g_logprob is not None else None, inv_temperature,
                lse.data_ptr() + o4, ex.data_ptr() + o4 if g_entropy is not None else None,
                g_logprob.data_ptr() + o4 if g_logprob is not None else None,
                g_entropy.data_ptr() + o4 if g_entropy is not None else None,
                out.data_ptr() + ooff * es, ostride, flags, stream)
            _lib.check(rc, "siirl_logprob_entropy_bwd")
            done += rows


@torch.library.custom_op(f"{_NS}::logprob_entropy_bwd", mutates_args=())
def logprob_entropy_bwd(logits: torch.Tensor, labels: Optional[torch.Tensor], inv_temperature: float,
                        lse: torch.Tensor, ex: Optional[torch.Tensor], g_logprob: Optional[torch.Tensor],
                        g_entropy: Optional[torch.Tensor], skip_zero_rows: bool) -> torch.Tensor:
    """Gradient w.r.t. ``logits`` as a fresh contiguous tensor of the logits' dtype and shape."""
    out = torch.empty(logits.shape, dtype=logits.dtype, device=logits.device)
    _bwd_launch(logits, labels, inv_temperature, lse, ex, g_logprob, g_entropy, out, skip_zero_rows)
    return out


@logprob_entropy_bwd.register_fake
def _(logits, labels, inv_temperature, lse, ex, g_logprob, g_entropy, skip_zero_rows):
    return logits.new_empty(logits.shape)


@torch.library.custom_op(f"{_NS}::logprob_entropy_bwd_", mutates_args=("logits",))
def logprob_entropy_bwd_(logits: torch.Tensor, labels: Optional[torch.Tensor], inv_temperature: float,
                         lse: torch.Tensor, ex: Optional[torch.Tensor], g_logprob: Optional[torch.Tensor],
                         g_entropy: Optional[torch.Tensor], skip_zero_rows: bool) -> None:
    """In-place variant: overwrites ``logits`` with its own gradient."""
    _bwd_launch(logits, labels, inv_temperature, lse, ex, g_logprob, g_entropy, logits, skip_zero_rows)


# ------------------------------------------------------------------------------------------------
# The [B, L] loss arithmetic, the group operations and the fused lm_head as ``torch.ops.siirl_hip.*``.
# Operands arrive prepared by the Python layer (fp32, contiguous, 2-D; masks in any dtype the library
# reads); every op allocates its outputs, runs on the current stream and has a fake kernel for tracing.


def _f32c(t: Optional[torch.Tensor], name: str):
    if t is None:
        return None
    _require_gpu(t, name)
    if t.dtype != torch.float32 or not t.is_contiguous():
        raise ValueError(f"siirl_amd: `{name}` must be a contiguous float32 tensor")
    return t


def _mask_code(mask: torch.Tensor) -> int:
    if not mask.is_contiguous():
        raise ValueError("siirl_amd: the mask must be contiguous")
    return _lib.dtype_code(mask.dtype)


def _loss_workspace(B: int, L: int, dev):
    n = _lib.lib().siirl_loss_workspace_bytes(B, L)
    return torch.empty(n, dtype=torch.uint8, device=dev), n


@torch.library.custom_op(f"{_NS}::grpo_advantage", mutates_args=())
def grpo_advantage(token_level_rewards: torch.Tensor, mask: torch.Tensor, uid: torch.Tensor, epsilon: float,
                   norm_by_std: bool) -> torch.Tensor:
    """``[B, L]`` fp32 group-normalised outcome advantage, masked (``uid`` int64 ``[B]``)."""
    r = _f32c(token_level_rewards, "token_level_rewards")
    B, L = r.shape
    dev = r.device
    if uid.dtype != torch.int64 or uid.numel() != B or tuple(mask.shape) != (B, L):
        raise ValueError("siirl_amd: uid must be int64 [B] and mask [B, L]")
    adv = torch.empty(B, L, dtype=torch.float32, device=dev)
    scratch = torch.empty(2 * max(B, 1), dtype=torch.float32, device=dev)
    with torch.cuda.device(dev):
        rc = _lib.lib().siirl_grpo_outcome_advantage(_lib.ptr(r), _lib.ptr(mask), _mask_code(mask),
                                                     _lib.ptr(uid.contiguous()), B, L, epsilon, int(norm_by_std),
                                                     _lib.ptr(adv), _lib.ptr(scratch), _lib.current_stream(dev))
    _lib.check(rc, "siirl_grpo_outcome_advantage")
    return adv


@grpo_advantage.register_fake
def _(token_level_rewards, mask, uid, epsilon, norm_by_std):
    return token_level_rewards.new_empty(token_level_rewards.shape, dtype=torch.float32)


@torch.library.custom_op(f"{_NS}::group_keep_mask", mutates_args=())
def group_keep_mask(metric: torch.Tensor, uid: torch.Tensor) -> Tuple[torch.Tensor, torch.Tensor]:
    """-> (keep uint8 ``[B]``, group_size int32 ``[B]``) for a fp32 / fp64 metric and int64 uids."""
    _require_gpu(metric, "metric")
    B = uid.numel()
    dev = metric.device
    if metric.numel() != B or uid.dtype != torch.int64:
        raise ValueError("siirl_amd: metric and uid must have one entry per trajectory, uid int64")
    keep = torch.empty(B, dtype=torch.uint8, device=dev)
    gsz = torch.empty(B, dtype=torch.int32, device=dev)
    met = metric.contiguous()
    with torch.cuda.device(dev):
        rc = _lib.lib().siirl_group_keep_mask(_lib.ptr(met), _lib.dtype_code(met.dtype), _lib.ptr(uid.contiguous()), B,
                                              _lib.ptr(keep), _lib.ptr(gsz), _lib.current_stream(dev))
    _lib.check(rc, "siirl_group_keep_mask")
    return keep, gsz


@group_keep_mask.register_fake
def _(metric, uid):
    return uid.new_empty(uid.shape, dtype=torch.uint8), uid.new_empty(uid.shape, dtype=torch.int32)


@torch.library.custom_op(f"{_NS}::agg_loss_fwd", mutates_args=())
def agg_loss_fwd(loss_mat: torch.Tensor, mask: torch.Tensor, agg_mode: int) -> Tuple[torch.Tensor, torch.Tensor]:
    """-> (out16, row_msum): the aggregate is ``out16[1]``; both are what ``agg_loss_bwd`` needs."""
    v = _f32c(loss_mat, "loss_mat")
    B, L = v.shape
    dev = v.device
    out16 = torch.empty(16, dtype=torch.float32, device=dev)
    row_msum = torch.empty(B, dtype=torch.float32, device=dev)
    ws, nws = _loss_workspace(B, L, dev)
    with torch.cuda.device(dev):
        rc = _lib.lib().siirl_agg_loss_fwd(_lib.ptr(v), _lib.ptr(mask), _mask_code(mask), B, L, agg_mode,
                                           _lib.ptr(out16), _lib.ptr(row_msum), _lib.ptr(ws), nws,
                                           _lib.current_stream(dev))
    _lib.check(rc, "siirl_agg_loss_fwd")
    return out16, row_msum


@agg_loss_fwd.register_fake
def _(loss_mat, mask, agg_mode):
    return loss_mat.new_empty(16, dtype=torch.float32), loss_mat.new_empty(loss_mat.shape[0], dtype=torch.float32)


@torch.library.custom_op(f"{_NS}::agg_loss_bwd", mutates_args=())
def agg_loss_bwd(g: torch.Tensor, mask: torch.Tensor, out16: torch.Tensor, row_msum: torch.Tensor,
                 agg_mode: int) -> torch.Tensor:
    B, L = mask.shape
    dev = out16.device
    g = _f32c(g, "g")
    d = torch.empty(B, L, dtype=torch.float32, device=dev)
    with torch.cuda.device(dev):
        rc = _lib.lib().siirl_agg_loss_bwd(_lib.ptr(g), _lib.ptr(mask), _mask_code(mask), _lib.ptr(out16),
                                           _lib.ptr(row_msum), B, L, agg_mode, _lib.ptr(d), _lib.current_stream(dev))
    _lib.check(rc, "siirl_agg_loss_bwd")
    return d


@agg_loss_bwd.register_fake
def _(g, mask, out16, row_msum, agg_mode):
    return out16.new_empty(mask.shape, dtype=torch.float32)


@torch.library.custom_op(f"{_NS}::policy_loss_fwd", mutates_args=())
def policy_loss_fwd(old_log_prob: torch.Tensor, log_prob: torch.Tensor, advantages: torch.Tensor, mask: torch.Tensor,
                    is_weights: Optional[torch.Tensor], entropy: Optional[torch.Tensor],
                    ref_log_prob: Optional[torch.Tensor], loss_mode: int, clip_low: float, clip_high: float,
                    clip_c: float, log_ratio_clamp: float, agg_mode: int, entropy_coeff: float, kl_mode: int,
                    kl_straight_through: bool, kl_coef: float, policy_drift_coeff: float,
                    loss_scale: float) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    """The actor's loss of one micro-batch -> (out16, row_msum, row_s).  ``out16`` holds the scaled total, the
    policy loss and the logged scalars (``SIIRL_OUT_*`` of the C header); the other two feed the backward."""
    lp = _f32c(log_prob, "log_prob")
    B, L = lp.shape
    dev = lp.device
    old, adv = _f32c(old_log_prob, "old_log_prob"), _f32c(advantages, "advantages")
    isw, ent, ref = _f32c(is_weights, "is_weights"), _f32c(entropy, "entropy"), _f32c(ref_log_prob, "ref_log_prob")
    out16 = torch.empty(16, dtype=torch.float32, device=dev)
    row_msum = torch.empty(B, dtype=torch.float32, device=dev)
    row_s = torch.empty(B, dtype=torch.float32, device=dev)
    ws, nws = _loss_workspace(B, L, dev)
    with torch.cuda.device(dev):
        rc = _lib.lib().siirl_actor_loss_fwd(
            _lib.ptr(old), _lib.ptr(lp), _lib.ptr(adv), _lib.ptr(mask), _mask_code(mask), _lib.ptr(isw), _lib.ptr(ent),
            _lib.ptr(ref), B, L, loss_mode, clip_low, clip_high, clip_c, log_ratio_clamp, agg_mode, entropy_coeff,
            kl_mode, int(kl_straight_through), kl_coef, policy_drift_coeff, loss_scale, _lib.ptr(out16),
            _lib.ptr(row_msum), _lib.ptr(row_s), _lib.ptr(ws), nws, _lib.current_stream(dev))
    _lib.check(rc, "siirl_actor_loss_fwd")
    return out16, row_msum, row_s


@policy_loss_fwd.register_fake
def _(old_log_prob, log_prob, advantages, mask, is_weights, entropy, ref_log_prob, loss_mode, clip_low, clip_high,
      clip_c, log_ratio_clamp, agg_mode, entropy_coeff, kl_mode, kl_straight_through, kl_coef, policy_drift_coeff,
      loss_scale):
    B = log_prob.shape[0]
    mk = lambda n: log_prob.new_empty(n, dtype=torch.float32)  # noqa: E731
    return mk(16), mk(B), mk(B)


@torch.library.custom_op(f"{_NS}::policy_loss_bwd", mutates_args=())
def policy_loss_bwd(g_loss: torch.Tensor, old_log_prob: torch.Tensor, log_prob: torch.Tensor, advantages: torch.Tensor,
                    mask: torch.Tensor, is_weights: Optional[torch.Tensor], entropy: Optional[torch.Tensor],
                    ref_log_prob: Optional[torch.Tensor], loss_mode: int, clip_low: float, clip_high: float,
                    clip_c: float, log_ratio_clamp: float, agg_mode: int, entropy_coeff: float, kl_mode: int,
                    kl_straight_through: bool, kl_coef: float, policy_drift_coeff: float, loss_scale: float,
                    out16: torch.Tensor, row_msum: torch.Tensor,
                    row_s: torch.Tensor) -> Tuple[torch.Tensor, torch.Tensor]:
    """-> (d_log_prob ``[B, L]``, d_entropy ``[B, L]`` or empty when no entropy was given)."""
    lp = _f32c(log_prob, "log_prob")
    B, L = lp.shape
    dev = lp.device
    g = _f32c(g_loss, "g_loss")
    old, adv = _f32c(old_log_prob, "old_log_prob"), _f32c(advantages, "advantages")
    isw, ent, ref = _f32c(is_weights, "is_weights"), _f32c(entropy, "entropy"), _f32c(ref_log_prob, "ref_log_prob")
    d_lp = torch.empty(B, L, dtype=torch.float32, device=dev)
    d_ent = torch.empty((B, L) if ent is not None else (0,), dtype=torch.float32, device=dev)
    with torch.cuda.device(dev):
        rc = _lib.lib().siirl_actor_loss_bwd(
            _lib.ptr(g), _lib.ptr(old), _lib.ptr(lp), _lib.ptr(adv), _lib.ptr(mask), _mask_code(mask), _lib.ptr(isw),
            _lib.ptr(ent), _lib.ptr(ref), B, L, loss_mode, clip_low, clip_high, clip_c, log_ratio_clamp, agg_mode,
            entropy_coeff, kl_mode, int(kl_straight_through), kl_coef, policy_drift_coeff, loss_scale,
            _lib.ptr(out16), _lib.ptr(row_msum), _lib.ptr(row_s), _lib.ptr(d_lp),
            _lib.ptr(d_ent) if ent is not None else None, _lib.current_stream(dev))
    _lib.check(rc, "siirl_actor_loss_bwd")
    return d_lp, d_ent


@policy_loss_bwd.register_fake
def _(g_loss, old_log_prob, log_prob, advantages, mask, is_weights, entropy, ref_log_prob, loss_mode, clip_low,
      clip_high, clip_c, log_ratio_clamp, agg_mode, entropy_coeff, kl_mode, kl_straight_through, kl_coef,
      policy_drift_coeff, loss_scale, out16, row_msum, row_s):
    return (log_prob.new_empty(log_prob.shape, dtype=torch.float32),
            log_prob.new_empty(log_prob.shape if entropy is not None else (0,), dtype=torch.float32))


@torch.library.custom_op(f"{_NS}::kl_penalty_fwd", mutates_args=())
def kl_penalty_fwd(log_prob: torch.Tensor, ref_log_prob: torch.Tensor, kl_mode: int) -> torch.Tensor:
    lp, ref = _f32c(log_prob, "log_prob"), _f32c(ref_log_prob, "ref_log_prob")
    if ref.shape != lp.shape:
        raise ValueError("siirl_amd: log_prob and ref_log_prob must have one shape")
    out = torch.empty_like(lp)
    with torch.cuda.device(lp.device):
        rc = _lib.lib().siirl_kl_penalty_fwd(_lib.ptr(lp), _lib.ptr(ref), lp.numel(), kl_mode, _lib.ptr(out),
                                             _lib.current_stream(lp.device))
    _lib.check(rc, "siirl_kl_penalty_fwd")
    return out


@kl_penalty_fwd.register_fake
def _(log_prob, ref_log_prob, kl_mode):
    return log_prob.new_empty(log_prob.shape, dtype=torch.float32)


@torch.library.custom_op(f"{_NS}::kl_penalty_bwd", mutates_args=())
def kl_penalty_bwd(g: torch.Tensor, log_prob: torch.Tensor, ref_log_prob: torch.Tensor, kl_mode: int,
                   straight_through: bool, need_log_prob: bool, need_ref: bool) -> Tuple[torch.Tensor, torch.Tensor]:
    """-> (d_log_prob, d_ref_log_prob); a gradient that is not needed comes back empty."""
    g, lp, ref = _f32c(g, "g"), _f32c(log_prob, "log_prob"), _f32c(ref_log_prob, "ref_log_prob")
    d_lp = torch.empty(lp.shape if need_log_prob else (0,), dtype=torch.float32, device=lp.device)
    d_ref = torch.empty(lp.shape if need_ref else (0,), dtype=torch.float32, device=lp.device)
    if need_log_prob or need_ref:
        with torch.cuda.device(lp.device):
            rc = _lib.lib().siirl_kl_penalty_bwd(_lib.ptr(g), _lib.ptr(lp), _lib.ptr(ref), lp.numel(), kl_mode,
                                                 int(straight_through), _lib.ptr(d_lp) if need_log_prob else None,
                                                 _lib.ptr(d_ref) if need_ref else None, _lib.current_stream(lp.device))
        _lib.check(rc, "siirl_kl_penalty_bwd")
    return d_lp, d_ref


@kl_penalty_bwd.register_fake
def _(g, log_prob, ref_log_prob, kl_mode, straight_through, need_log_prob, need_ref):
    mk = lambda need: log_prob.new_empty(log_prob.shape if need else (0,), dtype=torch.float32)  # noqa: E731
    return mk(need_log_prob), mk(need_ref)


def _bf16_2d(t: torch.Tensor, name: str):
    _require_gpu(t, name)
    if t.dtype != torch.bfloat16 or t.dim() != 2 or not t.is_contiguous():
        raise TypeError(f"siirl_amd: `{name}` must be a contiguous 2-D bfloat16 tensor")
    return t


@torch.library.custom_op(f"{_NS}::fused_linear_logprob_entropy_fwd", mutates_args=())
def fused_linear_logprob_entropy_fwd(hidden: torch.Tensor, weight: torch.Tensor, labels: torch.Tensor,
                                     inv_temperature: float, save_logits: bool = False
                                     ) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor, torch.Tensor, torch.Tensor]:
    """lm_head projection fused with log-prob / entropy -> (logprob, entropy, lse, ex, saved), fp32 ``[T]``.
    ``saved`` is empty unless ``save_logits``: then it holds the fp32 logit tiles in the kernel's own order (4 bytes
    per logit) for the backward to read instead of recomputing them."""
    h, w = _bf16_2d(hidden, "hidden"), _bf16_2d(weight, "weight")
    T, H = h.shape
    V = w.shape[0]
    dev = h.device
    if w.shape[1] != H or tuple(labels.shape) != (T,) or labels.dtype != torch.int64:
        raise ValueError(f"shape mismatch: hidden {tuple(h.shape)}, weight {tuple(w.shape)}, labels {tuple(labels.shape)}")
    L = _lib.lib()
    lp, ent, lse, ex = (torch.empty(T, dtype=torch.float32, device=dev) for _ in range(4))
    saved = torch.empty(0, dtype=torch.float32, device=dev)
    if save_logits:
        try:
            saved = torch.empty(L.siirl_fused_linear_saved_logits_bytes(T, V) // 4, dtype=torch.float32, device=dev)
        except torch.OutOfMemoryError:
            save_logits = False  # no room to keep the logits: the backward recomputes them
    nws = L.siirl_fused_linear_fwd_workspace_bytes(T, H, V)
    ws = torch.empty(max(nws, 256), dtype=torch.uint8, device=dev)
    y = labels.contiguous()
    with torch.cuda.device(dev):
        rc = L.siirl_fused_linear_logprob_entropy_fwd(_lib.ptr(h), _lib.ptr(w), _lib.BF16, _lib.ptr(y), T, H, V,
                                                      inv_temperature, _lib.ptr(lp), _lib.ptr(ent), _lib.ptr(lse),
                                                      _lib.ptr(ex), _lib.ptr(saved) if save_logits else None,
                                                      _lib.ptr(ws), nws, _lib.current_stream(dev))
    _lib.check(rc, "siirl_fused_linear_logprob_entropy_fwd")
    return lp, ent, lse, ex, saved


@fused_linear_logprob_entropy_fwd.register_fake
def _(hidden, weight, labels, inv_temperature, save_logits=False):
    mk = lambda: hidden.new_empty(hidden.shape[0], dtype=torch.float32)  # noqa: E731
    T, V = hidden.shape[0], weight.shape[0]
    n = ((V + 255) // 256) * ((T + 255) // 256) * 65536 if save_logits else 0
    return mk(), mk(), mk(), mk(), hidden.new_empty(n, dtype=torch.float32)


@torch.library.custom_op(f"{_NS}::fused_linear_logprob_entropy_bwd", mutates_args=())
def fused_linear_logprob_entropy_bwd(hidden: torch.Tensor, weight: torch.Tensor, labels: torch.Tensor,
                                     inv_temperature: float, lse: torch.Tensor, ex: torch.Tensor,
                                     g_logprob: Optional[torch.Tensor], g_entropy: Optional[torch.Tensor],
                                     need_hidden: bool, need_weight: bool,
                                     saved: Optional[torch.Tensor] = None) -> Tuple[torch.Tensor, torch.Tensor]:
    """-> (d_hidden, d_weight), bf16; a gradient that is not needed comes back empty.  ``saved``: the fifth output
    of the forward op (empty or None: the logits are recomputed)."""
    h, w = _bf16_2d(hidden, "hidden"), _bf16_2d(weight, "weight")
    T, H = h.shape
    V = w.shape[0]
    dev = h.device
    g_lp, g_ent = _f32c(g_logprob, "g_logprob"), _f32c(g_entropy, "g_entropy")
    d_h = torch.empty(h.shape if need_hidden else (0,), dtype=h.dtype, device=dev)
    d_w = torch.empty(w.shape if need_weight else (0,), dtype=w.dtype, device=dev)
    L = _lib.lib()
    if saved is not None and saved.numel() == 0:
        saved = None
    if saved is not None:
        _require_gpu(saved, "saved")
        if saved.dtype != torch.float32 or not saved.is_contiguous() or \
                saved.numel() * 4 != L.siirl_fused_linear_saved_logits_bytes(T, V):
            raise ValueError("saved is not the buffer the forward op returned for these shapes")
    nws = L.siirl_fused_linear_bwd_workspace_bytes(T, H, V, int(need_hidden), int(need_weight))
    ws = torch.empty(max(nws, 256), dtype=torch.uint8, device=dev)
    y = labels.contiguous()
    with torch.cuda.device(dev):
        rc = L.siirl_fused_linear_logprob_entropy_bwd(_lib.ptr(h), _lib.ptr(w), _lib.BF16, _lib.ptr(y), T, H, V,
                                                      inv_temperature, _lib.ptr(lse), _lib.ptr(ex), _lib.ptr(saved),
                                                      _lib.ptr(g_lp), _lib.ptr(g_ent),
                                                      _lib.ptr(d_h) if need_hidden else None,
                                                      _lib.ptr(d_w) if need_weight else None, _lib.ptr(ws), nws,
                                                      _lib.current_stream(dev))
    _lib.check(rc, "siirl_fused_linear_logprob_entropy_bwd")
    return d_h, d_w


@fused_linear_logprob_entropy_bwd.register_fake
def _(hidden, weight, labels, inv_temperature, lse, ex, g_logprob, g_entropy, need_hidden, need_weight, saved=None):
    return (hidden.new_empty(hidden.shape if need_hidden else (0,)),
            weight.new_empty(weight.shape if need_weight else (0,)))
